// Copies between a layout whose two innermost joint dims are one dense run (long x short, the short
// dim fastest) and one that keeps the long dim at unit stride, the short dim selecting a plane:
// tall-and-skinny transposes such as (N, 3) <-> (3, N):t() and the NCHW <-> NHWC conversions of
// images with few channels. The 64 x 128 tiles of the tiled kernels are nearly empty on a short dim
// of 3..64 elements (a (2^22, 16) transpose ran at 0.09 of peak through them, and the element-wise
// strided kernel at 0.33-0.38 on 3 or 4 planes). Here a tile is T long-dim positions x all S
// short-dim positions, about 16 KiB: on the dense side one contiguous run of T * S elements, on the
// planar side S runs of T elements. Both sides move 16-byte packs, at element-aligned addresses where
// a run starts off the 16-byte grid; the tile changes order in LDS, laid out lds[s * pitch + t].
// (what the reference's one strided apply does for these copies: lib/THC/THCApply.cuh:426-640,
// called from lib/THC/THCTensorCopy.cu:26-122)
#pragma once
#include <algorithm>
#include <cstdint>
#include <type_traits>

#include "apply_plan.hpp"
#include "common.hpp"
#include "device_util.hpp"

namespace thc {
namespace {

struct SkinnyArgs {
  uint32_t S;             // extent of the short dim
  uint32_t T;             // long-dim positions per tile (a multiple of 16)
  uint32_t pitch;         // LDS elements between planes
  uint32_t totalTiles;
  uint64_t longSize;      // extent of the long dim
  int64_t planeStride;    // planar side: elements between planes
  int nbatch;             // dims outside the two, innermost first
  int ntStore;
  Divisor<uint32_t> sdiv;           // by S
  Divisor<uint32_t> tilesPerSlice;  // tiles along the long dim
  Divisor<uint32_t> bsize[kMaxDims];
  int64_t denseBatchStride[kMaxDims], planarBatchStride[kMaxDims];
};

// TO_PLANAR: the source is the dense side. VD / VP: packs on the dense / planar side. ES / ED: source
// and destination element types (raw unsigned integers of the element size for same-type copies); a
// converting copy converts on the way into LDS, which holds destination elements.
template <typename ES, typename ED, bool TO_PLANAR, bool VD, bool VP>
__global__ __launch_bounds__(kBlock) void skinny_copy_kernel(ED* __restrict__ dst, const ES* __restrict__ src,
                                                             SkinnyArgs a) {
  constexpr uint32_t VS = 16 / sizeof(ES), VT = 16 / sizeof(ED);
  using PS = Pack<ES, VS>;
  using PT = Pack<ED, VT>;
  extern __shared__ __align__(16) unsigned char lds_raw[];
  ED* lds = reinterpret_cast<ED*>(lds_raw);
  auto cvt = [](ES x) -> ED {
    if constexpr (std::is_same<ES, ED>::value) return x;
    else return convert_value<ED, ES>(x);
  };
  const uint32_t S = a.S, pitch = a.pitch;
  for (uint32_t b = blockIdx.x; b < a.totalTiles; b += gridDim.x) {
    uint32_t rest, tl;
    a.tilesPerSlice.divmod(b, rest, tl);
    int64_t dOff = 0, pOff = 0;
    for (int j = 0; j < a.nbatch; ++j) {
      uint32_t r;
      a.bsize[j].divmod(rest, rest, r);
      dOff += (int64_t)r * a.denseBatchStride[j];
      pOff += (int64_t)r * a.planarBatchStride[j];
    }
    const uint64_t t0 = (uint64_t)tl * a.T;
    const uint32_t tn = (uint32_t)min((uint64_t)a.T, a.longSize - t0);  // long-dim positions of this tile
    const uint32_t n = tn * S;                                            // elements of this tile
    dOff += (int64_t)(t0 * S);
    pOff += (int64_t)t0;
    // ---- into LDS
    if (TO_PLANAR) {
      const ES* dsrc = src + dOff;
      const uint32_t packs = VD ? n / VS : 0;
      constexpr int U = 4;
      for (uint32_t k0 = threadIdx.x; k0 < packs; k0 += U * kBlock) {
        PS v[U];
#pragma unroll
        for (int u = 0; u < U; ++u)
          v[u] = load_pack_unaligned<true, PS>(dsrc + (size_t)min(k0 + u * kBlock, packs - 1) * VS);
#pragma unroll
        for (int u = 0; u < U; ++u) {
          const uint32_t k = k0 + u * kBlock;
          if (k < packs) {
            uint32_t t, s;
            a.sdiv.divmod(k * VS, t, s);
#pragma unroll
            for (uint32_t e = 0; e < VS; ++e) {
              lds[s * pitch + t] = cvt(v[u].v[e]);
              if (++s == S) {
                s = 0;
                ++t;
              }
            }
          }
        }
      }
      for (uint32_t m = packs * VS + threadIdx.x; m < n; m += kBlock) {
        uint32_t t, s;
        a.sdiv.divmod(m, t, s);
        lds[s * pitch + t] = cvt(dsrc[m]);
      }
    } else {
      const ES* psrc = src + pOff;
      const uint32_t planePacks = VP ? tn / VS : 0;  // whole packs of a plane's run
      const uint32_t packs = planePacks * S;
      constexpr int U = 4;
      for (uint32_t k0 = threadIdx.x; VP && k0 < packs; k0 += U * kBlock) {
        PS v[U];
#pragma unroll
        for (int u = 0; u < U; ++u) {
          const uint32_t k = min(k0 + u * kBlock, packs - 1);
          const uint32_t s = k / (VP ? planePacks : 1u), j = k - s * planePacks;
          v[u] = load_pack_unaligned<true, PS>(psrc + (int64_t)s * a.planeStride + (int64_t)j * VS);
        }
#pragma unroll
        for (int u = 0; u < U; ++u) {
          const uint32_t k = k0 + u * kBlock;
          if (k < packs) {
            const uint32_t s = k / (VP ? planePacks : 1u), j = k - s * planePacks;
#pragma unroll
            for (uint32_t e = 0; e < VS; ++e) lds[s * pitch + j * VS + e] = cvt(v[u].v[e]);
          }
        }
      }
      // what the packs leave: the end of every plane's run, or all of it
      const uint32_t left = tn - planePacks * VS;
      for (uint32_t m = threadIdx.x; m < left * S; m += kBlock) {
        const uint32_t s = m / left, t = planePacks * VS + (m - s * left);
        lds[s * pitch + t] = cvt(psrc[(int64_t)s * a.planeStride + t]);
      }
    }
    __syncthreads();
    // ---- out of LDS
    if (TO_PLANAR) {
      ED* pdst = dst + pOff;
      const uint32_t planePacks = VP ? tn / VT : 0;
      const uint32_t packs = planePacks * S;
      for (uint32_t k = threadIdx.x; VP && k < packs; k += kBlock) {
        const uint32_t s = k / (VP ? planePacks : 1u), j = k - s * planePacks;
        PT v;
#pragma unroll
        for (uint32_t e = 0; e < VT; ++e) v.v[e] = lds[s * pitch + j * VT + e];
        ED* at = pdst + (int64_t)s * a.planeStride + (int64_t)j * VT;
        if (a.ntStore) store_pack_unaligned<true, PT>(at, v);
        else store_pack_unaligned<false, PT>(at, v);
      }
      const uint32_t left = tn - planePacks * VT;
      for (uint32_t m = threadIdx.x; m < left * S; m += kBlock) {
        const uint32_t s = m / left, t = planePacks * VT + (m - s * left);
        pdst[(int64_t)s * a.planeStride + t] = lds[s * pitch + t];
      }
    } else {
      ED* ddst = dst + dOff;
      const uint32_t packs = VD ? n / VT : 0;
      for (uint32_t k = threadIdx.x; k < packs; k += kBlock) {
        uint32_t t, s;
        a.sdiv.divmod(k * VT, t, s);
        PT v;
#pragma unroll
        for (uint32_t e = 0; e < VT; ++e) {
          v.v[e] = lds[s * pitch + t];
          if (++s == S) {
            s = 0;
            ++t;
          }
        }
        ED* at = ddst + (size_t)k * VT;
        if (a.ntStore) store_pack_unaligned<true, PT>(at, v);
        else store_pack_unaligned<false, PT>(at, v);
      }
      for (uint32_t m = packs * VT + threadIdx.x; m < n; m += kBlock) {
        uint32_t t, s;
        a.sdiv.divmod(m, t, s);
        ddst[m] = lds[s * pitch + t];
      }
    }
    __syncthreads();  // the tile is refilled by the next round
  }
}

// `pl` is the jointly collapsed plan of a copy, dims ordered by the destination's strides
// (operand 0 = destination, 1 = source). Returns false when the layouts are not of this kind.
template <typename ES, typename ED = ES>
bool launch_skinny_copy(THCState* s, const Plan& pl) {
  using E = typename std::conditional<(sizeof(ES) > sizeof(ED)), ES, ED>::type;  // the wider element sizes the tiles
  if (!tuning("apply.skinny", 1) || pl.nops != 2) return false;
  const int nd = pl.lay[0].dims;
  if (nd < 2 || pl.numel >= (int64_t(1) << 40)) return false;
  const Layout& out = pl.lay[0];
  const Layout& in = pl.lay[1];
  const int q = nd - 1, p = nd - 2;
  // which operand is the dense side, and which of the two dims is the short one (small shapes can be
  // read both ways: the shorter short dim wins)
  int dense = -1, ds = -1, dl = -1;
  const int64_t maxShortBytes = tuning("apply.skinny.max_short_bytes", 256);
  auto consider = [&](int cand, int cs, int cl) {
    const int64_t S = pl.lay[cand].size[cs], L = pl.lay[cand].size[cl];
    if (S < 2 || L < 64 || S * (int64_t)sizeof(E) > maxShortBytes) return;
    if (dense >= 0 && pl.lay[dense].size[ds] <= S) return;
    dense = cand, ds = cs, dl = cl;
  };
  // planes of the source gathered into dense rows of the destination
  if (out.stride[q] == 1 && out.stride[p] == out.size[q] && in.stride[p] == 1 && in.stride[q] > 0) consider(0, q, p);
  // dense rows of the source scattered into planes of the destination
  if (in.stride[p] == 1 && in.stride[q] == in.size[p] && out.stride[q] == 1 && out.stride[p] > 0) consider(1, p, q);
  if (dense < 0) return false;
  const Layout& dn = pl.lay[dense];
  const Layout& pn = pl.lay[1 - dense];
  const int64_t S = dn.size[ds], L = dn.size[dl];
  for (int k = 0; k < 2; ++k)
    for (int d = 0; d < nd; ++d)
      if (pl.lay[k].stride[d] < 0) return false;
  SkinnyArgs a{};
  a.S = (uint32_t)S;
  a.longSize = (uint64_t)L;
  a.planeStride = pn.stride[ds];
  int64_t T = std::max<int64_t>(64, (tuning("apply.skinny.tile_bytes", 16384) / (S * (int64_t)sizeof(E))) / 16 * 16);
  T = std::min<int64_t>(T, (L + 15) / 16 * 16);
  a.T = (uint32_t)T;
  a.pitch = (uint32_t)(T + 16 / sizeof(ED) + 1) | 1u;
  a.sdiv.set((uint64_t)S);
  const int64_t tiles = (L + T - 1) / T;
  a.tilesPerSlice.set((uint64_t)tiles);
  int64_t total = tiles;
  a.nbatch = 0;
  for (int d = nd - 3; d >= 0; --d) {
    a.bsize[a.nbatch].set((uint64_t)dn.size[d]);
    a.denseBatchStride[a.nbatch] = dn.stride[d];
    a.planarBatchStride[a.nbatch] = pn.stride[d];
    ++a.nbatch;
    total *= dn.size[d];
  }
  if (total >= (int64_t(1) << 31)) return false;
  a.totalTiles = (uint32_t)total;
  a.ntStore = streaming_store("apply.tiled.nt_store", pl.numel * (int64_t)sizeof(ED)) ? 1 : 0;
  // packs: every tile's run starts on a 16-byte boundary (operand 0 holds ED elements, operand 1 ES)
  // (`apply.skinny.aligned_packs_only`: packs only where every tile's run starts on a 16-byte boundary, the
  // element-wise variants elsewhere; by default packs sit at element-aligned addresses, which this target allows)
  auto aligned = [](const void* ptr) { return reinterpret_cast<uintptr_t>(ptr) % 16 == 0; };
  const int64_t denseBytes = dense == 0 ? sizeof(ED) : sizeof(ES), planarBytes = dense == 0 ? sizeof(ES) : sizeof(ED);
  bool vd = true, vp = true;
  if (tuning("apply.skinny.aligned_packs_only", 0)) {
    vd = aligned(pl.ptr[dense]);
    vp = aligned(pl.ptr[1 - dense]) && (a.planeStride * planarBytes) % 16 == 0;
    for (int j = 0; j < a.nbatch; ++j) {
      vd = vd && (a.denseBatchStride[j] * denseBytes) % 16 == 0;
      vp = vp && (a.planarBatchStride[j] * planarBytes) % 16 == 0;
    }
  }
  const size_t ldsBytes = ((size_t)S * a.pitch * sizeof(ED) + 15) & ~size_t(15);
  if (ldsBytes > 64 * 1024) return false;
  const int grid = (int)std::max<int64_t>(1, std::min<int64_t>(total, (int64_t)num_compute_units(s) * 64));
  ED* dst = (ED*)pl.ptr[0];
  const ES* src = (const ES*)pl.ptr[1];
  hipStream_t st = current_stream(s);
#define THC_SKINNY(TP, D, Pk) \
  hipLaunchKernelGGL((skinny_copy_kernel<ES, ED, TP, D, Pk>), dim3(grid), dim3(kBlock), ldsBytes, st, dst, src, a)
  if (dense == 1) {
    if (vd && vp) THC_SKINNY(true, true, true);
    else if (vd) THC_SKINNY(true, true, false);
    else if (vp) THC_SKINNY(true, false, true);
    else THC_SKINNY(true, false, false);
  } else {
    if (vd && vp) THC_SKINNY(false, true, true);
    else if (vd) THC_SKINNY(false, true, false);
    else if (vp) THC_SKINNY(false, false, true);
    else THC_SKINNY(false, false, false);
  }
#undef THC_SKINNY
  note_kernel("skinny");
  return true;
}


// Batches of small dense matrices transposed ((B, P, Q) <- (B, Q, P) with P, Q below 64: per-pixel
// 3 x 3 or 4 x 4 matrices, 16 x 16 blocks): a 64 x 128 tile of the tiled kernels holds one such matrix
// and little else (2^18 x 16 x 16 ran at 0.12 of peak, 2^20 x 8 x 8 at 0.035). A tile here is K whole
// matrices, about 16 KiB, one contiguous run on BOTH sides: packs in, packs out, the order changed in
// LDS (source rows at a pitch of P + 1 elements).
struct SmallTransposeArgs {
  uint32_t P, Q, K;        // out is (.., P, Q), source rows are P long; K matrices per tile
  uint32_t pitch;          // LDS elements per matrix
  uint32_t totalTiles;
  uint64_t batch;          // matrices in the innermost batch dim (contiguous on both sides)
  int nbatch;              // dims outside that one, innermost first
  int ntStore;
  Divisor<uint32_t> pdiv, qdiv, pqdiv, tilesPerRun;
  Divisor<uint32_t> bsize[kMaxDims];
  int64_t dstBatchStride[kMaxDims], srcBatchStride[kMaxDims];
};

template <typename ES, typename ED, bool VIN, bool VOUT>
__global__ __launch_bounds__(kBlock) void small_transpose_kernel(ED* __restrict__ dst, const ES* __restrict__ src,
                                                                 SmallTransposeArgs a) {
  constexpr uint32_t VS = 16 / sizeof(ES), VT = 16 / sizeof(ED);
  using PS = Pack<ES, VS>;
  using PT = Pack<ED, VT>;
  extern __shared__ __align__(16) unsigned char lds_raw[];
  ED* lds = reinterpret_cast<ED*>(lds_raw);
  auto cvt = [](ES x) -> ED {
    if constexpr (std::is_same<ES, ED>::value) return x;
    else return convert_value<ED, ES>(x);
  };
  const uint32_t P = a.P, PQ = a.P * a.Q, rowPitch = a.P + 1;
  // source element m of a tile is (k, q, p) = (m / PQ, (m % PQ) / P, m % P); it waits at
  // lds[k * pitch + q * (P + 1) + p] for destination element (k, p, q)
  auto src_slot = [&](uint32_t m) {
    uint32_t k, r, q, pp;
    a.pqdiv.divmod(m, k, r);
    a.pdiv.divmod(r, q, pp);
    return k * a.pitch + q * rowPitch + pp;
  };
  auto dst_slot = [&](uint32_t m) {
    uint32_t k, r, pp, q;
    a.pqdiv.divmod(m, k, r);
    a.qdiv.divmod(r, pp, q);
    return k * a.pitch + q * rowPitch + pp;
  };
  for (uint32_t b = blockIdx.x; b < a.totalTiles; b += gridDim.x) {
    uint32_t rest, tl;
    a.tilesPerRun.divmod(b, rest, tl);
    int64_t dOff = 0, sOff = 0;
    for (int j = 0; j < a.nbatch; ++j) {
      uint32_t r;
      a.bsize[j].divmod(rest, rest, r);
      dOff += (int64_t)r * a.dstBatchStride[j];
      sOff += (int64_t)r * a.srcBatchStride[j];
    }
    const uint64_t k0 = (uint64_t)tl * a.K;
    const uint32_t kn = (uint32_t)min((uint64_t)a.K, a.batch - k0);
    const uint32_t n = kn * PQ;
    const ES* in = src + sOff + (int64_t)(k0 * PQ);
    ED* out = dst + dOff + (int64_t)(k0 * PQ);
    const uint32_t packsIn = VIN ? n / VS : 0;
    constexpr int U = 4;
    for (uint32_t i0 = threadIdx.x; i0 < packsIn; i0 += U * kBlock) {
      PS v[U];
#pragma unroll
      for (int u = 0; u < U; ++u) v[u] = load_pack_unaligned<true, PS>(in + (size_t)min(i0 + u * kBlock, packsIn - 1) * VS);
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const uint32_t i = i0 + u * kBlock;
        if (i < packsIn) {
#pragma unroll
          for (uint32_t e = 0; e < VS; ++e) lds[src_slot(i * VS + e)] = cvt(v[u].v[e]);
        }
      }
    }
    for (uint32_t m = packsIn * VS + threadIdx.x; m < n; m += kBlock) lds[src_slot(m)] = cvt(in[m]);
    __syncthreads();
    const uint32_t packsOut = VOUT ? n / VT : 0;
    for (uint32_t i = threadIdx.x; i < packsOut; i += kBlock) {
      PT v;
#pragma unroll
      for (uint32_t e = 0; e < VT; ++e) v.v[e] = lds[dst_slot(i * VT + e)];
      ED* at = out + (size_t)i * VT;
      if (a.ntStore) store_pack_unaligned<true, PT>(at, v);
      else store_pack_unaligned<false, PT>(at, v);
    }
    for (uint32_t m = packsOut * VT + threadIdx.x; m < n; m += kBlock) out[m] = lds[dst_slot(m)];
    __syncthreads();  // the tile is refilled by the next round
  }
}

// `pl` as for launch_skinny_copy. Returns false when the layouts are not of this kind.
template <typename ES, typename ED = ES>
bool launch_small_transpose(THCState* s, const Plan& pl) {
  using E = typename std::conditional<(sizeof(ES) > sizeof(ED)), ES, ED>::type;
  if (!tuning("apply.small_transpose", 1) || pl.nops != 2) return false;
  const int nd = pl.lay[0].dims;
  if (nd < 3 || pl.numel >= (int64_t(1) << 40)) return false;
  const Layout& out = pl.lay[0];
  const Layout& in = pl.lay[1];
  const int q = nd - 1, p = nd - 2, bd = nd - 3;
  const int64_t P = out.size[p], Q = out.size[q], PQ = P * Q;
  if (P < 2 || Q < 2 || P >= 64 || Q >= 64) return false;
  if (out.stride[q] != 1 || out.stride[p] != Q || in.stride[p] != 1 || in.stride[q] != P) return false;
  if (out.stride[bd] != PQ || in.stride[bd] != PQ || out.size[bd] < 8) return false;
  for (int k = 0; k < 2; ++k)
    for (int d = 0; d < nd; ++d)
      if (pl.lay[k].stride[d] < 0) return false;
  SmallTransposeArgs a{};
  a.P = (uint32_t)P;
  a.Q = (uint32_t)Q;
  a.batch = (uint64_t)out.size[bd];
  // K matrices per tile: about 16 KiB, a whole number of 16-element groups so that tiles start on pack boundaries
  int64_t K = std::max<int64_t>(1, tuning("apply.skinny.tile_bytes", 16384) / (PQ * (int64_t)sizeof(E)));
  int64_t unit = 16;
  for (int64_t g = PQ; g % 2 == 0 && unit > 1; g /= 2) unit /= 2;  // 16 / gcd(PQ, 16)
  K = std::max<int64_t>(unit, K / unit * unit);
  K = std::min<int64_t>(K, (out.size[bd] + unit - 1) / unit * unit);
  a.K = (uint32_t)K;
  a.pitch = (uint32_t)(Q * (P + 1));
  a.pdiv.set((uint64_t)P);
  a.qdiv.set((uint64_t)Q);
  a.pqdiv.set((uint64_t)PQ);
  const int64_t tiles = (out.size[bd] + K - 1) / K;
  a.tilesPerRun.set((uint64_t)tiles);
  int64_t total = tiles;
  a.nbatch = 0;
  for (int d = nd - 4; d >= 0; --d) {
    a.bsize[a.nbatch].set((uint64_t)out.size[d]);
    a.dstBatchStride[a.nbatch] = out.stride[d];
    a.srcBatchStride[a.nbatch] = in.stride[d];
    ++a.nbatch;
    total *= out.size[d];
  }
  if (total >= (int64_t(1) << 31)) return false;
  a.totalTiles = (uint32_t)total;
  a.ntStore = streaming_store("apply.tiled.nt_store", pl.numel * (int64_t)sizeof(ED)) ? 1 : 0;
  auto aligned = [](const void* ptr) { return reinterpret_cast<uintptr_t>(ptr) % 16 == 0; };
  bool vout = true, vin = true;
  if (tuning("apply.skinny.aligned_packs_only", 0)) {
    vout = aligned(pl.ptr[0]);
    vin = aligned(pl.ptr[1]);
    for (int j = 0; j < a.nbatch; ++j) {
      vout = vout && (a.dstBatchStride[j] * (int64_t)sizeof(ED)) % 16 == 0;
      vin = vin && (a.srcBatchStride[j] * (int64_t)sizeof(ES)) % 16 == 0;
    }
  }
  const size_t ldsBytes = ((size_t)K * a.pitch * sizeof(ED) + 15) & ~size_t(15);
  if (ldsBytes > 64 * 1024) return false;
  const int grid = (int)std::max<int64_t>(1, std::min<int64_t>(total, (int64_t)num_compute_units(s) * 64));
  ED* dst = (ED*)pl.ptr[0];
  const ES* src = (const ES*)pl.ptr[1];
  hipStream_t st = current_stream(s);
#define THC_SMALLT(VI, VO) \
  hipLaunchKernelGGL((small_transpose_kernel<ES, ED, VI, VO>), dim3(grid), dim3(kBlock), ldsBytes, st, dst, src, a)
  if (vin && vout) THC_SMALLT(true, true);
  else if (vin) THC_SMALLT(true, false);
  else if (vout) THC_SMALLT(false, true);
  else THC_SMALLT(false, false);
#undef THC_SMALLT
  note_kernel("small-transpose");
  return true;
}

}  // namespace
}  // namespace thc
