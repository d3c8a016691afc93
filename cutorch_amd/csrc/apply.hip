// Strided pointwise apply engine for gfx950 (wave64, 256 CUs, HBM-bound).
//
// Role of THC_pointwiseApply1/2/3 + kernelPointwiseApply1/2/3
// (lib/THC/THCApply.cuh:19-98,124-640): run an elementwise functor over
// operands that are each addressed through their own sizes/strides. The
// design differs from the reference on purpose:
//   * the operands are described in ONE joint iteration space (shared sizes,
//     per-operand strides), so the index -> coordinate division chain runs
//     once per 16-byte pack, not once per element and operand;
//   * four kernel families instead of one:
//       contig   every operand is a flat run: dwordx4 grid-stride streaming
//       strided  all operands have unit stride in the innermost joint dim:
//                dwordx4 packs along it, outer coordinates by multiply-shift
//                division
//       tiled    an operand whose unit-stride dim is not the output's goes
//                through an LDS tile so that both sides of the transpose are
//                accessed in 256-byte coalesced rows
//       generic  operands of different shapes (paired by logical linear
//                index) or with no unit-stride dim: per-element offsets
//   * 32-bit index arithmetic when every count and offset is < 2^31, 64-bit
//     otherwise (tile origins are the only 64-bit quantities in the tiled
//     kernel; inside a tile all arithmetic is 32-bit).
#include <hip/hip_fp16.h>

#include "common.hpp"

namespace thc {

// ------------------------------------------------------------------------
// Element packs and functors
// ------------------------------------------------------------------------
template <typename T, int N>
struct alignas(sizeof(T) * N) Pack {
  T v[N];
};

template <typename T>
struct Cvt {
  static __device__ __forceinline__ float up(T x) { return (float)x; }
  static __device__ __forceinline__ T down(float x) { return (T)x; }
};
template <>
struct Cvt<__half> {
  static __device__ __forceinline__ float up(__half x) { return __half2float(x); }
  static __device__ __forceinline__ __half down(float x) { return __float2half_rn(x); }
};

// Arithmetic is done in fp32 and rounded once to the element type; the build
// disables fp contraction so a*b+c stays two roundings (the CPU contract).
struct OpCopy {
  static constexpr int NIN = 1;
  template <typename T>
  __device__ __forceinline__ T operator()(T a, T, T) const {
    return a;
  }
};
struct OpFill {
  static constexpr int NIN = 0;
  float v;
  template <typename T>
  __device__ __forceinline__ T operator()(T, T, T) const {
    return Cvt<T>::down(v);
  }
};
#define THC_ARITH_OP(Name, NIN_, EXPR)                                  \
  struct Name {                                                         \
    static constexpr int NIN = NIN_;                                    \
    float v;                                                            \
    template <typename T>                                               \
    __device__ __forceinline__ T operator()(T a_, T b_, T c_) const {   \
      const float a = Cvt<T>::up(a_), b = Cvt<T>::up(b_), c = Cvt<T>::up(c_); \
      (void)a; (void)b; (void)c;                                        \
      return Cvt<T>::down(EXPR);                                        \
    }                                                                   \
  };
THC_ARITH_OP(OpAddC, 1, a + v)
THC_ARITH_OP(OpSubC, 1, a - v)
THC_ARITH_OP(OpMulC, 1, a * v)
THC_ARITH_OP(OpDivC, 1, a / v)
THC_ARITH_OP(OpPow, 1, powf(a, v))
THC_ARITH_OP(OpAdd, 2, a + b)
THC_ARITH_OP(OpSub, 2, a - b)
THC_ARITH_OP(OpMul, 2, a * b)
THC_ARITH_OP(OpDiv, 2, a / b)
THC_ARITH_OP(OpCAdd, 2, a + v * b)
THC_ARITH_OP(OpAddCMul, 3, a + v * (b * c))
THC_ARITH_OP(OpAddCDiv, 3, a + v * (b / c))
#undef THC_ARITH_OP

int point_op_inputs(PointOp op) {
  switch (op) {
    case PointOp::Fill: return 0;
    case PointOp::Copy: case PointOp::AddC: case PointOp::SubC: case PointOp::MulC:
    case PointOp::DivC: case PointOp::Pow: return 1;
    case PointOp::Add: case PointOp::Sub: case PointOp::Mul: case PointOp::Div:
    case PointOp::CAdd: return 2;
    default: return 3;
  }
}

// ------------------------------------------------------------------------
// Division by a launch-invariant divisor
// ------------------------------------------------------------------------
// 32-bit: round-up multiply-shift (Granlund & Montgomery, "Division by
// invariant integers using multiplication", 1994): with s = ceil(log2 d) and
// m = floor(2^32 (2^s - d) / d) + 1, floor(n / d) = (mulhi(n, m) + n) >> s for
// every n < 2^31 (the sum cannot carry out of 32 bits).
template <typename I>
struct Divisor;
template <>
struct Divisor<uint32_t> {
  uint32_t d, m, s;
  __host__ void set(uint64_t div) {
    d = (uint32_t)div;
    for (s = 0; s < 32; ++s)
      if ((uint64_t(1) << s) >= div) break;
    m = (uint32_t)(((uint64_t(1) << 32) * ((uint64_t(1) << s) - div)) / div + 1);
  }
  __device__ __forceinline__ void divmod(uint32_t n, uint32_t& q, uint32_t& r) const {
    q = (__umulhi(n, m) + n) >> s;
    r = n - q * d;
  }
};
template <>
struct Divisor<uint64_t> {
  uint64_t d;
  __host__ void set(uint64_t div) { d = div; }
  __device__ __forceinline__ void divmod(uint64_t n, uint64_t& q, uint64_t& r) const {
    q = n / d;
    r = n - q * d;
  }
};

constexpr int kMaxOps = 4;
constexpr int kBlock = 256;

// ------------------------------------------------------------------------
// contig: flat streaming, one 16-byte pack per operand per step
// ------------------------------------------------------------------------
template <typename T, typename Op, int VEC, int UNROLL>
__global__ __launch_bounds__(kBlock) void apply_contig_kernel(T* out, const T* in0, const T* in1,
                                                              const T* in2, uint64_t n, Op op) {
  using P = Pack<T, VEC>;
  const uint64_t npack = n / VEC;
  const uint64_t step = (uint64_t)gridDim.x * (kBlock * UNROLL);
  for (uint64_t base = (uint64_t)blockIdx.x * (kBlock * UNROLL) + threadIdx.x; base < npack;
       base += step) {
    P a[UNROLL], b[UNROLL], c[UNROLL];
#pragma unroll
    for (int u = 0; u < UNROLL; ++u) {
      const uint64_t i = base + (uint64_t)u * kBlock;
      if (i < npack) {
        if (Op::NIN > 0) a[u] = reinterpret_cast<const P*>(in0)[i];
        if (Op::NIN > 1) b[u] = reinterpret_cast<const P*>(in1)[i];
        if (Op::NIN > 2) c[u] = reinterpret_cast<const P*>(in2)[i];
      }
    }
#pragma unroll
    for (int u = 0; u < UNROLL; ++u) {
      const uint64_t i = base + (uint64_t)u * kBlock;
      if (i < npack) {
        P r;
#pragma unroll
        for (int e = 0; e < VEC; ++e) r.v[e] = op(a[u].v[e], b[u].v[e], c[u].v[e]);
        reinterpret_cast<P*>(out)[i] = r;
      }
    }
  }
  // the n % VEC trailing elements
  const uint64_t tail = npack * VEC + (uint64_t)blockIdx.x * kBlock + threadIdx.x;
  if (VEC > 1 && tail < n) {
    T a{}, b{}, c{};
    if (Op::NIN > 0) a = in0[tail];
    if (Op::NIN > 1) b = in1[tail];
    if (Op::NIN > 2) c = in2[tail];
    out[tail] = op(a, b, c);
  }
}

// ------------------------------------------------------------------------
// strided / generic: linear index -> per-operand offsets
// ------------------------------------------------------------------------
template <typename I>
struct IndexedArgs {
  int dims[kMaxOps];                  // JOINT: only dims[0] is used
  Divisor<I> size[kMaxOps][kMaxDims]; // JOINT: only size[0][*] is used
  I stride[kMaxOps][kMaxDims];        // in elements; pre-multiplied by VEC in the packed dim
};

// JOINT = all operands share sizes (one division chain); VEC packs along the
// innermost dim (then that dim's size is already divided by VEC on the host).
template <typename T, typename Op, typename I, int VEC, bool JOINT>
__global__ __launch_bounds__(kBlock) void apply_indexed_kernel(T* out, const T* in0, const T* in1,
                                                               const T* in2, I total,
                                                               IndexedArgs<I> args, Op op) {
  using P = Pack<T, VEC>;
  constexpr int NOPS = Op::NIN + 1;
  const I step = (I)gridDim.x * kBlock;
  for (I lin = (I)blockIdx.x * kBlock + threadIdx.x; lin < total; lin += step) {
    I off[kMaxOps] = {0, 0, 0, 0};
    if (JOINT) {
      I rest = lin;
      for (int d = args.dims[0] - 1; d > 0; --d) {
        I q, r;
        args.size[0][d].divmod(rest, q, r);
        rest = q;
#pragma unroll
        for (int k = 0; k < NOPS; ++k) off[k] += r * args.stride[k][d];
      }
#pragma unroll
      for (int k = 0; k < NOPS; ++k) off[k] += rest * args.stride[k][0];
    } else {
#pragma unroll
      for (int k = 0; k < NOPS; ++k) {
        I rest = lin;
        for (int d = args.dims[k] - 1; d > 0; --d) {
          I q, r;
          args.size[k][d].divmod(rest, q, r);
          rest = q;
          off[k] += r * args.stride[k][d];
        }
        off[k] += rest * args.stride[k][0];
      }
    }
    P a{}, b{}, c{};
    if (Op::NIN > 0) a = *reinterpret_cast<const P*>(in0 + off[1]);
    if (Op::NIN > 1) b = *reinterpret_cast<const P*>(in1 + off[2]);
    if (Op::NIN > 2) c = *reinterpret_cast<const P*>(in2 + off[3]);
    P r;
#pragma unroll
    for (int e = 0; e < VEC; ++e) r.v[e] = op(a.v[e], b.v[e], c.v[e]);
    *reinterpret_cast<P*>(out + off[0]) = r;
  }
}

// ------------------------------------------------------------------------
// tiled: operands whose unit-stride dim is `p` meet operands whose
// unit-stride dim is `q` in a TILE x TILE patch staged through LDS.
// ------------------------------------------------------------------------
template <typename I>
struct TiledArgs {
  int dims;
  int p, q;
  int staged[kMaxOps];             // operand k is accessed along p (through LDS)
  I size[kMaxDims];
  Divisor<I> bsize[kMaxDims];      // divisors of the batch dims (all but p, q)
  I stride[kMaxOps][kMaxDims];
  Divisor<I> tilesP, tilesQ;
  I totalTiles;
};

// LX lanes cover one tile row with VEC elements each: TILE = LX * VEC.
template <typename T, typename Op, typename I, int VEC, int LX>
__global__ __launch_bounds__(kBlock) void apply_tiled_kernel(T* out, const T* in0, const T* in1,
                                                             const T* in2, TiledArgs<I> args,
                                                             Op op) {
  constexpr int NOPS = Op::NIN + 1;
  constexpr int TILE = LX * VEC;
  constexpr int ROWS = kBlock / LX;      // tile rows covered per pass
  constexpr int PASSES = TILE / ROWS;
  constexpr int PITCH = TILE + 1;        // odd pitch: conflict-free transposed reads
  using P = Pack<T, VEC>;
  extern __shared__ __align__(16) unsigned char lds_raw[];
  T* lds = reinterpret_cast<T*>(lds_raw);

  const T* ptr[kMaxOps] = {out, in0, in1, in2};
  const int lx = threadIdx.x % LX;
  const int ly = threadIdx.x / LX;
  int slot[kMaxOps];  // LDS slab of a staged operand
  {
    int s = 0;
#pragma unroll
    for (int k = 0; k < NOPS; ++k) slot[k] = args.staged[k] ? s++ : -1;
  }

  for (I tile = blockIdx.x; tile < args.totalTiles; tile += gridDim.x) {
    I rest, tq, tp;
    args.tilesQ.divmod(tile, rest, tq);
    args.tilesP.divmod(rest, rest, tp);
    I base[kMaxOps] = {0, 0, 0, 0};
    for (int d = args.dims - 1; d >= 0; --d) {
      if (d == args.p || d == args.q) continue;
      I r;
      args.bsize[d].divmod(rest, rest, r);
#pragma unroll
      for (int k = 0; k < NOPS; ++k) base[k] += r * args.stride[k][d];
    }
    const I p0 = tp * TILE, q0 = tq * TILE;
    const uint32_t pn = (uint32_t)min((I)TILE, args.size[args.p] - p0);  // valid rows/cols
    const uint32_t qn = (uint32_t)min((I)TILE, args.size[args.q] - q0);
#pragma unroll
    for (int k = 0; k < NOPS; ++k)
      base[k] += p0 * args.stride[k][args.p] + q0 * args.stride[k][args.q];

    // phase 1: staged inputs, lanes along p, into lds[slot][q][p]
#pragma unroll
    for (int k = 1; k < NOPS; ++k) {
      if (!args.staged[k]) continue;
      T* slab = lds + slot[k] * (TILE * PITCH);
      const I sq = args.stride[k][args.q];
#pragma unroll
      for (int r = 0; r < PASSES; ++r) {
        const uint32_t qi = ly + r * ROWS, pi = lx * VEC;
        if (qi < qn && pi < pn) {
          const P v = *reinterpret_cast<const P*>(ptr[k] + base[k] + (I)qi * sq + pi);
#pragma unroll
          for (int e = 0; e < VEC; ++e) slab[qi * PITCH + pi + e] = v.v[e];
        }
      }
    }
    __syncthreads();

    // phase 2: compute with lanes along q
#pragma unroll
    for (int r = 0; r < PASSES; ++r) {
      const uint32_t pi = ly + r * ROWS, qi = lx * VEC;
      if (pi < pn && qi < qn) {
        P in[3] = {};
#pragma unroll
        for (int k = 1; k < NOPS; ++k) {
          if (args.staged[k]) {
            const T* slab = lds + slot[k] * (TILE * PITCH);
#pragma unroll
            for (int e = 0; e < VEC; ++e) in[k - 1].v[e] = slab[(qi + e) * PITCH + pi];
          } else if (VEC > 1) {
            in[k - 1] = *reinterpret_cast<const P*>(ptr[k] + base[k] +
                                                    (I)pi * args.stride[k][args.p] + qi);
          } else {
            in[k - 1].v[0] = ptr[k][base[k] + (I)pi * args.stride[k][args.p] +
                                    (I)qi * args.stride[k][args.q]];
          }
        }
        P res;
#pragma unroll
        for (int e = 0; e < VEC; ++e) res.v[e] = op(in[0].v[e], in[1].v[e], in[2].v[e]);
        if (args.staged[0]) {
          T* slab = lds + slot[0] * (TILE * PITCH);
#pragma unroll
          for (int e = 0; e < VEC; ++e) slab[(qi + e) * PITCH + pi] = res.v[e];
        } else if (VEC > 1) {
          *reinterpret_cast<P*>(out + base[0] + (I)pi * args.stride[0][args.p] + qi) = res;
        } else {
          out[base[0] + (I)pi * args.stride[0][args.p] + (I)qi * args.stride[0][args.q]] =
              res.v[0];
        }
      }
    }

    // phase 3: a staged output leaves with lanes along p
    if (args.staged[0]) {
      __syncthreads();
      const T* slab = lds + slot[0] * (TILE * PITCH);
      const I sq = args.stride[0][args.q];
#pragma unroll
      for (int r = 0; r < PASSES; ++r) {
        const uint32_t qi = ly + r * ROWS, pi = lx * VEC;
        if (qi < qn && pi < pn) {
          P v;
#pragma unroll
          for (int e = 0; e < VEC; ++e) v.v[e] = slab[qi * PITCH + pi + e];
          *reinterpret_cast<P*>(out + base[0] + (I)qi * sq + pi) = v;
        }
      }
    }
    __syncthreads();  // the slabs are reused by the next tile
  }
}

// ------------------------------------------------------------------------
// Host side: planning and launch
// ------------------------------------------------------------------------
namespace {

struct Plan {
  int nops;
  void* ptr[kMaxOps];
  Layout lay[kMaxOps];
  int64_t numel;
};

template <typename T>
bool aligned16(const void* p) {
  return (reinterpret_cast<uintptr_t>(p) & 15u) == 0;
}

int grid_for(THCState* s, int64_t work_items, int per_block, const char* key, int default_per_cu) {
  const int64_t blocks = (work_items + per_block - 1) / per_block;
  const int64_t cap = (int64_t)num_compute_units(s) * tuning(key, default_per_cu);
  return (int)std::max<int64_t>(1, std::min(blocks, cap));
}

template <typename T, typename Op>
void launch_contig(THCState* s, const Plan& pl, Op op) {
  constexpr int VEC = 16 / sizeof(T);
  bool vec = true;
  for (int k = 0; k < pl.nops; ++k) vec = vec && aligned16<T>(pl.ptr[k]);
  T* out = (T*)pl.ptr[0];
  const T* i0 = (const T*)pl.ptr[1];
  const T* i1 = (const T*)pl.ptr[2];
  const T* i2 = (const T*)pl.ptr[3];
  const uint64_t n = (uint64_t)pl.numel;
  hipStream_t st = current_stream(s);
  if (vec) {
    constexpr int U = 4;
    const int grid = grid_for(s, (int64_t)(n / VEC) + 1, kBlock * U, "apply.contig.blocks_per_cu", 16);
    hipLaunchKernelGGL((apply_contig_kernel<T, Op, VEC, U>), dim3(grid), dim3(kBlock), 0, st, out,
                       i0, i1, i2, n, op);
    note_kernel("contig");
  } else {
    constexpr int U = 4;
    const int grid = grid_for(s, (int64_t)n, kBlock * U, "apply.contig.blocks_per_cu", 16);
    hipLaunchKernelGGL((apply_contig_kernel<T, Op, 1, U>), dim3(grid), dim3(kBlock), 0, st, out, i0,
                       i1, i2, n, op);
    note_kernel("contig-scalar");
  }
}

template <typename T, typename Op, typename I, bool JOINT>
void launch_indexed(THCState* s, const Plan& pl, Op op) {
  constexpr int VEC = 16 / sizeof(T);
  IndexedArgs<I> args{};
  bool vec = JOINT;
  if (JOINT) {
    const int nd = pl.lay[0].dims;
    vec = vec && pl.lay[0].size[nd - 1] % VEC == 0;
    for (int k = 0; k < pl.nops && vec; ++k) {
      vec = aligned16<T>(pl.ptr[k]) && pl.lay[k].stride[nd - 1] == 1;
      for (int d = 0; d < nd - 1 && vec; ++d) vec = pl.lay[k].stride[d] % VEC == 0;
    }
  }
  const int pack = vec ? VEC : 1;
  for (int k = 0; k < pl.nops; ++k) {
    const int nd = pl.lay[k].dims;
    args.dims[k] = nd;
    for (int d = 0; d < nd; ++d) {
      int64_t sz = pl.lay[k].size[d];
      int64_t sd = pl.lay[k].stride[d];
      if (vec && d == nd - 1) {
        sz /= pack;
        sd *= pack;
      }
      args.size[k][d].set((uint64_t)sz);
      args.stride[k][d] = (I)sd;
    }
  }
  const int64_t total = pl.numel / pack;
  const int grid = grid_for(s, total, kBlock, "apply.indexed.blocks_per_cu", 32);
  T* out = (T*)pl.ptr[0];
  const T* i0 = (const T*)pl.ptr[1];
  const T* i1 = (const T*)pl.ptr[2];
  const T* i2 = (const T*)pl.ptr[3];
  hipStream_t st = current_stream(s);
  if (vec) {
    hipLaunchKernelGGL((apply_indexed_kernel<T, Op, I, VEC, JOINT>), dim3(grid), dim3(kBlock), 0, st,
                       out, i0, i1, i2, (I)total, args, op);
  } else {
    hipLaunchKernelGGL((apply_indexed_kernel<T, Op, I, 1, JOINT>), dim3(grid), dim3(kBlock), 0, st,
                       out, i0, i1, i2, (I)total, args, op);
  }
  note_kernel(JOINT ? (vec ? "strided" : "strided-scalar") : "generic");
}

// Pick (p, q) for the tiled kernel. q = innermost joint dim. An operand is
// staged when its unit-stride dim is p != q. Returns false when no operand
// wants a transpose (or the transposed operands disagree about p).
bool tile_plan(const Plan& pl, int& p, int& q, int staged[kMaxOps]) {
  const int nd = pl.lay[0].dims;
  if (nd < 2) return false;
  q = nd - 1;
  p = -1;
  for (int k = 0; k < pl.nops; ++k) {
    staged[k] = 0;
    if (pl.lay[k].stride[q] == 1) continue;
    int unit = -1;
    for (int d = 0; d < nd - 1; ++d)
      if (pl.lay[k].stride[d] == 1) unit = d;
    if (unit < 0) continue;  // no unit-stride dim at all: direct (uncoalesced) access
    if (p < 0) p = unit;
    if (unit == p) staged[k] = 1;
  }
  if (p < 0) return false;
  // Tiny tile dims make the LDS detour pointless.
  if (pl.lay[0].size[p] < 8 || pl.lay[0].size[q] < 8) return false;
  return true;
}

template <typename T, typename Op, typename I>
bool launch_tiled(THCState* s, const Plan& pl, Op op) {
  int p, q, staged[kMaxOps] = {0, 0, 0, 0};
  if (!tile_plan(pl, p, q, staged)) return false;
  constexpr int VEC = 16 / sizeof(T);
  constexpr int LX = 16;
  const int nd = pl.lay[0].dims;
  int nstaged = 0;
  for (int k = 0; k < pl.nops; ++k) nstaged += staged[k];

  // 16-byte packs need every pack fully inside the tensor and aligned.
  bool vec = pl.lay[0].size[p] % VEC == 0 && pl.lay[0].size[q] % VEC == 0;
  for (int k = 0; k < pl.nops && vec; ++k) {
    const int fast = staged[k] ? p : q;
    vec = aligned16<T>(pl.ptr[k]) && pl.lay[k].stride[fast] == 1;
    for (int d = 0; d < nd && vec; ++d)
      if (d != fast) vec = pl.lay[k].stride[d] % VEC == 0;
  }
  const size_t tileV = LX * VEC, tileS = 64;
  const size_t ldsV = nstaged * tileV * (tileV + 1) * sizeof(T);
  const size_t ldsS = nstaged * tileS * (tileS + 1) * sizeof(T);
  if (vec && ldsV > 64 * 1024) vec = false;
  if (!vec && ldsS > 64 * 1024) return false;
  const int64_t tile = vec ? (int64_t)tileV : (int64_t)tileS;

  TiledArgs<I> args{};
  args.dims = nd;
  args.p = p;
  args.q = q;
  int64_t batch = 1;
  for (int d = 0; d < nd; ++d) {
    args.size[d] = (I)pl.lay[0].size[d];
    args.bsize[d].set((uint64_t)pl.lay[0].size[d]);
    if (d != p && d != q) batch *= pl.lay[0].size[d];
    for (int k = 0; k < pl.nops; ++k) args.stride[k][d] = (I)pl.lay[k].stride[d];
  }
  for (int k = 0; k < pl.nops; ++k) args.staged[k] = staged[k];
  const int64_t tp = (pl.lay[0].size[p] + tile - 1) / tile;
  const int64_t tq = (pl.lay[0].size[q] + tile - 1) / tile;
  args.tilesP.set((uint64_t)tp);
  args.tilesQ.set((uint64_t)tq);
  const int64_t total = batch * tp * tq;
  if (sizeof(I) == 4 && total >= kIndex32Limit) return false;
  args.totalTiles = (I)total;
  const int64_t cap = (int64_t)num_compute_units(s) * tuning("apply.tiled.blocks_per_cu", 4096);
  const int grid = (int)std::max<int64_t>(1, std::min<int64_t>(total, std::min<int64_t>(cap, 1 << 30)));
  T* out = (T*)pl.ptr[0];
  const T* i0 = (const T*)pl.ptr[1];
  const T* i1 = (const T*)pl.ptr[2];
  const T* i2 = (const T*)pl.ptr[3];
  hipStream_t st = current_stream(s);
  if (vec) {
    hipLaunchKernelGGL((apply_tiled_kernel<T, Op, I, VEC, LX>), dim3(grid), dim3(kBlock), ldsV, st,
                       out, i0, i1, i2, args, op);
    note_kernel("tiled");
  } else {
    hipLaunchKernelGGL((apply_tiled_kernel<T, Op, I, 1, 64>), dim3(grid), dim3(kBlock), ldsS, st,
                       out, i0, i1, i2, args, op);
    note_kernel("tiled-scalar");
  }
  return true;
}

template <typename T, typename Op>
void run_plan(THCState* s, Plan& pl, bool sameShape, Op op) {
  bool wide = force_64bit_index();
  for (int k = 0; k < pl.nops; ++k) {
    wide = wide || !fits_32bit(pl.lay[k]);
    for (int d = 0; d < pl.lay[k].dims; ++d) wide = wide || pl.lay[k].stride[d] < 0;
  }
  if (sameShape && joint_collapse(pl.nops, pl.lay, /*reorder=*/true)) {
    bool flat = pl.lay[0].dims == 1;
    for (int k = 0; k < pl.nops && flat; ++k) flat = pl.lay[k].stride[0] == 1;
    if (flat) {
      launch_contig<T>(s, pl, op);
      return;
    }
    if (tuning("apply.tiled.enable", 1)) {
      if (wide ? launch_tiled<T, Op, uint64_t>(s, pl, op) : launch_tiled<T, Op, uint32_t>(s, pl, op))
        return;
    }
    if (wide)
      launch_indexed<T, Op, uint64_t, true>(s, pl, op);
    else
      launch_indexed<T, Op, uint32_t, true>(s, pl, op);
    return;
  }
  for (int k = 0; k < pl.nops; ++k) collapse(pl.lay[k]);
  if (wide)
    launch_indexed<T, Op, uint64_t, false>(s, pl, op);
  else
    launch_indexed<T, Op, uint32_t, false>(s, pl, op);
}

template <typename T>
void dispatch_op(THCState* s, Plan& pl, bool sameShape, PointOp op, float v) {
  switch (op) {
    case PointOp::Fill: run_plan<T>(s, pl, sameShape, OpFill{v}); break;
    case PointOp::AddC: run_plan<T>(s, pl, sameShape, OpAddC{v}); break;
    case PointOp::SubC: run_plan<T>(s, pl, sameShape, OpSubC{v}); break;
    case PointOp::MulC: run_plan<T>(s, pl, sameShape, OpMulC{v}); break;
    case PointOp::DivC: run_plan<T>(s, pl, sameShape, OpDivC{v}); break;
    case PointOp::Pow: run_plan<T>(s, pl, sameShape, OpPow{v}); break;
    case PointOp::Add: run_plan<T>(s, pl, sameShape, OpAdd{v}); break;
    case PointOp::Sub: run_plan<T>(s, pl, sameShape, OpSub{v}); break;
    case PointOp::Mul: run_plan<T>(s, pl, sameShape, OpMul{v}); break;
    case PointOp::Div: run_plan<T>(s, pl, sameShape, OpDiv{v}); break;
    case PointOp::CAdd: run_plan<T>(s, pl, sameShape, OpCAdd{v}); break;
    case PointOp::AddCMul: run_plan<T>(s, pl, sameShape, OpAddCMul{v}); break;
    case PointOp::AddCDiv: run_plan<T>(s, pl, sameShape, OpAddCDiv{v}); break;
    default: raise_error("pointwise op not available for this element type");
  }
}

}  // namespace

bool pointwise_apply(THCState* s, DType dt, PointOp op, float value, AnyTensor* out, AnyTensor* in0,
                     AnyTensor* in1, AnyTensor* in2, bool ignoreOverlap) {
  AnyTensor* t[kMaxOps] = {out, in0, in1, in2};
  const int nops = point_op_inputs(op) + 1;
  const ptrdiff_t n = tensor_numel(out);
  for (int k = 0; k < nops; ++k) {
    if (tensor_numel(t[k]) != n) return false;          // THCApply.cuh:434-439
    if (t[k]->nDimension > kMaxDims) return false;      // :441-445
  }
  if (out->nDimension == 0) return true;                // :447-450

  // An output that addresses one element through several indices is computed
  // into a dense temporary and copied back, last writer wins (:472-489).
  if (!ignoreOverlap && overlapping(tensor_layout(out))) {
    TensorRef tmp(s, tensor_new_with_size(s, out->nDimension, out->size, dt));
    if (!pointwise_apply(s, dt, op, value, tmp.t, in0, in1, in2, true)) return false;
    copy_tensor(s, dt, out, tmp.t, /*ignoreOverlap=*/true);
    return true;
  }

  Plan pl{};
  pl.nops = nops;
  pl.numel = n;
  bool sameShape = true;
  for (int k = 0; k < nops; ++k) {
    pl.ptr[k] = tensor_data(t[k], dt);
    pl.lay[k] = tensor_layout(t[k]);
    if (!pl.ptr[k]) raise_error("pointwise apply on a tensor without storage");
    if (k > 0) {
      sameShape = sameShape && pl.lay[k].dims == pl.lay[0].dims;
      for (int d = 0; sameShape && d < pl.lay[0].dims; ++d)
        sameShape = pl.lay[k].size[d] == pl.lay[0].size[d];
    }
  }
  switch (dt) {
    case DType::F32:
      if (op == PointOp::Copy) run_plan<uint32_t>(s, pl, sameShape, OpCopy{});
      else dispatch_op<float>(s, pl, sameShape, op, value);
      break;
    case DType::F16:
      if (op == PointOp::Copy) run_plan<uint16_t>(s, pl, sameShape, OpCopy{});
      else dispatch_op<__half>(s, pl, sameShape, op, value);
      break;
    case DType::I64:
      if (op != PointOp::Copy) raise_error("only copy is available for long tensors");
      run_plan<uint64_t>(s, pl, sameShape, OpCopy{});
      break;
  }
  THC_CHECK(hipGetLastError());
  return true;
}

void copy_tensor(THCState* s, DType dt, AnyTensor* dst, AnyTensor* src, bool ignoreOverlap) {
  if (dst == src) return;
  const ptrdiff_t n = tensor_numel(dst);
  THC_ARG_CHECK(n == tensor_numel(src), 2, "sizes do not match");  // THCTensorCopy.cu:29-31
  if (dst->nDimension == 0) return;
  if ((tensor_is_contiguous(dst) && tensor_is_contiguous(src)) || n == 1) {
    THC_CHECK(hipMemcpyAsync(tensor_data(dst, dt), tensor_data(src, dt), (size_t)n * dtype_size(dt),
                             hipMemcpyDeviceToDevice, current_stream(s)));
    return;
  }
  if (!pointwise_apply(s, dt, PointOp::Copy, 0.f, dst, src, nullptr, nullptr, ignoreOverlap))
    raise_arg_error(2, "%s", kDimWarning);
}

// ------------------------------------------------------------------------
// fp16 <-> fp32 copies
// ------------------------------------------------------------------------
template <typename D, typename S>
__global__ __launch_bounds__(kBlock) void convert_kernel(D* dst, const S* src, uint64_t n) {
  const uint64_t step = (uint64_t)gridDim.x * kBlock;
  for (uint64_t i = (uint64_t)blockIdx.x * kBlock + threadIdx.x; i < n; i += step)
    dst[i] = Cvt<D>::down(Cvt<S>::up(src[i]));
}

void convert_copy(THCState* s, DType dstT, AnyTensor* dst, DType srcT, AnyTensor* src) {
  const ptrdiff_t n = tensor_numel(dst);
  THC_ARG_CHECK(n == tensor_numel(src), 2, "sizes do not match");
  if (n == 0) return;
  TensorRef cs(s, tensor_new_contiguous(s, src, srcT));
  const bool direct = tensor_is_contiguous(dst);
  TensorRef cd(s, direct ? (tensor_retain(dst), dst)
                         : tensor_new_with_size(s, dst->nDimension, dst->size, dstT));
  const int grid = grid_for(s, n, kBlock * 4, "apply.contig.blocks_per_cu", 16);
  hipStream_t st = current_stream(s);
  if (dstT == DType::F32 && srcT == DType::F16)
    hipLaunchKernelGGL((convert_kernel<float, __half>), dim3(grid), dim3(kBlock), 0, st,
                       (float*)tensor_data(cd.t, dstT), (const __half*)tensor_data(cs.t, srcT),
                       (uint64_t)n);
  else if (dstT == DType::F16 && srcT == DType::F32)
    hipLaunchKernelGGL((convert_kernel<__half, float>), dim3(grid), dim3(kBlock), 0, st,
                       (__half*)tensor_data(cd.t, dstT), (const float*)tensor_data(cs.t, srcT),
                       (uint64_t)n);
  else
    raise_error("unsupported conversion");
  THC_CHECK(hipGetLastError());
  if (!direct) copy_tensor(s, dstT, dst, cd.t, false);
}

}  // namespace thc
