// The LDS-tile kernel of the apply engine for every functor and element-type
// pair (included by apply_impl.hpp).
//
// lib/THC/THCApply.cuh:426-640 runs every op of every type through one
// strided kernel. Here the specialised tiled kernels of apply_impl.hpp keep
// their direct operands in registers and are instantiated per staging mask,
// which is affordable for the plain arithmetic of the hot path only. This
// kernel is the general form for a transposed operand: EVERY input of a
// TP x TQ tile goes through LDS (inputs whose unit-stride dim is p are
// written transposed, the others as they are), so that
//   * the loads of a tile are issued as one batch into registers and, the
//     kernel being persistent, the NEXT tile's batch is in flight while the
//     current tile is computed out of LDS;
//   * the compute loop is rolled and reads LDS only, so a code-dispatched
//     functor is decoded once per tile around that loop (one copy of every
//     function per kernel instead of one per unrolled element);
//   * which inputs are transposed is a run-time flag (no instantiation per
//     staging mask), the index type is 64-bit for tile origins only, and the
//     input and output element types may differ (comparisons, conversions).
// Rows that are not whole aligned packs (odd sizes, views at odd offsets) take
// the same kernel with ALIGNED = false: every global access is still an aligned
// pack covering a window that starts at or below the row piece's first
// element; the element-wise LDS accesses absorb each operand's own shift.
#pragma once

namespace thc {

// fn(integral_constant<int, B>) ... fn(integral_constant<int, E - 1>): a loop whose index is a
// compile-time constant in every iteration. The packs a lane holds across the tile loop are
// an array indexed by such loops only; with ordinary unrolled loops the compiler left part of one
// rolled in the unaligned kernels, indexed the array at run time and therefore kept two of its
// packs in scratch memory, each stored there right behind its load (a full memory wait in the
// middle of the requests that are meant to stay in flight while the tile is computed).
template <int B, int E, typename Fn>
__device__ __forceinline__ void static_for(Fn&& fn) {
  if constexpr (B < E) {
    fn(std::integral_constant<int, B>{});
    static_for<B + 1, E>(fn);
  }
}

struct LdsTileArgs {
  int staged[kMaxOps];   // input k is read along p and transposed on its way into LDS
  int sameGrid[kMaxOps]; // input k is read along q and its rows share the output rows' 16-byte grid (unaligned rows)
  uint32_t sizeP, sizeQ;
  int64_t strideP[kMaxOps];  // elements
  int64_t strideQ[kMaxOps];
  int nbatch;            // remaining joint dims
  Divisor<uint32_t> bsize[kMaxDims];
  int64_t bstride[kMaxOps][kMaxDims];
  Divisor<uint32_t> tilesP, tilesQ;
  uint32_t totalTiles;
  uint32_t xcdPer;   // tiles per XCD when workgroup slot b takes tile (b % 8) * xcdPer + b / 8; 0 = identity
  uint32_t groupP;   // tiles are walked in bands of groupP tiles along p (p fastest inside a band); 1 = q fastest
  uint32_t ntStore;  // whole packs of the output go out with the streaming hint
};

// Geometry shared by the kernel and the host (LDS bytes, tile extents).
//
// ALIGNED: the tile is the window, WP x WQ; the transposed slab is [WQ][PITCH_S], the plain slab
// [WP][WQ].
// Otherwise a tile advances by TP = WP - VEC and TQ = WQ - VEC, one pack less than the window, and
//   * along p (transposed inputs) a row's window starts at the aligned pack at or below the tile's
//     first element of that row, so window element w is tile coordinate w - m, m < VEC the row's
//     own misalignment;
//   * along q every OUTPUT row cuts the tensor at its own pack boundaries: with mo < VEC the
//     misalignment of the output row at column q0, the tile owns of that row the 31 whole packs
//     [q0 - mo, q0 - mo + TQ). No pack is split between two tiles, so partial (element-wise) stores
//     only happen at the two ends of a tensor row. (Cutting every row at q0 left two partial packs
//     per row and tile; stores narrower than 4 bytes make the memory side read, merge and write a
//     whole sector each: a transposed half / short operand of odd shape moved 2.3 x its bytes.)
//     The transposed slab therefore holds tile rows q0 - VEC .. q0 + TQ - 1 (slab row = tile
//     coordinate + VEC), and a plain input's window starts at the aligned pack at or below ITS
//     element at column q0 - mo.
template <typename T, typename TOut, int LXP, int LXQ, bool ALIGNED>
struct LdsTileShape {
  static constexpr int W = sizeof(T) > sizeof(TOut) ? sizeof(T) : sizeof(TOut);
  static constexpr int VEC = 16 / W;
  static constexpr int WP = LXP * VEC, WQ = LXQ * VEC;  // window: lanes x pack
  static constexpr int TP = ALIGNED ? WP : WP - VEC, TQ = ALIGNED ? WQ : WQ - VEC;
  static constexpr int ROWS_P = kBlock / LXP, ROWS_Q = kBlock / LXQ;
  static constexpr int NP_S = WQ / ROWS_P;                 // packs per lane, lanes along p
  static constexpr int NP_D = (TP + ROWS_Q - 1) / ROWS_Q;  // packs per lane, lanes along q
  static constexpr int NP = NP_S > NP_D ? NP_S : NP_D;
  static_assert(WQ % ROWS_P == 0, "whole passes over the window's rows");
  static constexpr int MARG = ALIGNED ? 0 : VEC;
  // Pitch of the transposed slab: a whole, ODD number of 32-bit words. Whole words keep a lane's
  // pack of sub-word elements word-aligned in LDS (16-byte LDS writes at 2-byte alignment stall the
  // LDS pipeline: half and short tiles spent a fifth of their time in such stalls); the odd word
  // count spreads rows over the banks.
  static constexpr int EPW = sizeof(T) >= 4 ? 1 : 4 / (int)sizeof(T);   // elements per word
  // Unaligned rows of sub-word elements: the transposed slab keeps every row's WINDOW as loaded
  // (pack j at column j * VEC, a word-aligned LDS write) instead of shifting it into place, and
  // the readers add the row's shift, which they derive from the row number.
  static constexpr bool WIN = !ALIGNED && sizeof(T) < 4;
  // (shifted into place, a row occupies columns MARG - (VEC - 1) .. MARG + WP - 1)
  static constexpr int PITCH_S = (((ALIGNED || WIN ? WP : WP + VEC) + EPW - 1) / EPW | 1) * EPW;
  static constexpr int ROWS_S = ALIGNED ? WQ : WQ + VEC;   // (lane 31 of an unaligned tile reads past row WQ: never stored)
  // plain slab: row p's window from column MARG on; readers look up to 2 VEC - 2 columns beyond it
  static constexpr int PITCH_D = ALIGNED ? WQ : WQ + 3 * VEC;
  static constexpr int ROWS_D = WP;
  static_assert(NP * ROWS_Q <= ROWS_D && NP * ROWS_P <= ROWS_S, "every lane's row lies inside the slab");
  // Reading the transposed slab, lane lxq takes rows VEC * lxq + e: VEC rows are VEC * odd words, so
  // lanes 32 / VEC apart would meet in one bank. Row r therefore starts skew(r) = (r / 32) words late:
  // one bank further for every such group of lanes. (Unaligned rows: only the window layout, whose
  // readers compute an offset per element anyway.)
  static constexpr int SKEW_UNIT = (ALIGNED || WIN) && sizeof(T) <= 4 ? EPW : 0;
  static constexpr int skew(int r) { return SKEW_UNIT ? (r / 32) * SKEW_UNIT : 0; }
  static constexpr int SLAB_S = ROWS_S * PITCH_S + skew(ROWS_S);
  static constexpr int SLAB_RAW = SLAB_S > ROWS_D * PITCH_D ? SLAB_S : ROWS_D * PITCH_D;
  static constexpr int SLAB = (SLAB_RAW + VEC - 1) / VEC * VEC;  // elements of T per input
  static constexpr size_t lds_bytes(int nin) { return (size_t)nin * SLAB * sizeof(T); }
};

// NTL: inputs are read with the streaming (nontemporal) hint. A compile-time choice: a run-time one
// makes the compiler merge the two forms of every load into one plain load.
template <typename T, typename TOut, typename Op, int LXP, int LXQ, bool ALIGNED, bool NTL = true>
__global__ __launch_bounds__(kBlock) void apply_ldstile_kernel(TOut* out, const T* in0, const T* in1,
                                                               const T* in2, LdsTileArgs args, Op op) {
  using S = LdsTileShape<T, TOut, LXP, LXQ, ALIGNED>;
  constexpr int NIN = Op::NIN;
  constexpr int VEC = S::VEC, TP = S::TP, TQ = S::TQ, ROWS_P = S::ROWS_P, ROWS_Q = S::ROWS_Q;
  constexpr int NP = S::NP, NP_S = S::NP_S, NP_D = S::NP_D, PITCH_S = S::PITCH_S, PITCH_D = S::PITCH_D, MARG = S::MARG;
  constexpr bool WIN = S::WIN;
  static_assert(NIN >= 1 && NIN <= 3, "one to three inputs");
  using PIN = Pack<T, VEC>;
  using POUT = Pack<TOut, VEC>;
  // Packs travel from global memory to LDS as raw register images: a pack of sub-word elements kept
  // as a struct across the tile loop ended up in scratch memory (272 bytes a lane for two inputs of
  // 16-bit elements, which tripled the kernel's memory traffic).
  using RAW = typename RawBits<sizeof(PIN)>::type;
  extern __shared__ __align__(16) unsigned char lds_raw[];
  T* lds = reinterpret_cast<T*>(lds_raw);

  const T* ptr[3] = {in0, in1, in2};
  const uint32_t lxp = threadIdx.x % LXP, lyp = threadIdx.x / LXP;
  const uint32_t lxq = threadIdx.x % LXQ, lyq = threadIdx.x / LXQ;
  const int sizeQ = (int)args.sizeQ;
  auto mis_in = [](const T* row) { return (int)((reinterpret_cast<uintptr_t>(row) / sizeof(T)) & (uintptr_t)(VEC - 1)); };
  auto mis_out = [](const TOut* row) { return (int)((reinterpret_cast<uintptr_t>(row) / sizeof(TOut)) & (uintptr_t)(VEC - 1)); };
  auto load = [&](const T* at) -> RAW {
    if constexpr (NTL) return __builtin_nontemporal_load(reinterpret_cast<const RAW*>(at));
    else return *reinterpret_cast<const RAW*>(at);
  };

  struct Tile {       // uniform over the workgroup
    const T* tb[3];   // tile origin (p0, q0) of input k
    TOut* ob;         // tile origin of the output
    int pn;           // valid extent along p
    int qn;           // ALIGNED: valid extent along q
    int q0;           // first column (unaligned tiles reach back to q0 - VEC + 1 and on to q0 + TQ - 1)
  };
  const uint32_t slots = args.xcdPer ? args.xcdPer * 8 : args.totalTiles;
  // First valid tile at or after slot b (b advances by the grid size); false when none is left.
  auto locate = [&](uint32_t& b, Tile& t) -> bool {
    uint32_t tile = 0;
    for (;; b += gridDim.x) {
      if (b >= slots) return false;
      tile = args.xcdPer ? (b % 8) * args.xcdPer + b / 8 : b;
      if (tile < args.totalTiles) break;
    }
    uint32_t rest, tq, tp;
    if (args.groupP > 1) {
      const uint32_t perBatch = args.tilesP.d * args.tilesQ.d;
      rest = tile / perBatch;
      const uint32_t tt = tile - rest * perBatch;
      const uint32_t band = tt / (args.groupP * args.tilesQ.d);
      const uint32_t r = tt - band * (args.groupP * args.tilesQ.d);
      const uint32_t gp = min(args.groupP, args.tilesP.d - band * args.groupP);  // ragged last band
      tq = r / gp;
      tp = band * args.groupP + (r - tq * gp);
    } else {
      args.tilesQ.divmod(tile, rest, tq);
      args.tilesP.divmod(rest, rest, tp);
    }
    int64_t base[kMaxOps] = {0, 0, 0, 0};
    for (int j = 0; j < args.nbatch; ++j) {
      uint32_t r;
      args.bsize[j].divmod(rest, rest, r);
#pragma unroll
      for (int k = 0; k <= NIN; ++k) base[k] += (int64_t)r * args.bstride[k][j];
    }
    const uint32_t p0 = tp * TP, q0 = tq * TQ;
    t.pn = (int)min((uint32_t)TP, args.sizeP - p0);
    t.qn = (int)min((int64_t)TQ, (int64_t)args.sizeQ - (int64_t)q0);
    t.q0 = (int)q0;
    t.ob = out + (base[0] + (int64_t)p0 * args.strideP[0] + (int64_t)q0 * args.strideQ[0]);
#pragma unroll
    for (int k = 0; k < NIN; ++k)
      t.tb[k] = ptr[k] + (base[k + 1] + (int64_t)p0 * args.strideP[k + 1] + (int64_t)q0 * args.strideQ[k + 1]);
    return true;
  };

  // Row of transposed input k that lane row `qi` of the staging pass loads: tile coordinate
  // qi (ALIGNED) or qi - VEC, kept inside the tensor.
  auto staged_row = [&](const Tile& t, int k, int qi) -> const T* {
    const int sq = (int)args.strideQ[k + 1];
    if (ALIGNED) return t.tb[k] + (uint32_t)min(qi, t.qn - 1) * (uint32_t)sq;
    const int j = min(max(qi - VEC, -t.q0), sizeQ - 1 - t.q0);
    return t.tb[k] + (ptrdiff_t)(j * sq);
  };
  // First column (relative to q0) of the run that output row `pi` owns in this tile, kept inside
  // the tensor: q0 - mo for an unaligned row.
  auto row_start = [&](const Tile& t, int pi) -> int {
    if (ALIGNED) return 0;
    const int mo = mis_out(t.ob + (uint32_t)pi * (uint32_t)args.strideP[0]);
    return min(max(-mo, -t.q0), sizeQ - 1 - t.q0);
  };

  // Requests every pack of the tile's inputs. No load carries a predicate: lanes past the
  // tile's valid extent re-read a pack inside it, so a later wait covers exactly these loads.
  auto issue = [&](const Tile& t, RAW (&v)[NIN][NP]) {
    static_for<0, NIN>([&](auto kTag) {
      constexpr int k = decltype(kTag)::value;
      if (args.staged[k + 1]) {
        static_for<0, NP>([&](auto rTag) {
          constexpr int r = decltype(rTag)::value;
          const T* row = staged_row(t, k, (int)lyp + r * ROWS_P);
          int first = (int)(lxp * VEC) - (ALIGNED ? 0 : mis_in(row));
          if (first >= t.pn) first = ALIGNED ? 0 : -mis_in(row);
          v[k][r] = load(row + first);
        });
      } else {
        const uint32_t sp = (uint32_t)args.strideP[k + 1];
        // (NP, not NP_D, passes: both branches then fill the same registers. With one pass fewer
        // here the compiler merged the last load of either branch into one block that picks its
        // destination at run time, which put two packs of the array into scratch memory, each
        // stored behind a full memory wait. The extra pass re-reads the tile's last row.)
        static_for<0, NP>([&](auto rTag) {
          constexpr int r = decltype(rTag)::value;
          const int pi = min((int)lyq + r * ROWS_Q, t.pn - 1);
          const int cs = row_start(t, pi);
          const T* at = t.tb[k] + (uint32_t)pi * sp + (ptrdiff_t)cs;   // this row's element at the run's start
          int first = (int)(lxq * VEC) - (ALIGNED ? 0 : mis_in(at));
          if (ALIGNED ? first >= t.qn : t.q0 + cs + first >= sizeQ) first = ALIGNED ? 0 : -mis_in(at);
          v[k][r] = load(at + first);
        });
      }
    });
  };

  // Registers -> LDS, without predicates (the slabs have room for every lane's pack). Transposed
  // inputs land at [q][p] (shifted into place element by element, or as the window they were
  // loaded as); the others keep their window (pack j of row p at column MARG + j * VEC).
  auto commit = [&](const Tile& t, const RAW (&v)[NIN][NP]) {
    static_for<0, NIN>([&](auto kTag) {
      constexpr int k = decltype(kTag)::value;
      T* slab = lds + k * S::SLAB;
      if (args.staged[k + 1]) {
        static_for<0, NP>([&](auto rTag) {
          constexpr int r = decltype(rTag)::value;
          const int qi = (int)lyp + r * ROWS_P;
          if constexpr (WIN) {
            // word by word: the row starts at a multiple of 4 bytes, not of 16, and a 16-byte LDS
            // write there stalls the LDS pipeline (SQ_LDS_UNALIGNED_STALL)
            T* at = slab + qi * PITCH_S + S::skew(qi) + lxp * VEC;
            if constexpr (sizeof(RAW) == 16) {
              // (may_alias: the slab is read back as elements of T)
              typedef uint32_t __attribute__((may_alias)) Word;
              Word* w = reinterpret_cast<Word*>(at);
              w[0] = v[k][r].x;
              w[1] = v[k][r].y;
              w[2] = v[k][r].z;
              w[3] = v[k][r].w;
            } else {
              *reinterpret_cast<RAW*>(at) = v[k][r];
            }
          } else {
            int first = (int)(lxp * VEC);
            if (!ALIGNED) first -= mis_in(staged_row(t, k, qi));
            T* at = slab + qi * PITCH_S + S::skew(qi) + (first + MARG);
            PIN pk;
            __builtin_memcpy(&pk, &v[k][r], sizeof(PIN));
#pragma unroll
            for (int e = 0; e < VEC; ++e) at[e] = pk.v[e];
          }
        });
      } else {
        static_for<0, NP>([&](auto rTag) {
          constexpr int r = decltype(rTag)::value;
          const int pi = (int)lyq + r * ROWS_Q;
          *reinterpret_cast<RAW*>(slab + pi * PITCH_D + MARG + lxq * VEC) = v[k][r];
        });
      }
    });
  };

  // LDS -> functor -> global, lanes along q. Rolled: the functor's code is fixed outside.
  auto compute = [&](const Tile& t) {
    with_fixed_code(op, [&](auto f) {
#pragma unroll 2
      for (int r = 0; r < NP_D; ++r) {
        const int pi = (int)lyq + r * ROWS_Q;
        const int pic = ALIGNED ? pi : min(pi, t.pn - 1);
        TOut* orow = t.ob + (uint32_t)pic * (uint32_t)args.strideP[0];
        // tile coordinate of the lane's first element; its slab row is first + MARG
        const int first = (int)(lxq * VEC) - (ALIGNED ? 0 : mis_out(orow));
        // (elements are gathered and results kept as scalars: packs of sub-word elements that are
        // filled or read element by element do not stay in registers)
        T x[3][VEC] = {};
#pragma unroll
        for (int k = 0; k < NIN; ++k) {
          const T* slab = lds + k * S::SLAB;
          if (args.staged[k + 1] && WIN) {
            // row j's window starts mis(row j) elements before its first tile element
            const int sq = (int)((uint32_t)args.strideQ[k + 1] & (uint32_t)(VEC - 1));
            int m = (mis_in(t.tb[k]) + first * sq) & (VEC - 1);
            const T* at = slab + (first + MARG) * PITCH_S + pic;
#pragma unroll
            for (int e = 0; e < VEC; ++e) {
              x[k][e] = at[e * PITCH_S + m + S::skew(first + MARG + e)];
              m = (m + sq) & (VEC - 1);
            }
          } else if (args.staged[k + 1]) {
            const T* at = slab + (first + MARG) * PITCH_S + S::skew(first) + (pic + MARG);  // (skew: ALIGNED only)
#pragma unroll
            for (int e = 0; e < VEC; ++e) x[k][e] = at[e * PITCH_S];
          } else if (ALIGNED) {
            const RAW raw = *reinterpret_cast<const RAW*>(slab + pic * PITCH_D + first);
            PIN pk;
            __builtin_memcpy(&pk, &raw, sizeof(PIN));
#pragma unroll
            for (int e = 0; e < VEC; ++e) x[k][e] = pk.v[e];
          } else if (args.sameGrid[k + 1]) {
            // every row of this input starts as far from a 16-byte boundary as the output's row does
            // (operands of one shape and pitch): the window's packs are the output row's packs
            const RAW raw = *reinterpret_cast<const RAW*>(slab + pic * PITCH_D + MARG + lxq * VEC);
            PIN pk;
            __builtin_memcpy(&pk, &raw, sizeof(PIN));
#pragma unroll
            for (int e = 0; e < VEC; ++e) x[k][e] = pk.v[e];
          } else {
            // the window of row pic starts mis(element at the run's start) before that element
            const int cs = row_start(t, pic);
            const int m = mis_in(t.tb[k] + (uint32_t)pic * (uint32_t)args.strideP[k + 1] + (ptrdiff_t)cs);
            const T* at = slab + pic * PITCH_D + (first - cs + m + MARG);
#pragma unroll
            for (int e = 0; e < VEC; ++e) x[k][e] = at[e];
          }
        }
        TOut y[VEC];
#pragma unroll
        for (int e = 0; e < VEC; ++e) y[e] = f(x[0][e], x[1][e], x[2][e]);
        POUT res;
#pragma unroll
        for (int e = 0; e < VEC; ++e) res.v[e] = y[e];
        if constexpr (ALIGNED) {
          if (pi < t.pn && first < t.qn) {
            if (args.ntStore) store_pack<true>(reinterpret_cast<POUT*>(orow + first), res);
            else store_pack<false>(reinterpret_cast<POUT*>(orow + first), res);
          }
        } else {
          const int g = t.q0 + first;   // column of the pack's first element; lanes 0 .. LXQ - 2 own packs
          if (pi < t.pn && lxq < LXQ - 1 && g + VEC > 0 && g < sizeQ) {
            if (g >= 0 && g + VEC <= sizeQ) {
              if (args.ntStore) store_pack<true>(reinterpret_cast<POUT*>(orow + first), res);
              else store_pack<false>(reinterpret_cast<POUT*>(orow + first), res);
            } else {   // the two ends of a tensor row
#pragma unroll
              for (int e = 0; e < VEC; ++e)
                if (g + e >= 0 && g + e < sizeQ) orow[first + e] = y[e];
            }
          }
        }
      }
    });
  };

  uint32_t b = blockIdx.x;
  Tile cur, nxt;
  RAW v[NIN][NP];
  bool have = locate(b, cur);
  if (have) issue(cur, v);
  while (have) {
    commit(cur, v);
    lds_barrier();
    b += gridDim.x;
    const bool more = locate(b, nxt);
    if (more) issue(nxt, v);  // in flight while this tile is computed
    compute(cur);
    lds_barrier();            // the slabs are rewritten for the next tile
    cur = nxt;
    have = more;
  }
}

// Plans and launches the LDS-tile kernel; false (nothing launched) when the plan has no
// transposed operand or does not fit (no unit stride along an operand's fast dim, negative
// strides, a tile that spans 2^31 elements, more than 2^32 tiles).
template <typename T, typename Op, typename TOut>
bool launch_ldstile(THCState* s, const Plan& pl, Op op) {
  if constexpr (Op::NIN < 1 || Op::NIN > 3) {
    return false;
  } else {
    int p, q, staged[kMaxOps] = {0, 0, 0, 0};
    if (!tuning("apply.ldstile.enable", 1) || !tile_plan(pl, p, q, staged)) return false;
    constexpr int W = sizeof(T) > sizeof(TOut) ? sizeof(T) : sizeof(TOut);
    constexpr int VEC = 16 / W;
    // 512-byte rows (of the wider type) along q; along p 128 bytes of the input type at least
    // (64 bytes for 1-byte elements, whose 128 x 512 tile would take 66 KiB of LDS per input)
    constexpr int LXQ = 32;
    constexpr int LXP = (sizeof(T) == 1 && VEC == 16) ? 4 : ((128 / (int)sizeof(T)) / VEC < 8 ? 8 : (128 / (int)sizeof(T)) / VEC);
    const int nd = pl.lay[0].dims;
    auto elem_size = [](int k) { return k == 0 ? sizeof(TOut) : sizeof(T); };
    bool aligned = pl.lay[0].size[p] % VEC == 0 && pl.lay[0].size[q] % VEC == 0;
    for (int k = 0; k < pl.nops; ++k) {
      const int fast = staged[k] ? p : q;
      if (pl.lay[k].stride[fast] != 1) return false;
      if (reinterpret_cast<uintptr_t>(pl.ptr[k]) % elem_size(k) != 0) return false;
      aligned = aligned && reinterpret_cast<uintptr_t>(pl.ptr[k]) % (VEC * elem_size(k)) == 0;
      for (int d = 0; d < nd; ++d) {
        if (pl.lay[k].stride[d] < 0) return false;
        if (d != fast) aligned = aligned && pl.lay[k].stride[d] % VEC == 0;
      }
      // lane offsets inside a tile are 32-bit
      const int64_t span = (int64_t)(LXQ * VEC) * std::max(pl.lay[k].stride[p], pl.lay[k].stride[q]) + 4096;
      if (span >= (int64_t(1) << 31)) return false;
    }
    LdsTileArgs args{};
    for (int k = 0; k < pl.nops; ++k) {
      args.staged[k] = staged[k];
      args.strideP[k] = pl.lay[k].stride[p];
      args.strideQ[k] = pl.lay[k].stride[q];
      // an input read along q whose rows all start as far from a 16-byte boundary as the output's
      bool same = k > 0 && !staged[k] && tuning("apply.ldstile.same_grid", 1) &&
                  (reinterpret_cast<uintptr_t>(pl.ptr[k]) / elem_size(k)) % VEC ==
                      (reinterpret_cast<uintptr_t>(pl.ptr[0]) / elem_size(0)) % VEC;
      for (int d = 0; d < nd && same; ++d)
        if (d != q) same = pl.lay[k].stride[d] % VEC == pl.lay[0].stride[d] % VEC;
      args.sameGrid[k] = same ? 1 : 0;
    }
    if (pl.lay[0].size[p] >= kIndex32Limit || pl.lay[0].size[q] >= kIndex32Limit) return false;
    args.sizeP = (uint32_t)pl.lay[0].size[p];
    args.sizeQ = (uint32_t)pl.lay[0].size[q];
    int64_t batch = 1;
    for (int d = nd - 1; d >= 0; --d) {
      if (d == p || d == q) continue;
      args.bsize[args.nbatch].set((uint64_t)pl.lay[0].size[d]);
      for (int k = 0; k < pl.nops; ++k) args.bstride[k][args.nbatch] = pl.lay[k].stride[d];
      ++args.nbatch;
      batch *= pl.lay[0].size[d];
    }
    using SA = LdsTileShape<T, TOut, LXP, LXQ, true>;
    using SU = LdsTileShape<T, TOut, LXP, LXQ, false>;
    const int64_t tileP = aligned ? SA::TP : SU::TP, tileQ = aligned ? SA::TQ : SU::TQ;
    // (an unaligned row's first run starts up to VEC - 1 columns before the row does)
    const int64_t tp = (args.sizeP + tileP - 1) / tileP, tq = (args.sizeQ + (aligned ? 0 : VEC - 1) + tileQ - 1) / tileQ;
    args.tilesP.set((uint64_t)tp);
    args.tilesQ.set((uint64_t)tq);
    const int64_t total = batch * tp * tq;
    if (total >= (int64_t(1) << 31)) return false;
    args.totalTiles = (uint32_t)total;
    const int64_t ntKnob = tuning("apply.tiled.nt_store", -1);
    args.ntStore = (ntKnob >= 0 ? ntKnob != 0 : pl.numel * (int64_t)sizeof(TOut) >= (int64_t(64) << 20)) ? 1u : 0u;
    // single-input ops: bands along p (their only read stream is the transposed one); unaligned rows: bands
    // keep the lines that p-neighbours share in L2, and an XCD gets a contiguous range of tiles
    int64_t band = tuning("apply.ldstile.group_p", -1);
    if (band < 0) band = Op::NIN == 1 ? 16 : (aligned ? 1 : 8);
    args.groupP = (uint32_t)std::max<int64_t>(1, band);
    if ((int64_t)args.groupP * 2 > tp) args.groupP = 1;
    if (!aligned && tuning("apply.ldstile.xcd_swizzle", 1) && total >= 64 && total < (int64_t(1) << 28))
      args.xcdPer = (uint32_t)((total + 7) / 8);
    const size_t ldsBytes = aligned ? SA::lds_bytes(Op::NIN) : SU::lds_bytes(Op::NIN);
    if (ldsBytes > 160 * 1024) return false;
    // persistent grid: as many workgroups as the LDS admits per CU (160 KiB), capped by registers at 8
    const int64_t perCu = std::max<int64_t>(1, std::min<int64_t>(tuning("apply.ldstile.max_per_cu", 8),
                                                                 (int64_t)(160 * 1024) / (int64_t)ldsBytes));
    const int64_t slots = args.xcdPer ? (int64_t)args.xcdPer * 8 : total;
    int64_t gridCap = tuning("apply.ldstile.max_grid", -1);
    if (gridCap <= 0) gridCap = perCu * num_compute_units(s);
    const int grid = (int)std::max<int64_t>(1, std::min<int64_t>(slots, gridCap));
    hipStream_t st = current_stream(s);
    TOut* o = (TOut*)pl.ptr[0];
    const T* i0 = (const T*)pl.ptr[1];
    const T* i1 = (const T*)pl.ptr[2];
    const T* i2 = (const T*)pl.ptr[3];
    // Load policy. Ops with two or three inputs always read with the streaming hint (plain loads:
    // 0.75 -> 0.61 of peak on a transposed cmax of 8192 x 8192 floats). With ONE input both forms are
    // built and the choice is made here.
    bool ntl = true;
    if constexpr (Op::NIN == 1) {
      const int64_t knob = tuning("apply.ldstile.nt_load", -1);
      ntl = knob >= 0 ? knob != 0 : !(sizeof(T) == sizeof(TOut) && sizeof(T) < 4);
    }
    auto go = [&](auto alignedTag, auto ntlTag) {
      hipLaunchKernelGGL((apply_ldstile_kernel<T, TOut, Op, LXP, LXQ, decltype(alignedTag)::value, decltype(ntlTag)::value>),
                         dim3(grid), dim3(kBlock), ldsBytes, st, o, i0, i1, i2, args, op);
    };
    if constexpr (Op::NIN == 1) {
      if (aligned && ntl) go(std::true_type{}, std::true_type{});
      else if (aligned) go(std::true_type{}, std::false_type{});
      else if (ntl) go(std::false_type{}, std::true_type{});
      else go(std::false_type{}, std::false_type{});
    } else {
      if (aligned) go(std::true_type{}, std::true_type{});
      else go(std::false_type{}, std::true_type{});
    }
    note_kernel(aligned ? "lds-tile" : "lds-tile-shift");
    return true;
  }
}

}  // namespace thc
