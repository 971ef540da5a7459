/*
 * Row-regime selection shared by the softmax and RMSNorm launchers.
 *
 * A row of `packs` 128-bit packs is processed by a group of G threads (G = 64 ... 1024), each
 * holding NV packs in registers between the reduction and the write, so the row is read from
 * HBM once. HBM streams fastest here with many small waves each moving one or two packs, so
 * the plan takes the narrowest group that covers the row at a target NV (2 for softmax, 1 for
 * RMSNorm) and only lets NV grow once the group is 1024 threads wide:
 *   short rows         up to 16 packs: 1, 2, 4, 8 or 16 lanes a row, a pack a lane, packs that
 *                      start at the row's first element whatever its alignment (ShortRow);
 *   G = 8, 16, 32      several short rows per wavefront, DPP reductions inside 8-, 16- or
 *                      32-lane parts of the wave, so rows of a few hundred bytes keep all lanes busy
 *                      (8 lanes only for rows of at most eight packs, one pack a lane);
 *   G = 64             one wavefront per row, cross-lane (DPP / permlane-swap) reductions only;
 *   G = 128 ... 1024   per-wave partials combined through LDS with one barrier per reduction;
 *   stream             rows too long for registers: an online first pass and a second pass that
 *                      re-reads the row (served by L2 / the memory-side cache where it fits).
 * The reference has one regime only: a 32-lane warp per row striding the row with 4-byte loads
 * (src/cuda/nvcc_src/reduce_ij_i.cu:13-32).
 */
#ifndef MP_ROW_DISPATCH_H
#define MP_ROW_DISPATCH_H

#include "kernel_header.h"

#include <type_traits>

#if defined(__cplusplus) && defined(__HIPCC__)

namespace mp {

/* 0 = automatic; 1..5 force G = 64, 128, 256, 512, 1024; 6 forces the streaming kernels;
 * 7 forces the cluster path of the softmax forward; 8 and 9 force sub-wave groups of 16 and 32
 * lanes. A launcher without the forced path treats the value as automatic. */
enum RowRegime { REGIME_AUTO = 0, REGIME_G64 = 1, REGIME_G128 = 2, REGIME_G256 = 3, REGIME_G512 = 4,
                 REGIME_G1024 = 5, REGIME_STREAM = 6, REGIME_CLUSTER = 7, REGIME_G16 = 8, REGIME_G32 = 9 };

/* The regime the launchers plan with. The library as shipped has no switch: this is the constant
 * AUTO, the launchers hold no mutable state and the workspace sizes are functions of
 * (dtype, m, n) alone. Only the test build (MP_DIAGNOSTICS, linked into a library of its own that
 * the parity tests load to drive every regime) keeps a process-wide override behind
 * mpSetRowRegime. */
#ifdef MP_DIAGNOSTICS
inline int& row_regime_override() {
  static int regime = REGIME_AUTO;
  return regime;
}
#else
constexpr int row_regime_override() { return REGIME_AUTO; }
#endif

/* Largest NV a kernel may use, from the 32-bit registers it can spend on ONE row-shaped
 * register array (a 1024-thread workgroup leaves 128 registers per lane in total). */
template <class T> constexpr int max_nv_for(int regs_per_array) {
  using P = typename precision<T>::type;
  const int per_pack = (PACK_BYTES / (int)sizeof(T)) * (int)(sizeof(P) / 4);
  int nv = 1;
  while (nv * 2 * per_pack <= regs_per_array && nv < 16) nv *= 2;
  return nv;
}

struct RowPlan {
  int G;   /* threads per row; 0 = streaming */
  int NV;  /* packs per thread */
};

/* nv_target: packs per thread the automatic plan aims for before it widens the group.
 * min_group: 64, or 16 or 8 when the kernel also comes in groups of 8, 16 and 32 lanes (several
 * rows per wavefront), which keeps every lane busy on rows shorter than a wavefront's worth of
 * packs. Ragged rows need 16: a group's first lanes hold one head or tail element each, and a row
 * of two-byte values can have fourteen of them. */
inline RowPlan plan_row(size_t packs, int max_nv, int nv_target, int min_group = WAVE) {
  const bool subwave = min_group < WAVE;
  static const int ladder[] = {16, 32, 64, 128, 256, 512, 1024};
  constexpr int RUNGS = 7;
  int forced = row_regime_override();
  if (forced == REGIME_CLUSTER || (!subwave && (forced == REGIME_G16 || forced == REGIME_G32))) forced = REGIME_AUTO;
  if (forced == REGIME_STREAM) return RowPlan{0, 0};
  const int first_rung = subwave ? 0 : 2;
  if (forced == REGIME_AUTO) {
    if (min_group <= 8 && packs <= 8) return RowPlan{8, 1};
    const int want = nv_target < max_nv ? nv_target : max_nv;
    for (int r = first_rung; r < RUNGS; ++r) {
      const int nv = packs_per_thread(packs, ladder[r], want);
      if (nv) return RowPlan{ladder[r], nv};
    }
    const int nv = packs_per_thread(packs, 1024, max_nv);
    return nv ? RowPlan{1024, nv} : RowPlan{0, 0};
  }
  /* a forced group that cannot hold the row moves on to the next wider one */
  const int start = forced == REGIME_G16 ? 0 : forced == REGIME_G32 ? 1 : forced + 1;
  for (int r = start; r < RUNGS; ++r) {
    const int nv = packs_per_thread(packs, ladder[r], max_nv);
    if (nv) return RowPlan{ladder[r], nv};
  }
  return RowPlan{0, 0};
}

/* plan_row, reconsidered for rows that leave more than an eighth of the planned group idle (a row
 * of 1280 packs on 1024 threads x 2 packs uses five lanes in eight): the group and the packs a
 * thread, now any number up to max_nv, that waste the fewest lanes; among equals the count
 * closest to nv_target, then the narrower group. Rows of a power of two of packs keep their plan. */
inline RowPlan plan_row_fit(size_t packs, int max_nv, int nv_target, int min_group = WAVE) {
  const RowPlan base = plan_row(packs, max_nv, nv_target, min_group);
  if (row_regime_override() != REGIME_AUTO || base.G < WAVE || packs == 0) return base;
  const size_t base_slots = (size_t)base.G * base.NV;
  if (packs * 8 >= base_slots * 7) return base;
  static const int ladder[] = {64, 128, 256, 512, 1024};
  RowPlan best = base;
  size_t best_slots = base_slots;
  auto off_target = [&](int nv) { return nv > nv_target ? nv - nv_target : nv_target - nv; };
  for (int g : ladder)
    for (int nv = 1; nv <= (max_nv < 8 ? max_nv : 8); ++nv) {
      const size_t slots = (size_t)g * nv;
      if (slots < packs) continue;
      const bool better = slots < best_slots ||
                          (slots == best_slots && (off_target(nv) < off_target(best.NV) ||
                                                   (off_target(nv) == off_target(best.NV) && g < best.G)));
      if (better) {
        best = RowPlan{g, nv};
        best_slots = slots;
      }
    }
  return best;
}

/* Calls f.template operator()<G, NV>() for the plan; returns false for the streaming plan. */
/* ODD: the plan may hold 3, 5, 6 or 7 packs a thread (plan_row_fit); only callers that ask for such plans
 * pay for the extra kernels. */
template <int MAXNV, bool SUBWAVE = false, bool ODD = false, class F> inline bool for_row_plan(const RowPlan& plan, F&& f) {
#define MP_PLAN_CASE(G_, NV_) \
  if constexpr (NV_ <= MAXNV) { \
    if (plan.G == G_ && plan.NV == NV_) { f.template operator()<G_, NV_>(); return true; } \
  }
#define MP_PLAN_GROUP(G_) \
  MP_PLAN_CASE(G_, 1) MP_PLAN_CASE(G_, 2) MP_PLAN_CASE(G_, 4) MP_PLAN_CASE(G_, 8) MP_PLAN_CASE(G_, 16) \
  if constexpr (ODD) { MP_PLAN_CASE(G_, 3) MP_PLAN_CASE(G_, 5) MP_PLAN_CASE(G_, 6) MP_PLAN_CASE(G_, 7) }
  if constexpr (SUBWAVE) {
    MP_PLAN_CASE(8, 1)
    MP_PLAN_GROUP(16)
    MP_PLAN_GROUP(32)
  }
  MP_PLAN_GROUP(64)
  MP_PLAN_GROUP(128)
  MP_PLAN_GROUP(256)
  MP_PLAN_GROUP(512)
  MP_PLAN_GROUP(1024)
#undef MP_PLAN_GROUP
#undef MP_PLAN_CASE
  return false;
}

constexpr int STREAM_THREADS = 1024;

/* The hardware hands consecutive workgroups of a grid to the eight XCDs in turn, and every XCD
 * has its own L2. Rows that are not a whole number of 128-byte cache lines share a line with
 * their neighbours: if neighbouring rows sit on different XCDs the line is fetched into two L2s
 * and written back in halves. This mapping gives every XCD a contiguous range of the grid's
 * logical blocks instead, so neighbours meet in one L2 (measured with n = 1000: softmax r16
 * 5.3 -> 5.9 TB/s forward, r32 reverse 5.3 -> 5.8; the RMSNorm reverse gains 2 %, and its
 * forward, whose 256-thread workgroups already hold several neighbouring rows, nothing). Rows of
 * whole cache lines lose by it (n = 1024 r32 6.4 -> 5.5: eight far-apart streams instead of one
 * front), so launchers turn it on by row length only. */
constexpr unsigned XCDS = 8;
__device__ __forceinline__ unsigned xcd_contiguous_block(unsigned block, unsigned blocks) {
  const unsigned per = blocks / XCDS, rem = blocks % XCDS, xcd = block % XCDS, idx = block / XCDS;
  return xcd * per + (xcd < rem ? xcd : rem) + idx;
}
template <class T> inline unsigned rows_share_lines(size_t n) { return (n * sizeof(T)) % 128 != 0 ? 1u : 0u; }

/* A row as packs counted from its first element: npk = ceil(n / W) packs,
 * the last of which holds `last` elements (W when n is a multiple of W). A thread owns the same
 * columns in every row (their gain, and in the reverse their dg sums, stay in registers),
 * whatever the alignment:
 * LOOSE = false: every operand 16-byte aligned and n % W == 0, so every pack is whole and aligned;
 * LOOSE = true: packs start at any element (see loose_vec_of; free for these streaming reads,
 * about 5 % on the stores) and the cut pack of a row moves element by element, zero-filled
 * (predicated single accesses in line; moved in pieces behind branches, as the short rows do,
 * these kernels lose 10-25 %: r16 n = 2047 forward 4.6 -> 3.4 TB/s). */
template <class T, int W, bool LOOSE> struct RowPacks {
  using P = typename precision<T>::type;
  using V = typename vec_of<T, W>::type;
  using VL = typename std::conditional<LOOSE, typename loose_vec_of<T, W>::type, V>::type;
  int npk, last;
  __device__ __forceinline__ explicit RowPacks(size_t n)
      : npk(LOOSE ? (int)((n + W - 1) / W) : (int)(n / W)),
        last(LOOSE ? (int)(n - (size_t)((int)((n + W - 1) / W) - 1) * W) : W) {}
  /* elements of pack p that exist (p < npk) */
  __device__ __forceinline__ int valid(int p) const { return LOOSE && p == npk - 1 ? last : W; }
  /* pack p < npk of the row at `row`, in the storage type */
  template <bool NT> __device__ __forceinline__ V raw(const T* row, int p) const {
    const T* at = row + (size_t)(unsigned)p * W;
    if (!LOOSE || valid(p) == W) {
      if constexpr (NT) return __builtin_nontemporal_load(reinterpret_cast<const VL*>(at));
      else return *reinterpret_cast<const VL*>(at);
    }
    V v;
#pragma unroll
    for (int i = 0; i < W; ++i) v[i] = i < last ? at[i] : (T)0;
    return v;
  }
  template <bool NT> __device__ __forceinline__ void load(const T* row, int p, P (&out)[W]) const {
    const V v = raw<NT>(row, p);
#pragma unroll
    for (int i = 0; i < W; ++i) out[i] = (P)v[i];
  }
  __device__ __forceinline__ void store(T* row, int p, const P (&in)[W]) const {
    T* at = row + (size_t)(unsigned)p * W;
    if (!LOOSE || valid(p) == W) {
      V v;
#pragma unroll
      for (int i = 0; i < W; ++i) v[i] = (T)in[i];
      __builtin_nontemporal_store(v, reinterpret_cast<VL*>(at));
    } else {
#pragma unroll
      for (int i = 0; i < W; ++i)
        if (i < last) at[i] = (T)in[i];
    }
  }
};

/* ---------------------------------------------------------------------------------------
 * short rows: up to SHORT_MAX_PACKS packs, a pack a lane, 1, 2, 4, 8 or 16 lanes a row
 * ------------------------------------------------------------------------------------- */

constexpr int SHORT_MAX_PACKS = 16;
constexpr int SHORT_THREADS = 256;

inline unsigned short_row_grid(size_t m, int G) {
  const size_t blocks = (m * (size_t)G + SHORT_THREADS - 1) / SHORT_THREADS;
  require(blocks < 0x7fffffffull, "row launch: too many rows for one grid");
  return (unsigned)blocks;
}

/* f.template operator()<G, CUT>() for rows of n elements in packs of W: G, the lanes a row, is the
 * next power of two from its packs; CUT says that the last pack is cut (code for it costs the
 * rows of whole packs 10 % when compiled in: r16 n = 48 3.8 -> 4.2 TB/s without). */
template <class F> inline void for_short_row(size_t n, int W, F&& f) {
  const size_t packs = (n + W - 1) / W;
#define MP_SHORT_LANES(CUT_)                          \
  do {                                                \
    if (packs <= 1) f.template operator()<1, CUT_>(); \
    else if (packs <= 2) f.template operator()<2, CUT_>(); \
    else if (packs <= 4) f.template operator()<4, CUT_>(); \
    else if (packs <= 8) f.template operator()<8, CUT_>(); \
    else f.template operator()<16, CUT_>();           \
  } while (0)
  if (n % W != 0) MP_SHORT_LANES(true);
  else MP_SHORT_LANES(false);
#undef MP_SHORT_LANES
}

/* A row of up to G packs in the registers of G lanes, a pack each, so that a wavefront's access
 * is one contiguous kilobyte (two packs a lane over half the lanes: r32 n = 16 3.3 instead of
 * 5.8 TB/s). Packs start at the row's first element whatever its alignment (one 128-bit access
 * all the same), so rows of any length and base need no lanes for a head and a tail; the pack
 * that the end of the row cuts moves in pieces (load_cut_pack_from). The groups wide rows take would
 * leave most lanes idle here (measured, softmax r16 [4M, 8]: 1.1 TB/s at 8 lanes a row, 4.7 at
 * one). */
template <class T, int W, int G, bool CUT> struct ShortRow {
  using P = typename precision<T>::type;
  P v[W];

  /* NT: the row is read once (a streaming load); false for a vector that every row reuses */
  template <bool NT = true> __device__ __forceinline__ void load(const T* row, unsigned n, int lane, P fill) {
    const unsigned j = (unsigned)lane * W;
    if (j + W <= n) {
      if constexpr (NT) load_pack_nt_loose<T, W>(row + j, v);
      else load_pack_loose<T, W>(row + j, v);
    } else {
#pragma unroll
      for (int i = 0; i < W; ++i) v[i] = fill;
      if constexpr (CUT)
        if (j < n) load_cut_pack_from<T, W, 0, W / 2>(row + j, v, n - j);
    }
  }
  __device__ __forceinline__ void store(T* row, unsigned n, int lane) const {
    const unsigned j = (unsigned)lane * W;
    if (j + W <= n) store_pack_nt_loose<T, W>(row + j, v);
    else if constexpr (CUT)
      if (j < n) store_cut_pack<T, W>(row + j, v, n - j);
  }
};

/* The row of this thread's group and whether it exists: a dead group of a live wavefront works
 * on the last row, because the cross-lane steps need every lane, and stores nothing. Workgroups
 * whose rows end inside a cache line are numbered so that neighbours share an L2. */
template <int G> __device__ __forceinline__ size_t short_row_of(size_t m, unsigned by_xcd, bool& live) {
  const unsigned block = by_xcd ? xcd_contiguous_block(blockIdx.x, gridDim.x) : blockIdx.x;
  const size_t want = ((size_t)block * SHORT_THREADS + threadIdx.x) / G;
  live = want < m;
  return live ? want : m - 1;
}

/* whether the rows of one short-row workgroup end inside a cache line */
template <class T> inline unsigned short_rows_share_lines(size_t n, int G) {
  return ((size_t)(SHORT_THREADS / G) * n * sizeof(T)) % 128 != 0 ? 1u : 0u;
}

/* workgroups for m rows when a workgroup of max(G, 64) threads holds max(1, 64 / G) rows */
inline unsigned row_grid(size_t m, int G) {
  const size_t rows_per_block = G < WAVE ? WAVE / G : 1;
  const size_t blocks = (m + rows_per_block - 1) / rows_per_block;
  require(blocks < 0x7fffffffull, "row launch: too many rows for one grid");
  return (unsigned)blocks;
}

}  // namespace mp

#endif
#endif
