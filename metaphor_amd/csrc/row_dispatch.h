/*
 * Row-regime selection shared by the softmax and RMSNorm launchers.
 *
 * A row of `packs` 128-bit packs is processed by a group of G threads, each holding NV packs
 * in registers between the reduction and the write, so the row is read from HBM once:
 *   wave   G = 64    one wavefront per row, four rows per 256-thread workgroup, cross-lane
 *                    reductions only (rows up to 4 KiB by default);
 *   block  G = 256   one workgroup per row, per-wave partials combined through LDS
 *                    (rows up to 32 KiB);
 *   wide   G = 1024  one 16-wave workgroup per row (rows up to 256 KiB);
 *   stream           rows too long for registers: an online first pass and a second pass that
 *                    re-reads the row (served by L2 / the memory-side cache where it fits).
 * The reference has one regime only: a 32-lane warp per row striding the row with 4-byte loads
 * (src/cuda/nvcc_src/reduce_ij_i.cu:13-32).
 */
#ifndef MP_ROW_DISPATCH_H
#define MP_ROW_DISPATCH_H

#include "kernel_header.h"

#if defined(__cplusplus) && defined(__HIPCC__)

namespace mp {

enum RowRegime { REGIME_AUTO = 0, REGIME_WAVE = 1, REGIME_BLOCK = 2, REGIME_WIDE = 3, REGIME_STREAM = 4 };

/* Diagnostic override set through mpSetRowRegime (device_utils); AUTO in normal use. */
inline int& row_regime_override() {
  static int regime = REGIME_AUTO;
  return regime;
}

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

/* Default regime limits, in packs per thread: a wave takes rows up to 4 KiB, a 256-thread
 * group up to 32 KiB, a 1024-thread group up to 256 KiB, each clipped to max_nv. */
inline RowPlan plan_row(size_t packs, int max_nv) {
  static const int group_of[] = {0, 64, 256, 1024};
  static const int auto_cap[] = {0, 4, 8, 16};
  const int forced = row_regime_override();
  if (forced == REGIME_STREAM) return RowPlan{0, 0};
  /* a forced regime that cannot hold the row moves on to the next wider one */
  for (int r = (forced == REGIME_AUTO ? REGIME_WAVE : forced); r <= REGIME_WIDE; ++r) {
    const int cap = forced == REGIME_AUTO && auto_cap[r] < max_nv ? auto_cap[r] : max_nv;
    const int nv = packs_per_thread(packs, group_of[r], cap);
    if (nv) return RowPlan{group_of[r], nv};
  }
  return RowPlan{0, 0};
}

/* Calls f.template operator()<G, NV>() for the plan; returns false for the streaming plan. */
template <int MAXNV, class F> inline bool for_row_plan(const RowPlan& plan, F&& f) {
#define MP_PLAN_CASE(G_, NV_) \
  if constexpr (NV_ <= MAXNV) { \
    if (plan.G == G_ && plan.NV == NV_) { f.template operator()<G_, NV_>(); return true; } \
  }
#define MP_PLAN_GROUP(G_) \
  MP_PLAN_CASE(G_, 1) MP_PLAN_CASE(G_, 2) MP_PLAN_CASE(G_, 4) MP_PLAN_CASE(G_, 8) MP_PLAN_CASE(G_, 16)
  MP_PLAN_GROUP(64)
  MP_PLAN_GROUP(256)
  MP_PLAN_GROUP(1024)
#undef MP_PLAN_GROUP
#undef MP_PLAN_CASE
  return false;
}

constexpr int STREAM_THREADS = 1024;

template <int G> constexpr int block_threads() { return G < 256 ? 256 : G; }

inline unsigned row_grid(size_t m, int G) {
  const size_t rows_per_block = G < 256 ? 256 / G : 1;
  const size_t blocks = (m + rows_per_block - 1) / rows_per_block;
  require(blocks < 0x7fffffffull, "row launch: too many rows for one grid");
  return (unsigned)blocks;
}

}  // namespace mp

#endif
#endif
