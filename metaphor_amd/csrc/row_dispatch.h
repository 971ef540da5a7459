/*
 * Row-regime selection shared by the softmax and RMSNorm launchers.
 *
 * A row of `packs` 128-bit packs is processed by a group of G threads (G = 64 ... 1024), each
 * holding NV packs in registers between the reduction and the write, so the row is read from
 * HBM once. HBM streams fastest here with many small waves each moving one or two packs, so
 * the plan takes the narrowest group that covers the row at a target NV (2 for softmax, 1 for
 * RMSNorm) and only lets NV grow once the group is 1024 threads wide:
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

#if defined(__cplusplus) && defined(__HIPCC__)

namespace mp {

/* 0 = automatic; 1..5 force G = 64, 128, 256, 512, 1024; 6 forces the streaming kernels;
 * 7 forces the cluster path of the softmax forward (the other launchers treat it as automatic). */
enum RowRegime { REGIME_AUTO = 0, REGIME_G64 = 1, REGIME_G128 = 2, REGIME_G256 = 3, REGIME_G512 = 4,
                 REGIME_G1024 = 5, REGIME_STREAM = 6, REGIME_CLUSTER = 7 };

/* Diagnostic override set through mpSetRowRegime; AUTO in normal use. */
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

/* nv_target: packs per thread the automatic plan aims for before it widens the group. */
inline RowPlan plan_row(size_t packs, int max_nv, int nv_target) {
  static const int group_of[] = {0, 64, 128, 256, 512, 1024};
  int forced = row_regime_override();
  if (forced == REGIME_CLUSTER) forced = REGIME_AUTO;
  if (forced == REGIME_STREAM) return RowPlan{0, 0};
  if (forced == REGIME_AUTO) {
    const int want = nv_target < max_nv ? nv_target : max_nv;
    for (int r = REGIME_G64; r <= REGIME_G1024; ++r) {
      const int nv = packs_per_thread(packs, group_of[r], want);
      if (nv) return RowPlan{group_of[r], nv};
    }
    const int nv = packs_per_thread(packs, 1024, max_nv);
    return nv ? RowPlan{1024, nv} : RowPlan{0, 0};
  }
  /* a forced group that cannot hold the row moves on to the next wider one */
  for (int r = forced; r <= REGIME_G1024; ++r) {
    const int nv = packs_per_thread(packs, group_of[r], max_nv);
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
  MP_PLAN_GROUP(128)
  MP_PLAN_GROUP(256)
  MP_PLAN_GROUP(512)
  MP_PLAN_GROUP(1024)
#undef MP_PLAN_GROUP
#undef MP_PLAN_CASE
  return false;
}

constexpr int STREAM_THREADS = 1024;

inline unsigned row_grid(size_t m) {
  require(m < 0x7fffffffull, "row launch: too many rows for one grid");
  return (unsigned)m;
}

}  // namespace mp

#endif
#endif
