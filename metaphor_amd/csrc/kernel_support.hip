/*
 * Exports of the kernel library that are not per-dtype launchers: workspace sizing and (test
 * build only) the row-regime and cluster-tuning overrides. Compiled once (no `Scalar` replication).
 */
#include "row_reduce.h"
#include "row_softmax.h"

// Bytes of caller-owned scratch that launch_rmsnorm_ij_j_reverse_<dtype> needs for an [m, n]
// problem: one row of n accumulators (fp32 for r16/r32, fp64 for r64) per workgroup, at most
// two workgroups per compute unit. dtype is the dispatch key 0 = r16, 1 = r32, 2 = r64
// (the order of the reference's scalar.Tag, src/core/scalar.zig:35-40).
extern "C" len_t mpRmsnormReverseScratchBytes(len_t dtype, len_t m, len_t n) {
  switch (dtype) {
    case MP_R16: return mp::rmsnorm_reverse_scratch_bytes<r16>(m, n);
    case MP_R32: return mp::rmsnorm_reverse_scratch_bytes<r32>(m, n);
    case MP_R64: return mp::rmsnorm_reverse_scratch_bytes<r64>(m, n);
    default: mp::require(false, "mpRmsnormReverseScratchBytes: dtype must be 0, 1 or 2"); return 0;
  }
}

// Bytes of caller-owned scratch that launch_softmax_ij_j_<dtype> can use for an [m, n] problem:
// two accumulator words per workgroup of a row that is shared by several workgroups, 0 when a
// row fits one workgroup. Passing NULL instead is allowed and costs a second read of long rows.
extern "C" len_t mpSoftmaxScratchBytes(len_t dtype, len_t m, len_t n) {
  switch (dtype) {
    case MP_R16: return mp::softmax_scratch_bytes<r16>(m, n);
    case MP_R32: return mp::softmax_scratch_bytes<r32>(m, n);
    case MP_R64: return mp::softmax_scratch_bytes<r64>(m, n);
    default: mp::require(false, "mpSoftmaxScratchBytes: dtype must be 0, 1 or 2"); return 0;
  }
}

// The same for launch_rmsnorm_ij_j_<dtype>: one word per workgroup of a shared row.
extern "C" len_t mpRmsnormScratchBytes(len_t dtype, len_t m, len_t n) {
  switch (dtype) {
    case MP_R16: return mp::rmsnorm_scratch_bytes<r16>(m, n);
    case MP_R32: return mp::rmsnorm_scratch_bytes<r32>(m, n);
    case MP_R64: return mp::rmsnorm_scratch_bytes<r64>(m, n);
    default: mp::require(false, "mpRmsnormScratchBytes: dtype must be 0, 1 or 2"); return 0;
  }
}

// The same for launch_softmax_ij_j_reverse_<dtype>: one word per workgroup of a shared row.
extern "C" len_t mpSoftmaxReverseScratchBytes(len_t dtype, len_t m, len_t n) {
  switch (dtype) {
    case MP_R16: return mp::softmax_reverse_scratch_bytes<r16>(m, n);
    case MP_R32: return mp::softmax_reverse_scratch_bytes<r32>(m, n);
    case MP_R64: return mp::softmax_reverse_scratch_bytes<r64>(m, n);
    default: mp::require(false, "mpSoftmaxReverseScratchBytes: dtype must be 0, 1 or 2"); return 0;
  }
}

// Bytes of caller-owned scratch that launch_reduce_ij_j_scratch_<dtype> can use for an [m, n]
// problem: one partial row of accumulators per row chunk, 0 when the column strips alone fill the GPU.
extern "C" len_t mpReduceScratchBytes(len_t dtype, len_t m, len_t n) {
  switch (dtype) {
    case MP_R16: return mp::reduce_cols_scratch_bytes<r16>(m, n);
    case MP_R32: return mp::reduce_cols_scratch_bytes<r32>(m, n);
    case MP_R64: return mp::reduce_cols_scratch_bytes<r64>(m, n);
    default: mp::require(false, "mpReduceScratchBytes: dtype must be 0, 1 or 2"); return 0;
  }
}

#ifdef MP_DIAGNOSTICS
// Test build only: neither function exists in the library as shipped.
// Diagnostic: force the row regime of the softmax / RMSNorm launchers (0 auto; 1..5 = groups of
// 64, 128, 256, 512, 1024 threads per row; 6 = streaming; 7 = shared rows (cluster path) of the
// softmax launchers; 8, 9 = sub-wave groups of 16 and 32 lanes of the softmax kernels). A group that cannot hold a row falls through to the next wider one. Process-wide; meant for tests and tuning, not for concurrent use with launches.
extern "C" void mpSetRowRegime(len_t regime) {
  mp::require(regime <= mp::REGIME_G32, "mpSetRowRegime: regime must be 0..9");
  mp::row_regime_override() = (int)regime;
}

// Diagnostic: packs (16-byte units) of a row handled per workgroup on the cluster path of the
// softmax forward (0 = default, one pack per thread less than the register tile; larger values
// are clipped to the tile) and the number of polls a workgroup
// waits for its partners before it folds the row itself. Tests set a tiny spin limit to drive
// that second path. Process-wide, like mpSetRowRegime.
extern "C" void mpSetClusterTuning(len_t packs_per_block, len_t spin_limit) {
  mp::require(packs_per_block <= 0x7fffffffull, "mpSetClusterTuning: packs_per_block out of range");
  mp::cluster_tuning().packs_per_block = (int)packs_per_block;
  mp::cluster_tuning().spin_limit = (unsigned)spin_limit;
}

// Diagnostic: which kernel the RMSNorm reverse runs on shared rows of four-byte types: 0 by the
// launcher's rule (the pipelined kernel from 8193 packs a row on), 1 always the pipelined kernel,
// 2 never. Tests use 1 to drive that kernel on small rows. Process-wide.
extern "C" void mpSetClusterDeep(len_t which) {
  mp::require(which <= 2, "mpSetClusterDeep: 0, 1 or 2");
  mp::cluster_tuning().deep = (int)which;
}

// Diagnostic: where the stamped exchange words of the shared-row softmax kernels live: 1 (as
// shipped) in the library's own device memory where a region is to be had, 0 always in the
// caller's workspace, which is then cleared in front of every launch. Process-wide.
extern "C" void mpSetClusterWords(len_t own) {
  mp::require(own <= 1, "mpSetClusterWords: 0 or 1");
  mp::cluster_tuning().own_words = (int)own;
}

// Diagnostic: what the forward kernels leave in the memory-side cache for their reverse (the RMSNorm
// forward's loads of x, the softmax forward's stores of y): 0 nothing (streaming accesses whatever the
// size), 1 always, 2 (as shipped) by the size of the tensor. Process-wide.
extern "C" void mpSetKeepInput(len_t mode) {
  mp::require(mode <= 2, "mpSetKeepInput: 0, 1 or 2");
  mp::cluster_tuning().keep_input = mode == 2 ? -1 : (int)mode;
}

// Diagnostic: what the row launchers decide for [m, n] rows of a dtype on a GPU of `cus` compute
// units, for every n in [n_lo, n_hi), without a GPU: each launcher runs its whole dispatch on a dry
// run (kernel_header.h: MpPlanNote) and the kernel it would enqueue is written to notes[n - n_lo],
// the bytes the matching workspace-size function asks for to sizes[n - n_lo]. op: 0 softmax
// forward, 1 softmax reverse, 2 RMSNorm forward, 3 RMSNorm reverse. shift: 0 every operand 16-byte
// aligned, 1 every operand one element past that, 2 the output one element past the inputs.
// Operands are made-up addresses that nothing dereferences. Returns how many n were noted.
#include "kernel_decls.h"
extern "C" len_t mpDescribeRowPlans(len_t op, len_t dtype, len_t m, len_t n_lo, len_t n_hi, len_t cus, len_t shift,
                                    MpPlanNote* notes, len_t* sizes) {
  mp::require(op <= 3 && dtype <= 2 && shift <= 2 && cus >= 1 && n_lo <= n_hi, "mpDescribeRowPlans: bad arguments");
  const size_t elem = dtype == MP_R16 ? 2 : dtype == MP_R32 ? 4 : 8;
  auto at = [&](int k, bool shifted) {
    return reinterpret_cast<void*>((uintptr_t)0x100000000000ull + (uintptr_t)k * 0x4000000000ull + (shifted ? elem : 0));
  };
  const bool in_shift = shift == 1, out_shift = shift >= 1;
  void *a = at(0, in_shift), *b = at(1, in_shift), *g = at(2, in_shift), *o = at(3, out_shift), *o2 = at(4, false), *ws = at(5, false);
  StreamContext ctx{};
  MpPlanProbe& probe = mp_plan_probe();
  probe.dry = true;
  probe.cus = (int)cus;
  len_t noted = 0;
  for (len_t n = n_lo; n < n_hi; ++n) {
    probe.noted = false;
    probe.note = MpPlanNote{-1, 0, 0, 0, 0, 0, 0, 0, 0, 0};
    len_t need = 0;
#define MP_BY_DTYPE(STEM, ...) \
    do { if (dtype == MP_R16) launch_##STEM##_r16(__VA_ARGS__); else if (dtype == MP_R32) launch_##STEM##_r32(__VA_ARGS__); \
         else launch_##STEM##_r64(__VA_ARGS__); } while (0)
    switch (op) {
      case 0: need = mpSoftmaxScratchBytes(dtype, m, n); MP_BY_DTYPE(softmax_ij_j, a, o, ws, m, n, ctx); break;
      case 1: need = mpSoftmaxReverseScratchBytes(dtype, m, n); MP_BY_DTYPE(softmax_ij_j_reverse, a, b, o, ws, 0.0, m, n, ctx); break;
      case 2: need = mpRmsnormScratchBytes(dtype, m, n); MP_BY_DTYPE(rmsnorm_ij_j, a, g, o, ws, 1e-6, m, n, ctx); break;
      default: need = mpRmsnormReverseScratchBytes(dtype, m, n); MP_BY_DTYPE(rmsnorm_ij_j_reverse, a, g, b, o, o2, ws, 1e-6, 0.0, m, n, ctx); break;
    }
#undef MP_BY_DTYPE
    notes[n - n_lo] = probe.note;
    sizes[n - n_lo] = need;
    noted += probe.noted ? 1 : 0;
  }
  probe.dry = false;
  probe.cus = 0;
  return noted;
}
#endif
