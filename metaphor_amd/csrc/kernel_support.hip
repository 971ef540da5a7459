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
#endif
