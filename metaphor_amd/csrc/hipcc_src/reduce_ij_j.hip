#include "../gemm_dispatch.h"

// dst[j] = sum_i src[i,j] + alpha*dst[j]. Replaces src/cuda/nvcc_src/reduce_ij_j.cu:3-66, whose
// output line reads dst[threadIdx.x] instead of its own column (:42-43) and whose grid runs
// over m instead of n (:56); this follows the stated intent (src/ops/reduce.zig:142-165).
// Tall matrices split their rows through the workspace that the stream context owns (work on
// one stream is ordered, so launchers share it); a context without one walks every row per strip.
extern "C" void launch_reduce_ij_j_Scalar(
  const void* src,
  void* dst,
  double alpha,
  len_t m,
  len_t n,
  StreamContext stream
) {
  MpBlasContext* state = get_blas(stream);
  mp::reduce_cols<Scalar>(static_cast<const Scalar*>(src), nullptr, static_cast<Scalar*>(dst),
                          state ? state->workspace : nullptr, 1.0, alpha, m, n, get_stream(stream),
                          state ? state->workspace_bytes : 0);
}
