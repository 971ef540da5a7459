#include "../gemm_dispatch.h"

// dst[i] = sum_j src[i,j] + alpha*dst[i]. Replaces src/cuda/nvcc_src/reduce_ij_i.cu:3-54
// (called with alpha = 0 by src/ops/reduce.zig:98-121). A few very long rows (the sum of a whole
// tensor) are cut into segments through the workspace that the stream context owns.
extern "C" void launch_reduce_ij_i_Scalar(
  const void* src,
  void* dst,
  double alpha,
  len_t m,
  len_t n,
  StreamContext stream
) {
  MpBlasContext* state = get_blas(stream);
  mp::reduce_rows<Scalar>(static_cast<const Scalar*>(src), static_cast<Scalar*>(dst), alpha, m, n,
                          get_stream(stream), state ? state->workspace : nullptr,
                          state ? state->workspace_bytes : 0);
}
