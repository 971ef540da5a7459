#include "../row_reduce.h"

// dst[i] = sum_j src[i,j] + alpha*dst[i]. Replaces src/cuda/nvcc_src/reduce_ij_i.cu:3-54
// (called with alpha = 0 by src/ops/reduce.zig:98-121).
extern "C" void launch_reduce_ij_i_Scalar(
  const void* src,
  void* dst,
  double alpha,
  len_t m,
  len_t n,
  StreamContext stream
) {
  mp::reduce_rows<Scalar>(static_cast<const Scalar*>(src), static_cast<Scalar*>(dst), alpha, m, n,
                          get_stream(stream));
}
