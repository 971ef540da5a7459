#include "../row_reduce.h"

// dst[i,j] = src[i] + alpha*dst[i,j]. Replaces src/cuda/nvcc_src/broadcast_i_ij.cu:9-59; the
// reverse of reduce_ij_i calls it with alpha = 1 (src/ops/reduce.zig:123-140).
extern "C" void launch_broadcast_i_ij_Scalar(
  const void* src,
  void* dst,
  double alpha,
  len_t m,
  len_t n,
  StreamContext stream
) {
  mp::broadcast<Scalar, true>(static_cast<const Scalar*>(src), static_cast<Scalar*>(dst), alpha, m, n,
                              get_stream(stream));
}
