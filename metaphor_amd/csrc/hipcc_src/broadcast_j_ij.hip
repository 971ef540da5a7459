#include "../row_reduce.h"

// dst[i,j] = src[j] + alpha*dst[i,j]. Replaces src/cuda/nvcc_src/broadcast_j_ij.cu:9-57; the
// reverse of reduce_ij_j calls it with alpha = 1 (src/ops/reduce.zig:167-182).
extern "C" void launch_broadcast_j_ij_Scalar(
  const void* src,
  void* dst,
  double alpha,
  len_t m,
  len_t n,
  StreamContext stream
) {
  mp::broadcast<Scalar, false>(static_cast<const Scalar*>(src), static_cast<Scalar*>(dst), alpha, m, n,
                               get_stream(stream));
}
