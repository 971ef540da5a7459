#include "../row_reduce.h"

// dst[j] = sum_i src[i,j] + alpha*dst[j]. Replaces src/cuda/nvcc_src/reduce_ij_j.cu:3-66, whose
// output line reads dst[threadIdx.x] instead of its own column (:42-43) and whose grid runs
// over m instead of n (:56); this follows the stated intent (src/ops/reduce.zig:142-165).
extern "C" void launch_reduce_ij_j_Scalar(
  const void* src,
  void* dst,
  double alpha,
  len_t m,
  len_t n,
  StreamContext stream
) {
  mp::reduce_cols<Scalar>(static_cast<const Scalar*>(src), static_cast<Scalar*>(dst), nullptr, alpha, m, n,
                          get_stream(stream));
}
