#include "../row_reduce.h"

// dst[j] = sum_i src[i,j] + alpha*dst[j], like launch_reduce_ij_j, with caller-owned scratch of
// mpReduceScratchBytes(dtype, m, n) bytes (NULL allowed). No reference launcher: the reference's
// column sum has no workspace parameter (src/cuda/nvcc_src/reduce_ij_j.cu:46-53), so a tall, narrow
// matrix (a bias gradient: [tokens, hidden]) can only be walked by one workgroup per column
// strip. With scratch the rows are split into chunks, every chunk leaves a partial row, and a
// second kernel adds the partial rows in a fixed order.
extern "C" void launch_reduce_ij_j_scratch_Scalar(
  const void* src,
  void* dst,
  void* scratch,
  double alpha,
  len_t m,
  len_t n,
  StreamContext stream
) {
  mp::reduce_cols<Scalar>(static_cast<const Scalar*>(src), static_cast<Scalar*>(dst), scratch, alpha, m, n,
                          get_stream(stream));
}
