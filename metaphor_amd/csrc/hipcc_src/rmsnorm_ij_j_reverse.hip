#include "../row_rmsnorm.h"

// With r_i = 1/sqrt(mean_j src[i,:]^2 + eps) and c_i = mean_j(dst_grads*gain*src)[i,:]:
//   src_grads[i,j] = r_i * (dst_grads[i,j]*gain[j] - src[i,j] * r_i^2 * c_i) + alpha*src_grads[i,j]
//   gain_grads[j]  = sum_i dst_grads[i,j] * src[i,j] * r_i                   + alpha*gain_grads[j]
// scratch is caller-owned workspace of mpRmsnormReverseScratchBytes(dtype, m, n) bytes (the
// reference hands kernels their workspace from the per-stream scratch, src/core/utils.zig:20-36).
// Two kernels are enqueued: the row pass and the fixed-order sum of the partial gain rows.
extern "C" void launch_rmsnorm_ij_j_reverse_Scalar(
  const void* src,
  const void* gain,
  const void* dst_grads,
  void* src_grads,
  void* gain_grads,
  void* scratch,
  double eps,
  double alpha,
  len_t m,
  len_t n,
  StreamContext stream
) {
  mp::rmsnorm_reverse<Scalar>(static_cast<const Scalar*>(src), static_cast<const Scalar*>(gain),
                              static_cast<const Scalar*>(dst_grads), static_cast<Scalar*>(src_grads),
                              static_cast<Scalar*>(gain_grads), scratch, eps, alpha, m, n,
                              get_stream(stream));
}
