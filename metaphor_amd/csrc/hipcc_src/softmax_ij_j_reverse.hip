#include "../row_softmax.h"

// src_grads[i,j] = dst_value[i,j] * (dst_grads[i,j] - sum_j dst_value[i,j]*dst_grads[i,j])
//                  + alpha * src_grads[i,j].
// Takes the forward OUTPUT, not the input. alpha follows the blend convention of the
// reference's row launchers (src/cuda/nvcc_src/reduce_ij_i.cu:31): 0 overwrites, 1 accumulates.
// scratch: mpSoftmaxReverseScratchBytes(dtype, m, n) bytes owned by the caller, or NULL (rows too
// long for one workgroup are then read twice); the reference's softmax call sites pass one too
// (src/loss/loss.zig:204,226).
extern "C" void launch_softmax_ij_j_reverse_Scalar(
  const void* dst_value,
  const void* dst_grads,
  void* src_grads,
  void* scratch,
  double alpha,
  len_t m,
  len_t n,
  StreamContext stream
) {
  mp::softmax_reverse<Scalar>(static_cast<const Scalar*>(dst_value),
                              static_cast<const Scalar*>(dst_grads),
                              static_cast<Scalar*>(src_grads), scratch, alpha, m, n, get_stream(stream));
}
