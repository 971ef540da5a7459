#include "../row_softmax.h"

// dst[i,j] = exp(src[i,j] - max_j src[i,:]) / sum_j exp(src[i,j] - max_j src[i,:]).
// No reference kernel exists (NOTES.md:28); the (src, dst, m, n) shape follows the row
// launchers (src/cuda/nvcc_src/reduce_ij_i.cu:35-42) and the "ij|j" name the parser stub of
// src/ops/expression_parsing.zig:320-340. dst may be src.
extern "C" void launch_softmax_ij_j_Scalar(
  const void* src,
  void* dst,
  len_t m,
  len_t n,
  StreamContext stream
) {
  mp::softmax_forward<Scalar>(static_cast<const Scalar*>(src), static_cast<Scalar*>(dst), m, n,
                              get_stream(stream));
}
