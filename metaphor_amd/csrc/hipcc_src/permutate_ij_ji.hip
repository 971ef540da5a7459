#include "../permutate.h"

// dst[j,i] = src[i,j] + alpha*dst[j,i] for a row-major [row, col] source; src and dst must not
// overlap. Replaces src/cuda/nvcc_src/permutate_ij_ji.cu:7-71 (called with alpha = 0 forward
// and alpha = 1 in reverse by src/ops/permutate.zig:45-69).
extern "C" void launch_permutate_ij_ji_Scalar(
  const void* src,
  void* dst,
  double alpha,
  len_t row,
  len_t col,
  StreamContext ctx
) {
  mp::permutate<Scalar>(static_cast<const Scalar*>(src), static_cast<Scalar*>(dst), alpha, row, col,
                        get_stream(ctx));
}
