#include "../gemm_dispatch.h"

// c[m,k] = alpha * transpose(a[n,m]) . b[n,k] + beta * c[m,k], row-major. No reference launcher:
// src/ops/inner_product.zig:372-383 transposes a into scratch (permutate_ij_ji) and then calls
// inner_product_ij_jk_ik; here the transposition is an operation flag of the library call.
extern "C" void launch_inner_product_ji_jk_ik_Scalar(
  const void* a_data,
  const void* b_data,
  double alpha,
  void* c_data,
  double beta,
  len_t m, len_t n, len_t k,
  StreamContext stream
) {
  mp::gemm_row_major<Scalar>(stream, true, false, a_data, b_data, alpha, c_data, beta, m, n, k);
}
