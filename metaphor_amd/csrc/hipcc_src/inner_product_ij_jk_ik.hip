#include "../gemm_dispatch.h"

// c[m,k] = alpha * a[m,n] . b[n,k] + beta * c[m,k], row-major. Replaces
// src/cuda/nvcc_src/inner_product_ij_jk_ik.cu:3-27 (called by src/ops/inner_product.zig:286-303).
// The stream context must carry the BLAS handle that mpInitStream creates.
extern "C" void launch_inner_product_ij_jk_ik_Scalar(
  const void* a_data,
  const void* b_data,
  double alpha,
  void* c_data,
  double beta,
  len_t m, len_t n, len_t k,
  StreamContext stream
) {
  mp::gemm_row_major<Scalar>(stream, false, false, a_data, b_data, alpha, c_data, beta, m, n, k);
}
