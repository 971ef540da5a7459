/*
 * Row-major matrix products on rocBLAS, C[m,k] = alpha * op(A) * op(B) + beta * C with the
 * contraction running over n. Takes the place of src/cuda/gemm_dispatch.cuh:1-115 (cublasHgemm /
 * Sgemm / Dgemm behind mp_gemm<T>) and of the column-major argument swap in
 * src/cuda/nvcc_src/inner_product_ij_jk_ik.cu:12-26.
 *
 * The handle travels behind the second slot of the StreamContext, as the reference's cuBLAS handle
 * does (src/cuda/kernel_header.h:58-60); mpInitStream creates it and binds it to the stream.
 * r16 multiplies half inputs with fp32 accumulation (the up-cast rule of
 * src/cuda/tensor_types.h:51-69; the reference's cublasHgemm accumulates in half), r32 and r64
 * compute in their own type. Transposed operands are passed as operation flags, so no operand
 * is ever transposed into scratch first (the reference does that, src/ops/inner_product.zig:316-327).
 */
#ifndef MP_GEMM_DISPATCH_H
#define MP_GEMM_DISPATCH_H

#include "row_reduce.h"

#if defined(__cplusplus) && defined(__HIPCC__)

#include <rocblas/rocblas.h>

/* What the second slot of a StreamContext points to: the rocBLAS handle bound to the stream and a
 * workspace the vector products may split their rows through (owned here, so a launcher
 * allocates nothing). Made by mpInitStream / mpAdoptStream, released by mpDeinitStream /
 * mpReleaseStream; work that uses the workspace is ordered by the stream. */
struct MpBlasContext {
  rocblas_handle rocblas;
  void* workspace;
  size_t workspace_bytes;
  hipStream_t stream;
};
constexpr size_t MP_BLAS_WORKSPACE_BYTES = 16u << 20;

inline MpBlasContext* get_blas(StreamContext context) {
  return static_cast<MpBlasContext*>(context.blas_handle.ptr);
}
inline rocblas_handle get_handle(StreamContext context) {
  MpBlasContext* c = get_blas(context);
  return c ? c->rocblas : nullptr;
}

#define ROCBLAS_ASSERT(err) (mpHandleBlasError((err), __FILE__, __LINE__))
inline void mpHandleBlasError(rocblas_status err, const char* file, int line) {
  if (err != rocblas_status_success) {
    fprintf(stderr, "rocBLAS failure (%s) in %s at line %d\n", rocblas_status_to_string(err), file, line);
    exit(EXIT_FAILURE);
  }
}

inline MpBlasContext* mpCreateBlasContext(hipStream_t stream) {
  MpBlasContext* c = new MpBlasContext{nullptr, nullptr, MP_BLAS_WORKSPACE_BYTES, stream};
  ROCBLAS_ASSERT(rocblas_create_handle(&c->rocblas));
  ROCBLAS_ASSERT(rocblas_set_stream(c->rocblas, stream));
  HIP_ASSERT(hipMalloc(&c->workspace, c->workspace_bytes));
  return c;
}
inline void mpDestroyBlasContext(MpBlasContext* c) {
  if (c == nullptr) return;
  HIP_ASSERT(hipFree(c->workspace));
  ROCBLAS_ASSERT(rocblas_destroy_handle(c->rocblas));
  delete c;
}

namespace mp {

template <class T> struct gemm_types;
template <> struct gemm_types<r16> { static constexpr rocblas_datatype data = rocblas_datatype_f16_r, compute = rocblas_datatype_f32_r; };
template <> struct gemm_types<r32> { static constexpr rocblas_datatype data = rocblas_datatype_f32_r, compute = rocblas_datatype_f32_r; };
template <> struct gemm_types<r64> { static constexpr rocblas_datatype data = rocblas_datatype_f64_r, compute = rocblas_datatype_f64_r; };

/* A is [m,n] (or [n,m] when a_transposed), B is [n,k] (or [k,n] when b_transposed), C is [m,k];
 * all row-major and dense. In column-major terms C^T[k,m] = op(B)^T * op(A)^T, which is one
 * library call with the operands exchanged. */
template <class T>
inline void gemm_row_major(StreamContext ctx, bool a_transposed, bool b_transposed, const void* a, const void* b,
                           double alpha, void* c, double beta, size_t m, size_t n, size_t k) {
  if (m == 0 || k == 0) return;
  /* Products with a vector are HBM-bound reads (or, for the outer product, writes) of the one
   * matrix involved: they run on the row / column sum kernels of this library (measured through
   * the library's GEMM with a unit dimension: 0.1 - 2.3 TB/s for r32; here 5 - 6.5). No handle needed. */
  if (n >= 1 && (k == 1 || m == 1 || n == 1)) {
    const T* A = static_cast<const T*>(a);
    const T* B = static_cast<const T*>(b);
    T* C = static_cast<T*>(c);
    hipStream_t stream = get_stream(ctx);
    MpBlasContext* blas = get_blas(ctx); /* may be absent: the column sums then walk all rows per strip */
    void* ws = blas ? blas->workspace : nullptr;
    const size_t ws_bytes = blas ? blas->workspace_bytes : 0;
    if (n == 1) outer_product<T>(A, B, C, alpha, beta, m, k, stream);
    else if (k == 1 && !a_transposed) reduce_rows<T>(A, B, C, alpha, beta, m, n, stream, ws, ws_bytes);
    else if (k == 1) reduce_cols<T>(A, B, C, ws, alpha, beta, n, m, stream, ws_bytes);
    else if (!b_transposed) reduce_cols<T>(B, A, C, ws, alpha, beta, n, k, stream, ws_bytes);
    else reduce_rows<T>(B, A, C, alpha, beta, k, n, stream, ws, ws_bytes);
    return;
  }
  const rocblas_handle handle = get_handle(ctx);
  require(handle != nullptr, "inner_product: the stream context carries no BLAS handle (create the stream with mpInitStream)");
  using P = typename precision<T>::type;
  const P al = (P)alpha, be = (P)beta;
  const int64_t ldb = (int64_t)(b_transposed ? n : k), lda = (int64_t)(a_transposed ? m : n);
  ROCBLAS_ASSERT(rocblas_gemm_ex_64(
      handle, b_transposed ? rocblas_operation_transpose : rocblas_operation_none,
      a_transposed ? rocblas_operation_transpose : rocblas_operation_none, (int64_t)k, (int64_t)m, (int64_t)n, &al,
      b, gemm_types<T>::data, ldb > 0 ? ldb : 1, a, gemm_types<T>::data, lda > 0 ? lda : 1, &be,
      c, gemm_types<T>::data, (int64_t)k, c, gemm_types<T>::data, (int64_t)k, gemm_types<T>::compute,
      rocblas_gemm_algo_standard, 0, 0));
}

}  // namespace mp

#endif
#endif
