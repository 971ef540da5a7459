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

/* ------------------------------------------------------------------ few outputs, long contraction */

/* C[m,k] with m, k <= R (4 or 8) and a long contraction n: up to 64 dot products over operands that
 * are read once, an HBM-bound pass that the library's GEMM runs on a single workgroup (measured
 * through it, r32 [4, 1M] x [1M, 4]: 30 ms, 1 GB/s). Here a thread takes W contraction steps at a
 * time and keeps all m*k sums in registers; the workgroups walk the contraction, each leaves one
 * partial C (scaled by alpha) in the stream's workspace and sum_partial_rows adds them in a fixed
 * order with the beta blend.
 * An operand is LONG when the contraction index is its contiguous one (A as [m,n], B as [k,n]):
 * a step is then one pack of each of its rows; otherwise (A as [n,m], B as [n,k]) a step is W rows
 * of up to R elements, each read as one R-element vector from the row's first element (which
 * reads past a row shorter than R: the main loop stops R steps before the end, and the last
 * elements go one by one). */
constexpr size_t SMALL_PRODUCT_MIN_N = 8192; /* shorter contractions stay with the library */
constexpr int SMALL_PRODUCT_THREADS = 256;

template <class T, int W, int R, bool LONG>
__device__ __forceinline__ void small_product_step(const T* x, unsigned r, size_t n, size_t j0,
                                                   typename precision<T>::type (&out)[R][W]) {
  using P = typename precision<T>::type;
  if constexpr (LONG) {
#pragma unroll
    for (int i = 0; i < R; ++i) {
      if (i < (int)r) {
        load_pack_nt_loose<T, W>(x + (size_t)i * n + j0, out[i]);
      } else {
#pragma unroll
        for (int w = 0; w < W; ++w) out[i][w] = (P)0;
      }
    }
  } else {
#pragma unroll
    for (int w = 0; w < W; ++w) {
      P row[R];
      load_pack_nt_loose<T, R>(x + (j0 + w) * r, row);
#pragma unroll
      for (int i = 0; i < R; ++i) out[i][w] = i < (int)r ? row[i] : (P)0;
    }
  }
}

template <class T, int W, int R, bool A_LONG, bool B_LONG>
__global__ __launch_bounds__(SMALL_PRODUCT_THREADS) void small_product_kernel(
    const T* a, const T* b, typename precision<T>::type* partials, typename precision<T>::type scale,
    unsigned m, unsigned k, size_t n, size_t steps) {
  using P = typename precision<T>::type;
  constexpr int THREADS = SMALL_PRODUCT_THREADS, WAVES = THREADS / WAVE;
  __shared__ P part[WAVES][R * R];
  P acc[R][R];
#pragma unroll
  for (int i = 0; i < R; ++i)
#pragma unroll
    for (int l = 0; l < R; ++l) acc[i][l] = (P)0;

  for (size_t s = (size_t)blockIdx.x * THREADS + threadIdx.x; s < steps; s += (size_t)gridDim.x * THREADS) {
    P av[R][W], bv[R][W];
    small_product_step<T, W, R, A_LONG>(a, m, n, s * W, av);
    small_product_step<T, W, R, B_LONG>(b, k, n, s * W, bv);
#pragma unroll
    for (int i = 0; i < R; ++i)
#pragma unroll
      for (int l = 0; l < R; ++l)
#pragma unroll
        for (int w = 0; w < W; ++w) acc[i][l] += av[i][w] * bv[l][w];
  }

#pragma unroll
  for (int i = 0; i < R; ++i)
#pragma unroll
    for (int l = 0; l < R; ++l) {
      const P v = wave_allreduce<AddOP>(acc[i][l]);
      if (threadIdx.x % WAVE == 0) part[threadIdx.x / WAVE][i * R + l] = v;
    }
  __syncthreads();
  const unsigned i = threadIdx.x / R, l = threadIdx.x % R;
  if (threadIdx.x < R * R && i < m && l < k) {
    P t = (P)0;
#pragma unroll
    for (int w = 0; w < WAVES; ++w) t += part[w][threadIdx.x];
    if (blockIdx.x == 0) { /* the contraction steps behind the last whole one */
      for (size_t j = steps * W; j < n; ++j) {
        const P x = (P)(A_LONG ? a[(size_t)i * n + j] : a[j * m + i]);
        const P y = (P)(B_LONG ? b[(size_t)l * n + j] : b[j * k + l]);
        t += x * y;
      }
    }
    partials[(size_t)blockIdx.x * (m * k) + i * k + l] = scale * t;
  }
}

/* Whether the product goes to the kernel above, and with how many workgroups (0: no). */
template <class T> inline unsigned small_product_blocks(size_t m, size_t n, size_t k, size_t workspace_bytes) {
  using P = typename precision<T>::type;
  constexpr int W = PACK_BYTES / (int)sizeof(T);
  if (m > 8 || k > 8 || n < SMALL_PRODUCT_MIN_N) return 0;
  const size_t steps = (n - 8) / W;
  size_t blocks = (steps + SMALL_PRODUCT_THREADS - 1) / SMALL_PRODUCT_THREADS; /* a step a thread at least */
  const size_t most = (size_t)compute_units() * 4, fit = workspace_bytes / (m * k * sizeof(P));
  if (blocks > most) blocks = most;
  if (blocks > fit) blocks = fit;
  return (unsigned)blocks;
}

template <class T>
inline void small_product(const T* a, const T* b, T* c, bool a_transposed, bool b_transposed, double alpha, double beta,
                          size_t m, size_t n, size_t k, unsigned blocks, void* workspace, hipStream_t stream) {
  using P = typename precision<T>::type;
  constexpr int W = PACK_BYTES / (int)sizeof(T);
  P* partials = static_cast<P*>(workspace);
  const dim3 grid(blocks), block(SMALL_PRODUCT_THREADS);
#define MP_SMALL_PRODUCT(R_, AL_, BL_) \
  small_product_kernel<T, W, R_, AL_, BL_><<<grid, block, 0, stream>>>(a, b, partials, (P)alpha, (unsigned)m, (unsigned)k, n, (n - R_) / W)
#define MP_SMALL_PRODUCT_R(R_)                                   \
  do {                                                           \
    if (!a_transposed && b_transposed) MP_SMALL_PRODUCT(R_, true, true);        \
    else if (!a_transposed) MP_SMALL_PRODUCT(R_, true, false);   \
    else if (b_transposed) MP_SMALL_PRODUCT(R_, false, true);    \
    else MP_SMALL_PRODUCT(R_, false, false);                     \
  } while (0)
  if (m <= 4 && k <= 4) MP_SMALL_PRODUCT_R(4);
  else MP_SMALL_PRODUCT_R(8);
#undef MP_SMALL_PRODUCT_R
#undef MP_SMALL_PRODUCT
  MP_CHECK_LAUNCH();
  sum_partial_rows<T>(partials, c, beta, blocks, m * k, stream);
}

/* ------------------------------------------------------------------ many rows through a tiny matrix */

/* C[m,k] = alpha * op(A)[m,n] * op(B)[n,k] + beta * C with n, k <= R (4 or 8) and many rows: every
 * row of C is a few values made from a few values, an HBM-bound pass over A and C that the
 * library's GEMM runs at 0.2 TB/s (r32 [4M, 4] x [4, 4]). A thread takes one row: B sits in
 * registers (its loads are uniform), the row of A comes as one R-element vector from the row's first
 * element (past the row's end when n < R, so the last rows of the matrix go element by element),
 * or, for A stored [n, m], as n coalesced loads; the row of C leaves as one vector when k == R and
 * in pieces otherwise (store_cut_pack). */
constexpr size_t TINY_MAP_MIN_ROWS = 1024; /* fewer rows stay with the library */

template <class T, int R, bool A_T, bool B_T, bool BLEND>
__global__ __launch_bounds__(256) void tiny_map_kernel(
    const T* a, const T* b, T* c, typename precision<T>::type alpha, typename precision<T>::type beta,
    size_t m, unsigned n, unsigned k) {
  using P = typename precision<T>::type;
  P bm[R][R];
#pragma unroll
  for (int j = 0; j < R; ++j)
#pragma unroll
    for (int l = 0; l < R; ++l)
      bm[j][l] = j < (int)n && l < (int)k ? (P)(B_T ? b[(size_t)l * n + j] : b[(size_t)j * k + l]) : (P)0;

  const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= m) return;
  /* whether R elements from this row's start stay inside A, inside C */
  const bool inside_a = i * n + R <= m * n, inside_c = i * k + R <= m * k;

  P x[R];
  if constexpr (A_T) {
#pragma unroll
    for (int j = 0; j < R; ++j) x[j] = j < (int)n ? (P)__builtin_nontemporal_load(a + (size_t)j * m + i) : (P)0;
  } else {
    if (inside_a) {
      load_pack_nt_loose<T, R>(a + i * n, x);
    } else {
#pragma unroll
      for (int j = 0; j < R; ++j) x[j] = j < (int)n ? (P)a[i * n + j] : (P)0;
    }
#pragma unroll
    for (int j = 0; j < R; ++j) x[j] = j < (int)n ? x[j] : (P)0;
  }

  P y[R];
#pragma unroll
  for (int l = 0; l < R; ++l) {
    P t = (P)0;
#pragma unroll
    for (int j = 0; j < R; ++j) t += x[j] * bm[j][l];
    y[l] = alpha * t;
  }
  T* out = c + i * k;
  if constexpr (BLEND) {
    P old[R];
    if (inside_c) {
      load_pack_nt_loose<T, R>(out, old);
    } else {
#pragma unroll
      for (int l = 0; l < R; ++l) old[l] = l < (int)k ? (P)out[l] : (P)0;
    }
#pragma unroll
    for (int l = 0; l < R; ++l) y[l] += beta * (l < (int)k ? old[l] : (P)0);
  }
  if (k == R) store_pack_nt_loose<T, R>(out, y);
  else store_cut_pack<T, R>(out, y, k);
}

template <class T>
inline void tiny_map(const T* a, const T* b, T* c, bool a_transposed, bool b_transposed, double alpha, double beta,
                     size_t m, size_t n, size_t k, hipStream_t stream) {
  using P = typename precision<T>::type;
  const size_t blocks = (m + 255) / 256;
  require(blocks < 0x7fffffffull, "inner_product: too many rows for one grid");
  const dim3 grid((unsigned)blocks), block(256);
#define MP_TINY_MAP(R_, AT_, BT_)                                                                                              \
  do {                                                                                                                         \
    if (beta != 0.0) tiny_map_kernel<T, R_, AT_, BT_, true><<<grid, block, 0, stream>>>(a, b, c, (P)alpha, (P)beta, m, (unsigned)n, (unsigned)k); \
    else tiny_map_kernel<T, R_, AT_, BT_, false><<<grid, block, 0, stream>>>(a, b, c, (P)alpha, (P)beta, m, (unsigned)n, (unsigned)k);         \
  } while (0)
#define MP_TINY_MAP_R(R_)                                     \
  do {                                                        \
    if (a_transposed && b_transposed) MP_TINY_MAP(R_, true, true);   \
    else if (a_transposed) MP_TINY_MAP(R_, true, false);      \
    else if (b_transposed) MP_TINY_MAP(R_, false, true);      \
    else MP_TINY_MAP(R_, false, false);                       \
  } while (0)
  if (n <= 4 && k <= 4) MP_TINY_MAP_R(4);
  else MP_TINY_MAP_R(8);
#undef MP_TINY_MAP_R
#undef MP_TINY_MAP
  MP_CHECK_LAUNCH();
}

/* ------------------------------------------------------------------ a few dot products per row */

/* C[m,k] = alpha * A[m,n] * op(B) + beta * C with 2 <= k <= 8 outputs per row and many rows of any
 * length (a router's logits over a few experts, a head with a few classes): one HBM-bound read of
 * A, which the library's GEMM runs at 0.7 - 2.4 TB/s for r32. A group of G threads takes ROWS
 * consecutive rows at once, so that every pack of the k vectors it loads (from L2; Bt is [k,n],
 * contiguous along the contraction) meets ROWS packs of A: vector traffic k / ROWS of the matrix
 * traffic. Packs count from each row's first element at whatever alignment it has (element-aligned
 * 128-bit accesses), so a pack column is the same in every row and in every vector; the n % W
 * elements behind the last whole pack go one to a lane. The ROWS * k sums are folded across the
 * group in a fixed order (lanes, then wavefronts through LDS behind one barrier) and leave as one
 * contiguous run of ROWS * k values. */
constexpr int FEW_DOTS_ROWS = 4; /* rows a group walks at once (8 measured slower for k = 8: the folds and the stores weigh more than the vector loads) */
constexpr size_t FEW_DOTS_MIN_ROWS = 1024;       /* fewer rows, or a smaller matrix, stay with the library */
constexpr size_t FEW_DOTS_MIN_ELEMENTS = 1u << 21;

template <class T>
__global__ __launch_bounds__(256) void few_dots_transpose_kernel(const T* b, T* bt, size_t n, unsigned k) {
  const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; /* index into Bt[k,n] */
  if (i < n * k) bt[i] = b[(i % n) * k + i / n];
}

template <class T, int W, int G, int K, int R, bool BLEND>
__global__ __launch_bounds__(G < 256 ? 256 : G) void few_dots_kernel(
    const T* a, const T* bt, T* c, typename precision<T>::type alpha, typename precision<T>::type beta, size_t m,
    size_t n, unsigned k) {
  using P = typename precision<T>::type;
  constexpr int BLOCK = G < 256 ? 256 : G, RPB = BLOCK / G, NW = G < WAVE ? 1 : G / WAVE;
  __shared__ P slots[G > WAVE ? R * K : 1][NW];
  const int sub = threadIdx.x / G, lane = threadIdx.x % G;
  const size_t group = (size_t)blockIdx.x * RPB + sub;
  const bool live = group * R < m; /* a dead group of a live workgroup walks the first rows and stores nothing */
  const size_t row0 = live ? group * R : 0;

  const T* rows[R];
#pragma unroll
  for (int r = 0; r < R; ++r) rows[r] = a + (row0 + r < m ? row0 + r : m - 1) * n;
  const T* vecs[K];
#pragma unroll
  for (int j = 0; j < K; ++j) vecs[j] = bt + (size_t)(j < (int)k ? j : 0) * n; /* vectors past k repeat the first */

  P s[R][K];
#pragma unroll
  for (int r = 0; r < R; ++r)
#pragma unroll
    for (int j = 0; j < K; ++j) s[r][j] = (P)0;

  const size_t packs = n / W;
  if constexpr (sizeof(T) == 2) {
    /* v_dot2_f32_f16 on the packs as loaded: two exact half products added to an fp32 sum per
     * instruction, instead of two conversions and a multiply-add per element */
    using V = typename vec_of<T, W>::type;
    using LV = typename loose_vec_of<T, W>::type;
    typedef _Float16 half2_t __attribute__((ext_vector_type(2)));
    for (size_t p = lane; p < packs; p += G) {
      V av[R];
#pragma unroll
      for (int r = 0; r < R; ++r) av[r] = __builtin_nontemporal_load(reinterpret_cast<const LV*>(rows[r] + p * W));
#pragma unroll
      for (int j = 0; j < K; ++j) {
        const V bv = *reinterpret_cast<const LV*>(vecs[j] + p * W);
#pragma unroll
        for (int r = 0; r < R; ++r)
#pragma unroll
          for (int i = 0; i < W; i += 2)
            s[r][j] = __builtin_amdgcn_fdot2(half2_t{av[r][i], av[r][i + 1]}, half2_t{bv[i], bv[i + 1]}, s[r][j], false);
      }
    }
  } else
  for (size_t p = lane; p < packs; p += G) {
    P av[R][W];
#pragma unroll
    for (int r = 0; r < R; ++r) load_pack_nt_loose<T, W>(rows[r] + p * W, av[r]);
#pragma unroll
    for (int j = 0; j < K; ++j) {
      P bv[W];
      load_pack_loose<T, W>(vecs[j] + p * W, bv);
#pragma unroll
      for (int r = 0; r < R; ++r)
#pragma unroll
        for (int i = 0; i < W; ++i) s[r][j] += av[r][i] * bv[i];
    }
  }
  if (W > 1 && (size_t)lane < n - packs * W) {
    const size_t e = packs * W + lane;
#pragma unroll
    for (int j = 0; j < K; ++j) {
      const P bv = (P)vecs[j][e];
#pragma unroll
      for (int r = 0; r < R; ++r) s[r][j] += (P)rows[r][e] * bv;
    }
  }

#pragma unroll
  for (int r = 0; r < R; ++r)
#pragma unroll
    for (int j = 0; j < K; ++j) {
      if constexpr (G <= WAVE) {
        s[r][j] = lanes_allreduce<AddOP, G>(s[r][j]);
      } else {
        s[r][j] = wave_allreduce<AddOP>(s[r][j]);
        if ((lane & (WAVE - 1)) == 0) slots[r * K + j][lane / WAVE] = s[r][j];
      }
    }
  if constexpr (G > WAVE) {
    __syncthreads();
#pragma unroll
    for (int r = 0; r < R; ++r)
#pragma unroll
      for (int j = 0; j < K; ++j) s[r][j] = fold_partials<AddOP, NW>(slots[r * K + j][lane & (NW - 1)]);
  }

  /* lane o of the group writes the o-th of the group's values, C[row0 * k + o] */
  const size_t left = m - row0 < (size_t)R ? m - row0 : (size_t)R;
  const unsigned count = live ? (unsigned)left * k : 0;
#pragma unroll
  for (int base = 0; base < R * K; base += G) {
    const unsigned o = (unsigned)(base + lane);
    P val = (P)0;
#pragma unroll
    for (int r = 0; r < R; ++r)
#pragma unroll
      for (int j = 0; j < K; ++j)
        if (j < (int)k && o == (unsigned)r * k + (unsigned)j) val = s[r][j];
    if (o < count) {
      T* out = c + row0 * k + o;
      val *= alpha;
      if constexpr (BLEND) val += beta * (P)*out;
      *out = (T)val;
    }
  }
}

/* Bt: the k vectors, each n long. */
template <class T>
inline void few_dots(const T* a, const T* bt, T* c, double alpha, double beta, size_t m, size_t n, size_t k,
                     hipStream_t stream) {
  using P = typename precision<T>::type;
  constexpr int W = PACK_BYTES / (int)sizeof(T);
  constexpr size_t R = FEW_DOTS_ROWS;
  const size_t packs = n / W, groups = (m + R - 1) / R;
  require(groups < 0x7fffffffull, "inner_product: too many rows for one grid");
#define MP_FEW_DOTS(G_, K_, R_)                                                                                   \
  do {                                                                                                         \
    const dim3 grid((unsigned)((groups + (G_ < 256 ? 256 / G_ : 1) - 1) / (G_ < 256 ? 256 / G_ : 1))), block(G_ < 256 ? 256 : G_); \
    if (beta != 0.0) few_dots_kernel<T, W, G_, K_, R_, true><<<grid, block, 0, stream>>>(a, bt, c, (P)alpha, (P)beta, m, n, (unsigned)k); \
    else few_dots_kernel<T, W, G_, K_, R_, false><<<grid, block, 0, stream>>>(a, bt, c, (P)alpha, (P)beta, m, n, (unsigned)k);          \
  } while (0)
#define MP_FEW_DOTS_K(G_)              \
  do {                                 \
    if (k <= 2) MP_FEW_DOTS(G_, 2, FEW_DOTS_ROWS);    \
    else if (k <= 4) MP_FEW_DOTS(G_, 4, FEW_DOTS_ROWS); \
    else MP_FEW_DOTS(G_, 8, FEW_DOTS_ROWS);           \
  } while (0)
  if (packs <= 64) MP_FEW_DOTS_K(16);
  else if (packs <= 512) MP_FEW_DOTS_K(64);
  else MP_FEW_DOTS_K(256);
#undef MP_FEW_DOTS_K
#undef MP_FEW_DOTS
  MP_CHECK_LAUNCH();
}

/* ------------------------------------------------------------------ rows made of a few terms */

/* C[m,k] = alpha * A[m,n] * op(B) + beta * C with a contraction of 2 <= n <= 8 and long rows of C
 * (the gradient that a layer with a few outputs sends back to its input: every row of C is a
 * combination of the n rows of B): one HBM-bound write of C, which the library's GEMM runs at
 * 1.3 TB/s for r32 [1M, 8] x [8, 64]. A thread owns one pack column of C for FEW_TERMS_ROWS
 * consecutive rows: its n x W piece of B sits in registers (read once per FEW_TERMS_ROWS packs
 * written), a row of A comes as one 4- or 8-element vector from the row's first element (the last rows
 * of the matrix, where that would pass the end, element by element), packs count from each row's
 * first element at whatever alignment it has, and the pack that the row's end cuts leaves in
 * pieces. Measured 2.2 - 3.4 TB/s for r32 (rows of C of 16 and 64 elements: 0.5 and 1.3 through
 * the GEMM, which wins from rows of about a thousand on), and lower with fewer rows a
 * thread: the limit is the vector memory pipeline, through which every lane of a row asks for
 * the same 32 bytes of A and every thread for its piece of B, not HBM. */
constexpr int FEW_TERMS_ROWS = 4;
constexpr size_t FEW_TERMS_MIN_ELEMENTS = 1u << 21; /* a smaller C stays with the library */
constexpr size_t FEW_TERMS_MAX_ROW = 128;           /* and so do longer rows of C: r32 k = 1024: 5.9 TB/s there, 3.4 here */

template <class T, int W, int N, bool B_T, bool BLEND>
__global__ __launch_bounds__(256) void few_terms_kernel(
    const T* a, const T* b, T* c, typename precision<T>::type alpha, typename precision<T>::type beta, size_t m,
    unsigned n, size_t k, size_t packs_per_row, size_t row_groups) {
  using P = typename precision<T>::type;
  constexpr int R = FEW_TERMS_ROWS; /* N: the contraction rounded up to 4 or 8, the width of the read of a row of A */
  const size_t t = (size_t)blockIdx.x * 256 + threadIdx.x;
  if (t >= row_groups * packs_per_row) return;
  size_t group, col;
  if (row_groups * packs_per_row <= 0xffffffffull) { /* the common case without a 64-bit division */
    const unsigned q = (unsigned)t / (unsigned)packs_per_row;
    group = q;
    col = (size_t)((unsigned)t - q * (unsigned)packs_per_row) * W;
  } else {
    group = t / packs_per_row;
    col = (t % packs_per_row) * W;
  }
  const unsigned width = k - col < (size_t)W ? (unsigned)(k - col) : (unsigned)W;

  P bm[N][W];
#pragma unroll
  for (int j = 0; j < N; ++j)
#pragma unroll
    for (int i = 0; i < W; ++i) bm[j][i] = (P)0;
  if constexpr (!B_T) {
#pragma unroll
    for (int j = 0; j < N; ++j)
      if (j < (int)n) {
        const T* src = b + (size_t)j * k + col;
        if (width == W) {
          load_pack_loose<T, W>(src, bm[j]);
        } else {
#pragma unroll
          for (int i = 0; i < W; ++i)
            if (i < (int)width) bm[j][i] = (P)src[i];
        }
      }
  } else {
#pragma unroll
    for (int i = 0; i < W; ++i)
      if (i < (int)width) {
        const T* src = b + (col + i) * n;
        if ((col + i) * n + N <= k * n) {
          P piece[N];
          load_pack_loose<T, N>(src, piece);
#pragma unroll
          for (int j = 0; j < N; ++j) bm[j][i] = j < (int)n ? piece[j] : (P)0;
        } else {
#pragma unroll
          for (int j = 0; j < N; ++j)
            if (j < (int)n) bm[j][i] = (P)src[j];
        }
      }
  }

#pragma unroll
  for (int r = 0; r < R; ++r) {
    const size_t row = group * R + r;
    if (row >= m) break;
    P x[N];
    if (row * n + N <= m * n) {
      load_pack_nt_loose<T, N>(a + row * n, x);
#pragma unroll
      for (int j = 0; j < N; ++j) x[j] = j < (int)n ? x[j] : (P)0;
    } else {
#pragma unroll
      for (int j = 0; j < N; ++j) x[j] = j < (int)n ? (P)a[row * n + j] : (P)0;
    }
    P y[W];
#pragma unroll
    for (int i = 0; i < W; ++i) {
      P sum = (P)0;
#pragma unroll
      for (int j = 0; j < N; ++j) sum += x[j] * bm[j][i];
      y[i] = alpha * sum;
    }
    T* out = c + row * k + col;
    if constexpr (BLEND) {
      if (width == W) {
        P old[W];
        load_pack_nt_loose<T, W>(out, old);
#pragma unroll
        for (int i = 0; i < W; ++i) y[i] += beta * old[i];
      } else {
#pragma unroll
        for (int i = 0; i < W; ++i)
          if (i < (int)width) y[i] += beta * (P)out[i];
      }
    }
    if (width == W) store_pack_nt_loose<T, W>(out, y);
    else store_cut_pack<T, W>(out, y, width);
  }
}

template <class T>
inline void few_terms(const T* a, const T* b, T* c, bool b_transposed, double alpha, double beta, size_t m, size_t n,
                      size_t k, hipStream_t stream) {
  using P = typename precision<T>::type;
  constexpr int W = PACK_BYTES / (int)sizeof(T);
  const size_t packs_per_row = (k + W - 1) / W, row_groups = (m + FEW_TERMS_ROWS - 1) / FEW_TERMS_ROWS;
  const size_t blocks = (row_groups * packs_per_row + 255) / 256;
  require(blocks < 0x7fffffffull, "inner_product: too many outputs for one grid");
  const dim3 grid((unsigned)blocks), block(256);
#define MP_FEW_TERMS(N_, BT_)                                                                                       \
  do {                                                                                                              \
    if (beta != 0.0) few_terms_kernel<T, W, N_, BT_, true><<<grid, block, 0, stream>>>(a, b, c, (P)alpha, (P)beta, m, (unsigned)n, k, packs_per_row, row_groups); \
    else few_terms_kernel<T, W, N_, BT_, false><<<grid, block, 0, stream>>>(a, b, c, (P)alpha, (P)beta, m, (unsigned)n, k, packs_per_row, row_groups);          \
  } while (0)
  if (n <= 4) {
    if (b_transposed) MP_FEW_TERMS(4, true);
    else MP_FEW_TERMS(4, false);
  } else {
    if (b_transposed) MP_FEW_TERMS(8, true);
    else MP_FEW_TERMS(8, false);
  }
#undef MP_FEW_TERMS
  MP_CHECK_LAUNCH();
}

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
  if (n <= 8 && k <= 8 && m >= TINY_MAP_MIN_ROWS) {
    tiny_map<T>(static_cast<const T*>(a), static_cast<const T*>(b), static_cast<T*>(c), a_transposed, b_transposed, alpha,
                beta, m, n, k, get_stream(ctx));
    return;
  }
  if (!a_transposed && n >= 2 && n <= 8 && k > 8 && k <= FEW_TERMS_MAX_ROW && m * k >= FEW_TERMS_MIN_ELEMENTS) {
    few_terms<T>(static_cast<const T*>(a), static_cast<const T*>(b), static_cast<T*>(c), b_transposed, alpha, beta, m, n, k,
                 get_stream(ctx));
    return;
  }
  if (!a_transposed && k >= 2 && k <= 8 && n > 8 && m >= FEW_DOTS_MIN_ROWS && m * n >= FEW_DOTS_MIN_ELEMENTS) {
    const T* A = static_cast<const T*>(a);
    const T* B = static_cast<const T*>(b);
    T* C = static_cast<T*>(c);
    hipStream_t stream = get_stream(ctx);
    if (b_transposed) {
      few_dots<T>(A, B, C, alpha, beta, m, n, k, stream);
      return;
    }
    /* B stored [n,k]: its k columns are laid out as vectors in the stream's workspace first */
    MpBlasContext* blas = get_blas(ctx);
    if (blas && blas->workspace && n * k * sizeof(T) <= blas->workspace_bytes) {
      T* bt = static_cast<T*>(blas->workspace);
      few_dots_transpose_kernel<T><<<dim3((unsigned)((n * k + 255) / 256)), dim3(256), 0, stream>>>(B, bt, n, (unsigned)k);
      few_dots<T>(A, bt, C, alpha, beta, m, n, k, stream);
      return;
    }
  }
  if (MpBlasContext* blas = get_blas(ctx)) {
    if (const unsigned blocks = small_product_blocks<T>(m, n, k, blas->workspace ? blas->workspace_bytes : 0)) {
      small_product<T>(static_cast<const T*>(a), static_cast<const T*>(b), static_cast<T*>(c), a_transposed, b_transposed,
                       alpha, beta, m, n, k, blocks, blas->workspace, get_stream(ctx));
      return;
    }
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
