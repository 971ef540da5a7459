/*
 * TEST INFRASTRUCTURE — CPU oracle for the row-reduction / elementwise hot path.
 *
 * Scalar restatement, in fp64, of the math behind the launchers declared in
 * include/kernel_decls.h. Only tests, the smoke check and the benchmark's cpu_baseline leg
 * may load this file; the product path never calls it.
 *
 * Inputs are read in their storage type (dtype key 0 = r16, 1 = r32, 2 = r64, the order of
 * the reference's scalar.Tag, src/core/scalar.zig:35-40) and widened to double. Every
 * output is written as double, unrounded, so a test can state its tolerance against the
 * fp64 value. Layout is row-major (src/core/tensor_components.zig:50-67).
 *
 * What each function follows in the reference, and what pins it:
 *   oracle_addition          src/cuda/nvcc_src/addition.cu:12           c = a + b
 *   oracle_hadamard          src/cuda/nvcc_src/hadamard.cu:12           c = a * b
 *   oracle_hadamard_reverse  src/cuda/nvcc_src/hadamard_reverse.cu:12   c += a * b
 *   oracle_subtraction       src/cuda/nvcc_src/subtraction.cu:12        c = a - b
 *   oracle_negate            src/cuda/nvcc_src/negate.cu:11             b = -a
 *   oracle_relu / _reverse   src/cuda/nvcc_src/relu.cu:11-12, relu_reverse.cu:12-14   (a >= 0) convention
 *   oracle_stepwise          the step function (a >= 0) ? 1 : 0 that src/ops/relu.zig:54-57 needs as the
 *                            derivative of relu (the body of stepwise.cu:11-12 is a copy of relu)
 *   oracle_dilate / _reverse src/cuda/nvcc_src/dilate.cu:12, dilate_reverse.cu:12     c = a*v ; b += a*v
 *   oracle_translate         src/cuda/nvcc_src/translate.cu:12          c = a + v
 *   oracle_fill, _sequence   src/cuda/nvcc_src/fill.cu:11, sequence.cu:13             a = v ; a_i = init + step*i
 *   oracle_copy              src/cuda/nvcc_src/copy.cu:19-29            dst = src
 *                            Scalars are narrowed to the storage type first, as the reference launchers do.
 *   oracle_reduce_ij_i       src/cuda/nvcc_src/reduce_ij_i.cu:20-32     dst_i = sum_j + alpha*dst_i
 *   oracle_reduce_ij_j       src/cuda/nvcc_src/reduce_ij_j.cu:10-44     dst_j = sum_i + alpha*dst_j (the intent; the
 *                                                                       reference body mis-indexes dst, :42-43)
 *   oracle_broadcast_i_ij    src/cuda/nvcc_src/broadcast_i_ij.cu:35        dst_ij = src_i + alpha*dst_ij
 *   oracle_broadcast_j_ij    src/cuda/nvcc_src/broadcast_j_ij.cu:30        dst_ij = src_j + alpha*dst_ij
 *   oracle_permutate_ij_ji   src/cuda/nvcc_src/permutate_ij_ji.cu:20-44    dst_ji = src_ij + alpha*dst_ji
 *   oracle_inner_product     src/cuda/nvcc_src/inner_product_ij_jk_ik.cu:12-26 with the operand forms of
 *                            src/ops/inner_product.zig:286-383: c_ik = alpha * sum_j op(a)_ij op(b)_jk + beta*c_ik
 *                            (the arithmetic itself is cuBLAS in the reference, src/cuda/gemm_dispatch.cuh:24-110:
 *                            a closed-source library, restated here as the textbook triple loop)
 *   oracle_selu / _reverse   no reference kernel (only README.md:97); signature and the
 *                            accumulate-into-gradient convention follow relu.cu:11-12 and
 *                            relu_reverse.cu:12-14. Closed form stated below.
 *   oracle_fused_*           composition add -> hadamard -> selu shown in README.md:89-97.
 *   oracle_softmax_*         no reference kernel (NOTES.md:28 lists it as to-do); row-wise
 *                            over the last dim, the "ij|j" form of
 *                            src/ops/expression_parsing.zig:320-340.
 *   oracle_rmsnorm_*         no reference kernel; textbook closed form stated below.
 * The reference ships no tests or golden vectors for any of these, and its device code is
 * CUDA, which this toolchain cannot build. Each function is pinned instead by
 * tests/test_oracle.py: the known answers the reference's examples allow by hand
 * (src/examples/subgraphs.zig:34-45, src/examples/experimental.zig:19-50), library
 * routines in fp64 (torch.softmax, torch.nn.functional.selu / rms_norm and torch autograd
 * for every reverse), finite differences, and algebraic invariants.
 */
#include <math.h>
#include <stddef.h>
#include <stdint.h>
#include <string.h>

#define SELU_ALPHA 1.6732632
#define SELU_SCALE 1.0507010

/* ---- storage-type access ------------------------------------------------------------ */

static double half_bits_to_double(uint16_t h) {
  const int sign = (h >> 15) & 1, exp = (h >> 10) & 0x1f, man = h & 0x3ff;
  double v;
  if (exp == 0) v = ldexp((double)man, -24);
  else if (exp == 31) v = man ? NAN : INFINITY;
  else v = ldexp((double)(man | 0x400), exp - 25);
  return sign ? -v : v;
}

/* double -> IEEE binary16 bits, round to nearest even, directly (no float step). */
uint16_t oracle_double_to_half_bits(double x) {
  uint16_t sign = signbit(x) ? 0x8000u : 0;
  double a = fabs(x);
  if (isnan(x)) return (uint16_t)(sign | 0x7e00u);
  if (a >= 65520.0) return (uint16_t)(sign | 0x7c00u); /* rounds to inf */
  if (a < ldexp(1.0, -25)) return sign;                /* below half the least subnormal */
  int e;
  (void)frexp(a, &e); /* a = f * 2^e, f in [0.5,1) */
  int q = e - 11;     /* quantum exponent for normals: 11 significant bits */
  if (q < -24) q = -24;
  double scaled = ldexp(a, -q);         /* exact */
  double r = nearbyint(scaled);         /* default mode: ties to even */
  double v = ldexp(r, q);
  /* re-encode v, which is exactly representable */
  if (v >= 65520.0) return (uint16_t)(sign | 0x7c00u);
  if (v < ldexp(1.0, -14)) return (uint16_t)(sign | (uint16_t)ldexp(v, 24));
  (void)frexp(v, &e);
  int be = e - 1 + 15;
  uint16_t man = (uint16_t)(ldexp(v, 11 - e) - 1024.0);
  return (uint16_t)(sign | (be << 10) | man);
}

double oracle_half_bits_to_double(uint16_t h) { return half_bits_to_double(h); }

static inline double ld(int key, const void* p, size_t i) {
  switch (key) {
    case 0: return half_bits_to_double(((const uint16_t*)p)[i]);
    case 1: return (double)((const float*)p)[i];
    default: return ((const double*)p)[i];
  }
}

/* ---- elementwise ---------------------------------------------------------------------- */

void oracle_addition(int key, const void* a, const void* b, double* c, size_t N) {
#pragma omp parallel for schedule(static)
  for (size_t i = 0; i < N; ++i) c[i] = ld(key, a, i) + ld(key, b, i);
}

void oracle_hadamard(int key, const void* a, const void* b, double* c, size_t N) {
#pragma omp parallel for schedule(static)
  for (size_t i = 0; i < N; ++i) c[i] = ld(key, a, i) * ld(key, b, i);
}

/* c_out = c_in + a*b; c_in == NULL reads as zeros. */
void oracle_hadamard_reverse(int key, const void* a, const void* b, const void* c_in,
                             double* c_out, size_t N) {
#pragma omp parallel for schedule(static)
  for (size_t i = 0; i < N; ++i)
    c_out[i] = (c_in ? ld(key, c_in, i) : 0.0) + ld(key, a, i) * ld(key, b, i);
}

/* value rounded to the storage type of the dtype key */
static double narrow(int key, double v) {
  switch (key) {
    case 0: return half_bits_to_double(oracle_double_to_half_bits(v));
    case 1: return (double)(float)v;
    default: return v;
  }
}

void oracle_subtraction(int key, const void* a, const void* b, double* c, size_t N) {
#pragma omp parallel for schedule(static)
  for (size_t i = 0; i < N; ++i) c[i] = ld(key, a, i) - ld(key, b, i);
}

void oracle_negate(int key, const void* a, double* b, size_t N) {
#pragma omp parallel for schedule(static)
  for (size_t i = 0; i < N; ++i) b[i] = -ld(key, a, i);
}

void oracle_relu(int key, const void* a, double* b, size_t N) {
#pragma omp parallel for schedule(static)
  for (size_t i = 0; i < N; ++i) { const double v = ld(key, a, i); b[i] = v >= 0.0 ? v : 0.0; }
}

void oracle_relu_reverse(int key, const void* a_value, const void* a_grads_in, const void* b_grads,
                         double* a_grads_out, size_t N) {
#pragma omp parallel for schedule(static)
  for (size_t i = 0; i < N; ++i)
    a_grads_out[i] = (a_grads_in ? ld(key, a_grads_in, i) : 0.0) +
                     ld(key, b_grads, i) * (ld(key, a_value, i) >= 0.0 ? 1.0 : 0.0);
}

void oracle_stepwise(int key, const void* a, double* b, size_t N) {
#pragma omp parallel for schedule(static)
  for (size_t i = 0; i < N; ++i) b[i] = ld(key, a, i) >= 0.0 ? 1.0 : 0.0;
}

void oracle_dilate(int key, const void* a, double value, double* c, size_t N) {
  const double v = narrow(key, value);
#pragma omp parallel for schedule(static)
  for (size_t i = 0; i < N; ++i) c[i] = ld(key, a, i) * v;
}

void oracle_dilate_reverse(int key, const void* a, double value, const void* b_in, double* b_out, size_t N) {
  const double v = narrow(key, value);
#pragma omp parallel for schedule(static)
  for (size_t i = 0; i < N; ++i) b_out[i] = (b_in ? ld(key, b_in, i) : 0.0) + ld(key, a, i) * v;
}

void oracle_translate(int key, const void* a, double value, double* c, size_t N) {
  const double v = narrow(key, value);
#pragma omp parallel for schedule(static)
  for (size_t i = 0; i < N; ++i) c[i] = ld(key, a, i) + v;
}

void oracle_fill(int key, double value, double* a, size_t N) {
  const double v = narrow(key, value);
  for (size_t i = 0; i < N; ++i) a[i] = v;
}

void oracle_sequence(int key, double init, double step, double* a, size_t N) {
  const double i0 = narrow(key, init), st = narrow(key, step);
  for (size_t i = 0; i < N; ++i) a[i] = i0 + st * (double)i;
}

void oracle_copy(int key, const void* src, double* dst, size_t N) {
  for (size_t i = 0; i < N; ++i) dst[i] = ld(key, src, i);
}

/* selu(x) = scale*x for x > 0, scale*alpha*expm1(x) otherwise. */
static inline double selu_f(double x) {
  return x > 0.0 ? SELU_SCALE * x : SELU_SCALE * SELU_ALPHA * expm1(x);
}
/* d selu / dx = scale for x > 0, scale*alpha*exp(x) otherwise. */
static inline double selu_d(double x) {
  return x > 0.0 ? SELU_SCALE : SELU_SCALE * SELU_ALPHA * exp(x);
}

void oracle_selu(int key, const void* a, double* b, size_t N) {
#pragma omp parallel for schedule(static)
  for (size_t i = 0; i < N; ++i) b[i] = selu_f(ld(key, a, i));
}

/* a_grads_out = a_grads_in + b_grads * selu'(a_value); argument order of relu_reverse.cu:18-24. */
void oracle_selu_reverse(int key, const void* a_value, const void* a_grads_in,
                         const void* b_grads, double* a_grads_out, size_t N) {
#pragma omp parallel for schedule(static)
  for (size_t i = 0; i < N; ++i)
    a_grads_out[i] = (a_grads_in ? ld(key, a_grads_in, i) : 0.0) +
                     ld(key, b_grads, i) * selu_d(ld(key, a_value, i));
}

/* e = selu((a+b) * (c+d)) */
void oracle_fused_selu_hadamard_add_add(int key, const void* a, const void* b, const void* c,
                                        const void* d, double* e, size_t N) {
#pragma omp parallel for schedule(static)
  for (size_t i = 0; i < N; ++i) {
    const double u = ld(key, a, i) + ld(key, b, i);
    const double v = ld(key, c, i) + ld(key, d, i);
    e[i] = selu_f(u * v);
  }
}

/* With u = a+b, v = c+d, w = u*v, g = de*selu'(w):
 *   da = db = g*v,  dc = dd = g*u,  each blended as out = val + alpha*in (in == NULL: zeros). */
void oracle_fused_selu_hadamard_add_add_reverse(
    int key, const void* a, const void* b, const void* c, const void* d, const void* de,
    const void* da_in, const void* db_in, const void* dc_in, const void* dd_in,
    double* da, double* db, double* dc, double* dd, double alpha, size_t N) {
#pragma omp parallel for schedule(static)
  for (size_t i = 0; i < N; ++i) {
    const double u = ld(key, a, i) + ld(key, b, i);
    const double v = ld(key, c, i) + ld(key, d, i);
    const double g = ld(key, de, i) * selu_d(u * v);
    da[i] = g * v + (da_in ? alpha * ld(key, da_in, i) : 0.0);
    db[i] = g * v + (db_in ? alpha * ld(key, db_in, i) : 0.0);
    dc[i] = g * u + (dc_in ? alpha * ld(key, dc_in, i) : 0.0);
    dd[i] = g * u + (dd_in ? alpha * ld(key, dd_in, i) : 0.0);
  }
}

/* ---- reductions ----------------------------------------------------------------------- */

void oracle_reduce_ij_i(int key, const void* src, const void* dst_in, double* dst, double alpha,
                        size_t m, size_t n) {
#pragma omp parallel for schedule(static)
  for (size_t i = 0; i < m; ++i) {
    double s = 0.0;
    for (size_t j = 0; j < n; ++j) s += ld(key, src, i * n + j);
    dst[i] = s + (dst_in ? alpha * ld(key, dst_in, i) : 0.0);
  }
}

void oracle_reduce_ij_j(int key, const void* src, const void* dst_in, double* dst, double alpha,
                        size_t m, size_t n) {
#pragma omp parallel for schedule(static)
  for (size_t j = 0; j < n; ++j) {
    double s = 0.0;
    for (size_t i = 0; i < m; ++i) s += ld(key, src, i * n + j);
    dst[j] = s + (dst_in ? alpha * ld(key, dst_in, j) : 0.0);
  }
}

/* dst[i,j] = src[i] + alpha*dst_in[i,j]  (src/cuda/nvcc_src/broadcast_i_ij.cu:35) */
void oracle_broadcast_i_ij(int key, const void* src, const void* dst_in, double* dst, double alpha,
                           size_t m, size_t n) {
#pragma omp parallel for schedule(static)
  for (size_t i = 0; i < m; ++i)
    for (size_t j = 0; j < n; ++j)
      dst[i * n + j] = ld(key, src, i) + (dst_in ? alpha * ld(key, dst_in, i * n + j) : 0.0);
}

/* dst[i,j] = src[j] + alpha*dst_in[i,j]  (src/cuda/nvcc_src/broadcast_j_ij.cu:30) */
void oracle_broadcast_j_ij(int key, const void* src, const void* dst_in, double* dst, double alpha,
                           size_t m, size_t n) {
#pragma omp parallel for schedule(static)
  for (size_t i = 0; i < m; ++i)
    for (size_t j = 0; j < n; ++j)
      dst[i * n + j] = ld(key, src, j) + (dst_in ? alpha * ld(key, dst_in, i * n + j) : 0.0);
}

/* ---- softmax over the last dim -------------------------------------------------------- */

/* ---- transpose and matrix product ------------------------------------------------------- */

void oracle_permutate_ij_ji(int key, const void* src, const void* dst_in, double* dst, double alpha,
                            size_t rows, size_t cols) {
#pragma omp parallel for schedule(static)
  for (size_t j = 0; j < cols; ++j)
    for (size_t i = 0; i < rows; ++i)
      dst[j * rows + i] = ld(key, src, i * cols + j) + (dst_in ? alpha * ld(key, dst_in, j * rows + i) : 0.0);
}

/* a is [m,n] (stored [n,m] when ta), b is [n,k] (stored [k,n] when tb), c is [m,k]. `scale`, when
 * given, receives |alpha| * sum_j |op(a)_ij op(b)_jk| + |beta c_ik|: the size of the terms that a
 * finite-precision sum of the same products can lose to rounding. */
void oracle_inner_product(int key, int ta, int tb, const void* a, const void* b, double alpha,
                          const void* c_in, double beta, double* c, double* scale,
                          size_t m, size_t n, size_t k) {
#pragma omp parallel for schedule(static)
  for (size_t i = 0; i < m; ++i) {
    for (size_t l = 0; l < k; ++l) {
      double s = 0.0, mag = 0.0;
      for (size_t j = 0; j < n; ++j) {
        const double x = ta ? ld(key, a, j * m + i) : ld(key, a, i * n + j);
        const double y = tb ? ld(key, b, l * n + j) : ld(key, b, j * k + l);
        s += x * y;
        mag += fabs(x * y);
      }
      const double old = (c_in && beta != 0.0) ? beta * ld(key, c_in, i * k + l) : 0.0;
      c[i * k + l] = alpha * s + old;
      if (scale) scale[i * k + l] = fabs(alpha) * mag + fabs(old);
    }
  }
}


/* y_ij = exp(x_ij - max_j x_ij) / sum_j exp(x_ij - max_j x_ij); -inf entries give exactly 0.
 * A row with no finite entry (all -inf) yields NaN, as the closed form does. */
void oracle_softmax_ij_j(int key, const void* x, double* y, size_t m, size_t n) {
#pragma omp parallel for schedule(static)
  for (size_t i = 0; i < m; ++i) {
    const size_t o = i * n;
    double mx = -INFINITY;
    for (size_t j = 0; j < n; ++j) { const double v = ld(key, x, o + j); if (v > mx) mx = v; }
    double s = 0.0;
    for (size_t j = 0; j < n; ++j) { const double e = exp(ld(key, x, o + j) - mx); y[o + j] = e; s += e; }
    for (size_t j = 0; j < n; ++j) y[o + j] /= s;
  }
}

/* dx_ij = y_ij * (dy_ij - sum_j y_ij*dy_ij) + alpha*dx_in_ij */
void oracle_softmax_ij_j_reverse(int key, const void* y, const void* dy, const void* dx_in,
                                 double* dx, double alpha, size_t m, size_t n) {
#pragma omp parallel for schedule(static)
  for (size_t i = 0; i < m; ++i) {
    const size_t o = i * n;
    double dot = 0.0;
    for (size_t j = 0; j < n; ++j) dot += ld(key, y, o + j) * ld(key, dy, o + j);
    for (size_t j = 0; j < n; ++j)
      dx[o + j] = ld(key, y, o + j) * (ld(key, dy, o + j) - dot) +
                  (dx_in ? alpha * ld(key, dx_in, o + j) : 0.0);
  }
}

/* ---- RMSNorm over the last dim -------------------------------------------------------- */

/* r_i = (mean_j x_ij^2 + eps)^(-1/2);  y_ij = x_ij * r_i * g_j */
void oracle_rmsnorm_ij_j(int key, const void* x, const void* g, double* y, double eps,
                         size_t m, size_t n) {
#pragma omp parallel for schedule(static)
  for (size_t i = 0; i < m; ++i) {
    const size_t o = i * n;
    double ss = 0.0;
    for (size_t j = 0; j < n; ++j) { const double v = ld(key, x, o + j); ss += v * v; }
    const double r = 1.0 / sqrt(ss / (double)n + eps);
    for (size_t j = 0; j < n; ++j) y[o + j] = ld(key, x, o + j) * r * ld(key, g, j);
  }
}

/* c_i    = mean_j(dy_ij * g_j * x_ij)
 * dx_ij  = r_i * (dy_ij*g_j - x_ij * r_i^2 * c_i) + alpha*dx_in_ij
 * dg_j   = sum_i dy_ij * x_ij * r_i               + alpha*dg_in_j
 * The row loop for dg runs serially in i so the fp64 sum has one fixed order. */
void oracle_rmsnorm_ij_j_reverse(int key, const void* x, const void* g, const void* dy,
                                 const void* dx_in, const void* dg_in, double* dx, double* dg,
                                 double eps, double alpha, size_t m, size_t n) {
  for (size_t j = 0; j < n; ++j) dg[j] = 0.0;
  for (size_t i = 0; i < m; ++i) {
    const size_t o = i * n;
    double ss = 0.0, c = 0.0;
    for (size_t j = 0; j < n; ++j) {
      const double v = ld(key, x, o + j);
      ss += v * v;
      c += ld(key, dy, o + j) * ld(key, g, j) * v;
    }
    const double r = 1.0 / sqrt(ss / (double)n + eps);
    c /= (double)n;
    for (size_t j = 0; j < n; ++j) {
      const double v = ld(key, x, o + j), t = ld(key, dy, o + j);
      dx[o + j] = r * (t * ld(key, g, j) - v * r * r * c) +
                  (dx_in ? alpha * ld(key, dx_in, o + j) : 0.0);
      dg[j] += t * v * r;
    }
  }
  if (dg_in)
    for (size_t j = 0; j < n; ++j) dg[j] += alpha * ld(key, dg_in, j);
}

/* Row-parallel variant of the dx half above, for timing the CPU baseline on many cores;
 * dg is accumulated per thread in row order and the per-thread sums are added in thread order. */
void oracle_rmsnorm_ij_j_reverse_mt(int key, const void* x, const void* g, const void* dy,
                                    double* dx, double* dg, double eps, size_t m, size_t n);

#ifdef _OPENMP
#include <omp.h>
#include <stdlib.h>
int oracle_threads(void) { return omp_get_max_threads(); }
void oracle_set_threads(int t) { omp_set_num_threads(t); }
void oracle_rmsnorm_ij_j_reverse_mt(int key, const void* x, const void* g, const void* dy,
                                    double* dx, double* dg, double eps, size_t m, size_t n) {
  const int T = omp_get_max_threads();
  double* part = (double*)calloc((size_t)T * n, sizeof(double));
#pragma omp parallel num_threads(T)
  {
    double* mine = part + (size_t)omp_get_thread_num() * n;
#pragma omp for schedule(static)
    for (size_t i = 0; i < m; ++i) {
      const size_t o = i * n;
      double ss = 0.0, c = 0.0;
      for (size_t j = 0; j < n; ++j) {
        const double v = ld(key, x, o + j);
        ss += v * v;
        c += ld(key, dy, o + j) * ld(key, g, j) * v;
      }
      const double r = 1.0 / sqrt(ss / (double)n + eps);
      c /= (double)n;
      for (size_t j = 0; j < n; ++j) {
        const double v = ld(key, x, o + j), t = ld(key, dy, o + j);
        dx[o + j] = r * (t * ld(key, g, j) - v * r * r * c);
        mine[j] += t * v * r;
      }
    }
  }
  for (size_t j = 0; j < n; ++j) {
    double s = 0.0;
    for (int t = 0; t < T; ++t) s += part[(size_t)t * n + j];
    dg[j] = s;
  }
  free(part);
}
#else
int oracle_threads(void) { return 1; }
void oracle_set_threads(int t) { (void)t; }
void oracle_rmsnorm_ij_j_reverse_mt(int key, const void* x, const void* g, const void* dy,
                                    double* dx, double* dg, double eps, size_t m, size_t n) {
  oracle_rmsnorm_ij_j_reverse(key, x, g, dy, NULL, NULL, dx, dg, eps, 0.0, m, n);
}
#endif
