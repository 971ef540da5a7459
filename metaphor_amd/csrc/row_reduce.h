/*
 * Row / column sums and their reverses (broadcasts) of an [m, n] row-major matrix, with the
 * reference's blend `dst = value + alpha * dst`:
 *   reduce_ij_i     dst[i]   = sum_j src[i,j] + alpha*dst[i]     src/cuda/nvcc_src/reduce_ij_i.cu:3-54
 *   reduce_ij_j     dst[j]   = sum_i src[i,j] + alpha*dst[j]     src/cuda/nvcc_src/reduce_ij_j.cu:3-66
 *   broadcast_i_ij  dst[i,j] = src[i] + alpha*dst[i,j]           src/cuda/nvcc_src/broadcast_i_ij.cu:9-59
 *   broadcast_j_ij  dst[i,j] = src[j] + alpha*dst[i,j]           src/cuda/nvcc_src/broadcast_j_ij.cu:9-57
 * The reference sums a row with one 32-lane warp in the storage type and mis-indexes the output
 * of the column sum (reduce_ij_j.cu:42-43, grid over m instead of n at :56); here sums run in
 * precision<T>, rows are folded with the wave64 all-reduce, and the column sum is a single
 * deterministic pass (each workgroup owns a strip of columns and walks all rows). alpha == 0
 * never reads dst.
 */
#ifndef MP_ROW_REDUCE_H
#define MP_ROW_REDUCE_H

#include "row_dispatch.h"

#if defined(__cplusplus) && defined(__HIPCC__)

namespace mp {

/* ------------------------------------------------------------------ row sums */

/* One group of G threads per row (256/G rows per workgroup when G == 64). */
template <class T, int W, int G>
__global__ __launch_bounds__(G < 256 ? 256 : G) void reduce_rows_kernel(
    const T* src, T* dst, typename precision<T>::type alpha, size_t m, size_t n) {
  using P = typename precision<T>::type;
  constexpr int BLOCK = G < 256 ? 256 : G, RPB = BLOCK / G, U = 4;
  __shared__ P slots[G / WAVE];
  const int sub = threadIdx.x / G, lane = threadIdx.x % G;
  const size_t row = (size_t)blockIdx.x * RPB + sub;
  if (row >= m) return; /* whole waves; wider groups own one row per workgroup */

  const T* r = src + row * n;
  const RowGeom<T, W> g(r, n, true);
  const T* body = r + g.head;
  P s = (P)0;
  for (int p0 = lane; p0 < g.nvec; p0 += G * U) {
    P buf[U][W];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int p = p0 + u * G;
      if (p < g.nvec) {
        load_pack_nt<T, W>(body + (size_t)p * W, buf[u]);
      } else {
#pragma unroll
        for (int i = 0; i < W; ++i) buf[u][i] = (P)0;
      }
    }
#pragma unroll
    for (int u = 0; u < U; ++u)
#pragma unroll
      for (int i = 0; i < W; ++i) s += buf[u][i];
  }
  if (W > 1) {
    if (lane < g.head) s += (P)r[lane];
    else if (lane - g.head < g.tail) s += (P)body[(size_t)g.nvec * W + (lane - g.head)];
  }
  s = group_allreduce<AddOP, G>(s, slots, lane);
  if (lane == 0) dst[row] = (T)(alpha != (P)0 ? s + alpha * (P)dst[row] : s);
}

template <class T>
inline void reduce_rows(const T* src, T* dst, double alpha, size_t m, size_t n, hipStream_t stream) {
  if (m == 0) return;
  using P = typename precision<T>::type;
  constexpr int W = PACK_BYTES / (int)sizeof(T);
  require(n <= 0x40000000ull, "reduce_ij_i: row length must not exceed 2^30");
  require(m < 0x7fffffffull, "reduce_ij_i: too many rows for one grid");
  const size_t packs = (n + W - 1) / W;
  if (packs <= 256) {
    reduce_rows_kernel<T, W, 64><<<dim3((unsigned)((m + 3) / 4)), dim3(256), 0, stream>>>(src, dst, (P)alpha, m, n);
  } else if (packs <= 4096) {
    reduce_rows_kernel<T, W, 256><<<dim3((unsigned)m), dim3(256), 0, stream>>>(src, dst, (P)alpha, m, n);
  } else {
    reduce_rows_kernel<T, W, 1024><<<dim3((unsigned)m), dim3(1024), 0, stream>>>(src, dst, (P)alpha, m, n);
  }
  MP_CHECK_LAUNCH();
}

/* ------------------------------------------------------------------ column sums */

/* A workgroup owns LANES*CW columns; its SLICES slices take every SLICES-th row and are folded
 * through LDS in slice order, so the result does not depend on scheduling. */
template <class T, int CW, int LANES, int SLICES>
__global__ __launch_bounds__(LANES * SLICES) void reduce_cols_kernel(
    const T* src, T* dst, typename precision<T>::type alpha, size_t m, size_t n) {
  using P = typename precision<T>::type;
  __shared__ P part[SLICES][LANES * CW + 1];
  const int c = threadIdx.x % LANES, slice = threadIdx.x / LANES;
  const size_t col = ((size_t)blockIdx.x * LANES + c) * CW;
  P s[CW];
#pragma unroll
  for (int i = 0; i < CW; ++i) s[i] = (P)0;
  if (col < n) {
    size_t r = slice;
    for (; r + 3 * SLICES < m; r += 4 * SLICES) {
      P v[4][CW];
#pragma unroll
      for (int u = 0; u < 4; ++u) load_pack_nt<T, CW>(src + (r + (size_t)u * SLICES) * n + col, v[u]);
#pragma unroll
      for (int u = 0; u < 4; ++u)
#pragma unroll
        for (int i = 0; i < CW; ++i) s[i] += v[u][i];
    }
    for (; r < m; r += SLICES) {
      P v[CW];
      load_pack_nt<T, CW>(src + r * n + col, v);
#pragma unroll
      for (int i = 0; i < CW; ++i) s[i] += v[i];
    }
  }
#pragma unroll
  for (int i = 0; i < CW; ++i) part[slice][c * CW + i] = s[i];
  __syncthreads();
  const int mine = threadIdx.x;
  const size_t out = (size_t)blockIdx.x * LANES * CW + mine;
  if (mine < LANES * CW && out < n) {
    P t = (P)0;
    for (int i = 0; i < SLICES; ++i) t += part[i][mine];
    dst[out] = (T)(alpha != (P)0 ? t + alpha * (P)dst[out] : t);
  }
}

template <class T>
inline void reduce_cols(const T* src, T* dst, double alpha, size_t m, size_t n, hipStream_t stream) {
  if (n == 0) return;
  using P = typename precision<T>::type;
  constexpr int W = PACK_BYTES / (int)sizeof(T);
  const bool packed = aligned16(src) && (n % W) == 0;
  if (packed) { /* 8 lanes x one pack = 128 bytes of every row per workgroup */
    const size_t blocks = (n / W + 7) / 8;
    require(blocks < 0x7fffffffull, "reduce_ij_j: too many columns for one grid");
    reduce_cols_kernel<T, W, 8, 128><<<dim3((unsigned)blocks), dim3(1024), 0, stream>>>(src, dst, (P)alpha, m, n);
  } else {
    const size_t blocks = (n + 31) / 32;
    require(blocks < 0x7fffffffull, "reduce_ij_j: too many columns for one grid");
    reduce_cols_kernel<T, 1, 32, 32><<<dim3((unsigned)blocks), dim3(1024), 0, stream>>>(src, dst, (P)alpha, m, n);
  }
  MP_CHECK_LAUNCH();
}

/* ------------------------------------------------------------------ broadcasts */

/* BY_ROW: dst[i,j] = src[i] + alpha*dst[i,j]; otherwise dst[i,j] = src[j] + alpha*dst[i,j].
 * One workgroup walks rows blockIdx.x, blockIdx.x + gridDim.x, ... */
template <class T, int W, bool BY_ROW, bool BLEND>
__global__ __launch_bounds__(256) void broadcast_kernel(
    const T* src, T* dst, typename precision<T>::type alpha, size_t m, size_t n) {
  using P = typename precision<T>::type;
  const int lane = threadIdx.x;
  for (size_t row = blockIdx.x; row < m; row += gridDim.x) {
    T* r = dst + row * n;
    const RowGeom<T, W> g(r, n, true);
    T* body = r + g.head;
    const P rv = BY_ROW ? (P)src[row] : (P)0;
    for (int p = lane; p < g.nvec; p += 256) {
      P out[W];
#pragma unroll
      for (int i = 0; i < W; ++i) out[i] = BY_ROW ? rv : (P)src[(size_t)g.head + (size_t)p * W + i];
      if constexpr (BLEND) {
        P old[W];
        load_pack<T, W>(body + (size_t)p * W, old);
#pragma unroll
        for (int i = 0; i < W; ++i) out[i] += alpha * old[i];
      }
      store_pack_nt<T, W>(body + (size_t)p * W, out);
    }
    if (W > 1) {
      size_t e = (size_t)-1;
      if (lane < g.head) e = (size_t)lane;
      else if (lane - g.head < g.tail) e = (size_t)g.head + (size_t)g.nvec * W + (lane - g.head);
      if (e != (size_t)-1) {
        P out = BY_ROW ? rv : (P)src[e];
        if constexpr (BLEND) out += alpha * (P)r[e];
        r[e] = (T)out;
      }
    }
  }
}

template <class T, bool BY_ROW>
inline void broadcast(const T* src, T* dst, double alpha, size_t m, size_t n, hipStream_t stream) {
  if (m == 0 || n == 0) return;
  using P = typename precision<T>::type;
  constexpr int W = PACK_BYTES / (int)sizeof(T);
  require(n <= 0x40000000ull, "broadcast: row length must not exceed 2^30");
  const size_t cap = (size_t)compute_units() * 8;
  const dim3 grid((unsigned)(m < cap ? m : cap)), block(256);
  if (alpha != 0.0) broadcast_kernel<T, W, BY_ROW, true><<<grid, block, 0, stream>>>(src, dst, (P)alpha, m, n);
  else broadcast_kernel<T, W, BY_ROW, false><<<grid, block, 0, stream>>>(src, dst, (P)alpha, m, n);
  MP_CHECK_LAUNCH();
}

}  // namespace mp

#endif
#endif
