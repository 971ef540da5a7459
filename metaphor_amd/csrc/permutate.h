/*
 * Matrix transpose with the reference's blend, dst[j,i] = src[i,j] + alpha*dst[j,i], for a
 * row-major [rows, cols] source. Replaces src/cuda/nvcc_src/permutate_ij_ji.cu:7-71 (a 32x32
 * tile of scalar accesses through a padded shared array, eight rows per pass).
 *
 * Here a workgroup moves one tall tile: 64 packs of rows by 8 packs of columns (r32: 256 x 32
 * elements, r16: 512 x 64, r64: 128 x 16). It reads one 128-byte line from each of its source rows
 * and writes, for each of its source columns, one contiguous kilobyte of the destination; tiles
 * that follow each other along a source column band have consecutive workgroup indices, so the
 * workgroups in flight extend the same destination rows. Measured on the MI355X, long contiguous
 * writes are what a transpose needs: square 64 x 64 tiles in source order reach 4.1 TB/s on a
 * 16384 x 16384 r32 matrix, the same tiles in destination order 5.1 TB/s, this shape 6.0 TB/s
 * (a plain copy: 6.7 TB/s).
 * The tile is kept in LDS in source order with its packs swizzled inside each row (pack p of row r
 * sits in slot p ^ (r / W)), which keeps the 128-bit LDS writes aligned and spreads the transposed
 * reads over the banks. r16 tiles are gathered as 32-bit words (two neighbouring columns at
 * once) and separated in registers, so a thread issues W/2 LDS reads per output pack.
 * Operands whose rows are not 16-byte aligned (an odd row length, a shifted base) keep 128-bit
 * global accesses: every row segment is peeled so that its packs are aligned in memory, and only
 * the LDS side goes element by element.
 * HBM-bound: 2 * sizeof(T) bytes per element (3 when alpha != 0).
 */
#ifndef MP_PERMUTATE_H
#define MP_PERMUTATE_H

#include "kernel_header.h"

#if defined(__cplusplus) && defined(__HIPCC__)

namespace mp {

constexpr int TP_ROW_PACKS = 64; /* tile rows, in packs of the destination */
constexpr int TP_COL_PACKS = 8;  /* tile columns, in packs of the source: one 128-byte line per row */
template <class T> constexpr int tp_threads() { return sizeof(T) == 2 ? 512 : 256; }

typedef unsigned __attribute__((may_alias)) tp_word;

/* Index of element (r, c) of the tile in LDS. */
template <int W>
__device__ __forceinline__ int tp_at(int r, int c) {
  return r * (TP_COL_PACKS * W) + (((c / W) ^ (r / W)) & (TP_COL_PACKS - 1)) * W + (c % W);
}

template <class T, bool VIN, bool VOUT, bool BLEND>
__global__ __launch_bounds__(tp_threads<T>()) void permutate_kernel(
    const T* __restrict__ src, T* __restrict__ dst, typename precision<T>::type alpha,
    size_t rows, size_t cols, unsigned tiles_r) {
  using P = typename precision<T>::type;
  constexpr int W = pack_width<T>(), THREADS = tp_threads<T>(), RP = TP_ROW_PACKS, CP = TP_COL_PACKS;
  constexpr int TR = RP * W, TC = CP * W, STEPS = TR * CP / THREADS; /* packs per thread, in and out */
  using V = typename vec_of<T, W>::type;
  typedef V __attribute__((may_alias)) VA;
  __shared__ __align__(16) T tile[TR * TC];

  const int tid = threadIdx.x;
  const size_t r0 = (size_t)(blockIdx.x % tiles_r) * TR, c0 = (size_t)(blockIdx.x / tiles_r) * TC;

  if constexpr (VIN) {
    V v[STEPS];
#pragma unroll
    for (int s = 0; s < STEPS; ++s) {
      const int idx = s * THREADS + tid, r = idx / CP, p = idx % CP;
      /* every load is issued before the first is waited for: a pack outside the matrix reads the
       * first pack of the source instead and is zeroed below */
      const bool inside = r0 + r < rows && c0 + (size_t)p * W < cols;
      const T* from = inside ? src + (r0 + r) * cols + c0 + (size_t)p * W : src;
      v[s] = __builtin_nontemporal_load(reinterpret_cast<const V*>(from));
    }
#pragma unroll
    for (int s = 0; s < STEPS; ++s) {
      const int idx = s * THREADS + tid, r = idx / CP, p = idx % CP;
      if (!(r0 + r < rows && c0 + (size_t)p * W < cols)) {
#pragma unroll
        for (int i = 0; i < W; ++i) v[s][i] = (T)0;
      }
    }
#pragma unroll
    for (int s = 0; s < STEPS; ++s) {
      const int idx = s * THREADS + tid, r = idx / CP, p = idx % CP;
      *reinterpret_cast<VA*>(&tile[r * TC + ((p ^ (r / W)) & (CP - 1)) * W]) = v[s];
    }
  } else {
    /* Source rows whose length or base breaks the 16-byte alignment: each row's 128-byte segment
     * is peeled into [head scalars][packs aligned in MEMORY][tail scalars]; head and tail together
     * are exactly one pack's worth of elements, so the CP slots of a row still move W elements
     * each: CP - 1 aligned packs and one slot of scalars. A segment cut short by the matrix edge
     * is read element by element. Everything lands in LDS element by element. */
    const int len = cols - c0 < (size_t)TC ? (int)(cols - c0) : TC; /* uniform over the workgroup */
    T v[STEPS][W];
    /* tile column of element i of slot q of a row whose head is h elements long, -1: none */
    auto column = [&](int q, int h, int i) -> int {
      if (len != TC) return q * W + i < len ? q * W + i : -1;
      if (q < CP - (h ? 1 : 0)) return h + q * W + i;
      return i < h ? i : TC - W + i; /* the last slot of a misaligned row: its head and its tail */
    };
    auto head = [&](int r) -> int {
      const T* seg = src + (r0 + r) * cols + c0;
      return (int)(((16u - (unsigned)(reinterpret_cast<uintptr_t>(seg) & 15u)) & 15u) / sizeof(T));
    };
#pragma unroll
    for (int s = 0; s < STEPS; ++s) {
      const int idx = s * THREADS + tid, r = idx / CP, q = idx % CP;
#pragma unroll
      for (int i = 0; i < W; ++i) v[s][i] = (T)0;
      if (r0 + r < rows) {
        const T* seg = src + (r0 + r) * cols + c0;
        const int h = head(r);
        if (len == TC && q < CP - (h ? 1 : 0)) {
          const V pack = __builtin_nontemporal_load(reinterpret_cast<const V*>(seg + h + q * W));
#pragma unroll
          for (int i = 0; i < W; ++i) v[s][i] = pack[i];
        } else {
#pragma unroll
          for (int i = 0; i < W; ++i) {
            const int c = column(q, h, i);
            if (c >= 0) v[s][i] = seg[c];
          }
        }
      }
    }
#pragma unroll
    for (int s = 0; s < STEPS; ++s) {
      const int idx = s * THREADS + tid, r = idx / CP, q = idx % CP;
      if (r0 + r < rows) {
        const int h = head(r);
#pragma unroll
        for (int i = 0; i < W; ++i) {
          const int c = column(q, h, i);
          if (c >= 0) tile[tp_at<W>(r, c)] = v[s][i];
        }
      }
    }
  }
  __syncthreads();

  /* Output element (j, i) of the tile is source element (i, j). */
  if constexpr (VOUT) {
    /* Gather every output pack from LDS first (always inside the tile), then fetch the old
     * values when blending, then store: no step waits for the one before it. */
    V out[STEPS];
    size_t at[STEPS]; /* element offset of each output pack in dst, or npos outside the matrix */
    constexpr size_t npos = ~(size_t)0;
    if constexpr (sizeof(T) == 2) {
      /* Two output rows (source columns 2*jp and 2*jp + 1) per step: 32-bit words hold both. */
#pragma unroll
      for (int s = 0; s < STEPS / 2; ++s) {
        const int idx = s * THREADS + tid, jp = idx / RP, ip = idx % RP;
        unsigned w[W];
#pragma unroll
        for (int e = 0; e < W; ++e) w[e] = *reinterpret_cast<const tp_word*>(&tile[tp_at<W>(ip * W + e, 2 * jp)]);
        typedef unsigned words_t __attribute__((ext_vector_type(W / 2)));
        words_t lo, hi;
#pragma unroll
        for (int e = 0; e < W / 2; ++e) {
          lo[e] = (w[2 * e] & 0xffffu) | (w[2 * e + 1] << 16);
          hi[e] = (w[2 * e] >> 16) | (w[2 * e + 1] & 0xffff0000u);
        }
        out[2 * s] = __builtin_bit_cast(V, lo);
        out[2 * s + 1] = __builtin_bit_cast(V, hi);
        const size_t i = r0 + (size_t)ip * W, j = c0 + 2 * jp;
        at[2 * s] = (j < cols && i < rows) ? j * rows + i : npos;
        at[2 * s + 1] = (j + 1 < cols && i < rows) ? (j + 1) * rows + i : npos;
      }
    } else {
#pragma unroll
      for (int s = 0; s < STEPS; ++s) {
        const int idx = s * THREADS + tid, j = idx / RP, ip = idx % RP;
#pragma unroll
        for (int e = 0; e < W; ++e) out[s][e] = tile[tp_at<W>(ip * W + e, j)];
        const size_t i = r0 + (size_t)ip * W, jj = c0 + j;
        at[s] = (jj < cols && i < rows) ? jj * rows + i : npos;
      }
    }
    if constexpr (BLEND) {
      V old[STEPS];
#pragma unroll
      for (int s = 0; s < STEPS; ++s) old[s] = *reinterpret_cast<const V*>(dst + (at[s] != npos ? at[s] : 0));
#pragma unroll
      for (int s = 0; s < STEPS; ++s)
#pragma unroll
        for (int e = 0; e < W; ++e) out[s][e] = (T)((P)out[s][e] + alpha * (P)old[s][e]);
    }
#pragma unroll
    for (int s = 0; s < STEPS; ++s)
      if (at[s] != npos) __builtin_nontemporal_store(out[s], reinterpret_cast<V*>(dst + at[s]));
  } else {
    /* Destination rows that break the alignment: the same peeling on the way out. The LDS gather
     * is element by element in any case, so a pack may start at any row of the tile. */
    const int len = rows - r0 < (size_t)TR ? (int)(rows - r0) : TR;
#pragma unroll
    for (int s = 0; s < STEPS; ++s) {
      const int idx = s * THREADS + tid, j = idx / RP, q = idx % RP;
      if (c0 + j >= cols) continue;
      T* seg = dst + (c0 + j) * rows + r0;
      const int h = (int)(((16u - (unsigned)(reinterpret_cast<uintptr_t>(seg) & 15u)) & 15u) / sizeof(T));
      if (len == TR && q < RP - (h ? 1 : 0)) {
        const int i0 = h + q * W;
        V out;
#pragma unroll
        for (int e = 0; e < W; ++e) out[e] = tile[tp_at<W>(i0 + e, j)];
        if constexpr (BLEND) {
          const V old = *reinterpret_cast<const V*>(seg + i0);
#pragma unroll
          for (int e = 0; e < W; ++e) out[e] = (T)((P)out[e] + alpha * (P)old[e]);
        }
        __builtin_nontemporal_store(out, reinterpret_cast<V*>(seg + i0));
      } else {
#pragma unroll
        for (int e = 0; e < W; ++e) {
          const int i = len == TR ? (e < h ? e : TR - W + e) : q * W + e;
          if (i < len) {
            T x = tile[tp_at<W>(i, j)];
            if constexpr (BLEND) x = (T)((P)x + alpha * (P)seg[i]);
            seg[i] = x;
          }
        }
      }
    }
  }
}

template <class T>
inline void permutate(const T* src, T* dst, double alpha, size_t rows, size_t cols, hipStream_t stream) {
  if (rows == 0 || cols == 0) return;
  using P = typename precision<T>::type;
  constexpr int W = pack_width<T>(), TR = TP_ROW_PACKS * W, TC = TP_COL_PACKS * W;
  require(static_cast<const void*>(src) != static_cast<const void*>(dst), "permutate_ij_ji: source and destination must differ");
  const size_t tiles_r = (rows + TR - 1) / TR, tiles_c = (cols + TC - 1) / TC;
  require(tiles_r < 0x7fffffffull && tiles_c < 0x7fffffffull && tiles_r * tiles_c < 0x7fffffffull,
          "permutate_ij_ji: too many tiles for one grid");
  const bool vin = aligned16(src) && cols % W == 0, vout = aligned16(dst) && rows % W == 0, blend = alpha != 0.0;
  const dim3 grid((unsigned)(tiles_r * tiles_c)), block(tp_threads<T>());
  const unsigned tr = (unsigned)tiles_r; /* consecutive workgroups walk down a column band of the source */
#define MP_TP_LAUNCH(VIN, VOUT)                                                                                  \
  do {                                                                                                           \
    if (blend) permutate_kernel<T, VIN, VOUT, true><<<grid, block, 0, stream>>>(src, dst, (P)alpha, rows, cols, tr); \
    else permutate_kernel<T, VIN, VOUT, false><<<grid, block, 0, stream>>>(src, dst, (P)alpha, rows, cols, tr);  \
  } while (0)
  if (vin && vout) MP_TP_LAUNCH(true, true);
  else if (vin) MP_TP_LAUNCH(true, false);
  else if (vout) MP_TP_LAUNCH(false, true);
  else MP_TP_LAUNCH(false, false);
#undef MP_TP_LAUNCH
  MP_CHECK_LAUNCH();
}

}  // namespace mp

#endif
#endif
