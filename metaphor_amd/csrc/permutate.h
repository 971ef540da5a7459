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
 * The transposed reads still conflict (the counter shows conflicts in 11 % of the cycles), but they
 * do not bound the kernel: with a conflict-free read pattern it measures the same 6.1 TB/s.
 * Operands whose rows are not 16-byte aligned (an odd row length, a shifted base) keep 128-bit
 * accesses, global and LDS: their packs simply start at any element. A misaligned 128-byte row
 * segment touches two cache lines, which costs this kernel more than it costs a copy (measured:
 * 16384 x 16384 r32 with the source shifted by one element 4.9 TB/s, the destination 5.0, both
 * 4.2; [20000, 50257] r32 3.7, r16 4.4; element-wise fallbacks reached 2.9 and 1.7 there).
 * HBM-bound: 2 * sizeof(T) bytes per element (3 when alpha != 0).
 */
#ifndef MP_PERMUTATE_H
#define MP_PERMUTATE_H

#include "kernel_header.h"

#include <type_traits>

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

/* VIN / VOUT: the source / destination rows are 16-byte aligned (base and row length), so every
 * pack is whole and aligned. Otherwise packs start at any element (see loose_vec_of), the pack that
 * the matrix edge cuts moves element by element, and stores pay about 5 % for the misalignment. */
template <class T, bool VIN, bool VOUT, bool BLEND>
__global__ __launch_bounds__(tp_threads<T>()) void permutate_kernel(
    const T* __restrict__ src, T* __restrict__ dst, typename precision<T>::type alpha,
    size_t rows, size_t cols, unsigned tiles_r) {
  using P = typename precision<T>::type;
  constexpr int W = pack_width<T>(), THREADS = tp_threads<T>(), RP = TP_ROW_PACKS, CP = TP_COL_PACKS;
  constexpr int TR = RP * W, TC = CP * W, STEPS = TR * CP / THREADS; /* packs per thread, in and out */
  using V = typename vec_of<T, W>::type;
  using VI = typename std::conditional<VIN, V, typename loose_vec_of<T, W>::type>::type;
  using VO = typename std::conditional<VOUT, V, typename loose_vec_of<T, W>::type>::type;
  typedef V __attribute__((may_alias)) VA;
  __shared__ __align__(16) T tile[TR * TC];

  const int tid = threadIdx.x;
  const size_t r0 = (size_t)(blockIdx.x % tiles_r) * TR, c0 = (size_t)(blockIdx.x / tiles_r) * TC;

  {
    V v[STEPS];
    /* a pack is loaded whole when it lies inside the matrix; every load is issued before the first
     * is waited for: any other pack reads the first pack of the source instead and is zeroed below */
    auto whole = [&](int s) -> bool {
      const int idx = s * THREADS + tid, r = idx / CP, p = idx % CP;
      return r0 + r < rows && c0 + (size_t)p * W + W <= cols;
    };
    if (VIN || cols >= (size_t)W) { /* uniform: a source narrower than a pack has no first pack */
#pragma unroll
      for (int s = 0; s < STEPS; ++s) {
        const int idx = s * THREADS + tid, r = idx / CP, p = idx % CP;
        const T* from = whole(s) ? src + (r0 + r) * cols + c0 + (size_t)p * W : src;
        v[s] = __builtin_nontemporal_load(reinterpret_cast<const VI*>(from));
      }
    }
#pragma unroll
    for (int s = 0; s < STEPS; ++s) {
      if (!whole(s)) {
#pragma unroll
        for (int i = 0; i < W; ++i) v[s][i] = (T)0;
        if constexpr (!VIN) { /* the pack that the right edge cuts */
          const int idx = s * THREADS + tid, r = idx / CP, p = idx % CP;
          if (r0 + r < rows) {
            const T* row = src + (r0 + r) * cols;
#pragma unroll
            for (int i = 0; i < W; ++i) {
              const size_t c = c0 + (size_t)p * W + i;
              if (c < cols) v[s][i] = row[c];
            }
          }
        }
      }
    }
#pragma unroll
    for (int s = 0; s < STEPS; ++s) {
      const int idx = s * THREADS + tid, r = idx / CP, p = idx % CP;
      *reinterpret_cast<VA*>(&tile[r * TC + ((p ^ (r / W)) & (CP - 1)) * W]) = v[s];
    }
  }
  __syncthreads();

  /* Output element (j, i) of the tile is source element (i, j). Gather every output pack from LDS
   * first (always inside the tile), then fetch the old values when blending, then store: no step
   * waits for the one before it. */
  V out[STEPS];
  size_t at[STEPS]; /* element offset in dst of each output pack that is stored whole, else npos */
  constexpr size_t npos = ~(size_t)0;
  /* output pack s of this thread: destination row j, first column i (r16: the packs 2s and 2s + 1
   * are neighbouring destination rows, gathered together) */
  auto where = [&](int s, size_t& i, size_t& j) {
    if constexpr (sizeof(T) == 2) {
      const int idx = (s / 2) * THREADS + tid;
      j = c0 + 2 * (idx / RP) + (s & 1);
      i = r0 + (size_t)(idx % RP) * W;
    } else {
      const int idx = s * THREADS + tid;
      j = c0 + idx / RP;
      i = r0 + (size_t)(idx % RP) * W;
    }
  };
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
    }
  } else {
#pragma unroll
    for (int s = 0; s < STEPS; ++s) {
      const int idx = s * THREADS + tid, j = idx / RP, ip = idx % RP;
#pragma unroll
      for (int e = 0; e < W; ++e) out[s][e] = tile[tp_at<W>(ip * W + e, j)];
    }
  }
#pragma unroll
  for (int s = 0; s < STEPS; ++s) {
    size_t i, j;
    where(s, i, j);
    at[s] = j < cols && i + W <= rows ? j * rows + i : npos;
  }
  if constexpr (BLEND) {
    if (VOUT || rows >= (size_t)W) { /* uniform: a destination narrower than a pack has no first pack */
      V old[STEPS];
#pragma unroll
      for (int s = 0; s < STEPS; ++s) old[s] = *reinterpret_cast<const VO*>(dst + (at[s] != npos ? at[s] : 0));
#pragma unroll
      for (int s = 0; s < STEPS; ++s)
        if (at[s] != npos) {
#pragma unroll
          for (int e = 0; e < W; ++e) out[s][e] = (T)((P)out[s][e] + alpha * (P)old[s][e]);
        }
    }
  }
#pragma unroll
  for (int s = 0; s < STEPS; ++s)
    if (at[s] != npos) __builtin_nontemporal_store(out[s], reinterpret_cast<VO*>(dst + at[s]));
  if constexpr (!VOUT) {
    /* the pack of each destination row that the bottom edge cuts: only in the last tile of a band */
    if (rows - r0 < (size_t)TR && rows % W != 0) {
#pragma unroll
      for (int s = 0; s < STEPS; ++s) {
        size_t i, j;
        where(s, i, j);
        if (j < cols && i < rows && i + W > rows) {
          T* to = dst + j * rows + i;
          const int left = (int)(rows - i);
#pragma unroll
          for (int e = 0; e < W; ++e)
            if (e < left) {
              T x = out[s][e];
              if constexpr (BLEND) x = (T)((P)x + alpha * (P)to[e]);
              to[e] = x;
            }
        }
      }
    }
  }
}

/* ------------------------------------------------------------------ narrow matrices */

/* A matrix with a short side of n: [m, n] is an array of m records of n fields
 * (AoS), its transpose [n, m] one array per field (SoA). The tall tile above would use n of its
 * 8 packs of columns, or n of its 64 packs of rows (measured r32: [4M, 4] 2.5 TB/s, [4, 4M] 0.4).
 * Here a workgroup moves a chunk of R records: the AoS side is one contiguous run of R * n
 * elements, moved as linear packs, the SoA side n runs of R elements; in between the chunk lies in
 * LDS in AoS order, one pad word after every 32 words so that the gathers and scatters with a stride
 * of n elements spread over the banks. Packs on both sides start at any element. The more fields,
 * the fewer records fit a chunk and the shorter its runs on the field side: reads stand that
 * better than writes (measured against the tall tile, r32 fields to records n = 130: 3.9 -> 4.3 TB/s,
 * r16 n = 128: 3.6 -> 4.9; records to fields n = 96: 5.0 -> 3.4), hence the two limits. */
constexpr size_t TP_NARROW_MAX = 64;      /* records of up to this many fields are split into fields this way */
constexpr size_t TP_NARROW_MAX_BACK = 160; /* and fields are gathered into records of up to this many */
constexpr int TP_NARROW_BYTES = 32768; /* of a chunk in LDS, pads aside */
constexpr int TP_NARROW_THREADS = 256;

/* records per chunk: what fits, in whole packs */
template <class T> inline unsigned tp_narrow_records(size_t n) {
  constexpr int W = pack_width<T>();
  return (unsigned)(TP_NARROW_BYTES / sizeof(T) / n / W * W);
}

/* TO_SOA: src is [m, n] and dst [n, m]; otherwise src is [n, m] and dst [m, n]. */
template <class T, bool TO_SOA, bool BLEND>
__global__ __launch_bounds__(TP_NARROW_THREADS) void permutate_narrow_kernel(
    const T* __restrict__ src, T* __restrict__ dst, typename precision<T>::type alpha, size_t m, unsigned n, unsigned R) {
  using P = typename precision<T>::type;
  constexpr int W = pack_width<T>(), THREADS = TP_NARROW_THREADS;
  constexpr unsigned CAP = TP_NARROW_BYTES / sizeof(T);                   /* elements of a chunk */
  constexpr unsigned BLOCK = 128 / sizeof(T);                             /* elements in 32 words */
  constexpr unsigned PAD = sizeof(T) >= 4 ? 1 : 4 / sizeof(T);            /* elements of a pad: a word at least */
  using V = typename vec_of<T, W>::type;
  using VL = typename loose_vec_of<T, W>::type;
  __shared__ T tile[CAP + CAP / BLOCK * PAD];
  auto lds = [](unsigned e) -> unsigned { return e + e / BLOCK * PAD; };

  const unsigned tid = threadIdx.x;
  const size_t i0 = (size_t)blockIdx.x * R;
  const unsigned here = m - i0 < (size_t)R ? (unsigned)(m - i0) : R; /* records of this chunk */
  const unsigned count = here * n;                                   /* its elements */
  const unsigned ppr = (here + W - 1) / W;                           /* packs of one SoA run, the last one maybe cut */
  const T* aos_in = src + i0 * n;
  T* aos_out = dst + i0 * n;
  const T* soa_in = src + i0;
  T* soa_out = dst + i0;

  if constexpr (TO_SOA) {
    for (unsigned e = tid * W; e < count; e += THREADS * W) {
      if (e + W <= count) {
        *reinterpret_cast<VL*>(&tile[lds(e)]) = __builtin_nontemporal_load(reinterpret_cast<const VL*>(aos_in + e));
      } else {
        for (unsigned k = e; k < count; ++k) tile[lds(k)] = aos_in[k];
      }
    }
    __syncthreads();
    for (unsigned q = tid; q < n * ppr; q += THREADS) {
      const unsigned j = q / ppr, r0 = (q - j * ppr) * W;
      const bool whole = r0 + W <= here;
      V out;
#pragma unroll
      for (int r = 0; r < W; ++r) out[r] = r0 + r < here ? tile[lds((r0 + r) * n + j)] : (T)0;
      T* to = soa_out + (size_t)j * m + r0;
      if (whole) {
        if constexpr (BLEND) {
          const V old = *reinterpret_cast<const VL*>(to);
#pragma unroll
          for (int r = 0; r < W; ++r) out[r] = (T)((P)out[r] + alpha * (P)old[r]);
        }
        __builtin_nontemporal_store(out, reinterpret_cast<VL*>(to));
      } else {
#pragma unroll
        for (int r = 0; r < W; ++r)
          if (r0 + r < here) {
            T x = out[r];
            if constexpr (BLEND) x = (T)((P)x + alpha * (P)to[r]);
            to[r] = x;
          }
      }
    }
  } else {
    for (unsigned q = tid; q < n * ppr; q += THREADS) {
      const unsigned j = q / ppr, r0 = (q - j * ppr) * W;
      const T* from = soa_in + (size_t)j * m + r0;
      V v;
      if (r0 + W <= here) {
        v = __builtin_nontemporal_load(reinterpret_cast<const VL*>(from));
      } else {
#pragma unroll
        for (int r = 0; r < W; ++r) v[r] = r0 + r < here ? from[r] : (T)0;
      }
#pragma unroll
      for (int r = 0; r < W; ++r)
        if (r0 + r < here) tile[lds((r0 + r) * n + j)] = v[r];
    }
    __syncthreads();
    for (unsigned e = tid * W; e < count; e += THREADS * W) {
      T* to = aos_out + e;
      if (e + W <= count) {
        V out = *reinterpret_cast<const VL*>(&tile[lds(e)]);
        if constexpr (BLEND) {
          const V old = *reinterpret_cast<const VL*>(to);
#pragma unroll
          for (int r = 0; r < W; ++r) out[r] = (T)((P)out[r] + alpha * (P)old[r]);
        }
        __builtin_nontemporal_store(out, reinterpret_cast<VL*>(to));
      } else {
        for (unsigned k = e; k < count; ++k) {
          T x = tile[lds(k)];
          if constexpr (BLEND) x = (T)((P)x + alpha * (P)aos_out[k]);
          aos_out[k] = x;
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
  const bool blend = alpha != 0.0;
  const bool to_soa = cols <= rows; /* the short side are the fields of a record */
  if (to_soa ? cols <= TP_NARROW_MAX : rows <= TP_NARROW_MAX_BACK) {
    const size_t m = to_soa ? rows : cols, n = to_soa ? cols : rows;
    const unsigned R = tp_narrow_records<T>(n);
    const size_t chunks = (m + R - 1) / R;
    require(chunks < 0x7fffffffull, "permutate_ij_ji: too many chunks for one grid");
    const dim3 grid((unsigned)chunks), block(TP_NARROW_THREADS);
#define MP_TP_NARROW(TO_SOA)                                                                                      \
  do {                                                                                                            \
    if (blend) permutate_narrow_kernel<T, TO_SOA, true><<<grid, block, 0, stream>>>(src, dst, (P)alpha, m, (unsigned)n, R); \
    else permutate_narrow_kernel<T, TO_SOA, false><<<grid, block, 0, stream>>>(src, dst, (P)alpha, m, (unsigned)n, R);      \
  } while (0)
    if (to_soa) MP_TP_NARROW(true);
    else MP_TP_NARROW(false);
#undef MP_TP_NARROW
    MP_CHECK_LAUNCH();
    return;
  }
  const size_t tiles_r = (rows + TR - 1) / TR, tiles_c = (cols + TC - 1) / TC;
  require(tiles_r < 0x7fffffffull && tiles_c < 0x7fffffffull && tiles_r * tiles_c < 0x7fffffffull,
          "permutate_ij_ji: too many tiles for one grid");
  const bool vin = aligned16(src) && cols % W == 0, vout = aligned16(dst) && rows % W == 0;
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
