/*
 * Row / column sums and their reverses (broadcasts) of an [m, n] row-major matrix, with the
 * reference's blend `dst = value + alpha * dst`:
 *   reduce_ij_i     dst[i]   = sum_j src[i,j] + alpha*dst[i]     src/cuda/nvcc_src/reduce_ij_i.cu:3-54
 *   reduce_ij_j     dst[j]   = sum_i src[i,j] + alpha*dst[j]     src/cuda/nvcc_src/reduce_ij_j.cu:3-66
 *   broadcast_i_ij  dst[i,j] = src[i] + alpha*dst[i,j]           src/cuda/nvcc_src/broadcast_i_ij.cu:9-59
 *   broadcast_j_ij  dst[i,j] = src[j] + alpha*dst[i,j]           src/cuda/nvcc_src/broadcast_j_ij.cu:9-57
 * The reference sums a row with one 32-lane warp in the storage type and mis-indexes the output
 * of the column sum (reduce_ij_j.cu:42-43, grid over m instead of n at :56); here sums run in
 * precision<T>, rows are folded with the wave64 all-reduce, and the column sum is deterministic:
 * each workgroup owns a strip of columns and walks all rows, or, given a workspace, a chunk of
 * the rows, whose partial sums a second kernel adds in a fixed order. Operands at any alignment
 * and row length keep 128-bit accesses (packs that start at any element, see loose_vec_of).
 * alpha == 0 never reads dst.
 */
#ifndef MP_ROW_REDUCE_H
#define MP_ROW_REDUCE_H

#include <atomic>
#include "row_rmsnorm.h" /* sum_partial_rows */

#if defined(__cplusplus) && defined(__HIPCC__)

namespace mp {

/* ------------------------------------------------------------------ row sums */

/* One group of G threads per row; groups of 16, 32 or 64 lanes share a 256-thread workgroup
 * (several rows per wavefront below 64), wider groups own one row per workgroup. */
/* DOT: every element is multiplied by vec[column] first (a matrix-vector product, one dot
 * product per row). dst = scale * sum + blend * dst; blend == 0 never reads dst.
 * A row may be cut into `chunks` segments of chunk_len elements (the last one shorter): the
 * kernel then sees rows * chunks logical rows and writes one sum per segment (dst[row * chunks +
 * segment]), which a second
 * launch adds up; O is the type of those sums (the storage type, or precision<T> for partials). */
template <class T, class O, int W, int G, bool DOT>
__global__ __launch_bounds__(G < 256 ? 256 : G) void reduce_rows_kernel(
    const T* src, const T* vec, O* dst, typename precision<T>::type scale, typename precision<T>::type blend,
    size_t segments, size_t n, unsigned chunks, size_t chunk_len) {
  using P = typename precision<T>::type;
  constexpr int BLOCK = G < 256 ? 256 : G, RPB = BLOCK / G, U = 4;
  __shared__ P slots[G < WAVE ? 1 : G / WAVE];
  const int sub = threadIdx.x / G, lane = threadIdx.x % G;
  const size_t want = (size_t)blockIdx.x * RPB + sub;
  const bool live = want < segments; /* a dead group of a live wavefront walks the last segment and stores nothing */
  const size_t q = live ? want : segments - 1;
  /* Neighbouring workgroups take the same segment of neighbouring rows, so that every XCD reads a
   * product's piece of the vector from HBM once for the rows / XCDS rows it sees of it. With few
   * rows that is no reuse at all: then the workgroups that follow each other on one XCD (every
   * XCDS-th) take the same segment instead (measured on r32 [8, 16M] A.v: 3.3 -> 5.3 TB/s; with
   * many rows that order costs 10 %, [64, 2M]: 5.5 -> 4.8). */
  const size_t rows = segments / chunks;
  size_t row, piece;
  if (DOT && RPB == 1 && chunks % XCDS == 0 && rows < 4 * XCDS) {
    const size_t t = q / XCDS;
    row = t % rows;
    piece = t / rows * XCDS + q % XCDS;
  } else {
    row = q % rows;
    piece = q / rows;
  }
  const size_t first = piece * chunk_len;
  const size_t at = row * chunks + piece; /* chunks == 1: the whole row, at == q */
  const size_t len = n - first < chunk_len ? n - first : chunk_len;

  const T* r = src + row * n + first;
  const T* v = vec + first; /* DOT only */
  const RowGeom<T, W> g(r, len, true);
  const T* body = r + g.head;
  const T* vbody = v + g.head; /* the vector entries of the packed columns */
  const bool vec_packed = DOT && (reinterpret_cast<uintptr_t>(vbody) & 15u) == 0;
  P s = (P)0;
  if constexpr (DOT && sizeof(T) == 2) {
    /* v_dot2_f32_f16 on the packs as loaded: two exact half products added to an fp32 sum per
     * instruction, instead of two conversions and a multiply-add per element */
    using V = typename vec_of<T, W>::type;
    typedef _Float16 half2_t __attribute__((ext_vector_type(2)));
    for (int p0 = lane; p0 < g.nvec; p0 += G * U) {
      V a[U], b[U];
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const int p = p0 + u * G;
        if (p < g.nvec) {
          a[u] = __builtin_nontemporal_load(reinterpret_cast<const V*>(body + (size_t)p * W));
          b[u] = *reinterpret_cast<const typename loose_vec_of<T, W>::type*>(vbody + (size_t)p * W);
        } else {
          a[u] = b[u] = V{};
        }
      }
#pragma unroll
      for (int u = 0; u < U; ++u)
#pragma unroll
        for (int i = 0; i < W; i += 2)
          s = __builtin_amdgcn_fdot2(half2_t{a[u][i], a[u][i + 1]}, half2_t{b[u][i], b[u][i + 1]}, s, false);
    }
  } else {
    for (int p0 = lane; p0 < g.nvec; p0 += G * U) {
      P buf[U][W], wv[U][W];
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const int p = p0 + u * G;
        if (p < g.nvec) {
          load_pack_nt<T, W>(body + (size_t)p * W, buf[u]);
          if constexpr (DOT) {
            if (vec_packed) load_pack<T, W>(vbody + (size_t)p * W, wv[u]);
            else load_pack_loose<T, W>(vbody + (size_t)p * W, wv[u]); /* the row's packs are aligned, the vector's not */
          }
        } else {
#pragma unroll
          for (int i = 0; i < W; ++i) buf[u][i] = wv[u][i] = (P)0;
        }
      }
#pragma unroll
      for (int u = 0; u < U; ++u)
#pragma unroll
        for (int i = 0; i < W; ++i) s += DOT ? buf[u][i] * wv[u][i] : buf[u][i];
    }
  }
  if (W > 1) {
    size_t e = (size_t)-1;
    if (lane < g.head) e = (size_t)lane;
    else if (lane - g.head < g.tail) e = (size_t)g.head + (size_t)g.nvec * W + (lane - g.head);
    if (e != (size_t)-1) s += DOT ? (P)r[e] * (P)v[e] : (P)r[e];
  }
  s = group_allreduce<AddOP, G>(s, slots, lane);
  if (live && lane == 0) dst[at] = (O)(blend != (P)0 ? scale * s + blend * (P)dst[at] : scale * s);
}

/* Rows of up to sixteen packs: a pack a lane, 1 ... 16 lanes a row (ShortRow). Groups as wide as
 * the longer rows take would leave most lanes idle (measured on r32 [16M, 2]: 0.07 TB/s with
 * sixteen lanes a row). */
template <class T, class O, int W, int G, bool CUT, bool DOT>
__global__ __launch_bounds__(SHORT_THREADS) void reduce_short_rows_kernel(
    const T* src, const T* vec, O* dst, typename precision<T>::type scale, typename precision<T>::type blend,
    size_t rows, unsigned n) {
  using P = typename precision<T>::type;
  const int lane = threadIdx.x % G;
  bool live;
  const size_t row = short_row_of<G>(rows, 0, live);
  ShortRow<T, W, G, CUT> a;
  a.load(src + row * n, n, lane, (P)0);
  P s = (P)0;
  if constexpr (DOT) {
    ShortRow<T, W, G, CUT> b;
    b.template load<false>(vec, n, lane, (P)0);
#pragma unroll
    for (int i = 0; i < W; ++i) s += a.v[i] * b.v[i];
  } else {
#pragma unroll
    for (int i = 0; i < W; ++i) s += a.v[i];
  }
  s = fold_partials<AddOP, G>(s);
  if (live && lane == 0) dst[row] = (O)(blend != (P)0 ? scale * s + blend * (P)dst[row] : scale * s);
}

/* One launch of the kernel above: `rows` rows of n elements of S, each cut into `chunks` segments. */
template <class S, class O>
inline void launch_reduce_rows(const S* src, const S* vec, O* dst, double scale, double blend, size_t rows, size_t n,
                               size_t chunks, size_t chunk_len, hipStream_t stream) {
  using P = typename precision<S>::type;
  constexpr int W = PACK_BYTES / (int)sizeof(S);
  const size_t segments = rows * chunks;
  require(segments < 0x7fffffffull, "row sums: too many rows for one grid");
  if (chunks == 1 && n <= (size_t)(SHORT_MAX_PACKS * W)) {
    for_short_row(n, W, [&]<int G, bool CUT>() {
      const dim3 grid(short_row_grid(rows, G)), block(SHORT_THREADS);
      if (vec) reduce_short_rows_kernel<S, O, W, G, CUT, true><<<grid, block, 0, stream>>>(src, vec, dst, (P)scale, (P)blend, rows, (unsigned)n);
      else reduce_short_rows_kernel<S, O, W, G, CUT, false><<<grid, block, 0, stream>>>(src, vec, dst, (P)scale, (P)blend, rows, (unsigned)n);
    });
    MP_CHECK_LAUNCH();
    return;
  }
  const size_t packs = (chunk_len + W - 1) / W;
#define MP_ROWS_LAUNCH(G_)                                                                                          \
  do {                                                                                                              \
    const dim3 grid((unsigned)((segments + (G_ < 256 ? 256 / G_ : 1) - 1) / (G_ < 256 ? 256 / G_ : 1))), block(G_ < 256 ? 256 : G_); \
    if (vec) reduce_rows_kernel<S, O, W, G_, true><<<grid, block, 0, stream>>>(src, vec, dst, (P)scale, (P)blend, segments, n, (unsigned)chunks, chunk_len); \
    else reduce_rows_kernel<S, O, W, G_, false><<<grid, block, 0, stream>>>(src, vec, dst, (P)scale, (P)blend, segments, n, (unsigned)chunks, chunk_len);   \
  } while (0)
  if (packs <= 16) MP_ROWS_LAUNCH(16);
  else if (packs <= 32) MP_ROWS_LAUNCH(32);
  else if (packs <= 256) MP_ROWS_LAUNCH(64);
  else if (packs <= 4096) MP_ROWS_LAUNCH(256);
  else MP_ROWS_LAUNCH(1024);
#undef MP_ROWS_LAUNCH
  MP_CHECK_LAUNCH();
}

/* dst[i] = scale * sum_j src[i,j] (* vec[j] when vec is given) + blend * dst[i].
 * workspace (optional, workspace_bytes of it): a few very long rows (the sum or the dot product
 * of whole tensors) would otherwise keep one workgroup each busy; with it they are cut into
 * segments whose sums, kept in precision<T>, a second launch adds in a fixed order
 * (measured: r32 [1, 2^26] 0.06 TB/s without). */
template <class T>
inline void reduce_rows(const T* src, const T* vec, T* dst, double scale, double blend, size_t m, size_t n,
                        hipStream_t stream, void* workspace = nullptr, size_t workspace_bytes = 0) {
  if (m == 0) return;
  using P = typename precision<T>::type;
  constexpr int W = PACK_BYTES / (int)sizeof(T);
  require(n <= 0x40000000ull, "row sums: row length must not exceed 2^30");
  require(m < 0x7fffffffull, "row sums: too many rows for one grid");
  constexpr size_t SHORTEST = 16384; /* elements of a segment: sixteen packs a thread of a 256-thread group for r32 */
  const size_t want = (size_t)compute_units() * 16;
  size_t chunks = 1;
  if (workspace != nullptr && m < want && n >= 2 * SHORTEST) {
    chunks = (want + m - 1) / m;
    if (chunks > n / SHORTEST) chunks = n / SHORTEST;
    const size_t fit = workspace_bytes / (m * sizeof(P));
    if (chunks > fit) chunks = fit;
    if (chunks > 4096) chunks = 4096;
  }
  if (chunks > 1) {
    size_t chunk_len = (n + chunks - 1) / chunks;
    chunk_len = (chunk_len + W - 1) / W * W; /* whole packs, so that aligned rows give aligned segments */
    chunks = (n + chunk_len - 1) / chunk_len;
    P* partials = static_cast<P*>(workspace);
    launch_reduce_rows<T, P>(src, vec, partials, 1.0, 0.0, m, n, chunks, chunk_len, stream);
    launch_reduce_rows<P, T>(partials, nullptr, dst, scale, blend, m, chunks, 1, chunks, stream);
    return;
  }
  launch_reduce_rows<T, T>(src, vec, dst, scale, blend, m, n, 1, n, stream);
}

template <class T>
inline void reduce_rows(const T* src, T* dst, double alpha, size_t m, size_t n, hipStream_t stream,
                        void* workspace = nullptr, size_t workspace_bytes = 0) {
  reduce_rows<T>(src, nullptr, dst, 1.0, alpha, m, n, stream, workspace, workspace_bytes);
}

/* ------------------------------------------------------------------ column sums */

/* A workgroup owns LANES*CW columns of the rows [blockIdx.y * chunk, (blockIdx.y + 1) * chunk); its
 * SLICES slices take every SLICES-th of those rows. The slices of a wavefront (64 / LANES of them)
 * are folded with lane exchanges, the wavefronts through LDS in wavefront order, so the result
 * does not depend on scheduling. LANES is the power of two that holds the packs of a row of a
 * narrow matrix (every lane busy however narrow it is: LANES == 1 is a thread per row), else 8
 * or 64.
 * The sums go to `out + blockIdx.y * n`: the destination itself (O = T, one chunk holding every
 * row, alpha blend) or a partial row of accumulators (O = precision<T>, no blend) that
 * sum_partial_rows adds up afterwards. WEIGHTED: row r counts weight[r] times (a vector-matrix
 * product). LOOSE: rows that are not 16-byte aligned (an odd row length, a shifted base); the
 * packs then start at any element, which a streaming read does not feel, and the pack that the
 * end of the row cuts is read element by element. */
template <class T, class O, int CW, int LANES, int SLICES, bool WEIGHTED, bool LOOSE>
__global__ __launch_bounds__(LANES * SLICES) void reduce_cols_kernel(
    const T* src, const T* weight, O* out, typename precision<T>::type scale, typename precision<T>::type blend,
    size_t m, size_t n, size_t chunk) {
  using P = typename precision<T>::type;
  static_assert(LANES <= WAVE && (LANES & (LANES - 1)) == 0, "a wavefront holds whole slices");
  constexpr int WAVES = LANES * SLICES / WAVE;
  __shared__ P part[WAVES][LANES * CW + 1];
  const int c = threadIdx.x % LANES, slice = threadIdx.x / LANES;
  const size_t col = ((size_t)blockIdx.x * LANES + c) * CW;
  const size_t begin = (size_t)blockIdx.y * chunk, end = begin + chunk < m ? begin + chunk : m;
  O* dst = out + (size_t)blockIdx.y * n;
  P s[CW];
#pragma unroll
  for (int i = 0; i < CW; ++i) s[i] = (P)0;
  const bool whole = col + CW <= n;
  auto fetch = [&](size_t row, P(&v)[CW]) {
    const T* p = src + row * n + col;
    if constexpr (!LOOSE) {
      load_pack_nt<T, CW>(p, v);
    } else if (whole) {
      load_pack_nt_loose<T, CW>(p, v);
    } else {
#pragma unroll
      for (int i = 0; i < CW; ++i) v[i] = col + i < n ? (P)p[i] : (P)0;
    }
  };
  if (col < n) {
    size_t r = begin + slice;
    for (; r + 3 * SLICES < end; r += 4 * SLICES) {
      P v[4][CW], w[4];
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        fetch(r + (size_t)u * SLICES, v[u]);
        w[u] = WEIGHTED ? (P)weight[r + (size_t)u * SLICES] : (P)1;
      }
#pragma unroll
      for (int u = 0; u < 4; ++u)
#pragma unroll
        for (int i = 0; i < CW; ++i) s[i] += WEIGHTED ? w[u] * v[u][i] : v[u][i];
    }
    for (; r < end; r += SLICES) {
      P v[CW];
      fetch(r, v);
      const P w = WEIGHTED ? (P)weight[r] : (P)1;
#pragma unroll
      for (int i = 0; i < CW; ++i) s[i] += WEIGHTED ? w * v[i] : v[i];
    }
  }
#pragma unroll
  for (int i = 0; i < CW; ++i) {
#pragma unroll
    for (int mask = LANES; mask < WAVE; mask <<= 1) s[i] += __shfl_xor(s[i], mask, WAVE);
    if (threadIdx.x % WAVE < LANES) part[threadIdx.x / WAVE][c * CW + i] = s[i];
  }
  __syncthreads();
  for (int mine = threadIdx.x; mine < LANES * CW; mine += LANES * SLICES) { /* a small workgroup has fewer threads than columns */
    const size_t at = (size_t)blockIdx.x * LANES * CW + mine;
    if (at < n) {
      P t = (P)0;
#pragma unroll
      for (int i = 0; i < WAVES; ++i) t += part[i][mine];
      dst[at] = (O)(blend != (P)0 ? scale * t + blend * (P)dst[at] : scale * t);
    }
  }
}

constexpr size_t SHORT_MATRIX_ROWS = 256; /* up to here the column sum takes four slices a workgroup */

/* Lanes (packs) of a row per workgroup: as many as a narrow matrix has, so that no lane idles
 * (measured on r32 [4M, 4]: 0.4 TB/s with 8 lanes); 32 lanes x one pack = 512 bytes of every
 * aligned row of a wider one: strips of one 128-byte line a row, the first choice, leave a
 * quarter of what the memory gives on the table (interleaved repeats, 8 -> 32 lanes: r32
 * [16384, 16384] 5.47 -> 6.43 TB/s, [65536, 4096] 5.76 -> 6.16, [262144, 1024] 5.60 -> 6.43; r16 5.32 -> 6.06,
 * 5.29 -> 5.93, 5.13 -> 6.10; 64 lanes: the same for r32, r16 [65536, 4096] 4.05); a wavefront per
 * kilobyte of a row for wide rows that are not aligned, because a misaligned 128-byte segment
 * would touch two lines for the data of one (measured on r32 [20000, 50257]: 3.4 TB/s with 8
 * lanes, one element per lane 4.3); two-byte types stay at 32 lanes there as well (64 -> 32: r16
 * [20000, 50257] 4.76 -> 4.92 TB/s, [65536, 4099] 4.25 -> 4.88; r32 loses 6-11 % by it). */
template <class T> inline size_t reduce_cols_lanes(size_t n, bool loose) {
  constexpr int W = PACK_BYTES / (int)sizeof(T);
  const size_t packs = (n + W - 1) / W;
  if (packs <= 1) return 1;
  if (packs <= 2) return 2;
  if (packs <= 4) return 4;
  if (packs <= 8) return 8;
  if (packs <= 16) return 16;
  if (packs <= 32) return 32;
  return loose && sizeof(T) >= 4 ? 64 : 32;
}

/* Row chunks of the two-stage column sum: enough workgroups to fill the GPU when the matrix is
 * tall and narrow (a [262144, 1024] r32 matrix has 32 column strips), never chunks under four
 * rows a slice (512 rows at 8 lanes); 1 when the strips alone are enough or the matrix is short. */
template <class T> inline size_t reduce_cols_chunks(size_t m, size_t n) {
  constexpr int W = PACK_BYTES / (int)sizeof(T);
  const size_t lanes = reduce_cols_lanes<T>(n, n % W != 0); /* as reduce_cols picks them (a shifted base aside) */
  const size_t strips = ((n + W - 1) / W + lanes - 1) / lanes;
  const size_t want = (size_t)compute_units() * 4;
  if (strips >= want) return 1;
  size_t chunks = (want + strips - 1) / strips;
  const size_t least = lanes >= 8 ? 512 : 4096 / lanes; /* rows */
  const size_t most = m / least;
  if (chunks > most) chunks = most;
  if (chunks > 1024) chunks = 1024;
  return chunks > 1 ? chunks : 1;
}

template <class T> inline size_t reduce_cols_scratch_bytes(size_t m, size_t n) {
  const size_t chunks = reduce_cols_chunks<T>(m, n);
  return chunks > 1 ? chunks * n * sizeof(typename precision<T>::type) : 0;
}

/* A stream context put together by hand has no workspace: say once what that costs, since nothing
 * in the launcher's signature does. */
inline void note_missing_workspace(size_t m, size_t n, size_t blocks) {
  static std::atomic<bool> told{false};
  if (!told.exchange(true))
    fprintf(stderr,
            "note: column sums of [%zu, %zu] run on %zu workgroups because they were given no workspace (a stream "
            "context from mpInitStream / mpAdoptStream carries one, launch_reduce_ij_j_scratch takes one); said once\n",
            m, n, blocks);
}

/* dst[j] = scale * sum_i (weight[i] *) src[i,j] + blend * dst[j].
 * scratch: reduce_cols_scratch_bytes(m, n) bytes or NULL (then one workgroup per column strip
 * walks every row, which leaves most of the GPU idle on tall, narrow matrices). */
template <class T>
inline void reduce_cols(const T* src, const T* weight, T* dst, void* scratch, double scale, double blend, size_t m,
                        size_t n, hipStream_t stream, size_t scratch_bytes = ~(size_t)0) {
  if (n == 0) return;
  using P = typename precision<T>::type;
  constexpr int W = PACK_BYTES / (int)sizeof(T);
  const bool loose = !(aligned16(src) && (n % W) == 0);
#define MP_COLS_SHAPE(O_, LANES_, SLICES_, LOOSE_, GRID_, OUT_, SCALE_, BLEND_, CHUNK_)                                         \
  do {                                                                                                                       \
    if (weight) reduce_cols_kernel<T, O_, W, LANES_, SLICES_, true, LOOSE_><<<GRID_, dim3(LANES_ * SLICES_), 0, stream>>>(src, weight, OUT_, SCALE_, BLEND_, m, n, CHUNK_); \
    else reduce_cols_kernel<T, O_, W, LANES_, SLICES_, false, LOOSE_><<<GRID_, dim3(LANES_ * SLICES_), 0, stream>>>(src, weight, OUT_, SCALE_, BLEND_, m, n, CHUNK_);       \
  } while (0)
#define MP_COLS_AS(O_, LANES_, LOOSE_, GRID_, OUT_, SCALE_, BLEND_, CHUNK_) \
  MP_COLS_SHAPE(O_, LANES_, 1024 / LANES_, LOOSE_, GRID_, OUT_, SCALE_, BLEND_, CHUNK_)
#define MP_COLS(O_, GRID_, OUT_, SCALE_, BLEND_, CHUNK_)                              \
  do {                                                                              \
    if (lanes == 1) MP_COLS_AS(O_, 1, true, GRID_, OUT_, SCALE_, BLEND_, CHUNK_);   \
    else if (lanes == 2) MP_COLS_AS(O_, 2, true, GRID_, OUT_, SCALE_, BLEND_, CHUNK_); \
    else if (lanes == 4) MP_COLS_AS(O_, 4, true, GRID_, OUT_, SCALE_, BLEND_, CHUNK_); \
    else if (lanes == 16) MP_COLS_AS(O_, 16, true, GRID_, OUT_, SCALE_, BLEND_, CHUNK_); \
    else if (lanes == 32) MP_COLS_AS(O_, 32, true, GRID_, OUT_, SCALE_, BLEND_, CHUNK_); \
    else if (lanes == 64) MP_COLS_AS(O_, 64, true, GRID_, OUT_, SCALE_, BLEND_, CHUNK_); \
    else if (loose) MP_COLS_AS(O_, 8, true, GRID_, OUT_, SCALE_, BLEND_, CHUNK_);   \
    else MP_COLS_AS(O_, 8, false, GRID_, OUT_, SCALE_, BLEND_, CHUNK_);             \
  } while (0)
  /* A few long rows (the sum of a handful of vectors): the 128 slices of an 8-lane workgroup
   * would find eight rows to share (measured on r32 [8, 16M]: 0.34 TB/s, [256, 512K]: 4.1); a
   * wavefront per kilobyte of the rows and four slices (fewer for one or two rows) keep every
   * thread busy. */
  if (m <= SHORT_MATRIX_ROWS && (n + W - 1) / W >= 64) {
    const size_t wide = ((n + W - 1) / W + 63) / 64;
    require(wide < 0x7fffffffull, "column sums: too many columns for one grid");
    if (m == 1) MP_COLS_SHAPE(T, 64, 1, true, dim3((unsigned)wide), dst, (P)scale, (P)blend, m);
    else if (m == 2) MP_COLS_SHAPE(T, 64, 2, true, dim3((unsigned)wide), dst, (P)scale, (P)blend, m);
    else MP_COLS_SHAPE(T, 64, 4, true, dim3((unsigned)wide), dst, (P)scale, (P)blend, m);
    MP_CHECK_LAUNCH();
    return;
  }
  size_t lanes = reduce_cols_lanes<T>(n, loose); /* other than 8 lanes the kernel is always the loose one */
  size_t blocks = ((n + W - 1) / W + lanes - 1) / lanes;
  require(blocks < 0x7fffffffull, "column sums: too many columns for one grid");
  size_t chunks = scratch != nullptr ? reduce_cols_chunks<T>(m, n) : 1;
  if (scratch == nullptr && blocks * 4 < (size_t)compute_units() && reduce_cols_chunks<T>(m, n) > 1)
    note_missing_workspace(m, n, blocks);
  const size_t fit = scratch_bytes / (n * sizeof(P)); /* partial rows the workspace holds */
  if (chunks > fit) chunks = fit;
  /* without a workspace the strips are all the workgroups there are: an aligned matrix too narrow
   * to give every CU one at 32 lanes goes back to strips of a line */
  const bool too_few = chunks <= 1 && blocks < (size_t)compute_units();
  /* and the weighted sum of r16 rows keeps them as well (a vector times an r16 matrix, 32 lanes against 8:
   * [16384, 16384] 5.32 -> 4.95 TB/s, [65536, 4096] 5.23 -> 4.76; r32 gains there like the plain sum) */
  const bool weighted_r16 = weight != nullptr && sizeof(T) == 2;
  if (!loose && lanes == 32 && (too_few || weighted_r16)) {
    lanes = 8;
    blocks = ((n + W - 1) / W + lanes - 1) / lanes;
  }
  if (chunks > 1) {
    const size_t chunk = (m + chunks - 1) / chunks;
    P* partials = static_cast<P*>(scratch);
    MP_COLS(P, dim3((unsigned)blocks, (unsigned)chunks), partials, (P)scale, (P)0, chunk);
    MP_CHECK_LAUNCH();
    sum_partial_rows<T>(partials, dst, blend, (unsigned)chunks, n, stream);
    return;
  }
  MP_COLS(T, dim3((unsigned)blocks), dst, (P)scale, (P)blend, m);
#undef MP_COLS_SHAPE
#undef MP_COLS_AS
#undef MP_COLS
  MP_CHECK_LAUNCH();
}

template <class T>
inline void reduce_cols(const T* src, T* dst, void* scratch, double alpha, size_t m, size_t n, hipStream_t stream) {
  reduce_cols<T>(src, nullptr, dst, scratch, 1.0, alpha, m, n, stream);
}

/* c[i,l] = scale * a[i] * b[l] + blend * c[i,l]: the product of a column and a row vector, written
 * like a broadcast: c as one flat array, one pack per thread. ALIGNED: n % W == 0 and b 16-byte
 * aligned, so a pack lies inside one row and its b values are one aligned pack; otherwise a pack
 * may run over the end of its row (over several rows when n < W): the b values are then a pack
 * that starts at any element, or, for a pack that wraps, single loads. DALIGNED: c is 16-byte
 * aligned. The last workgroup also writes the m*n % W elements behind the last whole pack. */
template <class T, int W, bool BLEND, bool ALIGNED, bool DALIGNED>
__global__ __launch_bounds__(256) void outer_flat_kernel(
    const T* a, const T* b, T* c, typename precision<T>::type scale, typename precision<T>::type blend,
    size_t total, unsigned n) {
  using P = typename precision<T>::type;
  const size_t packs = total / W;
  const size_t base = (size_t)blockIdx.x * 256 * W;
  const size_t row0 = base / n;
  const unsigned off = (unsigned)(base - row0 * n) + threadIdx.x * W;
  const size_t idx = (size_t)blockIdx.x * 256 + threadIdx.x;
  if (idx < packs) {
    const size_t row = row0 + off / n;
    const unsigned col = off % n;
    P out[W];
    if (ALIGNED || col + W <= n) {
      if constexpr (ALIGNED) load_pack<T, W>(b + col, out);
      else load_pack_loose<T, W>(b + col, out);
      const P left = scale * (P)a[row];
#pragma unroll
      for (int i = 0; i < W; ++i) out[i] *= left;
    } else { /* walk the pack's elements: the row advances whenever the column reaches n */
      size_t r = row;
      unsigned l = col;
#pragma unroll
      for (int i = 0; i < W; ++i) {
        out[i] = scale * (P)a[r] * (P)b[l];
        if (++l == n) {
          l = 0;
          ++r;
        }
      }
    }
    T* o = c + idx * W;
    if constexpr (BLEND) {
      P old[W];
      if constexpr (DALIGNED) load_pack_nt<T, W>(o, old);
      else load_pack_nt_loose<T, W>(o, old);
#pragma unroll
      for (int i = 0; i < W; ++i) out[i] += blend * old[i];
    }
    if constexpr (DALIGNED) store_pack_nt<T, W>(o, out);
    else store_pack_nt_loose<T, W>(o, out);
  }
  if (W > 1 && blockIdx.x == gridDim.x - 1) {
    const size_t e = packs * W + threadIdx.x;
    if (threadIdx.x < W && e < total) {
      P v = scale * (P)a[e / n] * (P)b[e % n];
      if constexpr (BLEND) v += blend * (P)c[e];
      c[e] = (T)v;
    }
  }
}

template <class T>
inline void outer_product(const T* a, const T* b, T* c, double scale, double blend, size_t m, size_t n, hipStream_t stream) {
  if (m == 0 || n == 0) return;
  using P = typename precision<T>::type;
  constexpr int W = PACK_BYTES / (int)sizeof(T);
  require(n <= 0x40000000ull, "outer product: row length must not exceed 2^30");
  const size_t total = m * n, blocks = (total / W + 255) / 256 + 1; /* + 1: the tail always has a workgroup */
  require(blocks < 0x7fffffffull, "outer product: too many elements for one grid");
  const dim3 grid((unsigned)blocks), block(256);
  const bool aligned = n % W == 0 && aligned16(b);
#define MP_OUTER_AS(BLEND_, ALIGNED_, DALIGNED_) \
  outer_flat_kernel<T, W, BLEND_, ALIGNED_, DALIGNED_><<<grid, block, 0, stream>>>(a, b, c, (P)scale, (P)blend, total, (unsigned)n)
#define MP_OUTER(BLEND_, ALIGNED_) \
  do { if (aligned16(c)) MP_OUTER_AS(BLEND_, ALIGNED_, true); else MP_OUTER_AS(BLEND_, ALIGNED_, false); } while (0)
  if (aligned) { if (blend != 0.0) MP_OUTER(true, true); else MP_OUTER(false, true); }
  else { if (blend != 0.0) MP_OUTER(true, false); else MP_OUTER(false, false); }
#undef MP_OUTER
#undef MP_OUTER_AS
  MP_CHECK_LAUNCH();
}

/* ------------------------------------------------------------------ broadcasts */

/* BY_ROW: dst[i,j] = src[i] + alpha*dst[i,j]; otherwise dst[i,j] = src[j] + alpha*dst[i,j]. */

/* The destination as one flat array of m*n elements: one pack per thread in one-shot 256-thread
 * workgroups, the shape that writes fastest on this GPU, whatever the row length (short rows keep
 * every lane busy). ALIGNED: n % W == 0 and 16-byte aligned column values, so a pack lies inside
 * one row and its values are one aligned pack load; otherwise a pack may run over the end of its
 * row (over several rows when n < W): the column values are then a pack that starts at any
 * element, or, for a pack that wraps, W single loads. DALIGNED: the destination base is 16-byte
 * aligned; a destination that is not costs about 5 % (packs that start at any element). The last
 * workgroup also writes the m*n % W elements behind the last whole pack. */
template <class T, int W, bool BY_ROW, bool BLEND, bool ALIGNED, bool DALIGNED>
__global__ __launch_bounds__(256) void broadcast_flat_kernel(
    const T* src, T* dst, typename precision<T>::type alpha, size_t total, unsigned n) {
  using P = typename precision<T>::type;
  const size_t packs = total / W;
  const size_t base = (size_t)blockIdx.x * 256 * W; /* first element of the workgroup: uniform, so the */
  const size_t row0 = base / n;                     /* one 64-bit division is scalar work */
  const unsigned off = (unsigned)(base - row0 * n) + threadIdx.x * W;
  const size_t idx = (size_t)blockIdx.x * 256 + threadIdx.x;
  if (idx < packs) {
    const size_t row = row0 + off / n;
    const unsigned col = off % n;
    P out[W];
    if constexpr (BY_ROW && ALIGNED) {
      const P here = (P)src[row];
#pragma unroll
      for (int i = 0; i < W; ++i) out[i] = here;
    } else if constexpr (ALIGNED) {
      load_pack<T, W>(src + col, out);
    } else if (!BY_ROW && col + W <= n) {
      load_pack_loose<T, W>(src + col, out);
    } else { /* walk the pack's elements: the row advances whenever the column reaches n */
      size_t r = row;
      unsigned c = col;
#pragma unroll
      for (int i = 0; i < W; ++i) {
        out[i] = BY_ROW ? (P)src[r] : (P)src[c];
        if (++c == n) {
          c = 0;
          ++r;
        }
      }
    }
    T* o = dst + idx * W;
    if constexpr (BLEND) {
      P old[W];
      if constexpr (DALIGNED) load_pack_nt<T, W>(o, old);
      else load_pack_nt_loose<T, W>(o, old);
#pragma unroll
      for (int i = 0; i < W; ++i) out[i] += alpha * old[i];
    }
    if constexpr (DALIGNED) store_pack_nt<T, W>(o, out);
    else store_pack_nt_loose<T, W>(o, out);
  }
  if (W > 1 && blockIdx.x == gridDim.x - 1) {
    const size_t e = packs * W + threadIdx.x;
    if (threadIdx.x < W && e < total) {
      P v = BY_ROW ? (P)src[e / n] : (P)src[e % n];
      if constexpr (BLEND) v += alpha * (P)dst[e];
      dst[e] = (T)v;
    }
  }
}

template <class T, bool BY_ROW>
inline void broadcast(const T* src, T* dst, double alpha, size_t m, size_t n, hipStream_t stream) {
  if (m == 0 || n == 0) return;
  using P = typename precision<T>::type;
  constexpr int W = PACK_BYTES / (int)sizeof(T);
  require(n <= 0x40000000ull, "broadcast: row length must not exceed 2^30");
  const size_t total = m * n, blocks = (total / W + 255) / 256 + 1; /* + 1: the tail always has a workgroup */
  require(blocks < 0x7fffffffull, "broadcast: too many elements for one grid");
  const dim3 grid((unsigned)blocks), block(256);
  const bool aligned = n % W == 0 && (BY_ROW || aligned16(src));
  const bool blend = alpha != 0.0;
#define MP_FLAT_AS(BLEND_, ALIGNED_, DALIGNED_) \
  broadcast_flat_kernel<T, W, BY_ROW, BLEND_, ALIGNED_, DALIGNED_><<<grid, block, 0, stream>>>(src, dst, (P)alpha, total, (unsigned)n)
#define MP_FLAT(BLEND_, ALIGNED_) \
  do { if (aligned16(dst)) MP_FLAT_AS(BLEND_, ALIGNED_, true); else MP_FLAT_AS(BLEND_, ALIGNED_, false); } while (0)
  if (aligned) { if (blend) MP_FLAT(true, true); else MP_FLAT(false, true); }
  else { if (blend) MP_FLAT(true, false); else MP_FLAT(false, false); }
#undef MP_FLAT
#undef MP_FLAT_AS
  MP_CHECK_LAUNCH();
}

}  // namespace mp

#endif
#endif
