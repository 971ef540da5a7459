/*
 * RMSNorm over the last dimension, forward and reverse.
 *
 * The reference has no RMSNorm kernel; its row-reduce (src/cuda/nvcc_src/reduce_ij_i.cu:3-54)
 * and column-reduce (src/cuda/nvcc_src/reduce_ij_j.cu:3-66) are the nearest patterns. Math:
 *   forward   r_i   = (mean_j x_ij^2 + eps)^(-1/2),   y_ij = x_ij * r_i * g_j
 *   reverse   c_i   = mean_j(dy_ij * g_j * x_ij)
 *             dx_ij = r_i * (dy_ij*g_j - x_ij * r_i^2 * c_i) + alpha * dx_ij
 *             dg_j  = sum_i dy_ij * x_ij * r_i               + alpha * dg_j
 * Accumulation is in precision<T>; the last stage of dg sums in fp64.
 *
 * Workgroups are persistent: 1024 threads hold 1024/G rows at a time and walk the rows with
 * the gain vector (and, in reverse, the per-column dg sums) resident in registers. The
 * reverse reads x and dy once, folds both row reductions into one barrier, writes dx, and at
 * the end combines the workgroup's dg sums through LDS into ONE partial row per workgroup;
 * a second small kernel adds the partial rows in a fixed order, so dg is deterministic.
 */
#ifndef MP_ROW_RMSNORM_H
#define MP_ROW_RMSNORM_H

#include "row_cluster.h"

#include <type_traits>

#if defined(__cplusplus) && defined(__HIPCC__)

namespace mp {

constexpr int NORM_BLOCK = 1024;

/* Both values folded over a G-thread group with a single barrier. */
template <int G, class P>
__device__ __forceinline__ void group_allreduce_sum2(P& a, P& b, P* slots_a, P* slots_b, int lane) {
  a = lanes_allreduce<AddOP, (G < WAVE ? G : WAVE)>(a);
  b = lanes_allreduce<AddOP, (G < WAVE ? G : WAVE)>(b);
  if constexpr (G > WAVE) {
    if ((lane & (WAVE - 1)) == 0) {
      slots_a[lane / WAVE] = a;
      slots_b[lane / WAVE] = b;
    }
    __syncthreads();
    constexpr int NW = G / WAVE;
    a = fold_partials<AddOP, NW>(slots_a[lane & (NW - 1)]);
    b = fold_partials<AddOP, NW>(slots_b[lane & (NW - 1)]);
  }
}

/* ------------------------------------------------------------------ resident forward */

/* KEEP: x through ordinary loads, which leave it in the memory-side cache for the reverse
 * (keep_input, row_cluster.h). */
/* LOOSE = false: x, gain and y 16-byte aligned and n % W == 0. LOOSE = true: any alignment of the
 * three and any n; the packs start at the row's first element (see RowPacks), so a thread's
 * columns, and with them its gain, are the same in every row (gain read element by element for
 * rows that each peel differently: r32 n = 257 3.3 TB/s). */
template <class T, int W, int G, int NV, bool LOOSE, int BLOCK = NORM_BLOCK, bool KEEP = false>
__global__ __launch_bounds__(BLOCK) void rmsnorm_fwd_resident(
    const T* x, const T* gain, T* y, typename precision<T>::type eps, size_t m, size_t n) {
  using P = typename precision<T>::type;
  const P inv_n = (P)1 / (P)n; /* one division a thread, not two a row */
  constexpr int RPB = BLOCK / G;
  static_assert(G >= W, "the first lanes of a group hold the elements behind the last whole pack");
  __shared__ P slots[2][G < WAVE ? 1 : RPB][G < WAVE ? 1 : G / WAVE];

  const int sub = threadIdx.x / G, lane = threadIdx.x % G;
  /* the whole packs of a row; the n % W elements behind them go one to a lane (a single lane
   * moving them with W predicated accesses costs every wavefront those instructions: r16 n = 100
   * 3.2 -> 4.4 TB/s, r32 n = 257 5.0 -> 5.5; the reverse kernel, shorter of registers, loses by
   * the same change and keeps the cut pack on one lane) */
  const size_t body = n / W * W;
  const RowPacks<T, W, LOOSE> rp(body);
  const bool edged = LOOSE && (size_t)lane < n - body;

  P gv[NV][W];
#pragma unroll
  for (int k = 0; k < NV; ++k) {
    const int p = k * G + lane;
#pragma unroll
    for (int i = 0; i < W; ++i) gv[k][i] = (P)0;
    if (p < rp.npk) rp.template load<false>(gain, p, gv[k]);
  }
  const P ge = edged ? (P)gain[body + lane] : (P)0;

  int parity = 0;
  for (size_t base = (size_t)blockIdx.x * RPB; base < m; base += (size_t)gridDim.x * RPB, parity ^= 1) {
    const size_t row = base + sub;
    const bool live = row < m; /* uniform per wave; dead groups still meet the barrier */
    const T* xr = x + (live ? row : 0) * n;
    P xv[NV][W];
#pragma unroll
    for (int k = 0; k < NV; ++k) {
      const int p = k * G + lane;
      if (live && p < rp.npk) {
        rp.template load<!KEEP>(xr, p, xv[k]);
      } else {
#pragma unroll
        for (int i = 0; i < W; ++i) xv[k][i] = (P)0;
      }
    }
    P xe = (P)0;
    if constexpr (LOOSE)
      if (edged && live) xe = (P)xr[body + lane];

    P ss = xe * xe;
#pragma unroll
    for (int k = 0; k < NV; ++k)
#pragma unroll
      for (int i = 0; i < W; ++i) ss += xv[k][i] * xv[k][i];
    ss = group_allreduce<AddOP, G>(ss, slots[parity][G < WAVE ? 0 : sub], lane);
    const P r = rsqrt_of(ss * inv_n + eps);

    if (live) {
      T* yr = y + row * n;
#pragma unroll
      for (int k = 0; k < NV; ++k) {
        const int p = k * G + lane;
        if (p < rp.npk) {
#pragma unroll
          for (int i = 0; i < W; ++i) xv[k][i] *= r * gv[k][i];
          rp.store(yr, p, xv[k]);
        }
      }
      if constexpr (LOOSE)
        if (edged) yr[body + lane] = (T)(xe * r * ge);
    }
    if constexpr (G <= WAVE && BLOCK > WAVE) { /* keep the waves of a persistent workgroup on neighbouring rows */
      if (rp.npk >= G) __syncthreads();
    }
  }
}

/* The resident forward for aligned rows of whole packs held by `gw` wavefronts a row, any number
 * from 2 to 16 (a kernel argument), and as many rows a workgroup as the launch gives it threads
 * for: rows that a power of two of wavefronts would leave partly idle. Sums of a group fold over
 * sixteen slots of which the ones past gw read as zero. The next rows are loaded while these are
 * reduced and written, as in the paired reverse (against loading after the write, interleaved
 * repeats: r16 n = 1152 5.26 -> 5.67 TB/s, r32 n = 1280 5.78 -> 5.94, six other widths -2 ... +1 %). */
constexpr int ANY_MAX_ROWS = 8; /* groups per workgroup the LDS of the wavefront-group kernels is sized for */

template <class T, int W, int NV, bool KEEP = false>
__global__ __launch_bounds__(NORM_BLOCK) void rmsnorm_fwd_any(
    const T* x, const T* gain, T* y, typename precision<T>::type eps, size_t m, size_t n, int gw) {
  using P = typename precision<T>::type;
  const P inv_n = (P)1 / (P)n; /* one division a thread, not two a row */
  using V = typename vec_of<T, W>::type;
  constexpr int NW = NORM_BLOCK / WAVE;
  __shared__ P slots[2][ANY_MAX_ROWS][NW];
  const int G = gw * WAVE, RPB = (int)blockDim.x / G;
  const int sub = threadIdx.x / G, lane = threadIdx.x % G;
  const int npk = (int)(n / W);
  const size_t last = m - 1, stride = (size_t)gridDim.x * RPB;

  V gv[NV]; /* in the storage type, widened where it is used */
#pragma unroll
  for (int k = 0; k < NV; ++k) {
    const int p = k * G + lane;
    gv[k] = *reinterpret_cast<const V*>(gain + (size_t)(p < npk ? p : 0) * W);
  }
  /* loads without conditions: a row beyond the last reads the last, a pack beyond the row its
   * first; both are dropped */
  auto fetch = [&](V (&xs)[NV], size_t base) {
    size_t row = base + sub;
    row = row < last ? row : last;
    const T* xr = x + row * n;
#pragma unroll
    for (int k = 0; k < NV; ++k) {
      const int p = k * G + lane;
      const V* at = reinterpret_cast<const V*>(xr + (size_t)(p < npk ? p : 0) * W);
      xs[k] = KEEP ? *at : __builtin_nontemporal_load(at);
    }
  };
  auto finish = [&](const V (&xs)[NV], size_t base, P (*sl)[NW]) {
    const size_t row = base + sub;
    P ss = (P)0;
#pragma unroll
    for (int k = 0; k < NV; ++k) {
      if (k * G + lane < npk) {
#pragma unroll
        for (int i = 0; i < W; ++i) ss += (P)xs[k][i] * (P)xs[k][i];
      }
    }
    ss = wave_allreduce<AddOP>(ss);
    if ((lane & (WAVE - 1)) == 0) sl[sub][lane / WAVE] = ss;
    lds_barrier();
    const int slot = lane & (NW - 1);
    ss = fold_partials<AddOP, NW>(slot < gw ? sl[sub][slot] : (P)0);
    const P r = rsqrt_of(ss * inv_n + eps);
    if (row < m) {
      T* yr = y + row * n;
#pragma unroll
      for (int k = 0; k < NV; ++k) {
        const int p = k * G + lane;
        if (p < npk) {
          P out[W];
#pragma unroll
          for (int i = 0; i < W; ++i) out[i] = (P)xs[k][i] * (r * (P)gv[k][i]);
          store_pack_nt<T, W>(yr + (size_t)p * W, out);
        }
      }
    }
  };

  /* the next rows are on their way while these are reduced and written: two register sets that take turns */
  V ax[NV], bx[NV];
  size_t base = (size_t)blockIdx.x * RPB;
  fetch(ax, base);
#pragma unroll
  for (int k = 0; k < NV; ++k) settle(gv[k]);
  for (; base < m; base += 2 * stride) {
    fetch(bx, base + stride);
    __builtin_amdgcn_sched_barrier(0);
    finish(ax, base, slots[0]);
    fetch(ax, base + 2 * stride);
    __builtin_amdgcn_sched_barrier(0);
    finish(bx, base + stride, slots[1]);
  }
}

/* ------------------------------------------------------------------ streaming forward */

/* The packs of a row start where x's alignment puts them; the gain's, and with APART (y not
 * aligned like x) y's, start at any element. */
template <class T, int W, bool APART = false>
__global__ __launch_bounds__(STREAM_THREADS) void rmsnorm_fwd_stream(
    const T* x, const T* gain, T* y, typename precision<T>::type eps, size_t m, size_t n) {
  using P = typename precision<T>::type;
  const P inv_n = (P)1 / (P)n; /* one division a thread, not two a row */
  constexpr int G = STREAM_THREADS, U = 4;
  __shared__ P slots[2][G / WAVE];
  const int lane = threadIdx.x;
  int parity = 0;

  for (size_t row = blockIdx.x; row < m; row += gridDim.x, parity ^= 1) {
    const T* xr = x + row * n;
    T* yr = y + row * n;
    const RowGeom<T, W> g(xr, n, true);
    const T* body = xr + g.head;
    T* ybody = yr + g.head;

    P ss = (P)0;
    for (int p0 = lane; p0 < g.nvec; p0 += G * U) {
      P buf[U][W];
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const int p = p0 + u * G;
        if (p < g.nvec) {
          load_pack<T, W>(body + (size_t)p * W, buf[u]);
        } else {
#pragma unroll
          for (int i = 0; i < W; ++i) buf[u][i] = (P)0;
        }
      }
#pragma unroll
      for (int u = 0; u < U; ++u)
#pragma unroll
        for (int i = 0; i < W; ++i) ss += buf[u][i] * buf[u][i];
    }
    size_t edge = (size_t)-1;
    if (W > 1) {
      if (lane < g.head) edge = (size_t)lane;
      else if (lane - g.head < g.tail) edge = (size_t)g.head + (size_t)g.nvec * W + (lane - g.head);
      if (edge != (size_t)-1) ss += (P)xr[edge] * (P)xr[edge];
    }
    ss = group_allreduce<AddOP, G>(ss, slots[parity], lane);
    const P r = rsqrt_of(ss * inv_n + eps);

    for (int p = lane; p < g.nvec; p += G) {
      P buf[W], gv[W];
      load_pack_nt<T, W>(body + (size_t)p * W, buf);
      load_pack_loose<T, W>(gain + (size_t)g.head + (size_t)p * W, gv);
#pragma unroll
      for (int i = 0; i < W; ++i) buf[i] *= r * gv[i];
      if constexpr (APART) store_pack_nt_loose<T, W>(ybody + (size_t)p * W, buf);
      else store_pack_nt<T, W>(ybody + (size_t)p * W, buf);
    }
    if (W > 1 && edge != (size_t)-1) yr[edge] = (T)((P)xr[edge] * r * (P)gain[edge]);
  }
}

/* ------------------------------------------------------------------ shared-row forward */

/* Rows too long for one workgroup's registers: C consecutive workgroups share a row. Each keeps
 * its chunk of x in registers in the storage type, publishes its part of sum x^2, waits (bounded)
 * for the others and writes its chunk of y: the row is read once. A workgroup that stops
 * waiting reads the whole row again for the sum, which is why the path is not taken in place. */
constexpr int NORM_CLUSTER_NV = 5; /* packs per thread: 20 registers, two workgroups a CU */

template <class T, int W>
__global__ __launch_bounds__(CLUSTER_THREADS, 8) void rmsnorm_fwd_cluster(
    const T* x, const T* gain, T* y, typename precision<T>::type eps,
    typename slot_word<typename precision<T>::type>::type* slots,
    size_t m, size_t n, int C, int packs_per_block, unsigned spin_limit) {
  using P = typename precision<T>::type;
  const P inv_n = (P)1 / (P)n; /* one division a thread, not two a row */
  using V = typename vec_of<T, W>::type;
  constexpr int G = CLUSTER_THREADS, NV = NORM_CLUSTER_NV;
  __shared__ P red[2][G / WAVE];
  __shared__ P bc[2];
  const int lane = threadIdx.x;
  const size_t row = blockIdx.x / (unsigned)C;
  const int rank = (int)(blockIdx.x % (unsigned)C);
  const T* xr = x + row * n;
  T* yr = y + row * n;
  const RowGeom<T, W> g(xr, n, true);
  const T* body = xr + g.head;
  const int lo = rank * packs_per_block - cluster_skew(body, C, packs_per_block, g.nvec);
  const int hi = lo + packs_per_block < g.nvec ? lo + packs_per_block : g.nvec;

  V v[NV];
#pragma unroll
  for (int k = 0; k < NV; ++k) {
    const int p = lo + k * G + lane;
    if (p >= 0 && p < hi) {
      v[k] = __builtin_nontemporal_load(reinterpret_cast<const V*>(body + (size_t)p * W));
    } else {
#pragma unroll
      for (int i = 0; i < W; ++i) v[k][i] = (T)0;
    }
  }
  P edge = (P)0; /* rank 0 also holds the row's head / tail scalars */
  size_t edge_at = (size_t)-1;
  if (W > 1 && rank == 0) {
    if (lane < g.head) edge_at = (size_t)lane;
    else if (lane - g.head < g.tail) edge_at = (size_t)g.head + (size_t)g.nvec * W + (lane - g.head);
    if (edge_at != (size_t)-1) edge = (P)xr[edge_at];
  }

  P ss = edge * edge;
#pragma unroll
  for (int k = 0; k < NV; ++k)
#pragma unroll
    for (int i = 0; i < W; ++i) ss += (P)v[k][i] * (P)v[k][i];
  ss = group_allreduce<AddOP, G>(ss, red[0], lane);
#pragma unroll
  for (int k = 0; k < NV; ++k) forget(v[k]);

  if (C > 1) {
    P sums[1] = {ss};
    const bool complete = cluster_exchange_sums<1>(slots + (size_t)row * C, C, rank, sums, spin_limit, bc, lane);
    ss = sums[0];
    if (!complete) { /* gave up waiting: the whole row's sum here */
      P t = (P)0;
      for (int p = lane; p < g.nvec; p += G) {
        P u[W];
        load_pack<T, W>(body + (size_t)p * W, u);
#pragma unroll
        for (int i = 0; i < W; ++i) t += u[i] * u[i];
      }
      if (W > 1) {
        size_t e = (size_t)-1;
        if (lane < g.head) e = (size_t)lane;
        else if (lane - g.head < g.tail) e = (size_t)g.head + (size_t)g.nvec * W + (lane - g.head);
        if (e != (size_t)-1) t += (P)xr[e] * (P)xr[e];
      }
      ss = group_allreduce<AddOP, G>(t, red[1], lane);
    }
  }

  const P r = rsqrt_of(ss * inv_n + eps);
  T* ybody = yr + g.head;
  const T* gbody = gain + g.head;
  const bool gain_packed = (reinterpret_cast<uintptr_t>(gbody) & 15u) == 0;
#pragma unroll
  for (int k = 0; k < NV; ++k) {
    const int p = lo + k * G + lane;
    if (p >= 0 && p < hi) {
      P gv[W], out[W];
      if (gain_packed) {
        load_pack<T, W>(gbody + (size_t)p * W, gv);
      } else {
#pragma unroll
        for (int i = 0; i < W; ++i) gv[i] = (P)gbody[(size_t)p * W + i];
      }
#pragma unroll
      for (int i = 0; i < W; ++i) out[i] = (P)v[k][i] * r * gv[i];
      store_pack_nt<T, W>(ybody + (size_t)p * W, out);
    }
  }
  if (edge_at != (size_t)-1) yr[edge_at] = (T)(edge * r * (P)gain[edge_at]);
}

/* Workgroups per row when the forward shares rows; 0 when it does not. */
template <class T> inline int rmsnorm_cluster_size(size_t packs) {
  const int regime = row_regime_override();
  if (regime != REGIME_AUTO && regime != REGIME_CLUSTER) return 0;
  constexpr size_t resident = (size_t)NORM_BLOCK * max_nv_for<T>(32); /* what one workgroup holds */
  /* from three quarters of that on, two one-shot workgroups a row beat the persistent one with
   * its widest register tile (interleaved repeats: r32 n = 32768 5.33 -> 5.57 TB/s, 24576 equal;
   * r16 n = 24576 5.28 -> 5.49, 32768 5.39 -> 5.54) */
  if (regime == REGIME_AUTO && packs < resident / 4 * 3) return 0;
  constexpr size_t tile = (size_t)CLUSTER_THREADS * NORM_CLUSTER_NV;
  size_t ppb = (size_t)cluster_tuning().packs_per_block;
  if (ppb == 0 || ppb > tile) ppb = tile;
  const size_t c = (packs + ppb - 1) / ppb;
  return c >= 1 && c <= (size_t)CLUSTER_MAX ? (int)c : 0;
}

template <class T> inline size_t rmsnorm_scratch_bytes(size_t m, size_t n) {
  constexpr int W = PACK_BYTES / (int)sizeof(T);
  const size_t c = cluster_size_for_scratch(rmsnorm_cluster_size<T>((n + W - 1) / W));
  return m * c * sizeof(typename precision<T>::type);
}

/* ------------------------------------------------------------------ resident reverse */

/* partials holds gridDim.x rows of n values of precision<T>. */
template <class T, int W, int G, int NV, bool BLEND, bool LOOSE>
__global__ __launch_bounds__(NORM_BLOCK) void rmsnorm_rev_resident(
    const T* x, const T* gain, const T* dy, T* dx, typename precision<T>::type* partials,
    typename precision<T>::type eps, typename precision<T>::type alpha, size_t m, size_t n, unsigned by_xcd) {
  using P = typename precision<T>::type;
  const P inv_n = (P)1 / (P)n; /* one division a thread, not two a row */
  constexpr int RPB = NORM_BLOCK / G;
  __shared__ P slots[2][2][G < WAVE ? 1 : RPB][G < WAVE ? 1 : G / WAVE];
  __shared__ P comb[RPB > 1 ? NORM_BLOCK * NV * W : 1]; /* one row of dg sums per group of the workgroup */
  const unsigned block = by_xcd ? xcd_contiguous_block(blockIdx.x, gridDim.x) : blockIdx.x;

  const int sub = threadIdx.x / G, lane = threadIdx.x % G;
  const RowPacks<T, W, LOOSE> rp(n);

  P gv[NV][W], acc[NV][W];
#pragma unroll
  for (int k = 0; k < NV; ++k) {
    const int p = k * G + lane;
#pragma unroll
    for (int i = 0; i < W; ++i) acc[k][i] = gv[k][i] = (P)0;
    if (p < rp.npk) rp.template load<false>(gain, p, gv[k]);
  }

  int parity = 0;
  for (size_t base = (size_t)block * RPB; base < m; base += (size_t)gridDim.x * RPB, parity ^= 1) {
    const size_t row = base + sub;
    const bool live = row < m;
    const size_t off = (live ? row : 0) * n;

    P xv[NV][W], dv[NV][W];
#pragma unroll
    for (int k = 0; k < NV; ++k) {
      const int p = k * G + lane;
      if (live && p < rp.npk) {
        rp.template load<true>(x + off, p, xv[k]);
        rp.template load<true>(dy + off, p, dv[k]);
      } else {
#pragma unroll
        for (int i = 0; i < W; ++i) xv[k][i] = dv[k][i] = (P)0;
      }
    }

    P ss = (P)0, c = (P)0;
#pragma unroll
    for (int k = 0; k < NV; ++k)
#pragma unroll
      for (int i = 0; i < W; ++i) {
        ss += xv[k][i] * xv[k][i];
        c += dv[k][i] * gv[k][i] * xv[k][i];
      }
    group_allreduce_sum2<G>(ss, c, slots[parity][0][G < WAVE ? 0 : sub], slots[parity][1][G < WAVE ? 0 : sub], lane);
    const P r = rsqrt_of(ss * inv_n + eps);
    const P cc = c * inv_n * r * r;

    if (live) {
#pragma unroll
      for (int k = 0; k < NV; ++k) {
        const int p = k * G + lane;
        if (p < rp.npk) {
          P out[W];
#pragma unroll
          for (int i = 0; i < W; ++i) {
            out[i] = r * (dv[k][i] * gv[k][i] - xv[k][i] * cc);
            acc[k][i] += dv[k][i] * xv[k][i] * r;
          }
          if constexpr (BLEND) {
            P old[W];
            rp.template load<false>(dx + off, p, old);
#pragma unroll
            for (int i = 0; i < W; ++i) out[i] += alpha * old[i];
          }
          rp.store(dx + off, p, out);
        }
      }
    }
    /* Groups of a wavefront or less never meet a barrier in this loop; left alone, the waves of a
     * workgroup drift apart and its contiguous 16 KiB bursts dissolve into scattered kilobytes
     * (measured: r32 n = 256 5.3 TB/s without, 5.9 with). Rows that leave lanes idle are the exception. */
    if constexpr (G <= WAVE) {
      if (rp.npk >= G) __syncthreads();
    }
  }

  /* one partial row per workgroup */
  P* mine = partials + (size_t)blockIdx.x * n;
  if constexpr (RPB > 1) {
    /* every group leaves its sums in LDS; then one thread per column adds the RPB groups in order */
    constexpr int ROW = G * NV * W;
#pragma unroll
    for (int k = 0; k < NV; ++k)
#pragma unroll
      for (int i = 0; i < W; ++i) comb[sub * ROW + (k * G + lane) * W + i] = acc[k][i];
    __syncthreads();
    for (size_t col = threadIdx.x; col < n; col += NORM_BLOCK) {
      P t = (P)0;
      for (int s = 0; s < RPB; ++s) t += comb[s * ROW + col];
      mine[col] = t;
    }
  } else {
#pragma unroll
    for (int k = 0; k < NV; ++k) {
      const int p = k * G + lane;
      if (p < rp.npk) {
#pragma unroll
        for (int i = 0; i < W; ++i)
          if (i < rp.valid(p)) mine[(size_t)p * W + i] = acc[k][i];
      }
    }
  }
}

/* ------------------------------------------------------------------ resident reverse, rows in pairs */

/* Two sums folded over a G-thread group (G > 64) behind the LDS-only barrier. */
template <int G, class P>
__device__ __forceinline__ void group_allreduce_sum2_lds(P& a, P& b, P* slots_a, P* slots_b, int lane) {
  static_assert(G > WAVE, "groups of more than one wavefront");
  a = wave_allreduce<AddOP>(a);
  b = wave_allreduce<AddOP>(b);
  if ((lane & (WAVE - 1)) == 0) {
    slots_a[lane / WAVE] = a;
    slots_b[lane / WAVE] = b;
  }
  lds_barrier();
  constexpr int NW = G / WAVE;
  a = fold_partials<AddOP, NW>(slots_a[lane & (NW - 1)]);
  b = fold_partials<AddOP, NW>(slots_b[lane & (NW - 1)]);
}

/* The resident reverse for aligned rows of whole packs held by groups of 128 ... 1024 threads,
 * with the loads of the next row in flight while the current one is reduced and written: two
 * register sets (in the storage type) that take turns, loads without conditions (a row index
 * beyond the last row reads the last row, a pack index beyond the row reads the row's first pack;
 * both are dropped), and reductions behind a barrier that does not wait for global loads. One
 * workgroup per CU then moves what two of the unpaired kernel move (r32 [8192, 4096]: 66.4 -> 63.9 us,
 * against 63.1 for a plain two-reads-one-write pass over the same bytes), and leaves half as
 * many partial rows. EXACT: every thread's NV packs lie inside the row (n == G * NV * W).
 * DEPTH 3: three register sets, two rows on their way while a third is reduced; the launcher says
 * where that pays. */
template <class T, int W, int G, int NV, bool BLEND, bool EXACT, int DEPTH = 2>
__global__ __launch_bounds__(NORM_BLOCK) void rmsnorm_rev_paired(
    const T* x, const T* gain, const T* dy, T* dx, typename precision<T>::type* partials,
    typename precision<T>::type eps, typename precision<T>::type alpha, size_t m, size_t n) {
  using P = typename precision<T>::type;
  const P inv_n = (P)1 / (P)n; /* one division a thread, not two a row */
  using V = typename vec_of<T, W>::type;
  static_assert(G > WAVE && G <= NORM_BLOCK, "groups of 128 ... 1024 threads");
  constexpr int RPB = NORM_BLOCK / G;
  static_assert(DEPTH == 2 || DEPTH == 3, "two or three register sets");
  __shared__ P slots[DEPTH][2][RPB][G / WAVE];
  __shared__ P comb[RPB > 1 ? NORM_BLOCK * NV * W : 1];

  const int sub = threadIdx.x / G, lane = threadIdx.x % G;
  const int npk = (int)(n / W);
  const size_t last = m - 1, stride = (size_t)gridDim.x * RPB;

  P gv[NV][W], acc[NV][W];
#pragma unroll
  for (int k = 0; k < NV; ++k) {
    const int p = k * G + lane;
#pragma unroll
    for (int i = 0; i < W; ++i) acc[k][i] = gv[k][i] = (P)0;
    if (p < npk) load_pack<T, W>(gain + (size_t)p * W, gv[k]);
  }

  auto fetch = [&](V (&xs)[NV], V (&ds)[NV], size_t base) {
    size_t row = base + sub;
    row = row < last ? row : last;
    const T* xr = x + row * n;
    const T* dr = dy + row * n;
#pragma unroll
    for (int k = 0; k < NV; ++k) {
      const int p = k * G + lane;
      const size_t at = (size_t)(EXACT || p < npk ? p : 0) * W;
      xs[k] = __builtin_nontemporal_load(reinterpret_cast<const V*>(xr + at));
      ds[k] = __builtin_nontemporal_load(reinterpret_cast<const V*>(dr + at));
    }
  };
  auto finish = [&](const V (&xs)[NV], const V (&ds)[NV], size_t base, P (*sl)[RPB][G / WAVE]) {
    const size_t row = base + sub;
    const bool live = row < m;
    P xv[NV][W], dv[NV][W];
    P ss = (P)0, c = (P)0;
#pragma unroll
    for (int k = 0; k < NV; ++k) {
      const bool inside = EXACT || k * G + lane < npk;
#pragma unroll
      for (int i = 0; i < W; ++i) {
        xv[k][i] = inside ? (P)xs[k][i] : (P)0;
        dv[k][i] = inside ? (P)ds[k][i] : (P)0;
        ss += xv[k][i] * xv[k][i];
        c += dv[k][i] * gv[k][i] * xv[k][i];
      }
    }
    group_allreduce_sum2_lds<G>(ss, c, sl[0][sub], sl[1][sub], lane);
    const P r = rsqrt_of(ss * inv_n + eps);
    const P cc = c * inv_n * r * r;
    if (live) {
      T* out_row = dx + row * n;
#pragma unroll
      for (int k = 0; k < NV; ++k) {
        const int p = k * G + lane;
        if (EXACT || p < npk) {
          P out[W];
#pragma unroll
          for (int i = 0; i < W; ++i) {
            out[i] = r * (dv[k][i] * gv[k][i] - xv[k][i] * cc);
            acc[k][i] += dv[k][i] * xv[k][i] * r;
          }
          if constexpr (BLEND) {
            P old[W];
            load_pack<T, W>(out_row + (size_t)p * W, old);
#pragma unroll
            for (int i = 0; i < W; ++i) out[i] += alpha * old[i];
          }
          store_pack_nt<T, W>(out_row + (size_t)p * W, out);
        }
      }
    }
  };

  V ax[NV], ad[NV], bx[NV], bd[NV];
  size_t base = (size_t)blockIdx.x * RPB;
  fetch(ax, ad, base);
  if constexpr (DEPTH == 3) fetch(bx, bd, base + stride);
#pragma unroll
  for (int k = 0; k < NV; ++k)
#pragma unroll
    for (int i = 0; i < W; ++i) settle(gv[k][i]); /* the gain is waited for here, not inside the loop */
  if constexpr (DEPTH == 3) { /* two rows on their way while a third is reduced and written */
    V cx[NV], cd[NV];
    for (; base < m; base += 3 * stride) {
      fetch(cx, cd, base + 2 * stride);
      __builtin_amdgcn_sched_barrier(0);
      finish(ax, ad, base, slots[0]);
      fetch(ax, ad, base + 3 * stride);
      __builtin_amdgcn_sched_barrier(0);
      finish(bx, bd, base + stride, slots[1]);
      fetch(bx, bd, base + 4 * stride);
      __builtin_amdgcn_sched_barrier(0);
      finish(cx, cd, base + 2 * stride, slots[DEPTH - 1]);
    }
  } else {
    for (; base < m; base += 2 * stride) {
      fetch(bx, bd, base + stride);
      __builtin_amdgcn_sched_barrier(0);
      finish(ax, ad, base, slots[0]);
      fetch(ax, ad, base + 2 * stride);
      __builtin_amdgcn_sched_barrier(0);
      finish(bx, bd, base + stride, slots[1]);
    }
  }

  /* one partial row per workgroup */
  P* mine = partials + (size_t)blockIdx.x * n;
  if constexpr (RPB > 1) {
    constexpr int ROW = G * NV * W;
#pragma unroll
    for (int k = 0; k < NV; ++k)
#pragma unroll
      for (int i = 0; i < W; ++i) comb[sub * ROW + (k * G + lane) * W + i] = acc[k][i];
    __syncthreads();
    for (size_t col = threadIdx.x; col < n; col += NORM_BLOCK) {
      P t = (P)0;
      for (int s = 0; s < RPB; ++s) t += comb[s * ROW + col];
      mine[col] = t;
    }
  } else {
#pragma unroll
    for (int k = 0; k < NV; ++k) {
      const int p = k * G + lane;
      if (EXACT || p < npk) {
#pragma unroll
        for (int i = 0; i < W; ++i) mine[(size_t)p * W + i] = acc[k][i];
      }
    }
  }
}

/* The paired reverse for rows that a power of two of wavefronts would leave partly idle: a row is
 * held by `gw` wavefronts (any number from 1 to 16, chosen by the launcher as the fewest that cover
 * the row at NV packs a thread) and a workgroup is as many such groups as fit 1024 threads, so
 * every lane but the last wavefront's tail holds data (n = 5120 r16: 640 packs on ten wavefronts,
 * not on sixteen). The group's width is a kernel argument, not a template parameter: one kernel
 * per (type, packs a thread, blend) serves every width. Sums of a group fold over sixteen slots of
 * which the ones past gw read as zero. */

template <class T, int W, int NV, bool BLEND, int DEPTH = 2>
__global__ __launch_bounds__(NORM_BLOCK) void rmsnorm_rev_paired_any(
    const T* x, const T* gain, const T* dy, T* dx, typename precision<T>::type* partials,
    typename precision<T>::type eps, typename precision<T>::type alpha, size_t m, size_t n, int gw) {
  using P = typename precision<T>::type;
  const P inv_n = (P)1 / (P)n; /* one division a thread, not two a row */
  using V = typename vec_of<T, W>::type;
  constexpr int NW = NORM_BLOCK / WAVE;
  __shared__ P slots[DEPTH][2][ANY_MAX_ROWS][NW];
  constexpr int COMB = NORM_BLOCK * (NV * W < 8 ? NV * W : 8); /* one row of dg sums: the launcher keeps G * NV * W within it */
  __shared__ P comb[COMB];

  const int G = gw * WAVE, RPB = (int)blockDim.x / G;
  const int sub = threadIdx.x / G, lane = threadIdx.x % G;
  const int npk = (int)(n / W);
  const size_t last = m - 1, stride = (size_t)gridDim.x * RPB;

  /* the gain stays in the storage type like x and dy and is widened where it is used: for two-byte
   * types that is what lets two packs a thread fit beside the two register sets */
  V gv[NV];
  P acc[NV][W];
#pragma unroll
  for (int k = 0; k < NV; ++k) {
    const int p = k * G + lane;
#pragma unroll
    for (int i = 0; i < W; ++i) acc[k][i] = (P)0;
    gv[k] = *reinterpret_cast<const V*>(gain + (size_t)(p < npk ? p : 0) * W);
  }

  auto fetch = [&](V (&xs)[NV], V (&ds)[NV], size_t base) {
    size_t row = base + sub;
    row = row < last ? row : last;
    const T* xr = x + row * n;
    const T* dr = dy + row * n;
#pragma unroll
    for (int k = 0; k < NV; ++k) {
      const int p = k * G + lane;
      const size_t at = (size_t)(p < npk ? p : 0) * W;
      xs[k] = __builtin_nontemporal_load(reinterpret_cast<const V*>(xr + at));
      ds[k] = __builtin_nontemporal_load(reinterpret_cast<const V*>(dr + at));
    }
  };
  auto finish = [&](const V (&xs)[NV], const V (&ds)[NV], size_t base, P (*sl)[ANY_MAX_ROWS][NW]) {
    const size_t row = base + sub;
    const bool live = row < m;
    P ss = (P)0, c = (P)0;
#pragma unroll
    for (int k = 0; k < NV; ++k) {
      if (k * G + lane < npk) { /* a pack beyond the row was loaded from its start and is dropped */
#pragma unroll
        for (int i = 0; i < W; ++i) {
          const P xv = (P)xs[k][i];
          ss += xv * xv;
          c += (P)ds[k][i] * (P)gv[k][i] * xv;
        }
      }
    }
    ss = wave_allreduce<AddOP>(ss);
    c = wave_allreduce<AddOP>(c);
    if ((lane & (WAVE - 1)) == 0) {
      sl[0][sub][lane / WAVE] = ss;
      sl[1][sub][lane / WAVE] = c;
    }
    lds_barrier();
    const int slot = lane & (NW - 1);
    ss = fold_partials<AddOP, NW>(slot < gw ? sl[0][sub][slot] : (P)0);
    c = fold_partials<AddOP, NW>(slot < gw ? sl[1][sub][slot] : (P)0);
    const P r = rsqrt_of(ss * inv_n + eps);
    const P cc = c * inv_n * r * r;
    if (live) {
      T* out_row = dx + row * n;
#pragma unroll
      for (int k = 0; k < NV; ++k) {
        const int p = k * G + lane;
        if (p < npk) {
          P out[W];
#pragma unroll
          for (int i = 0; i < W; ++i) {
            const P xv = (P)xs[k][i], dv = (P)ds[k][i];
            out[i] = r * (dv * (P)gv[k][i] - xv * cc);
            acc[k][i] += dv * xv * r;
          }
          if constexpr (BLEND) {
            P old[W];
            load_pack<T, W>(out_row + (size_t)p * W, old);
#pragma unroll
            for (int i = 0; i < W; ++i) out[i] += alpha * old[i];
          }
          store_pack_nt<T, W>(out_row + (size_t)p * W, out);
        }
      }
    }
  };

  V ax[NV], ad[NV], bx[NV], bd[NV];
  size_t base = (size_t)blockIdx.x * RPB;
  fetch(ax, ad, base);
  if constexpr (DEPTH == 3) fetch(bx, bd, base + stride);
#pragma unroll
  for (int k = 0; k < NV; ++k) settle(gv[k]); /* the gain is waited for here, not inside the loop */
  if constexpr (DEPTH == 3) {
    V cx[NV], cd[NV];
    for (; base < m; base += 3 * stride) {
      fetch(cx, cd, base + 2 * stride);
      __builtin_amdgcn_sched_barrier(0);
      finish(ax, ad, base, slots[0]);
      fetch(ax, ad, base + 3 * stride);
      __builtin_amdgcn_sched_barrier(0);
      finish(bx, bd, base + stride, slots[1]);
      fetch(bx, bd, base + 4 * stride);
      __builtin_amdgcn_sched_barrier(0);
      finish(cx, cd, base + 2 * stride, slots[DEPTH - 1]);
    }
  } else {
    for (; base < m; base += 2 * stride) {
      fetch(bx, bd, base + stride);
      __builtin_amdgcn_sched_barrier(0);
      finish(ax, ad, base, slots[0]);
      fetch(ax, ad, base + 2 * stride);
      __builtin_amdgcn_sched_barrier(0);
      finish(bx, bd, base + stride, slots[1]);
    }
  }

  /* one partial row per workgroup: the groups add their sums into one row in LDS, one after the other */
  for (int turn = 0; turn < RPB; ++turn) {
    if (sub == turn) {
#pragma unroll
      for (int k = 0; k < NV; ++k)
#pragma unroll
        for (int i = 0; i < W; ++i) {
          P& cell = comb[(k * G + lane) * W + i];
          cell = turn == 0 ? acc[k][i] : cell + acc[k][i];
        }
    }
    __syncthreads();
  }
  P* mine = partials + (size_t)blockIdx.x * n;
  for (size_t col = threadIdx.x; col < n; col += blockDim.x) mine[col] = comb[col];
}

/* ------------------------------------------------------------------ streaming reverse */

/* Rows too long to keep x and dy in registers: they are read twice (the second read mostly from
 * cache). NA > 0: a thread still keeps the dg sums of its NA packs of columns in registers and the
 * workgroup writes one partial row at the end. NA == 0 (rows beyond 1024 * NA packs): each
 * workgroup adds every row it processes into its partial row in memory (first row: overwrite). */
template <class T> constexpr int stream_acc_packs() {
  using P = typename precision<T>::type;
  return 64 / ((PACK_BYTES / (int)sizeof(T)) * (int)(sizeof(P) / 4)); /* 64 registers of sums */
}

template <class T, int W, int NA, bool BLEND, bool LOOSE>
__global__ __launch_bounds__(STREAM_THREADS) void rmsnorm_rev_stream(
    const T* x, const T* gain, const T* dy, T* dx, typename precision<T>::type* partials,
    typename precision<T>::type eps, typename precision<T>::type alpha, size_t m, size_t n) {
  using P = typename precision<T>::type;
  const P inv_n = (P)1 / (P)n; /* one division a thread, not two a row */
  constexpr int G = STREAM_THREADS, U = 2;
  __shared__ P slots[2][2][G / WAVE];
  const int lane = threadIdx.x;
  const RowPacks<T, W, LOOSE> rp(n);
  P* mine = partials + (size_t)blockIdx.x * n;
  int parity = 0;
  bool first = true;
  P acc[NA > 0 ? NA : 1][W];
#pragma unroll
  for (int k = 0; k < (NA > 0 ? NA : 1); ++k)
#pragma unroll
    for (int i = 0; i < W; ++i) acc[k][i] = (P)0;

  for (size_t row = blockIdx.x; row < m; row += gridDim.x, parity ^= 1, first = false) {
    const size_t off = row * n;
    P ss = (P)0, c = (P)0;
    for (int p0 = lane; p0 < rp.npk; p0 += G * U) {
      P xv[U][W], dv[U][W], gv[U][W];
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const int p = p0 + u * G;
        if (p < rp.npk) {
          rp.template load<false>(x + off, p, xv[u]);
          rp.template load<false>(dy + off, p, dv[u]);
          rp.template load<false>(gain, p, gv[u]);
        } else {
#pragma unroll
          for (int i = 0; i < W; ++i) xv[u][i] = dv[u][i] = gv[u][i] = (P)0;
        }
      }
#pragma unroll
      for (int u = 0; u < U; ++u)
#pragma unroll
        for (int i = 0; i < W; ++i) {
          ss += xv[u][i] * xv[u][i];
          c += dv[u][i] * gv[u][i] * xv[u][i];
        }
    }
    group_allreduce_sum2<G>(ss, c, slots[parity][0], slots[parity][1], lane);
    const P r = rsqrt_of(ss * inv_n + eps);
    const P cc = c * inv_n * r * r;

    auto finish_pack = [&](int p, P (&sum)[W], bool in_registers) {
      P xv[W], dv[W], gv[W], out[W];
      rp.template load<true>(x + off, p, xv);
      rp.template load<true>(dy + off, p, dv);
      rp.template load<false>(gain, p, gv);
#pragma unroll
      for (int i = 0; i < W; ++i) {
        out[i] = r * (dv[i] * gv[i] - xv[i] * cc);
        const P t = dv[i] * xv[i] * r;
        if (in_registers) {
          sum[i] += t;
        } else if (i < rp.valid(p)) {
          P* slot = mine + (size_t)p * W + i;
          *slot = first ? t : *slot + t;
        }
      }
      if constexpr (BLEND) {
        P old[W];
        rp.template load<false>(dx + off, p, old);
#pragma unroll
        for (int i = 0; i < W; ++i) out[i] += alpha * old[i];
      }
      rp.store(dx + off, p, out);
    };
    if constexpr (NA > 0) {
#pragma unroll
      for (int k = 0; k < NA; ++k) {
        const int p = k * G + lane;
        if (p < rp.npk) finish_pack(p, acc[k], true);
      }
    } else {
      for (int p = lane; p < rp.npk; p += G) finish_pack(p, acc[0], false);
    }
  }

  if constexpr (NA > 0) {
#pragma unroll
    for (int k = 0; k < NA; ++k) {
      const int p = k * G + lane;
      if (p < rp.npk) {
#pragma unroll
        for (int i = 0; i < W; ++i)
          if (i < rp.valid(p)) mine[(size_t)p * W + i] = acc[k][i];
      }
    }
  }
}

/* ------------------------------------------------------------------ shared-row reverse */

/* Rows too long for one workgroup's registers: the grid is S slices of C
 * consecutive workgroups. The C workgroups of a slice share every row of the slice
 * (rows slice, slice + S, ...): each keeps the dg sums of its chunk in registers for the whole
 * kernel and, per row, its chunk of x, dy and (from L2) the gain; the two row sums (x^2 and dy*g*x) are
 * exchanged through scratch once per row, so x and dy are read once. All S * C workgroups fit the
 * GPU at once (one or two per CU, see norm_rev_cluster_per_cu), which keeps the per-row waits short; a workgroup that stops waiting
 * reads the whole row for the sums, so the kernel ends under any scheduling. Not taken when dx
 * overwrites x or dy. One partial row of dg per slice. */
/* Two packs of x, dy and (per row) gain per thread, in the storage type, and the dg sums beside
 * them. Four-byte and wider types then fit 64 registers with a small spill, which lets two
 * workgroups share a CU; measured on r32 against four packs and one workgroup per CU:
 * n = 32768 4.5 -> 5.5 TB/s, 65536 4.2 -> 5.4, 131072 4.6 -> 5.0. The dg sums of r16 are four
 * times as wide as its packs: it spills heavily at 64 registers (3.1 TB/s) and keeps one
 * workgroup per CU and 128 registers (4.5). */
template <class T> constexpr int norm_rev_cluster_nv() { return 2; }
template <class T> constexpr int norm_rev_cluster_per_cu() { return sizeof(T) == 2 ? 1 : 2; }

template <class T, int W, bool BLEND, bool LOOSE>
__global__ __launch_bounds__(CLUSTER_THREADS, 4 * norm_rev_cluster_per_cu<T>()) void rmsnorm_rev_cluster(
    const T* x, const T* gain, const T* dy, T* dx, typename precision<T>::type* partials,
    typename precision<T>::type eps, typename precision<T>::type alpha,
    typename slot_word<typename precision<T>::type>::type* slots,
    size_t m, size_t n, int C, int packs_per_block, unsigned spin_limit) {
  using P = typename precision<T>::type;
  const P inv_n = (P)1 / (P)n; /* one division a thread, not two a row */
  using V = typename vec_of<T, W>::type;
  constexpr int G = CLUSTER_THREADS, NV = norm_rev_cluster_nv<T>();
  __shared__ P red[2][2][G / WAVE];
  __shared__ P bc[3];
  const int lane = threadIdx.x;
  const int rank = (int)(blockIdx.x % (unsigned)C);
  const size_t slice = blockIdx.x / (unsigned)C, S = gridDim.x / (unsigned)C;
  const RowPacks<T, W, LOOSE> rp(n);
  const int lo = rank * packs_per_block;
  const int hi = lo + packs_per_block < rp.npk ? lo + packs_per_block : rp.npk;

  P acc[NV][W];
#pragma unroll
  for (int k = 0; k < NV; ++k)
#pragma unroll
    for (int i = 0; i < W; ++i) acc[k][i] = (P)0;

  /* A partner that is not running yet (the GPU shared with other work) is waited for once: after
   * the first wait that runs out, this workgroup stops waiting for the rest of the kernel (it
   * still publishes its sums first, so its partners are never held up by it). */
  unsigned patience = spin_limit;
  int parity = 0;
  /* r16 runs one workgroup per CU, so nothing else on the CU fills the wait for the partners:
   * the chunk of the next row is asked for before that wait (two-byte packs leave the registers) */
  constexpr bool AHEAD = sizeof(T) == 2;
  auto fetch = [&](size_t row, V (&xs)[NV], V (&ds)[NV]) {
    const size_t off = row * n;
#pragma unroll
    for (int k = 0; k < NV; ++k) {
      const int p = lo + k * G + lane;
      xs[k] = p < hi ? rp.template raw<true>(x + off, p) : V{};
    }
#pragma unroll
    for (int k = 0; k < NV; ++k) {
      const int p = lo + k * G + lane;
      ds[k] = p < hi ? rp.template raw<true>(dy + off, p) : V{};
    }
  };
  V xv[NV], dv[NV], xn[AHEAD ? NV : 1], dn[AHEAD ? NV : 1];
  if constexpr (AHEAD) {
    if (slice < m) fetch(slice, xv, dv);
  }
  for (size_t row = slice; row < m; row += S, parity ^= 1) {
    const size_t off = row * n;
    V gv[NV]; /* the gain chunk comes from L2 every row: registers go to the dg sums */
    if constexpr (!AHEAD) fetch(row, xv, dv);
#pragma unroll
    for (int k = 0; k < NV; ++k) {
      const int p = lo + k * G + lane;
      gv[k] = p < hi ? rp.template raw<false>(gain, p) : V{};
    }
    P ss = (P)0, c = (P)0;
#pragma unroll
    for (int k = 0; k < NV; ++k)
#pragma unroll
      for (int i = 0; i < W; ++i) {
        const P xf = (P)xv[k][i];
        ss += xf * xf;
        c += (P)dv[k][i] * (P)gv[k][i] * xf;
      }
    group_allreduce_sum2<G>(ss, c, red[parity][0], red[parity][1], lane);
    /* the chunk stays in the storage type: widened copies must not live across the exchange,
     * nor a widened gain across the loop */
#pragma unroll
    for (int k = 0; k < NV; ++k) {
      forget(xv[k]);
      forget(dv[k]);
      forget(gv[k]);
    }

    /* Asked for before the exchange, the next row's loads are what the polling wavefront waits for
     * first (a wavefront's loads return in order), and the workgroup with it; asked for after it,
     * they overlap less. Measured (interleaved repeats, r16): behind the exchange n = 20480 4.00 ->
     * 4.38 TB/s, 24576 4.42 -> 4.64, 32768 4.80 -> 5.13 (two workgroups a row); four a row -5 ... +6 %
     * from box to box, eight -8 %. */
    const bool fetch_late = C <= 2;
    if constexpr (AHEAD) {
      if (!fetch_late && row + S < m) fetch(row + S, xn, dn);
    }
    if (C > 1) {
      P sums[2] = {ss, c};
      const bool complete = cluster_exchange_sums<2>(slots + row * (size_t)C * 2, C, rank, sums, patience, bc, lane);
      ss = sums[0];
      c = sums[1];
      if (!complete) { /* gave up waiting: both sums over the whole row here, and no waiting for later rows */
        patience = 0;
        P s2 = (P)0, c2 = (P)0;
        for (int p = lane; p < rp.npk; p += G) {
          P u[W], d[W], g[W];
          rp.template load<false>(x + off, p, u);
          rp.template load<false>(dy + off, p, d);
          rp.template load<false>(gain, p, g);
#pragma unroll
          for (int i = 0; i < W; ++i) {
            s2 += u[i] * u[i];
            c2 += d[i] * g[i] * u[i];
          }
        }
        /* the barrier inside the exchange lies between the last read of red[parity] and this reuse */
        group_allreduce_sum2<G>(s2, c2, red[parity][0], red[parity][1], lane);
        ss = s2;
        c = c2;
      }
    }
    if constexpr (AHEAD) {
      if (fetch_late && row + S < m) fetch(row + S, xn, dn);
    }
    const P r = rsqrt_of(ss * inv_n + eps);
    const P cc = c * inv_n * r * r;

#pragma unroll
    for (int k = 0; k < NV; ++k) {
      const int p = lo + k * G + lane;
      if (p < hi) {
        P out[W];
#pragma unroll
        for (int i = 0; i < W; ++i) {
          const P xf = (P)xv[k][i], df = (P)dv[k][i];
          out[i] = r * (df * (P)gv[k][i] - xf * cc);
          acc[k][i] += df * xf * r;
        }
        if constexpr (BLEND) {
          P old[W];
          rp.template load<false>(dx + off, p, old);
#pragma unroll
          for (int i = 0; i < W; ++i) out[i] += alpha * old[i];
        }
        rp.store(dx + off, p, out);
      }
    }
    if constexpr (AHEAD) {
#pragma unroll
      for (int k = 0; k < NV; ++k) {
        xv[k] = xn[k];
        dv[k] = dn[k];
      }
    }
  }

  P* mine = partials + slice * n;
#pragma unroll
  for (int k = 0; k < NV; ++k) {
    const int p = lo + k * G + lane;
    if (p < hi) {
#pragma unroll
      for (int i = 0; i < W; ++i)
        if (i < rp.valid(p)) mine[(size_t)p * W + i] = acc[k][i];
    }
  }
}

/* The same as a pipeline over the rows of a slice. What the kernel above cannot hide is the exchange
 * itself: a row's sums are published and then waited for, and until the partners' words arrive
 * (another CU, often another XCD) the workgroup has nothing to do. Here the sums of row j + 2 are
 * published and the words of row j + 1 read while row j is written back, so the partners' words of
 * a row have had a whole iteration to arrive when they are asked for, and nobody waits while they
 * are fetched; the chunk of row j + 3 is on its way meanwhile. Four register sets take turns
 * (being written back, waiting for its totals, just reduced, loading).
 * A wavefront's loads return in order, so a wavefront that polled behind loads of its own would
 * wait for them first: the last wavefront of the workgroup holds no data and is the only one that
 * publishes and polls, the other fifteen hold the chunk (960 lanes, two packs each), the gain
 * chunk stays in registers and every barrier orders LDS only. One workgroup per CU. */
constexpr int DEEP_LANES = CLUSTER_THREADS - WAVE; /* lanes of a workgroup that hold data */
/* Which rows take it. Four-byte types only: the four register sets of r16 leave no room for its
 * dg sums, which are four times as wide as its packs (kept in LDS instead, the kernel spills
 * regardless and loses 12-21 % to the kernel above; as 512 threads at four packs a lane in 255
 * registers it spills nothing and runs at the rate of the kernel above, -5 ... +4 %), and r64
 * spills. From 8193 packs a row on
 * (interleaved repeats, r32: n = 50257 4.27 -> 5.10 TB/s, 65536 5.27 -> 5.44, 100352 4.74 -> 5.46,
 * 131072 4.92 -> 5.40, 151936 4.44 -> 5.27, 262144 3.99 -> 5.26; below: n = 20480 equal, 24576 5.36 ->
 * 4.77, 32768 5.53 -> 5.40). The test build can force either kernel. */
template <class T> inline bool norm_rev_deep(size_t packs) {
  if (sizeof(T) != 4) return false;
#ifdef MP_DIAGNOSTICS
  if (cluster_tuning().deep != 0) return cluster_tuning().deep == 1;
#endif
  return packs > 8192;
}
/* packs of a row that one workgroup of the shared-row reverse holds */
template <class T> inline size_t norm_rev_cluster_tile(size_t packs) {
  return norm_rev_deep<T>(packs) ? (size_t)DEEP_LANES * 2 : (size_t)CLUSTER_THREADS * norm_rev_cluster_nv<T>();
}

template <class T, int W, bool BLEND>
__global__ __launch_bounds__(CLUSTER_THREADS) void rmsnorm_rev_cluster_deep(
    const T* x, const T* gain, const T* dy, T* dx, typename precision<T>::type* partials,
    typename precision<T>::type eps, typename precision<T>::type alpha,
    typename slot_word<typename precision<T>::type>::type* slots,
    size_t m, size_t n, int C, int packs_per_block, unsigned spin_limit) {
  using P = typename precision<T>::type;
  const P inv_n = (P)1 / (P)n; /* one division a thread, not two a row */
  using V = typename vec_of<T, W>::type;
  using Word = typename slot_word<P>::type;
  constexpr int G = CLUSTER_THREADS, D = DEEP_LANES, NV = 2, NW = G / WAVE;
  /* the packs start at the row's first element whatever the alignment: the one variant serves
   * aligned rows as well (built for aligned rows only it needs 17 registers more and spills) */
  constexpr bool LOOSE = true;
  __shared__ P red[2][2][NW]; /* [row parity][sum][wavefront]; the sixteenth wavefront's slot stays zero */
  __shared__ P fb[2][NW];     /* the sums of a workgroup that folds a whole row itself */
  __shared__ P bc[2][3];      /* [row parity]: the row totals and whether a partner was missing */
  const int lane = threadIdx.x;
  const bool messenger = lane >= D;
  const int ml = lane - D;
  const int rank = (int)(blockIdx.x % (unsigned)C);
  const size_t slice = blockIdx.x / (unsigned)C, S = gridDim.x / (unsigned)C;
  const RowPacks<T, W, LOOSE> rp(n);
  const int lo = rank * packs_per_block;
  const int hi = messenger ? 0 : (lo + packs_per_block < rp.npk ? lo + packs_per_block : rp.npk);

  P acc[NV][W];
  V gv[NV];
#pragma unroll
  for (int k = 0; k < NV; ++k) {
#pragma unroll
    for (int i = 0; i < W; ++i) acc[k][i] = (P)0;
    const int p = lo + k * D + lane;
    gv[k] = p < hi ? rp.template raw<false>(gain, p) : V{};
  }
  if (lane < NW) red[0][0][lane] = red[0][1][lane] = red[1][0][lane] = red[1][1][lane] = (P)0;

  auto fetch = [&](size_t row, V (&xs)[NV], V (&ds)[NV]) {
    const size_t off = row * n;
#pragma unroll
    for (int k = 0; k < NV; ++k) {
      const int p = lo + k * D + lane;
      xs[k] = p < hi ? rp.template raw<true>(x + off, p) : V{};
    }
#pragma unroll
    for (int k = 0; k < NV; ++k) {
      const int p = lo + k * D + lane;
      ds[k] = p < hi ? rp.template raw<true>(dy + off, p) : V{};
    }
  };
  /* this workgroup's sums of a row into red[parity]; no barrier */
  auto sums = [&](V (&xv)[NV], V (&dv)[NV], int parity) {
    P ss = (P)0, c = (P)0;
#pragma unroll
    for (int k = 0; k < NV; ++k)
#pragma unroll
      for (int i = 0; i < W; ++i) {
        const P xf = (P)xv[k][i];
        ss += xf * xf;
        c += (P)dv[k][i] * (P)gv[k][i] * xf;
      }
    ss = wave_allreduce<AddOP>(ss);
    c = wave_allreduce<AddOP>(c);
    if (!messenger && (lane & (WAVE - 1)) == 0) {
      red[parity][0][lane / WAVE] = ss;
      red[parity][1][lane / WAVE] = c;
    }
#pragma unroll
    for (int k = 0; k < NV; ++k) { /* no widened copy lives on */
      forget(xv[k]);
      forget(dv[k]);
    }
  };
  unsigned patience = spin_limit; /* after the first wait that runs out, no later row is waited for */
  /* the messenger, between the two barriers of an iteration: the sums in red[parity] go out as row
   * `ahead`'s (when there is one), the words of row `now` come in */
  auto exchange = [&](bool has_ahead, size_t ahead, int parity, bool has_now, size_t now, int now_parity) {
    if (!messenger) return;
    if (has_ahead) {
      P mine[2] = {fold_partials<AddOP, NW>(red[parity][0][ml & (NW - 1)]), fold_partials<AddOP, NW>(red[parity][1][ml & (NW - 1)])};
      if (ml == 0) {
        Word* words = slots + ahead * (size_t)C * 2;
#pragma unroll
        for (int v = 0; v < 2; ++v) {
          const P part = mine[v] == (P)0 ? -(P)0 : mine[v];
          __hip_atomic_store(words + (size_t)rank * 2 + v, __builtin_bit_cast(Word, part), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
      }
    }
    if (has_now) {
      Word* words = slots + now * (size_t)C * 2;
      Word w[2] = {0, 0};
      bool heard = true;
      if (ml < C) {
        for (unsigned spins = 0;; ++spins) {
          heard = true;
#pragma unroll
          for (int v = 0; v < 2; ++v) {
            w[v] = __hip_atomic_load(words + (size_t)ml * 2 + v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            heard = heard && w[v] != 0;
          }
          if (heard || spins >= patience) break;
          __builtin_amdgcn_s_sleep(4);
        }
      }
      const P missing = wave_allreduce<AddOP>(heard ? (P)0 : (P)1);
      P total[2];
#pragma unroll
      for (int v = 0; v < 2; ++v) total[v] = wave_allreduce<AddOP>(ml < C && heard ? __builtin_bit_cast(P, w[v]) : (P)0);
      if (ml == 0) {
        bc[now_parity][0] = total[0];
        bc[now_parity][1] = total[1];
        bc[now_parity][2] = missing;
      }
    }
  };
  /* row totals from bc, then this chunk of dx and of the dg sums */
  auto finish = [&](size_t row, int parity, V (&xv)[NV], V (&dv)[NV]) {
    const size_t off = row * n;
    P ss = bc[parity][0], c = bc[parity][1];
    if (bc[parity][2] != (P)0) { /* a partner was not heard from: both sums over the whole row here */
      patience = 0;
      P s2 = (P)0, c2 = (P)0;
      for (int p = lane; p < rp.npk; p += G) {
        P u[W], d[W], g[W];
        rp.template load<false>(x + off, p, u);
        rp.template load<false>(dy + off, p, d);
        rp.template load<false>(gain, p, g);
#pragma unroll
        for (int i = 0; i < W; ++i) {
          s2 += u[i] * u[i];
          c2 += d[i] * g[i] * u[i];
        }
      }
      s2 = wave_allreduce<AddOP>(s2);
      c2 = wave_allreduce<AddOP>(c2);
      if ((lane & (WAVE - 1)) == 0) {
        fb[0][lane / WAVE] = s2;
        fb[1][lane / WAVE] = c2;
      }
      __syncthreads();
      ss = fold_partials<AddOP, NW>(fb[0][lane & (NW - 1)]);
      c = fold_partials<AddOP, NW>(fb[1][lane & (NW - 1)]);
      __syncthreads(); /* fb is free again */
    }
    const P r = rsqrt_of(ss * inv_n + eps);
    const P cc = c * inv_n * r * r;
#pragma unroll
    for (int k = 0; k < NV; ++k) {
      const int p = lo + k * D + lane;
      if (p < hi) {
        P out[W];
#pragma unroll
        for (int i = 0; i < W; ++i) {
          const P xf = (P)xv[k][i], df = (P)dv[k][i];
          out[i] = r * (df * (P)gv[k][i] - xf * cc);
          acc[k][i] += df * xf * r;
        }
        if constexpr (BLEND) {
          P old[W];
          rp.template load<false>(dx + off, p, old);
#pragma unroll
          for (int i = 0; i < W; ++i) out[i] += alpha * old[i];
        }
        rp.store(dx + off, p, out);
      }
    }
  };
  /* one iteration, between two barriers: row `row` (parity `parity`) is written back from `fx, fd`
   * with the totals that came in one iteration ago, while the messenger sends the sums of row + 2
   * (reduced from `sx, sd` just before) and reads the words of row + 1; row + 3 is asked for into
   * `lx, ld`. The set of row + 1 is not touched. */
  auto iteration = [&](size_t row, int parity, V (&fx)[NV], V (&fd)[NV], V (&sx)[NV], V (&sd)[NV], V (&lx)[NV], V (&ld)[NV]) {
    const bool has_one = row + S < m, has_two = row + 2 * S < m;
    if (row + 3 * S < m) fetch(row + 3 * S, lx, ld);
    __builtin_amdgcn_sched_barrier(0);
    if (has_two) sums(sx, sd, parity);
    lds_barrier();
    exchange(has_two, row + 2 * S, parity, has_one, row + S, parity ^ 1);
    finish(row, parity, fx, fd);
    lds_barrier();
  };

  V ax[NV], ad[NV], bx[NV], bd[NV], cx[NV], cd[NV], ex[NV], ed[NV];
  if (slice < m) fetch(slice, ax, ad);
  if (slice + S < m) fetch(slice + S, bx, bd);
  if (slice + 2 * S < m) fetch(slice + 2 * S, cx, cd);
#pragma unroll
  for (int k = 0; k < NV; ++k) settle(gv[k]);
  __syncthreads(); /* the zeroed slots */
  if (slice < m) { /* the sums of the first two rows go out, the totals of the first come in, before the loop */
    sums(ax, ad, 0);
    lds_barrier();
    exchange(true, slice, 0, false, 0, 0);
    lds_barrier();
    const bool has_one = slice + S < m;
    if (has_one) sums(bx, bd, 1);
    lds_barrier();
    exchange(has_one, slice + S, 1, true, slice, 0);
    lds_barrier();
  }
  for (size_t row = slice; row < m; row += 4 * S) { /* four rows a turn: their parities are 0, 1, 0, 1 */
    iteration(row, 0, ax, ad, cx, cd, ex, ed);
    if (row + S >= m) break;
    iteration(row + S, 1, bx, bd, ex, ed, ax, ad);
    if (row + 2 * S >= m) break;
    iteration(row + 2 * S, 0, cx, cd, ax, ad, bx, bd);
    if (row + 3 * S >= m) break;
    iteration(row + 3 * S, 1, ex, ed, bx, bd, cx, cd);
  }

  P* mine = partials + slice * n;
#pragma unroll
  for (int k = 0; k < NV; ++k) {
    const int p = lo + k * D + lane;
    if (p < hi) {
#pragma unroll
      for (int i = 0; i < W; ++i)
        if (i < rp.valid(p)) mine[(size_t)p * W + i] = acc[k][i];
    }
  }
}

/* Workgroups per row when the reverse shares rows; 0 when it does not. */
template <class T> inline int rmsnorm_rev_cluster_size(size_t n) {
  constexpr int W = PACK_BYTES / (int)sizeof(T);
  const size_t packs = (n + W - 1) / W;
  const int regime = row_regime_override();
  if (regime != REGIME_AUTO && regime != REGIME_CLUSTER) return 0;
  constexpr size_t resident = (size_t)NORM_BLOCK * max_nv_for<T>(16); /* what the resident reverse holds */
  if (regime == REGIME_AUTO && packs <= resident) return 0;
  const size_t tile = norm_rev_cluster_tile<T>(packs);
  size_t ppb = (size_t)cluster_tuning().packs_per_block;
  if (ppb == 0 || ppb > tile) ppb = tile;
  const size_t c = (packs + ppb - 1) / ppb;
  return c >= 1 && c <= (size_t)CLUSTER_MAX ? (int)c : 0;
}

/* dg_j = sum over partial rows (fixed order, fp64) + alpha * dg_j. A workgroup owns LANES * CW
 * columns (CW = 4 and a whole 128-byte line when the partial rows are 16-byte aligned, else single
 * columns); its FINISH_SLICES slices split the partial rows, and a thread keeps up to eight
 * CW-wide loads in flight. With whole lines a workgroup is 512 threads and 4096 columns make 128
 * workgroups (r32 [512, 4096] partial rows: 3.6 -> 2.9 us against 64 workgroups of 1024). */
constexpr int FINISH_SLICES = 64;
template <int CW> constexpr int finish_lanes() { return CW == 4 ? 8 : 16; }
template <class T, int CW>
__global__ __launch_bounds__(finish_lanes<CW>() * FINISH_SLICES) void rmsnorm_dgain_finish(
    const typename precision<T>::type* partials, T* dg, double alpha, int rows, size_t n) {
  using P = typename precision<T>::type;
  constexpr int LANES = finish_lanes<CW>();
  __shared__ double part[FINISH_SLICES][LANES * CW + 1];
  const int c = threadIdx.x % LANES, slice = threadIdx.x / LANES;
  const size_t col = ((size_t)blockIdx.x * LANES + c) * CW;
  double s[CW];
#pragma unroll
  for (int i = 0; i < CW; ++i) s[i] = 0.0;
  if (col < n) { /* n is a multiple of CW, so a thread's CW columns are all in range */
    int p = slice;
    auto take = [&]<int U>() {
      P v[U][CW];
#pragma unroll
      for (int u = 0; u < U; ++u) load_pack<P, CW>(partials + (size_t)(p + u * FINISH_SLICES) * n + col, v[u]);
#pragma unroll
      for (int u = 0; u < U; ++u)
#pragma unroll
        for (int i = 0; i < CW; ++i) s[i] += (double)v[u][i];
      p += U * FINISH_SLICES;
    };
    while (p + 7 * FINISH_SLICES < rows) take.template operator()<8>();
    if (p + 3 * FINISH_SLICES < rows) take.template operator()<4>();
    if (p + FINISH_SLICES < rows) take.template operator()<2>();
    if (p < rows) take.template operator()<1>();
  }
#pragma unroll
  for (int i = 0; i < CW; ++i) part[slice][c * CW + i] = s[i];
  __syncthreads();
  /* the first LANES * CW threads finish one column each */
  const int mine = threadIdx.x;
  const size_t out = (size_t)blockIdx.x * LANES * CW + mine;
  if (mine < LANES * CW && out < n) {
    double t = 0.0;
#pragma unroll 8
    for (int i = 0; i < FINISH_SLICES; ++i) t += part[i][mine];
    if (alpha != 0.0) t += alpha * (double)dg[out];
    dg[out] = (T)t;
  }
}

/* dst_j = sum of `rows` partial rows of n accumulators (fixed order, fp64) + alpha * dst_j. */
template <class T>
inline void sum_partial_rows(const typename precision<T>::type* partials, T* dst, double alpha, unsigned rows,
                             size_t n, hipStream_t stream) {
  using P = typename precision<T>::type;
  if (plan_dry_run()) return;
  /* wide loads need 16-byte aligned partial rows: fp32 accumulators, n % 4 == 0, aligned scratch */
  const bool wide = sizeof(P) == 4 && (n % 4) == 0 && aligned16(partials);
  if (wide) {
    constexpr int COLS = finish_lanes<4>() * 4;
    rmsnorm_dgain_finish<T, 4><<<dim3((unsigned)((n + COLS - 1) / COLS)), dim3(finish_lanes<4>() * FINISH_SLICES), 0, stream>>>(
        partials, dst, alpha, (int)rows, n);
  } else {
    constexpr int COLS = finish_lanes<1>();
    rmsnorm_dgain_finish<T, 1><<<dim3((unsigned)((n + COLS - 1) / COLS)), dim3(finish_lanes<1>() * FINISH_SLICES), 0, stream>>>(
        partials, dst, alpha, (int)rows, n);
  }
  MP_CHECK_LAUNCH();
}

/* ------------------------------------------------------------------ short rows */

/* Rows of up to sixteen packs (a norm over a head's few dozen values): a pack a lane, 1 ... 16
 * lanes a row (ShortRow), one-shot workgroups of 256 threads. */
template <class T, int W, int G, bool CUT>
__global__ __launch_bounds__(SHORT_THREADS) void rmsnorm_fwd_short(
    const T* x, const T* gain, T* y, typename precision<T>::type eps, size_t m, unsigned n, unsigned by_xcd) {
  using P = typename precision<T>::type;
  const P inv_n = (P)1 / (P)n; /* one division a thread, not two a row */
  const int lane = threadIdx.x % G;
  bool live;
  const size_t row = short_row_of<G>(m, by_xcd, live);
  ShortRow<T, W, G, CUT> t, g;
  t.load(x + row * n, n, lane, (P)0);
  g.template load<false>(gain, n, lane, (P)0);
  P ss = (P)0;
#pragma unroll
  for (int i = 0; i < W; ++i) ss += t.v[i] * t.v[i];
  ss = fold_partials<AddOP, G>(ss);
  const P r = rsqrt_of(ss * inv_n + eps);
#pragma unroll
  for (int i = 0; i < W; ++i) t.v[i] *= r * g.v[i];
  if (live) t.store(y + row * n, n, lane);
}

/* The reverse walks the rows with gridDim.x workgroups of NORM_BLOCK threads, because every
 * workgroup leaves one partial row of dg sums (partials holds gridDim.x rows of n values): the
 * groups of a wavefront are folded with lane exchanges, the wavefronts through LDS in order. */
template <class T, int W, int G, bool CUT, bool BLEND>
__global__ __launch_bounds__(NORM_BLOCK) void rmsnorm_rev_short(
    const T* x, const T* gain, const T* dy, T* dx, typename precision<T>::type* partials,
    typename precision<T>::type eps, typename precision<T>::type alpha, size_t m, unsigned n) {
  using P = typename precision<T>::type;
  const P inv_n = (P)1 / (P)n; /* one division a thread, not two a row */
  constexpr int RPB = NORM_BLOCK / G, WAVES = NORM_BLOCK / WAVE;
  __shared__ P comb[WAVES][G * W];
  const int lane = threadIdx.x % G, sub = threadIdx.x / G;
  ShortRow<T, W, G, CUT> gv;
  gv.template load<false>(gain, n, lane, (P)0);
  P acc[W];
#pragma unroll
  for (int i = 0; i < W; ++i) acc[i] = (P)0;

  for (size_t base = (size_t)blockIdx.x * RPB; base < m; base += (size_t)gridDim.x * RPB) {
    const size_t want = base + sub;
    const bool live = want < m; /* a dead group of a live wavefront reads the last row and keeps nothing */
    const size_t off = (live ? want : m - 1) * n;
    ShortRow<T, W, G, CUT> xv, dv;
    xv.load(x + off, n, lane, (P)0);
    dv.load(dy + off, n, lane, (P)0);
    P ss = (P)0, c = (P)0;
#pragma unroll
    for (int i = 0; i < W; ++i) {
      ss += xv.v[i] * xv.v[i];
      c += dv.v[i] * gv.v[i] * xv.v[i];
    }
    ss = fold_partials<AddOP, G>(ss);
    c = fold_partials<AddOP, G>(c);
    const P r = rsqrt_of(ss * inv_n + eps);
    const P cc = c * inv_n * r * r;
    if (live) {
      ShortRow<T, W, G, CUT> out;
#pragma unroll
      for (int i = 0; i < W; ++i) {
        out.v[i] = r * (dv.v[i] * gv.v[i] - xv.v[i] * cc);
        acc[i] += dv.v[i] * xv.v[i] * r;
      }
      if constexpr (BLEND) {
        ShortRow<T, W, G, CUT> old;
        old.template load<false>(dx + off, n, lane, (P)0);
#pragma unroll
        for (int i = 0; i < W; ++i) out.v[i] += alpha * old.v[i];
      }
      out.store(dx + off, n, lane);
    }
  }

#pragma unroll
  for (int i = 0; i < W; ++i) {
#pragma unroll
    for (int mask = G; mask < WAVE; mask <<= 1) acc[i] += __shfl_xor(acc[i], mask, WAVE);
    if (threadIdx.x % WAVE < G) comb[threadIdx.x / WAVE][lane * W + i] = acc[i];
  }
  __syncthreads();
  P* mine = partials + (size_t)blockIdx.x * n;
  for (unsigned col = threadIdx.x; col < n; col += NORM_BLOCK) {
    P t = (P)0;
#pragma unroll
    for (int w = 0; w < WAVES; ++w) t += comb[w][col];
    mine[col] = t;
  }
}

/* Whether the short-row kernels take rows of n elements. Up to four packs always (r32 [8M, 4]:
 * 1.5/1.9 -> 5.7/5.2 TB/s forward/reverse, r16 [4M, 8]: 1.3/1.0 -> 4.3/4.3). From five to sixteen
 * packs the groups of 8 and 16 lanes of the resident kernels are the same layout when the row
 * fills them, and the measurements decide: r32 rows of whole packs gain forward (n = 64: 5.3 ->
 * 5.6) and, below eight packs, in reverse (n = 24: 4.75 -> 4.87; n = 32 and 64 lose 6 %); r16 rows
 * of whole packs gain in reverse (n = 64: 3.7 -> 4.5, n = 128: 4.4 -> 4.5) and lose 6 % forward; rows
 * with a cut pack gain only forward in r16 up to eight packs (n = 33: 1.2 -> 1.7). */
template <class T> inline bool rmsnorm_short_rows(size_t n, bool reverse) {
  constexpr int W = PACK_BYTES / (int)sizeof(T);
  const size_t packs = (n + W - 1) / W;
  const bool whole = n % W == 0;
  if (row_regime_override() != REGIME_AUTO || packs > (size_t)SHORT_MAX_PACKS) return false;
  if (packs <= 4) return true;
  if (sizeof(T) == 2) return reverse ? whole : !whole && packs <= 8;
  return whole && (!reverse || packs < 8);
}

/* ------------------------------------------------------------------ host dispatch */

/* Partial rows the reverse may write: one per workgroup, at most two workgroups per CU. */
inline size_t rmsnorm_reverse_partial_rows(size_t m) {
  const size_t cap = (size_t)compute_units() * 2;
  return m < cap ? (m ? m : 1) : cap;
}

template <class T>
inline size_t rmsnorm_reverse_scratch_bytes(size_t m, size_t n) {
  /* the partial rows of dg, then (shared rows only) two words per row and workgroup of the row */
  const size_t c = cluster_size_for_scratch(rmsnorm_rev_cluster_size<T>(n));
  return (rmsnorm_reverse_partial_rows(m) * n + m * c * 2) * sizeof(typename precision<T>::type);
}

template <class T>
inline void rmsnorm_forward(const T* x, const T* gain, T* y, void* scratch, double eps, size_t m, size_t n,
                            hipStream_t stream) {
  if (m == 0 || n == 0) return;
  using P = typename precision<T>::type;
  constexpr int W = PACK_BYTES / (int)sizeof(T);
  require(n <= 0x40000000ull, "rmsnorm: row length must not exceed 2^30");
  const size_t cap = (size_t)compute_units() * 2;
  if (rmsnorm_short_rows<T>(n, false)) {
    for_short_row(n, W, [&]<int G, bool CUT>() {
      if (note_plan(PLAN_SHORT, G, 1, SHORT_THREADS / G, short_row_grid(m, G), SHORT_THREADS)) return;
      rmsnorm_fwd_short<T, W, G, CUT><<<dim3(short_row_grid(m, G)), dim3(SHORT_THREADS), 0, stream>>>(
          x, gain, y, (P)eps, m, (unsigned)n, short_rows_share_lines<T>(n, G));
    });
    MP_CHECK_LAUNCH();
    return;
  }
  /* rows of x and y that peel differently: the kernels that hold a row in registers take them (their
   * packs start at the row's first element), the others go element by element */
  const bool mismatch = misalign16(x) != misalign16(y);
  const bool loose = !(aligned16(x) && aligned16(y) && aligned16(gain) && (n % W) == 0);
  constexpr int MAXNV = max_nv_for<T>(32);
  if (!mismatch) {
    const int C = rmsnorm_cluster_size<T>((n + W - 1) / W);
    const bool shareable = scratch != nullptr && !ranges_overlap(x, y, m * n * sizeof(T));
    if (C >= 1 && (C == 1 || shareable) && m * (size_t)C < 0x7fffffffull) {
      using Word = typename slot_word<P>::type;
      Word* slots = static_cast<Word*>(scratch);
      const int ppb = cluster_chunk_packs((n + W - 1) / W, C, (size_t)CLUSTER_THREADS * NORM_CLUSTER_NV, CLUSTER_SKEW_MAX);
      require(ppb <= CLUSTER_THREADS * NORM_CLUSTER_NV, "rmsnorm: cluster chunk exceeds the register tile");
      if (note_plan(PLAN_CLUSTER, CLUSTER_THREADS, NORM_CLUSTER_NV, 1, m * C, CLUSTER_THREADS, C, ppb,
                    C > 1 ? m * (size_t)C * sizeof(Word) : 0))
        return;
      if (C > 1) {
        const size_t words = m * (size_t)C;
        cluster_zero_slots<Word><<<dim3((unsigned)((words + 255) / 256)), dim3(256), 0, stream>>>(slots, words);
      }
      rmsnorm_fwd_cluster<T, W><<<dim3((unsigned)(m * C)), dim3(CLUSTER_THREADS), 0, stream>>>(
          x, gain, y, (P)eps, slots, m, n, C, ppb, cluster_tuning().spin_limit);
      MP_CHECK_LAUNCH();
      return;
    }
  }
  const size_t packs = (n + W - 1) / W;
  /* Short rows: one-shot 256-thread workgroups (each loads the gain it needs, which stays in L2)
   * beat persistent 1024-thread ones: r32 n = 256: 5.5 -> 6.3 TB/s, n = 1024: 6.0 -> 6.4; r16 wants
   * two packs per thread for the same effect (n = 1024: 5.6 -> 6.1) and
   * nothing beats the persistent kernel below 32 packs a row. Measured on the MI355X. */
  constexpr int ONESHOT = 256;
  /* aligned rows of whole packs: x through loads that leave it in the memory-side cache for the reverse */
  const bool keep = keep_input(m * n * sizeof(T));
  /* rows whose packs start at any element: two packs a thread, so that a row one pack over a power
   * of two does not idle half of a group twice as wide (r32 n = 257: 4.1 -> 5.1 TB/s, n = 130: 3.8 -> 4.9) */
  const int nv_target = sizeof(T) == 2 || loose ? 2 : 1;
  const RowPlan shot = plan_row(packs, MAXNV, nv_target, 8);
  /* aligned rows that leave the planned group more than an eighth idle and need at most five
   * wavefronts at the planned packs a thread: persistent workgroups of three to eight such rows
   * (interleaved repeats: r16 n = 1152 4.44 -> 5.31 TB/s, 1280 4.99 -> 5.74, 2560 5.20 -> 5.86; r32
   * n = 576 5.20 -> 6.14, 640 5.57 -> 6.22, 1280 5.84 -> 6.19; one-shot workgroups of the same groups: -4 ... +7 %;
   * six wavefronts a row: -2 ... +2 %, left with the power-of-two groups) */
  /* r16 rows of 129 ... 223 packs (128 x 2 planned): persistent workgroups of eight such rows that load
   * after they have written beat both the wavefront-group kernel and one-shot workgroups there
   * (interleaved repeats: n = 1152 4.78 -> 5.34 TB/s, 1280 5.06 -> 5.54, 1408 5.21 -> 5.68, 1536 5.42 -> 5.71) */
  const bool eight_rows = !loose && !mismatch && sizeof(T) == 2 && row_regime_override() == REGIME_AUTO &&
                          shot.G == 128 && shot.NV == 2 && packs > 128 && packs * 8 < (size_t)shot.G * shot.NV * 7;
  if (eight_rows) {
    const size_t need = (m + NORM_BLOCK / 128 - 1) / (NORM_BLOCK / 128);
    const dim3 grid((unsigned)(need < cap ? need : cap)), block(NORM_BLOCK);
    if (note_plan(PLAN_RESIDENT, 128, 2, NORM_BLOCK / 128, grid.x, block.x, 1, 0, 0, keep)) return;
    if (keep) rmsnorm_fwd_resident<T, W, 128, 2, false, NORM_BLOCK, true><<<grid, block, 0, stream>>>(x, gain, y, (P)eps, m, n);
    else rmsnorm_fwd_resident<T, W, 128, 2, false><<<grid, block, 0, stream>>>(x, gain, y, (P)eps, m, n);
    MP_CHECK_LAUNCH();
    return;
  }
  if (!loose && !mismatch && row_regime_override() == REGIME_AUTO && shot.G >= 128 && shot.G <= 512 && shot.NV <= 2 &&
      packs * 8 < (size_t)shot.G * shot.NV * 7) {
    const int gw = (int)((packs + (size_t)WAVE * shot.NV - 1) / ((size_t)WAVE * shot.NV));
    if (gw >= 2 && gw <= 5) {
      const int rpb = NORM_BLOCK / WAVE / gw;
      const size_t need = (m + rpb - 1) / rpb;
      const dim3 grid((unsigned)(need < cap ? need : cap)), block(rpb * gw * WAVE);
      if (note_plan(PLAN_ANY, gw * WAVE, shot.NV, rpb, grid.x, block.x, 1, 0, 0, keep)) return;
      if (shot.NV == 1) {
        if (keep) rmsnorm_fwd_any<T, W, 1, true><<<grid, block, 0, stream>>>(x, gain, y, (P)eps, m, n, gw);
        else rmsnorm_fwd_any<T, W, 1><<<grid, block, 0, stream>>>(x, gain, y, (P)eps, m, n, gw);
      } else {
        if (keep) rmsnorm_fwd_any<T, W, 2, true><<<grid, block, 0, stream>>>(x, gain, y, (P)eps, m, n, gw);
        else rmsnorm_fwd_any<T, W, 2><<<grid, block, 0, stream>>>(x, gain, y, (P)eps, m, n, gw);
      }
      MP_CHECK_LAUNCH();
      return;
    }
  }
  const bool take_shot = row_regime_override() == REGIME_AUTO && shot.G > 0 && shot.G <= ONESHOT &&
                         (sizeof(T) != 2 || packs >= 32);
  if (take_shot) {
    const bool done = for_row_plan<MAXNV, true>(shot, [&]<int G, int NV>() {
      if constexpr (G <= ONESHOT) {
        const size_t need = (m + ONESHOT / G - 1) / (ONESHOT / G);
        require(need < 0x7fffffffull, "rmsnorm: too many rows for one grid");
        const dim3 grid((unsigned)need), block(ONESHOT);
        if (note_plan(PLAN_RESIDENT, G, NV, ONESHOT / G, grid.x, block.x, 1, 0, 0, keep && !loose)) return;
        if (loose) rmsnorm_fwd_resident<T, W, G, NV, true, ONESHOT><<<grid, block, 0, stream>>>(x, gain, y, (P)eps, m, n);
        else if (keep) rmsnorm_fwd_resident<T, W, G, NV, false, ONESHOT, true><<<grid, block, 0, stream>>>(x, gain, y, (P)eps, m, n);
        else rmsnorm_fwd_resident<T, W, G, NV, false, ONESHOT><<<grid, block, 0, stream>>>(x, gain, y, (P)eps, m, n);
      }
    });
    if (done) {
      MP_CHECK_LAUNCH();
      return;
    }
  }
  RowPlan plan = plan_row(packs, MAXNV, loose ? 2 : 1, 8);
  /* r32 rows of exactly 64 KiB: two rows a workgroup at eight packs a thread, not one at four
   * (interleaved repeats, n = 16384: 5.52 -> 5.79 TB/s in three runs; n = 15360 loses by it, r16 rows
   * of 64 KiB gain 3 % at most) */
  if (sizeof(T) == 4 && row_regime_override() == REGIME_AUTO && packs == 4096 && MAXNV >= 8 && plan.G == 1024) plan = RowPlan{512, 8};
  const bool resident = for_row_plan<MAXNV, true>(plan, [&]<int G, int NV>() {
    const size_t need = (m + NORM_BLOCK / G - 1) / (NORM_BLOCK / G);
    const dim3 grid((unsigned)(need < cap ? need : cap)), block(NORM_BLOCK);
    if (note_plan(PLAN_RESIDENT, G, NV, NORM_BLOCK / G, grid.x, block.x, 1, 0, 0, keep && !loose)) return;
    if (loose) rmsnorm_fwd_resident<T, W, G, NV, true><<<grid, block, 0, stream>>>(x, gain, y, (P)eps, m, n);
    else if (keep)
      rmsnorm_fwd_resident<T, W, G, NV, false, NORM_BLOCK, true><<<grid, block, 0, stream>>>(x, gain, y, (P)eps, m, n);
    else rmsnorm_fwd_resident<T, W, G, NV, false><<<grid, block, 0, stream>>>(x, gain, y, (P)eps, m, n);
  });
  if (!resident && !note_plan(PLAN_STREAM, STREAM_THREADS, 0, 1, m < cap ? m : cap, STREAM_THREADS)) {
    const size_t grid = m < cap ? m : cap;
    if (mismatch) rmsnorm_fwd_stream<T, W, true><<<dim3((unsigned)grid), dim3(STREAM_THREADS), 0, stream>>>(x, gain, y, (P)eps, m, n);
    else rmsnorm_fwd_stream<T, W><<<dim3((unsigned)grid), dim3(STREAM_THREADS), 0, stream>>>(x, gain, y, (P)eps, m, n);
  }
  MP_CHECK_LAUNCH();
}

template <class T, bool LOOSE>
inline void rmsnorm_reverse_as(const T* x, const T* gain, const T* dy, T* dx, T* dg, void* scratch,
                               double eps, double alpha, size_t m, size_t n, hipStream_t stream) {
  using P = typename precision<T>::type;
  constexpr int W = PACK_BYTES / (int)sizeof(T);
  P* partials = static_cast<P*>(scratch);
  const size_t max_rows = rmsnorm_reverse_partial_rows(m);
  const size_t packs = (n + W - 1) / W;
  const bool blend = alpha != 0.0;
  unsigned rows = 0;
  /* four register arrays per thread (x, dy, gain, dg sums): 16 registers each */
  constexpr int MAXNV = max_nv_for<T>(16);
  /* shared rows: dx distinct from x and dy (a workgroup that stops waiting re-reads the row), and
   * rows beyond the resident kernel unless the regime is forced */
  const bool distinct = !ranges_overlap(dx, x, m * n * sizeof(T)) && !ranges_overlap(dx, dy, m * n * sizeof(T));
  const int C = distinct ? rmsnorm_rev_cluster_size<T>(n) : 0;
  const bool force_shared = C >= 1 && row_regime_override() == REGIME_CLUSTER;
  RowPlan plan = force_shared ? RowPlan{0, 0} : plan_row(packs, MAXNV, 1, 8);
  /* a plan of several packs a thread that idles more than an eighth of its lanes gives way to the
   * tightest fit (r32 n = 5120: 1024 x 2 -> 512 x 3, 5.46 -> 5.98 TB/s; n = 6144: 5.63 -> 5.98); at
   * one pack a thread the wide group stays (n = 3072: 1024 x 1 6.00 against 256 x 3 5.85), and the
   * forward loses by the same change at every length tried (n = 5120: 5.68 -> 5.49) */
  if (plan.NV >= 2) plan = plan_row_fit(packs, MAXNV, 1, 8);
  /* aligned r32 rows of 129 ... 239 and 257 ... 479 packs: 128-thread groups at two or four packs a
   * thread, eight rows a workgroup (two packs: the paired kernel; four: the unpaired one, two
   * workgroups a CU), not a group of twice or four times the width at a pack a thread that they
   * would not fill (interleaved repeats against that and the wavefront-group kernel: n = 704 5.65 ->
   * 5.83 TB/s, 832 5.74 -> 5.98, 1152 5.43 -> 5.93, 1408 5.62 -> 5.95, 1664 5.21 -> 5.90, 1792 5.53 -> 5.85;
   * rows that fill the wide group lose, n = 1024 6.03 -> 5.82, 2048 6.02 -> 5.57, and keep it) */
  if (!LOOSE && sizeof(T) == 4 && !force_shared && row_regime_override() == REGIME_AUTO && packs > 128 && packs <= 512 && MAXNV >= 4 &&
      packs * 16 < (size_t)(packs <= 256 ? 256 : 512) * 15)
    plan = RowPlan{128, packs <= 256 ? 2 : 4};
  const bool resident = for_row_plan<MAXNV, true, true>(plan, [&]<int G, int NV>() {
    const size_t need = (m + NORM_BLOCK / G - 1) / (NORM_BLOCK / G);
    /* two register sets of x and dy beside the gain and the dg sums: up to eight registers an array
     * fit the 128 of a 1024-thread workgroup without spills */
    constexpr bool pairs_fit = NV * W * (int)(sizeof(P) / 4) <= 8;
    /* rows of 129 ... 223 and 257 ... 447 packs leave a 256- or 512-thread group more than an eighth
     * idle: three to six wavefronts a row and as many rows a workgroup as fit 1024 threads instead
     * (interleaved repeats: r16 n = 1152 4.01 -> 4.72 TB/s, 1280 4.59 -> 5.17, 2560 4.30 -> 5.43, 3072
     * 5.03 -> 5.48; r32 n = 576 4.78 -> 5.39, 1280 5.09 -> 5.50, 1536 5.40 -> 5.95). Wider rows gain nothing
     * from shedding their idle wavefronts (n = 5120 r16: 4.80 -> 4.87, with two such workgroups a CU
     * 4.73) and keep the power-of-two groups. Aligned r32 rows of these lengths no longer come here:
     * the plan above puts them on 128-thread groups, which beat this path in turn. */
    /* rows of 513 ... 896 packs on one 1024-thread group at a pack a thread: five to seven wavefronts
     * a row at two packs a thread and three or two rows a workgroup. r32 and r64 hold the widened
     * packs; r16 would not fit them twice over, so the kernel keeps x, dy and gain as loaded and
     * widens on use (r32 n = 2176: 4.75 -> 5.79 TB/s, 2560: 5.38 -> 6.00, 3328: 5.25 -> 5.85, 3584:
     * 5.31 -> 5.89, 3072: equal; r16 n = 4352: 4.26 -> 5.67, 5120: 4.80 -> 5.91, 6144: 5.49 -> 6.15,
     * 6656: 5.07 -> 5.73, 7168: 4.88 -> 5.69). Seven eighths of a 512- or 256-thread group: -2 ... +3 %,
     * left with the power-of-two groups. */
    if constexpr (!LOOSE && G == 1024 && NV == 1 && (2 * W * (int)(sizeof(P) / 4) <= 8 || sizeof(T) == 2)) {
      const int gw = (int)((packs + 2 * WAVE - 1) / (2 * WAVE));
      if (row_regime_override() == REGIME_AUTO && packs * 8 <= (size_t)G * 7 && gw >= 2 && gw * WAVE * 2 * W <= NORM_BLOCK * 8) {
        const int rpb = NORM_BLOCK / (gw * WAVE);
        const size_t need_any = (m + rpb - 1) / rpb, one_per_cu = (size_t)compute_units();
        rows = (unsigned)(need_any < one_per_cu ? need_any : one_per_cu);
        const dim3 grid(rows), block(rpb * gw * WAVE);
        if (note_plan(PLAN_ANY, gw * WAVE, 2, rpb, grid.x, block.x, 1, 0, (size_t)rows * n * sizeof(P))) return;
        if (blend) rmsnorm_rev_paired_any<T, W, 2, true><<<grid, block, 0, stream>>>(x, gain, dy, dx, partials, (P)eps, (P)alpha, m, n, gw);
        else rmsnorm_rev_paired_any<T, W, 2, false><<<grid, block, 0, stream>>>(x, gain, dy, dx, partials, (P)eps, (P)alpha, m, n, gw);
        return;
      }
    }
    if constexpr (!LOOSE && (G == 512 || G == 256) && NV == 1 && pairs_fit) {
      const int gw = (int)((packs + WAVE - 1) / WAVE);
      /* r16: only rows that fill the group to less than eleven sixteenths; fuller ones are better off on
       * the power-of-two group since it keeps three register sets (n = 1536: 5.55 -> 6.03 TB/s, 3072:
       * 5.79 -> 6.05) */
      const bool idle_enough = sizeof(T) == 2 ? packs * 16 < (size_t)G * 11 : packs * 8 < (size_t)G * 7;
      if (row_regime_override() == REGIME_AUTO && idle_enough && gw >= NORM_BLOCK / WAVE / ANY_MAX_ROWS) {
        const int rpb = NORM_BLOCK / (gw * WAVE);
        const size_t need_any = (m + rpb - 1) / rpb, one_per_cu = (size_t)compute_units();
        rows = (unsigned)(need_any < one_per_cu ? need_any : one_per_cu);
        const dim3 grid(rows), block(rpb * gw * WAVE);
        if (note_plan(PLAN_ANY, gw * WAVE, NV, rpb, grid.x, block.x, 1, 0, (size_t)rows * n * sizeof(P))) return;
        /* a third register set for two-byte types and for the shortest rows of four-byte ones (interleaved
         * repeats: r16 n = 1280 4.71 -> 5.99 TB/s, 3072 5.55 -> 5.87, 2560 equal; r32 n = 640 5.36 -> 5.71,
         * 1280 equal, 1536 5.86 -> 5.68) */
        const bool deep = sizeof(T) == 2 || (sizeof(T) == 4 && gw <= 4);
        auto go = [&]<bool BLEND, int DEPTH>() {
          rmsnorm_rev_paired_any<T, W, NV, BLEND, DEPTH><<<grid, block, 0, stream>>>(x, gain, dy, dx, partials, (P)eps, (P)alpha, m, n, gw);
        };
        if (blend) { if (deep) go.template operator()<true, 3>(); else go.template operator()<true, 2>(); }
        else { if (deep) go.template operator()<false, 3>(); else go.template operator()<false, 2>(); }
        return;
      }
    }
    if constexpr (!LOOSE && G > WAVE && pairs_fit) {
      /* aligned rows of whole packs in groups of more than a wavefront: rows in pairs, the next
       * row's loads in flight behind the current row's reduction, one workgroup per CU */
      const size_t one_per_cu = (size_t)compute_units();
      rows = (unsigned)(need < one_per_cu ? need : one_per_cu);
      const dim3 grid(rows), block(NORM_BLOCK);
      if (note_plan(PLAN_PAIRED, G, NV, NORM_BLOCK / G, grid.x, block.x, 1, 0, (size_t)rows * n * sizeof(P))) return;
      const bool exact = n == (size_t)G * NV * W;
      /* a third register set where a row is short enough that two sets in flight do not cover the
       * memory latency (interleaved repeats: r16 n = 1024 5.45 -> 6.09 TB/s, 2048 5.89 -> 6.08, 4096
       * 5.89 -> 6.10, 8192 6.16 -> 6.06; r32 n = 512 5.81 -> 6.04, 1024 6.09 -> 5.97, 2048 6.04 -> 5.57,
       * 4096 5.99 -> 5.81) */
      constexpr int DEPTH = NV == 1 && ((sizeof(T) == 2 && G <= 512) || G == 128) ? 3 : 2;
      auto go = [&]<bool BLEND, bool EXACT>() {
        rmsnorm_rev_paired<T, W, G, NV, BLEND, EXACT, DEPTH><<<grid, block, 0, stream>>>(x, gain, dy, dx, partials, (P)eps, (P)alpha, m, n);
      };
      if (blend) { if (exact) go.template operator()<true, true>(); else go.template operator()<true, false>(); }
      else { if (exact) go.template operator()<false, true>(); else go.template operator()<false, false>(); }
    } else {
      rows = (unsigned)(need < max_rows ? need : max_rows);
      const dim3 grid(rows), block(NORM_BLOCK);
      if (note_plan(PLAN_RESIDENT, G, NV, NORM_BLOCK / G, grid.x, block.x, 1, 0, (size_t)rows * n * sizeof(P))) return;
      if (blend) rmsnorm_rev_resident<T, W, G, NV, true, LOOSE><<<grid, block, 0, stream>>>(x, gain, dy, dx, partials, (P)eps, (P)alpha, m, n, rows_share_lines<T>(n));
      else rmsnorm_rev_resident<T, W, G, NV, false, LOOSE><<<grid, block, 0, stream>>>(x, gain, dy, dx, partials, (P)eps, (P)alpha, m, n, rows_share_lines<T>(n));
    }
  });
  bool shared = false;
  if (!resident && C >= 1) {
    using Word = typename slot_word<P>::type;
    const bool deep = norm_rev_deep<T>(packs);
    size_t S = (size_t)compute_units() * (deep ? 1 : norm_rev_cluster_per_cu<T>()) / (size_t)C; /* every workgroup resident at once */
    if (S > m) S = m;
    if (S == 0) S = 1;
    rows = (unsigned)S;
    const int ppb = cluster_chunk_packs(packs, C, norm_rev_cluster_tile<T>(packs));
    require((size_t)ppb <= norm_rev_cluster_tile<T>(packs), "rmsnorm reverse: cluster chunk exceeds the register tile");
    Word* slots = reinterpret_cast<Word*>(partials + rmsnorm_reverse_partial_rows(m) * n);
    if (note_plan(deep ? PLAN_DEEP : PLAN_CLUSTER, CLUSTER_THREADS, (int)((norm_rev_cluster_tile<T>(packs) + CLUSTER_THREADS - 1) / CLUSTER_THREADS), 1, S * C,
                  CLUSTER_THREADS, C, ppb,
                  (rmsnorm_reverse_partial_rows(m) * n + (C > 1 || deep ? m * (size_t)C * 2 : 0)) * sizeof(P)))
      return;
    if (C > 1 || deep) { /* the pipelined kernel hands its sums over through the words also when a row is one chunk (test build only) */
      const size_t words = m * (size_t)C * 2;
      cluster_zero_slots<Word><<<dim3((unsigned)((words + 255) / 256)), dim3(256), 0, stream>>>(slots, words);
    }
    const dim3 grid((unsigned)(S * C)), block(CLUSTER_THREADS);
    bool launched = false;
    if constexpr (sizeof(T) == 4) {
      if (deep) {
        if (blend) rmsnorm_rev_cluster_deep<T, W, true><<<grid, block, 0, stream>>>(x, gain, dy, dx, partials, (P)eps, (P)alpha, slots, m, n, C, ppb, cluster_tuning().spin_limit);
        else rmsnorm_rev_cluster_deep<T, W, false><<<grid, block, 0, stream>>>(x, gain, dy, dx, partials, (P)eps, (P)alpha, slots, m, n, C, ppb, cluster_tuning().spin_limit);
        launched = true;
      }
    }
    if (!launched) {
      if (blend) rmsnorm_rev_cluster<T, W, true, LOOSE><<<grid, block, 0, stream>>>(x, gain, dy, dx, partials, (P)eps, (P)alpha, slots, m, n, C, ppb, cluster_tuning().spin_limit);
      else rmsnorm_rev_cluster<T, W, false, LOOSE><<<grid, block, 0, stream>>>(x, gain, dy, dx, partials, (P)eps, (P)alpha, slots, m, n, C, ppb, cluster_tuning().spin_limit);
    }
    shared = true;
  }
  if (!resident && !shared) {
    rows = (unsigned)max_rows;
    const dim3 grid(rows), block(STREAM_THREADS);
    if (note_plan(PLAN_STREAM, STREAM_THREADS, 0, 1, grid.x, block.x, 1, 0, (size_t)rows * n * sizeof(P))) return;
    constexpr int NA = stream_acc_packs<T>();
    const bool sums_fit = packs <= (size_t)STREAM_THREADS * NA;
    if (sums_fit) {
      if (blend) rmsnorm_rev_stream<T, W, NA, true, LOOSE><<<grid, block, 0, stream>>>(x, gain, dy, dx, partials, (P)eps, (P)alpha, m, n);
      else rmsnorm_rev_stream<T, W, NA, false, LOOSE><<<grid, block, 0, stream>>>(x, gain, dy, dx, partials, (P)eps, (P)alpha, m, n);
    } else {
      if (blend) rmsnorm_rev_stream<T, W, 0, true, LOOSE><<<grid, block, 0, stream>>>(x, gain, dy, dx, partials, (P)eps, (P)alpha, m, n);
      else rmsnorm_rev_stream<T, W, 0, false, LOOSE><<<grid, block, 0, stream>>>(x, gain, dy, dx, partials, (P)eps, (P)alpha, m, n);
    }
  }
  MP_CHECK_LAUNCH();
  sum_partial_rows<T>(partials, dg, alpha, rows, n, stream);
}

template <class T>
inline void rmsnorm_reverse(const T* x, const T* gain, const T* dy, T* dx, T* dg, void* scratch,
                            double eps, double alpha, size_t m, size_t n, hipStream_t stream) {
  if (m == 0 || n == 0) return;
  constexpr int W = PACK_BYTES / (int)sizeof(T);
  require(n <= 0x40000000ull, "rmsnorm reverse: row length must not exceed 2^30");
  require(scratch != nullptr, "rmsnorm reverse: scratch must hold mpRmsnormReverseScratchBytes bytes");
  if (rmsnorm_short_rows<T>(n, true)) {
    using P = typename precision<T>::type;
    P* partials = static_cast<P*>(scratch);
    const size_t max_rows = rmsnorm_reverse_partial_rows(m);
    unsigned rows = 0;
    for_short_row(n, W, [&]<int G, bool CUT>() {
      const size_t need = (m + NORM_BLOCK / G - 1) / (NORM_BLOCK / G);
      rows = (unsigned)(need < max_rows ? need : max_rows);
      const dim3 grid(rows), block(NORM_BLOCK);
      if (note_plan(PLAN_SHORT, G, 1, NORM_BLOCK / G, grid.x, block.x, 1, 0, (size_t)rows * n * sizeof(P))) return;
      if (alpha != 0.0) rmsnorm_rev_short<T, W, G, CUT, true><<<grid, block, 0, stream>>>(x, gain, dy, dx, partials, (P)eps, (P)alpha, m, (unsigned)n);
      else rmsnorm_rev_short<T, W, G, CUT, false><<<grid, block, 0, stream>>>(x, gain, dy, dx, partials, (P)eps, (P)alpha, m, (unsigned)n);
    });
    MP_CHECK_LAUNCH();
    sum_partial_rows<T>(partials, dg, alpha, rows, n, stream);
    return;
  }
  const bool packed = aligned16(x) && aligned16(dy) && aligned16(dx) && aligned16(gain) && (n % W) == 0;
  if (packed) rmsnorm_reverse_as<T, false>(x, gain, dy, dx, dg, scratch, eps, alpha, m, n, stream);
  else rmsnorm_reverse_as<T, true>(x, gain, dy, dx, dg, scratch, eps, alpha, m, n, stream);
}

}  // namespace mp

#endif
#endif
