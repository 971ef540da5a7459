/*
 * Row-wise softmax over the last dimension, forward and reverse.
 *
 * The reference has no softmax kernel (NOTES.md:28 lists it as to-do; the "ij|j" notation is
 * src/ops/expression_parsing.zig:320-340). Math:
 *   forward   y_ij  = exp(x_ij - max_j x_ij) / sum_j exp(x_ij - max_j x_ij)
 *   reverse   dx_ij = y_ij * (dy_ij - sum_j y_ij*dy_ij) + alpha * dx_ij
 * Accumulation is in precision<T> (fp32 for r16/r32, fp64 for r64), following the up-cast rule
 * of src/cuda/tensor_types.h:51-69. -inf inputs give exactly 0; a row with no finite entry
 * gives NaN, as the closed form does.
 *
 * Resident kernels read each row once, keep it in registers across both reductions and write
 * it once; the reverse folds dot(y, dy) and the gradient write into the same pass over
 * registers. Rows longer than one workgroup's registers are shared by a cluster of consecutive
 * workgroups that exchange their (max, sum) through caller-owned scratch, still reading the row
 * once. Streaming kernels cover what is left (no scratch given, or rows beyond a cluster) with
 * one online max/sum pass (running maximum, running sum rescaled whenever the maximum moves)
 * and one write pass that re-reads the row.
 */
#ifndef MP_ROW_SOFTMAX_H
#define MP_ROW_SOFTMAX_H

#include "row_cluster.h"
#include <type_traits>

#if defined(__cplusplus) && defined(__HIPCC__)

namespace mp {

/* ------------------------------------------------------------------ short rows */

template <class T, int W, int G, bool CUT>
__global__ __launch_bounds__(SHORT_THREADS) void softmax_fwd_short(const T* x, T* y, size_t m, unsigned n, unsigned by_xcd) {
  using P = typename precision<T>::type;
  const int lane = threadIdx.x % G;
  bool live;
  const size_t row = short_row_of<G>(m, by_xcd, live);
  ShortRow<T, W, G, CUT> t;
  t.load(x + row * n, n, lane, neg_inf<P>());

  P mx = neg_inf<P>();
#pragma unroll
  for (int i = 0; i < W; ++i) mx = t.v[i] > mx ? t.v[i] : mx;
  mx = fold_partials<MaxOP, G>(mx);

  const P sh = shift_of(mx);
  P s = (P)0;
#pragma unroll
  for (int i = 0; i < W; ++i) {
    t.v[i] = exp_shifted(t.v[i], sh);
    s += t.v[i];
  }
  s = fold_partials<AddOP, G>(s);

  const P inv = reciprocal_of(s);
#pragma unroll
  for (int i = 0; i < W; ++i) t.v[i] *= inv;
  if (live) t.store(y + row * n, n, lane);
}

template <class T, int W, int G, bool CUT, bool BLEND>
__global__ __launch_bounds__(SHORT_THREADS) void softmax_rev_short(
    const T* y, const T* dy, T* dx, typename precision<T>::type alpha, size_t m, unsigned n, unsigned by_xcd) {
  using P = typename precision<T>::type;
  const int lane = threadIdx.x % G;
  bool live;
  const size_t row = short_row_of<G>(m, by_xcd, live);
  ShortRow<T, W, G, CUT> ty, tg;
  ty.load(y + row * n, n, lane, (P)0);
  tg.load(dy + row * n, n, lane, (P)0);

  P dot = (P)0;
#pragma unroll
  for (int i = 0; i < W; ++i) dot += ty.v[i] * tg.v[i];
  dot = fold_partials<AddOP, G>(dot);
  if (!live) return; /* nothing below crosses lanes */

#pragma unroll
  for (int i = 0; i < W; ++i) ty.v[i] *= tg.v[i] - dot;
  if constexpr (BLEND) {
    tg.load(dx + row * n, n, lane, (P)0);
#pragma unroll
    for (int i = 0; i < W; ++i) ty.v[i] += alpha * tg.v[i];
  }
  ty.store(dx + row * n, n, lane);
}

/* ------------------------------------------------------------------ resident forward */

/* KEEP: y through ordinary stores, which leave it in the memory-side cache for the reverse
 * (keep_output, row_cluster.h). */

template <class T, int W, int G, int NV, bool RAGGED, bool KEEP = false>
__global__ __launch_bounds__(G < WAVE ? WAVE : G) void softmax_fwd_resident(
    const T* x, T* y, size_t m, size_t n, unsigned by_xcd) {
  using P = typename precision<T>::type;
  constexpr int RPB = G < WAVE ? WAVE / G : 1; /* rows per workgroup: several only below a wave */
  __shared__ P slots[2][G < WAVE ? 1 : G / WAVE];

  const int lane = threadIdx.x % G;
  const unsigned block = by_xcd ? xcd_contiguous_block(blockIdx.x, gridDim.x) : blockIdx.x;
  const size_t row_at = (size_t)block * RPB + threadIdx.x / G;
  const bool live = row_at < m;            /* a dead part of a wave still runs the cross-lane steps */
  const size_t row = live ? row_at : m - 1;

  const T* xr = x + row * n;
  const RowGeom<T, W> g(xr, n, RAGGED);
  RowTile<T, W, G, NV, RAGGED> t;
  t.load(xr, g, lane, neg_inf<P>());

  P mx = neg_inf<P>();
  t.each([&](P& e) { mx = e > mx ? e : mx; });
  mx = group_allreduce<MaxOP, G>(mx, slots[0], lane);

  const P sh = shift_of(mx);
  P s = (P)0;
  t.each([&](P& e) { e = exp_shifted(e, sh); s += e; });
  s = group_allreduce<AddOP, G>(s, slots[1], lane);

  const P inv = reciprocal_of(s);
  t.each([&](P& e) { e *= inv; });
  if (live) t.template store<KEEP>(y + row * n, g, lane);
}

/* ------------------------------------------------------------------ resident reverse */

template <class T, int W, int G, int NV, bool RAGGED, bool BLEND>
__global__ __launch_bounds__(G < WAVE ? WAVE : G) void softmax_rev_resident(
    const T* y, const T* dy, T* dx, typename precision<T>::type alpha, size_t m, size_t n, unsigned by_xcd) {
  using P = typename precision<T>::type;
  constexpr int RPB = G < WAVE ? WAVE / G : 1;
  __shared__ P slots[G < WAVE ? 1 : G / WAVE];

  const int lane = threadIdx.x % G;
  const unsigned block = by_xcd ? xcd_contiguous_block(blockIdx.x, gridDim.x) : blockIdx.x;
  const size_t row_at = (size_t)block * RPB + threadIdx.x / G;
  const bool live = row_at < m;
  const size_t row = live ? row_at : m - 1;

  const T* yr = y + row * n;
  const T* gr = dy + row * n;
  T* dr = dx + row * n;
  const RowGeom<T, W> g(yr, n, RAGGED);
  RowTile<T, W, G, NV, RAGGED> ty, tg;
  ty.load(yr, g, lane, (P)0);
  tg.load(gr, g, lane, (P)0);

  P dot = (P)0;
#pragma unroll
  for (int k = 0; k < NV; ++k)
#pragma unroll
    for (int i = 0; i < W; ++i) dot += ty.v[k][i] * tg.v[k][i];
  if constexpr (RAGGED) dot += ty.edge * tg.edge;
  dot = group_allreduce<AddOP, G>(dot, slots, lane);
  if (!live) return; /* nothing below crosses lanes */

  T* body = dr + g.head;
#pragma unroll
  for (int k = 0; k < NV; ++k) {
    const int p = k * G + lane;
    if (p < g.nvec) {
      P out[W];
#pragma unroll
      for (int i = 0; i < W; ++i) out[i] = ty.v[k][i] * (tg.v[k][i] - dot);
      if constexpr (BLEND) {
        P old[W];
        load_pack<T, W>(body + (size_t)p * W, old);
#pragma unroll
        for (int i = 0; i < W; ++i) out[i] += alpha * old[i];
      }
      store_pack_nt<T, W>(body + (size_t)p * W, out);
    }
  }
  if constexpr (RAGGED) {
    T* e = nullptr;
    if (lane < g.head) e = dr + lane;
    else if (lane - g.head < g.tail) e = body + (size_t)g.nvec * W + (lane - g.head);
    if (e) {
      P out = ty.edge * (tg.edge - dot);
      if constexpr (BLEND) out += alpha * (P)*e;
      *e = (T)out;
    }
  }
}

/* ------------------------------------------------------------------ rows shifted apart */

/* The resident kernels for operands whose rows do not peel alike (x 16-byte aligned and y not, a
 * gradient at another offset than its output): packs counted from each row's first element
 * (RowPacks), at whatever alignment each operand has. Element by element these rows ran at
 * 0.3-1.7 TB/s. */
template <class T, int W, int G, int NV>
__global__ __launch_bounds__(G < WAVE ? WAVE : G) void softmax_fwd_loose(const T* x, T* y, size_t m, size_t n) {
  using P = typename precision<T>::type;
  constexpr int RPB = G < WAVE ? WAVE / G : 1;
  __shared__ P slots[2][G < WAVE ? 1 : G / WAVE];
  const int lane = threadIdx.x % G;
  const size_t row_at = (size_t)blockIdx.x * RPB + threadIdx.x / G;
  const bool live = row_at < m; /* a dead part of a wave still runs the cross-lane steps */
  const size_t row = live ? row_at : m - 1;
  const RowPacks<T, W, true> rp(n);

  P v[NV][W];
#pragma unroll
  for (int k = 0; k < NV; ++k) {
    const int p = k * G + lane;
    if (p < rp.npk) rp.template load<true>(x + row * n, p, v[k]);
#pragma unroll
    for (int i = 0; i < W; ++i)
      if (p >= rp.npk || i >= rp.valid(p)) v[k][i] = neg_inf<P>();
  }
  P mx = neg_inf<P>();
#pragma unroll
  for (int k = 0; k < NV; ++k)
#pragma unroll
    for (int i = 0; i < W; ++i) mx = v[k][i] > mx ? v[k][i] : mx;
  mx = group_allreduce<MaxOP, G>(mx, slots[0], lane);

  const P sh = shift_of(mx);
  P s = (P)0;
#pragma unroll
  for (int k = 0; k < NV; ++k)
#pragma unroll
    for (int i = 0; i < W; ++i) {
      v[k][i] = exp_shifted(v[k][i], sh);
      s += v[k][i];
    }
  s = group_allreduce<AddOP, G>(s, slots[1], lane);

  const P inv = reciprocal_of(s);
  if (!live) return;
#pragma unroll
  for (int k = 0; k < NV; ++k) {
    const int p = k * G + lane;
    if (p < rp.npk) {
#pragma unroll
      for (int i = 0; i < W; ++i) v[k][i] *= inv;
      rp.store(y + row * n, p, v[k]);
    }
  }
}

template <class T, int W, int G, int NV, bool BLEND>
__global__ __launch_bounds__(G < WAVE ? WAVE : G) void softmax_rev_loose(
    const T* y, const T* dy, T* dx, typename precision<T>::type alpha, size_t m, size_t n) {
  using P = typename precision<T>::type;
  constexpr int RPB = G < WAVE ? WAVE / G : 1;
  __shared__ P slots[G < WAVE ? 1 : G / WAVE];
  const int lane = threadIdx.x % G;
  const size_t row_at = (size_t)blockIdx.x * RPB + threadIdx.x / G;
  const bool live = row_at < m;
  const size_t row = live ? row_at : m - 1;
  const RowPacks<T, W, true> rp(n);

  P yv[NV][W], gv[NV][W];
  P dot = (P)0;
#pragma unroll
  for (int k = 0; k < NV; ++k) {
    const int p = k * G + lane;
    if (p < rp.npk) {
      rp.template load<true>(y + row * n, p, yv[k]);
      rp.template load<true>(dy + row * n, p, gv[k]);
    } else {
#pragma unroll
      for (int i = 0; i < W; ++i) yv[k][i] = gv[k][i] = (P)0;
    }
#pragma unroll
    for (int i = 0; i < W; ++i) dot += yv[k][i] * gv[k][i];
  }
  dot = group_allreduce<AddOP, G>(dot, slots, lane);
  if (!live) return; /* nothing below crosses lanes */

#pragma unroll
  for (int k = 0; k < NV; ++k) {
    const int p = k * G + lane;
    if (p < rp.npk) {
      P out[W];
#pragma unroll
      for (int i = 0; i < W; ++i) out[i] = yv[k][i] * (gv[k][i] - dot);
      if constexpr (BLEND) {
        P old[W];
        rp.template load<false>(dx + row * n, p, old);
#pragma unroll
        for (int i = 0; i < W; ++i) out[i] += alpha * old[i];
      }
      rp.store(dx + row * n, p, out);
    }
  }
}

/* ------------------------------------------------------------------ streaming forward */

/* Folds one value into a lane's running (max, sum of exp(x - max)). */
template <class P> __device__ __forceinline__ void online_rescale(P& run_max, P& run_sum, P chunk_max) {
  const P nm = chunk_max > run_max ? chunk_max : run_max;
  if (nm > run_max) { /* also taken on the first finite value: exp(-inf - nm) = 0 */
    run_sum *= exp_shifted(run_max, shift_of(nm));
    run_max = nm;
  }
}

/* One lane's share of a row folded online: running maximum and the sum of exp(x - maximum),
 * rescaled whenever the maximum moves. G threads stride the packs, U loads in flight. */
template <class T, int W, int G, int U>
__device__ __forceinline__ void row_online_max_sum(const T* xr, const RowGeom<T, W>& g, int lane,
                                                   typename precision<T>::type& run_max,
                                                   typename precision<T>::type& run_sum) {
  using P = typename precision<T>::type;
  const T* body = xr + g.head;
  run_max = neg_inf<P>();
  run_sum = (P)0;
  for (int p0 = lane; p0 < g.nvec; p0 += G * U) {
    P buf[U][W];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int p = p0 + u * G;
      if (p < g.nvec) {
        load_pack<T, W>(body + (size_t)p * W, buf[u]);
      } else {
#pragma unroll
        for (int i = 0; i < W; ++i) buf[u][i] = neg_inf<P>();
      }
    }
    P cm = neg_inf<P>();
#pragma unroll
    for (int u = 0; u < U; ++u)
#pragma unroll
      for (int i = 0; i < W; ++i) cm = buf[u][i] > cm ? buf[u][i] : cm;
    online_rescale(run_max, run_sum, cm);
    if (run_max > neg_inf<P>()) {
      const P sh = shift_of(run_max);
#pragma unroll
      for (int u = 0; u < U; ++u)
#pragma unroll
        for (int i = 0; i < W; ++i) run_sum += exp_shifted(buf[u][i], sh);
    }
  }
  if (W > 1) {
    P e = neg_inf<P>();
    if (lane < g.head) e = (P)xr[lane];
    else if (lane - g.head < g.tail) e = (P)body[(size_t)g.nvec * W + (lane - g.head)];
    online_rescale(run_max, run_sum, e);
    if (e > neg_inf<P>()) run_sum += exp_shifted(e, shift_of(run_max));
  }
}

/* APART: y is not aligned like x (whose alignment sets where the packs of a row start): its
 * packs then start at any element. */
template <class T, int W, bool APART = false>
__global__ __launch_bounds__(STREAM_THREADS) void softmax_fwd_stream(
    const T* x, T* y, size_t m, size_t n) {
  using P = typename precision<T>::type;
  constexpr int G = STREAM_THREADS, U = 4;
  __shared__ P slots[2][2][G / WAVE];
  const int lane = threadIdx.x;
  int parity = 0;

  for (size_t row = blockIdx.x; row < m; row += gridDim.x, parity ^= 1) {
    const T* xr = x + row * n;
    T* yr = y + row * n;
    const RowGeom<T, W> g(xr, n, true);
    const T* body = xr + g.head;

    /* pass 1: online max / sum */
    P run_max, run_sum;
    row_online_max_sum<T, W, G, 4>(xr, g, lane, run_max, run_sum);

    const P mx = group_allreduce<MaxOP, G>(run_max, slots[parity][0], lane);
    const P sh = shift_of(mx);
    const P scaled = run_max > neg_inf<P>() ? run_sum * exp_shifted(run_max, sh) : (P)0;
    const P s = group_allreduce<AddOP, G>(scaled, slots[parity][1], lane);
    const P inv = reciprocal_of(s);

    /* pass 2: the row again, normally still in cache */
    T* ybody = yr + g.head;
    for (int p0 = lane; p0 < g.nvec; p0 += G * U) {
      P buf[U][W];
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const int p = p0 + u * G;
        if (p < g.nvec) load_pack_nt<T, W>(body + (size_t)p * W, buf[u]);
      }
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const int p = p0 + u * G;
        if (p < g.nvec) {
#pragma unroll
          for (int i = 0; i < W; ++i) buf[u][i] = exp_shifted(buf[u][i], sh) * inv;
          if constexpr (APART) store_pack_nt_loose<T, W>(ybody + (size_t)p * W, buf[u]);
          else store_pack_nt<T, W>(ybody + (size_t)p * W, buf[u]);
        }
      }
    }
    if (W > 1) {
      if (lane < g.head) yr[lane] = (T)(exp_shifted((P)xr[lane], sh) * inv);
      else if (lane - g.head < g.tail) {
        const size_t o = (size_t)g.nvec * W + (lane - g.head);
        ybody[o] = (T)(exp_shifted((P)body[o], sh) * inv);
      }
    }
  }
}

/* ------------------------------------------------------------------ cluster forward */

/* Rows too long for one workgroup's registers but short enough for a few: C consecutive
 * workgroups share a row. Each keeps its chunk in registers, publishes its (max, sum) through
 * two agent-scope atomic words in caller-owned scratch, waits for the other C-1, and writes its
 * chunk: the row is still read once and written once.
 *
 * The words are stamped (row_cluster.h): a word counts as published when it carries the stamp of
 * this launch, which a workgroup derives from what its own word carried before, so no launch in
 * front has to clear anything when the words are the library's own.
 *
 * Waiting is bounded. Workgroups of one row have consecutive indices and a workgroup publishes
 * before it waits, so with in-order dispatch the wait is short; if spin_limit polls pass
 * anyway, the workgroup stops waiting and folds the whole row itself (one extra read of the row),
 * so every wave reaches the end whatever the scheduling. */
/* packs per thread, so that two workgroups fit a CU (64 registers): 24 registers of widened row
 * data for r32 and r64 (6 packs); r16 chunks stay in their storage type (four registers a
 * pack) and are widened where they are used, at the price of a second exponential per element,
 * which makes room for 7 packs: a 50257-wide r16 row then fits one workgroup and needs no
 * exchange (5.2 -> 5.6 TB/s; 8 packs spill) */
template <class T> constexpr int cluster_nv() {
  if (sizeof(T) == 2) return 7;
  return 24 / ((PACK_BYTES / (int)sizeof(T)) * (int)(sizeof(typename precision<T>::type) / 4));
}

template <class T, int W, bool KEEP = false>
__global__ __launch_bounds__(CLUSTER_THREADS, 8) void softmax_fwd_cluster(
    const T* x, T* y, share_word* callers_words, size_t region,
    size_t m, size_t n, int C, int packs_per_block, unsigned spin_limit) {
  using P = typename precision<T>::type;
  constexpr int G = CLUSTER_THREADS, NV = cluster_nv<T>(), WPS = 2 * share_parts<P>();
  __shared__ P red[4][G / WAVE];
  __shared__ P bc[3];
  const int lane = threadIdx.x;
  const size_t row = blockIdx.x / (unsigned)C;
  const int rank = (int)(blockIdx.x % (unsigned)C);
  share_word* row_words = share_words(callers_words, region) + row * (size_t)C * WPS;
  const share_word peeked = C > 1 ? share_peek(row_words + (size_t)rank * WPS, lane) : 0; /* on its way while the chunk loads */
  const T* xr = x + row * n;
  T* yr = y + row * n;
  const RowGeom<T, W> g(xr, n, true);
  const T* body = xr + g.head;
  const int lo = rank * packs_per_block - cluster_skew(body, C, packs_per_block, g.nvec);
  const int hi = lo + packs_per_block < g.nvec ? lo + packs_per_block : g.nvec;

  /* this workgroup's chunk; rank 0 also holds the row's head / tail scalars */
  constexpr bool RAW = sizeof(T) == 2; /* chunk kept in the storage type, exponentials taken twice */
  using V = typename vec_of<T, W>::type;
  using Held = typename std::conditional<RAW, V, P[W]>::type;
  Held v[NV];
#pragma unroll
  for (int k = 0; k < NV; ++k) {
    const int p = lo + k * G + lane;
    if (p >= 0 && p < hi) {
      if constexpr (RAW) v[k] = __builtin_nontemporal_load(reinterpret_cast<const V*>(body + (size_t)p * W));
      else load_pack_nt<T, W>(body + (size_t)p * W, v[k]);
    } else {
#pragma unroll
      for (int i = 0; i < W; ++i) v[k][i] = RAW ? (T)neg_inf<P>() : neg_inf<P>();
    }
  }
  P edge = neg_inf<P>();
  size_t edge_at = (size_t)-1;
  if (W > 1 && rank == 0) {
    if (lane < g.head) edge_at = (size_t)lane;
    else if (lane - g.head < g.tail) edge_at = (size_t)g.head + (size_t)g.nvec * W + (lane - g.head);
    if (edge_at != (size_t)-1) edge = (P)xr[edge_at];
  }

  P mx = edge;
  if constexpr (RAW) { /* packed half maxima (two elements an instruction), widened once at the end */
    V vm = v[0];
#pragma unroll
    for (int k = 1; k < NV; ++k) vm = __builtin_elementwise_max(vm, v[k]);
#pragma unroll
    for (int i = 0; i < W; ++i) mx = (P)vm[i] > mx ? (P)vm[i] : mx;
  } else {
#pragma unroll
    for (int k = 0; k < NV; ++k)
#pragma unroll
      for (int i = 0; i < W; ++i) mx = (P)v[k][i] > mx ? (P)v[k][i] : mx;
  }
  /* one exchange inside the workgroup for both reductions: every wavefront shifts by its own
   * maximum, and the (max, sum) pairs of the sixteen wavefronts meet behind one barrier (against a
   * barrier for the maximum and one for the sum: [512, 151936] 111.1 -> 109.7 us, [2048, 50257]
   * 146.9 -> 144.4, launcher times of interleaved repeats) */
  const P base_mx = wave_allreduce<MaxOP>(mx);
  if constexpr (RAW) {
#pragma unroll
    for (int k = 0; k < NV; ++k) forget(v[k]);
  }
  /* a chunk without a finite entry (fully masked) contributes exact zeros, not exp(-inf + inf) */
  const P sh = shift_of(base_mx > neg_inf<P>() ? base_mx : (P)0);
  P s = (P)0;
#pragma unroll
  for (int k = 0; k < NV; ++k)
#pragma unroll
    for (int i = 0; i < W; ++i) {
      const P e = exp_shifted((P)v[k][i], sh);
      if constexpr (!RAW) v[k][i] = e;
      s += e;
    }
  if constexpr (RAW) {
#pragma unroll
    for (int k = 0; k < NV; ++k) forget(v[k]);
  }
  const P edge_x = edge;
  edge = exp_shifted(edge, sh);
  s += edge;
  s = wave_allreduce<AddOP>(s);
  if ((lane & (WAVE - 1)) == 0) {
    red[0][lane / WAVE] = base_mx;
    red[1][lane / WAVE] = s;
  }
  __syncthreads();
  {
    constexpr int NW = G / WAVE;
    const P wm = red[0][lane & (NW - 1)], ws = red[1][lane & (NW - 1)];
    mx = fold_partials<MaxOP, NW>(wm); /* the chunk's maximum and, relative to it, its sum */
    s = fold_partials<AddOP, NW>(wm > neg_inf<P>() ? ws * exp_shifted(wm, shift_of(mx)) : (P)0);
  }
  P M = mx, S = s;
  if (C > 1) {
    if (lane < WAVE) { /* wave 0: lane b waits for workgroup b of this row */
      const unsigned stamp = share_stamp_of(peeked);
      if (lane == 0) { /* the sum of a chunk without a finite entry is ignored through its -inf maximum */
        const P mine[2] = {mx, s};
        share_publish<2>(row_words + (size_t)rank * WPS, stamp, mine);
      }
      P theirs[2] = {neg_inf<P>(), (P)0};
      bool ok = true;
      if (lane < C) {
        for (unsigned spins = 0;; ++spins) {
          ok = share_read<2>(row_words + (size_t)lane * WPS, stamp, theirs);
          if (ok || spins >= spin_limit) break;
          __builtin_amdgcn_s_sleep(4);
        }
      }
      const P om = theirs[0], os = theirs[1];
      const P all_ok = wave_allreduce<AddOP>(ok ? (P)0 : (P)1); /* every lane takes part */
      const P gm = wave_allreduce<MaxOP>(lane < C && ok ? om : neg_inf<P>());
      const P part = (lane < C && ok && om > neg_inf<P>()) ? os * exp_shifted(om, shift_of(gm)) : (P)0;
      const P gs = wave_allreduce<AddOP>(part);
      if (lane == 0) {
        bc[0] = gm;
        bc[1] = gs;
        bc[2] = all_ok;
      }
    }
    __syncthreads();
    M = bc[0];
    S = bc[1];
    if (bc[2] != (P)0) { /* gave up waiting: fold the whole row here */
      P run_max, run_sum;
      row_online_max_sum<T, W, G, 1>(xr, g, lane, run_max, run_sum); /* rare path: keep it lean */
      M = group_allreduce<MaxOP, G>(run_max, red[2], lane);
      const P scaled = run_max > neg_inf<P>() ? run_sum * exp_shifted(run_max, shift_of(M)) : (P)0;
      S = group_allreduce<AddOP, G>(scaled, red[3], lane);
    }
  }

  const P scale = exp_shifted(base_mx, shift_of(M)) * reciprocal_of(S);
  T* ybody = yr + g.head;
  if constexpr (RAW) {
    const P shM = shift_of(M), inv = reciprocal_of(S);
#pragma unroll
    for (int k = 0; k < NV; ++k) {
      const int p = lo + k * G + lane;
      if (p >= 0 && p < hi) {
        P out[W];
#pragma unroll
        for (int i = 0; i < W; ++i) out[i] = exp_shifted((P)v[k][i], shM) * inv;
        store_pack_kept<KEEP, T, W>(ybody + (size_t)p * W, out);
      }
    }
    if (edge_at != (size_t)-1) yr[edge_at] = (T)(exp_shifted(edge_x, shM) * inv);
  } else {
#pragma unroll
    for (int k = 0; k < NV; ++k) {
      const int p = lo + k * G + lane;
      if (p >= 0 && p < hi) {
#pragma unroll
        for (int i = 0; i < W; ++i) v[k][i] *= scale;
        store_pack_kept<KEEP, T, W>(ybody + (size_t)p * W, v[k]);
      }
    }
    if (edge_at != (size_t)-1) yr[edge_at] = (T)(edge * scale);
  }
}

/* Workgroups per row on the cluster path; 0 when the row does not take it. */
template <class T> inline int cluster_size(size_t packs) {
  const int regime = row_regime_override();
  if (regime != REGIME_AUTO && regime != REGIME_CLUSTER) return 0;
  /* up to two packs per thread a resident workgroup is the better kernel; measured exceptions: r32
   * rows of exactly 2048 packs (n = 8192: 5.8 resident, 6.1 here), and r16 chunks want the whole
   * register tile (n = 49152: 5.4 -> 5.7 TB/s) where r32 is better one pack per thread below it */
  const size_t resident = (size_t)CLUSTER_THREADS * 2 - (sizeof(T) == 4 ? 1 : 0); /* r64 at 2048 packs: 3.66 here, 5.8 resident */
  if (regime == REGIME_AUTO && packs <= resident) return 0;
  /* r32 rows of 32 ... 64 KiB stay with one workgroup of 1024 threads at four packs a thread
   * (interleaved repeats, 2^28 elements: n = 12288 6.12 TB/s against 5.94 shared, 16384 equal; above,
   * two workgroups a row win or tie: n = 24576 6.10 against 5.76, 32768 equal; sixteen packs a thread
   * in 256 or 512 threads, an earlier choice, 5.78 / 5.37 / 5.58 / 5.70) */
  if (regime == REGIME_AUTO && sizeof(T) == 4 && packs > resident + 1 && packs <= 4096) return 0;
  /* r16 rows of exactly 64 KiB as well (n = 32768: 5.51 -> 5.89 TB/s); every other length from 24576
   * to 32000 ties or is better here */
  if (regime == REGIME_AUTO && sizeof(T) == 2 && packs == 4096) return 0;
  constexpr size_t tile = (size_t)CLUSTER_THREADS * cluster_nv<T>();
  size_t ppb = (size_t)cluster_tuning().packs_per_block;
  if (ppb == 0) ppb = sizeof(T) == 2 ? tile : tile - CLUSTER_THREADS;
  if (ppb > tile) ppb = tile;
  size_t c = (packs + ppb - 1) / ppb;
  /* r32 rows of exactly 128 KiB: three workgroups a row, not two that start 64 KiB apart (interleaved
   * repeats, n = 32768: 5.83 -> 6.12 TB/s; r16 n = 65536 loses, 5.13 -> 4.95) */
  if (regime == REGIME_AUTO && cluster_tuning().packs_per_block == 0 && sizeof(T) == 4 && packs == 8192 && c == 2) c = 3;
  return c >= 1 && c <= (size_t)CLUSTER_MAX ? (int)c : 0;
}

template <class T> inline size_t softmax_scratch_bytes(size_t m, size_t n) {
  using P = typename precision<T>::type;
  constexpr int W = PACK_BYTES / (int)sizeof(T);
  const size_t c = cluster_size_for_scratch(cluster_size<T>((n + W - 1) / W));
  return m * c * 2 * share_parts<P>() * sizeof(share_word); /* (max, sum) as stamped words */
}

/* ------------------------------------------------------------------ streaming reverse */

/* APART: dy or dx is not aligned like y (whose alignment sets where the packs of a row start):
 * their packs then start at any element. */
template <class T, int W, bool BLEND, bool APART = false>
__global__ __launch_bounds__(STREAM_THREADS) void softmax_rev_stream(
    const T* y, const T* dy, T* dx, typename precision<T>::type alpha, size_t m, size_t n) {
  using P = typename precision<T>::type;
  constexpr int G = STREAM_THREADS, U = 2;
  __shared__ P slots[2][G / WAVE];
  const int lane = threadIdx.x;
  int parity = 0;

  for (size_t row = blockIdx.x; row < m; row += gridDim.x, parity ^= 1) {
    const T* yr = y + row * n;
    const T* gr = dy + row * n;
    T* dr = dx + row * n;
    const RowGeom<T, W> g(yr, n, true);
    const T* ybody = yr + g.head;
    const T* gbody = gr + g.head;
    T* dbody = dr + g.head;

    P dot = (P)0;
    for (int p0 = lane; p0 < g.nvec; p0 += G * U) {
      P a[U][W], b[U][W];
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const int p = p0 + u * G;
        if (p < g.nvec) {
          load_pack<T, W>(ybody + (size_t)p * W, a[u]);
          if constexpr (APART) load_pack_loose<T, W>(gbody + (size_t)p * W, b[u]);
          else load_pack<T, W>(gbody + (size_t)p * W, b[u]);
        } else {
#pragma unroll
          for (int i = 0; i < W; ++i) a[u][i] = b[u][i] = (P)0;
        }
      }
#pragma unroll
      for (int u = 0; u < U; ++u)
#pragma unroll
        for (int i = 0; i < W; ++i) dot += a[u][i] * b[u][i];
    }
    size_t edge = (size_t)-1; /* offset of this lane's edge element inside the row */
    if (W > 1) {
      if (lane < g.head) edge = (size_t)lane;
      else if (lane - g.head < g.tail) edge = (size_t)g.head + (size_t)g.nvec * W + (lane - g.head);
      if (edge != (size_t)-1) dot += (P)yr[edge] * (P)gr[edge];
    }
    dot = group_allreduce<AddOP, G>(dot, slots[parity], lane);

    for (int p0 = lane; p0 < g.nvec; p0 += G * U) {
      P a[U][W], b[U][W];
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const int p = p0 + u * G;
        if (p < g.nvec) {
          load_pack_nt<T, W>(ybody + (size_t)p * W, a[u]);
          if constexpr (APART) load_pack_nt_loose<T, W>(gbody + (size_t)p * W, b[u]);
          else load_pack_nt<T, W>(gbody + (size_t)p * W, b[u]);
        }
      }
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const int p = p0 + u * G;
        if (p < g.nvec) {
          P out[W];
#pragma unroll
          for (int i = 0; i < W; ++i) out[i] = a[u][i] * (b[u][i] - dot);
          if constexpr (BLEND) {
            P old[W];
            if constexpr (APART) load_pack_loose<T, W>(dbody + (size_t)p * W, old);
            else load_pack<T, W>(dbody + (size_t)p * W, old);
#pragma unroll
            for (int i = 0; i < W; ++i) out[i] += alpha * old[i];
          }
          if constexpr (APART) store_pack_nt_loose<T, W>(dbody + (size_t)p * W, out);
          else store_pack_nt<T, W>(dbody + (size_t)p * W, out);
        }
      }
    }
    if (W > 1 && edge != (size_t)-1) {
      P out = (P)yr[edge] * ((P)gr[edge] - dot);
      if constexpr (BLEND) out += alpha * (P)dr[edge];
      dr[edge] = (T)out;
    }
  }
}

/* ------------------------------------------------------------------ cluster reverse */

/* The reverse of a long row, shared like the forward: each of C consecutive workgroups keeps its
 * chunk of y and dy in registers, publishes its part of dot(y, dy) as a stamped word, waits for the
 * others with the same bounded poll, and writes its chunk of dx: y and dy are read once. A
 * workgroup that stops waiting reads the whole row again for the dot product, which is why the
 * shared path is not taken when dx overwrites y or dy. */
/* packs of y and of dy per thread: kept in their storage type (four registers a pack whatever T
 * is) and widened where they are used, so a workgroup holds the same 64 KiB of each for r16, r32
 * and r64 within 64 registers a thread (62-64 used, no spills), which keeps two workgroups a CU.
 * Measured on r32, 2 / 3 / 4 / 5 / 6 / 8 packs (5 and more: one workgroup a CU):
 * [512, 151936] 190 / 171 / 163 / 188 / 190 / 179 us, [2048, 50257] 244 / 217 / 211 / 238 / 243 / 225 us. */
constexpr int CLUSTER_REV_NV = 4;

template <class T, int W, bool BLEND>
__global__ __launch_bounds__(CLUSTER_THREADS, 8) void softmax_rev_cluster(
    const T* y, const T* dy, T* dx, typename precision<T>::type alpha,
    share_word* callers_words, size_t region,
    size_t m, size_t n, int C, int packs_per_block, unsigned spin_limit) {
  using P = typename precision<T>::type;
  constexpr int G = CLUSTER_THREADS, NV = CLUSTER_REV_NV, WPS = share_parts<P>();
  using V = typename vec_of<T, W>::type;
  __shared__ P red[2][G / WAVE];
  __shared__ P bc[2];
  const int lane = threadIdx.x;
  const size_t row = blockIdx.x / (unsigned)C;
  const int rank = (int)(blockIdx.x % (unsigned)C);
  share_word* row_words = share_words(callers_words, region) + row * (size_t)C * WPS;
  const share_word peeked = C > 1 ? share_peek(row_words + (size_t)rank * WPS, lane) : 0; /* on its way while the chunk loads */
  const T* yr = y + row * n;
  const T* gr = dy + row * n;
  T* dr = dx + row * n;
  const RowGeom<T, W> g(yr, n, true);
  const T* ybody = yr + g.head;
  const T* gbody = gr + g.head;
  T* dbody = dr + g.head;
  const int lo = rank * packs_per_block - cluster_skew(ybody, C, packs_per_block, g.nvec);
  const int hi = lo + packs_per_block < g.nvec ? lo + packs_per_block : g.nvec;

  V a[NV], b[NV];
#pragma unroll
  for (int k = 0; k < NV; ++k) {
    const int p = lo + k * G + lane;
    if (p >= 0 && p < hi) {
      a[k] = __builtin_nontemporal_load(reinterpret_cast<const V*>(ybody + (size_t)p * W));
      b[k] = __builtin_nontemporal_load(reinterpret_cast<const V*>(gbody + (size_t)p * W));
    } else {
#pragma unroll
      for (int i = 0; i < W; ++i) a[k][i] = b[k][i] = (T)0;
    }
  }
  P ey = (P)0, eg = (P)0; /* rank 0 also holds the row's head / tail scalars */
  size_t edge_at = (size_t)-1;
  if (W > 1 && rank == 0) {
    if (lane < g.head) edge_at = (size_t)lane;
    else if (lane - g.head < g.tail) edge_at = (size_t)g.head + (size_t)g.nvec * W + (lane - g.head);
    if (edge_at != (size_t)-1) {
      ey = (P)yr[edge_at];
      eg = (P)gr[edge_at];
    }
  }

  P dot = ey * eg;
#pragma unroll
  for (int k = 0; k < NV; ++k) {
    if constexpr (sizeof(T) == 2) {
      /* v_dot2_f32_f16: two exact half products added to an fp32 sum, no widening of the chunk
       * (which would not fit the registers of two workgroups a CU) */
      typedef _Float16 half2_t __attribute__((ext_vector_type(2)));
#pragma unroll
      for (int i = 0; i < W; i += 2)
        dot = __builtin_amdgcn_fdot2(half2_t{a[k][i], a[k][i + 1]}, half2_t{b[k][i], b[k][i + 1]}, dot, false);
    } else {
#pragma unroll
      for (int i = 0; i < W; ++i) dot += (P)a[k][i] * (P)b[k][i];
    }
  }
  dot = group_allreduce<AddOP, G>(dot, red[0], lane);

  if (C > 1) {
    P sums[1] = {dot};
    const bool complete = share_exchange_sums<1>(row_words, C, rank, peeked, sums, spin_limit, bc, lane);
    dot = sums[0];
    if (!complete) { /* gave up waiting: the whole row's dot product here */
      P d = (P)0;
      for (int p = lane; p < g.nvec; p += G) {
        P u[W], v[W];
        load_pack<T, W>(ybody + (size_t)p * W, u);
        load_pack<T, W>(gbody + (size_t)p * W, v);
#pragma unroll
        for (int i = 0; i < W; ++i) d += u[i] * v[i];
      }
      if (W > 1) {
        size_t e = (size_t)-1;
        if (lane < g.head) e = (size_t)lane;
        else if (lane - g.head < g.tail) e = (size_t)g.head + (size_t)g.nvec * W + (lane - g.head);
        if (e != (size_t)-1) d += (P)yr[e] * (P)gr[e];
      }
      dot = group_allreduce<AddOP, G>(d, red[1], lane);
    }
  }

#pragma unroll
  for (int k = 0; k < NV; ++k) {
    const int p = lo + k * G + lane;
    if (p >= 0 && p < hi) {
      P out[W];
#pragma unroll
      for (int i = 0; i < W; ++i) out[i] = (P)a[k][i] * ((P)b[k][i] - dot);
      if constexpr (BLEND) {
        P old[W];
        load_pack<T, W>(dbody + (size_t)p * W, old);
#pragma unroll
        for (int i = 0; i < W; ++i) out[i] += alpha * old[i];
      }
      store_pack_nt<T, W>(dbody + (size_t)p * W, out);
    }
  }
  if (edge_at != (size_t)-1) {
    P out = ey * (eg - dot);
    if constexpr (BLEND) out += alpha * (P)dr[edge_at];
    dr[edge_at] = (T)out;
  }
}

/* ------------------------------------------------------------------ host dispatch */

inline unsigned stream_grid(size_t m) {
  const size_t cap = (size_t)compute_units() * 2; /* two 1024-thread workgroups fit a CU */
  return (unsigned)(m < cap ? m : cap);
}

/* Whether the short-row kernels take rows of n elements: up to four packs always, up to sixteen
 * when no pack is cut (n % W == 0, whatever the base alignments) and up to eight for two-byte
 * values; the other rows of five to sixteen packs that are not whole packs would leave lanes
 * idle next to a cut pack, and the 16-lane groups with head and tail lanes are faster there
 * (measured forward/reverse on [1M, 33] r32, nine packs: 3.5/4.2 TB/s there, 2.8/3.3 here; r32 n = 50: 4.6/4.6
 * there, 4.2/4.4 here; r16 n = 100, thirteen packs: 3.2/3.7 there, 3.2/3.0 here; but r16 n = 33, five packs:
 * 1.5/1.8 there, 2.2/2.1 here, and r16 n = 50: 2.0/2.3 there, 2.9/2.8 here). */
template <class T> inline bool softmax_short_rows(size_t n) {
  constexpr int W = PACK_BYTES / (int)sizeof(T);
  const size_t packs = (n + W - 1) / W;
  if (row_regime_override() != REGIME_AUTO || packs > (size_t)SHORT_MAX_PACKS) return false;
  return packs <= 4 || n % W == 0 || (sizeof(T) == 2 && packs <= 8);
}

template <class T>
inline void softmax_forward(const T* x, T* y, void* scratch, size_t m, size_t n, hipStream_t stream) {
  if (m == 0 || n == 0) return;
  using P = typename precision<T>::type;
  constexpr int W = PACK_BYTES / (int)sizeof(T);
  require(n <= 0x40000000ull, "softmax: row length must not exceed 2^30");
  if (softmax_short_rows<T>(n)) {
    for_short_row(n, W, [&]<int G, bool CUT>() {
      if (note_plan(PLAN_SHORT, G, 1, SHORT_THREADS / G, short_row_grid(m, G), SHORT_THREADS)) return;
      softmax_fwd_short<T, W, G, CUT><<<dim3(short_row_grid(m, G)), dim3(SHORT_THREADS), 0, stream>>>(
          x, y, m, (unsigned)n, short_rows_share_lines<T>(n, G));
    });
    MP_CHECK_LAUNCH();
    return;
  }
  if (misalign16(x) != misalign16(y)) { /* rows of x and y peel differently */
    constexpr int MAXNV = max_nv_for<T>(64);
    const bool resident = for_row_plan<MAXNV, true>(plan_row((n + W - 1) / W, MAXNV, 2, 16), [&]<int G, int NV>() {
      if (note_plan(PLAN_LOOSE, G, NV, G < WAVE ? WAVE / G : 1, row_grid(m, G), G < WAVE ? WAVE : G)) return;
      softmax_fwd_loose<T, W, G, NV><<<dim3(row_grid(m, G)), dim3(G < WAVE ? WAVE : G), 0, stream>>>(x, y, m, n);
    });
    if (!resident && !note_plan(PLAN_STREAM, STREAM_THREADS, 0, 1, stream_grid(m), STREAM_THREADS)) /* rows beyond the registers of a workgroup */
      softmax_fwd_stream<T, W, true><<<dim3(stream_grid(m)), dim3(STREAM_THREADS), 0, stream>>>(x, y, m, n);
    MP_CHECK_LAUNCH();
    return;
  }
  const size_t packs = (n + W - 1) / W;
  const int C = cluster_size<T>(packs);
  /* in place, a workgroup that gives up waiting would re-read chunks its partners already
   * overwrote: shared rows need distinct buffers */
  const bool shareable = scratch != nullptr && !ranges_overlap(x, y, m * n * sizeof(T));
  if (C >= 1 && (C == 1 || shareable) && m * (size_t)C < 0x7fffffffull) {
    const int ppb = cluster_chunk_packs(packs, C, (size_t)CLUSTER_THREADS * cluster_nv<T>(), CLUSTER_SKEW_MAX);
    require(ppb <= CLUSTER_THREADS * cluster_nv<T>(), "softmax: cluster chunk exceeds the register tile");
    /* the stamped words of the rows: a region of the library's own for this workspace and geometry,
     * or (none to be had) the caller's workspace, cleared first */
    constexpr int WPS = 2 * share_parts<P>();
    share_word* callers = nullptr;
    long long region = 0;
    /* what the launch may touch of the caller's workspace: the words, when the library has none of its own for it */
    if (note_plan(PLAN_CLUSTER, CLUSTER_THREADS, cluster_nv<T>(), 1, m * C, CLUSTER_THREADS, C, ppb,
                  C > 1 ? m * (size_t)C * WPS * sizeof(share_word) : 0, keep_output(m * n * sizeof(T))))
      return;
    if (C > 1) {
      region = share_region(scratch, m, C, WPS);
      if (region < 0) {
        callers = static_cast<share_word*>(scratch);
        region = 0;
        const size_t words = m * (size_t)C * WPS;
        cluster_zero_slots<share_word><<<dim3((unsigned)((words + 255) / 256)), dim3(256), 0, stream>>>(callers, words);
      }
    }
    if (keep_output(m * n * sizeof(T)))
      softmax_fwd_cluster<T, W, true><<<dim3((unsigned)(m * C)), dim3(CLUSTER_THREADS), 0, stream>>>(
          x, y, callers, (size_t)region, m, n, C, ppb, cluster_tuning().spin_limit);
    else
      softmax_fwd_cluster<T, W><<<dim3((unsigned)(m * C)), dim3(CLUSTER_THREADS), 0, stream>>>(
          x, y, callers, (size_t)region, m, n, C, ppb, cluster_tuning().spin_limit);
    MP_CHECK_LAUNCH();
    return;
  }
  const bool ragged = !(aligned16(x) && (n % W) == 0);
  constexpr int MAXNV = max_nv_for<T>(64);
  RowPlan plan = row_regime_override() == REGIME_CLUSTER ? RowPlan{0, 0} : plan_row(packs, MAXNV, 2, 16);
  /* r16 rows that leave a 1024-thread group at two packs a thread more than an eighth idle take
   * the tightest fit instead (n = 10240: 1024 x 2 -> 256 x 5, 5.44 -> 5.88 TB/s; n = 12288: 512 x 3,
   * 5.68 -> 6.13; interleaved repeats). Everywhere else the wide group with idle lanes is the
   * faster one: the same change loses 1-6 % on r32 rows, on r16 rows planned at other shapes and in
   * the reverse. */
  constexpr bool FIT = sizeof(T) == 2;
  if (FIT && plan.G == 1024 && plan.NV == 2) plan = plan_row_fit(packs, MAXNV < 8 ? MAXNV : 8, 2, 16);
  /* and r16 rows that fill a narrower group at two packs a thread to eleven sixteenths or less run
   * on half the group at four (interleaved repeats: n = 1280 128 x 2 -> 64 x 4 5.63 -> 5.96 TB/s, 2560
   * 256 x 2 -> 128 x 4 5.88 -> 6.11, 4608 5.51 -> 6.11, 5120 512 x 2 -> 256 x 4 5.71 -> 6.18, 5632 5.91 ->
   * 6.06; fuller rows equal) */
  else if (FIT && row_regime_override() == REGIME_AUTO && plan.NV == 2 && plan.G >= 128 && plan.G <= 512 && MAXNV >= 4 &&
           packs * 16 <= (size_t)plan.G * 2 * 11)
    plan = RowPlan{plan.G / 2, 4};
  const unsigned flags = rows_share_lines<T>(n);
  const bool keep = keep_output(m * n * sizeof(T));
  const bool resident = for_row_plan<MAXNV, true, FIT>(plan, [&]<int G, int NV>() {
    const dim3 grid(row_grid(m, G)), block(G < WAVE ? WAVE : G);
    if (note_plan(PLAN_RESIDENT, G, NV, G < WAVE ? WAVE / G : 1, grid.x, block.x, 1, 0, 0, keep && !ragged)) return;
    if (ragged) softmax_fwd_resident<T, W, G, NV, true><<<grid, block, 0, stream>>>(x, y, m, n, flags);
    else if (keep) softmax_fwd_resident<T, W, G, NV, false, true><<<grid, block, 0, stream>>>(x, y, m, n, flags);
    else softmax_fwd_resident<T, W, G, NV, false><<<grid, block, 0, stream>>>(x, y, m, n, flags);
  });
  if (!resident && !note_plan(PLAN_STREAM, STREAM_THREADS, 0, 1, stream_grid(m), STREAM_THREADS))
    softmax_fwd_stream<T, W><<<dim3(stream_grid(m)), dim3(STREAM_THREADS), 0, stream>>>(x, y, m, n);
  MP_CHECK_LAUNCH();
}

/* Workgroups per row when the reverse shares rows; 0 when it does not. */
template <class T> inline int cluster_rev_size(size_t packs) {
  const int regime = row_regime_override();
  if (regime != REGIME_AUTO && regime != REGIME_CLUSTER) return 0;
  if (regime == REGIME_AUTO && packs <= (size_t)CLUSTER_THREADS * 2) return 0; /* one workgroup, two packs each */
  /* r16 rows of exactly 64 KiB stay with one persistent workgroup at four packs a thread (interleaved
   * repeats, n = 32768: 5.48 -> 5.75 TB/s; 24576 ... 32000: 1 ... 7 % better shared) */
  if (regime == REGIME_AUTO && sizeof(T) == 2 && packs == 4096) return 0;
  constexpr size_t tile = (size_t)CLUSTER_THREADS * CLUSTER_REV_NV;
  size_t ppb = (size_t)cluster_tuning().packs_per_block;
  if (ppb == 0 || ppb > tile) ppb = tile;
  size_t c = (packs + ppb - 1) / ppb;
  /* rows of exactly 8192 packs: three workgroups a row, not two that start 64 KiB apart (interleaved
   * repeats: r32 n = 32768 5.61 -> 6.21 TB/s, r16 n = 65536 5.27 -> 5.99) */
  if (regime == REGIME_AUTO && cluster_tuning().packs_per_block == 0 && packs == 8192 && c == 2) c = 3;
  return c >= 1 && c <= (size_t)CLUSTER_MAX ? (int)c : 0;
}

template <class T> inline size_t softmax_reverse_scratch_bytes(size_t m, size_t n) {
  using P = typename precision<T>::type;
  constexpr int W = PACK_BYTES / (int)sizeof(T);
  const size_t c = cluster_size_for_scratch(cluster_rev_size<T>((n + W - 1) / W));
  return m * c * share_parts<P>() * sizeof(share_word); /* the part of the dot product as stamped words */
}

template <class T>
inline void softmax_reverse(const T* y, const T* dy, T* dx, void* scratch, double alpha, size_t m, size_t n,
                            hipStream_t stream) {
  if (m == 0 || n == 0) return;
  using P = typename precision<T>::type;
  constexpr int W = PACK_BYTES / (int)sizeof(T);
  require(n <= 0x40000000ull, "softmax reverse: row length must not exceed 2^30");
  const P al = (P)alpha;
  const bool blend = alpha != 0.0;
  if (softmax_short_rows<T>(n)) {
    for_short_row(n, W, [&]<int G, bool CUT>() {
      const dim3 grid(short_row_grid(m, G)), block(SHORT_THREADS);
      const unsigned by_xcd = short_rows_share_lines<T>(n, G);
      if (note_plan(PLAN_SHORT, G, 1, SHORT_THREADS / G, grid.x, block.x)) return;
      if (blend) softmax_rev_short<T, W, G, CUT, true><<<grid, block, 0, stream>>>(y, dy, dx, al, m, (unsigned)n, by_xcd);
      else softmax_rev_short<T, W, G, CUT, false><<<grid, block, 0, stream>>>(y, dy, dx, al, m, (unsigned)n, by_xcd);
    });
    MP_CHECK_LAUNCH();
    return;
  }
  if (misalign16(y) != misalign16(dy) || misalign16(y) != misalign16(dx)) { /* rows that peel differently */
    constexpr int MAXNV = max_nv_for<T>(32);
    const bool resident = for_row_plan<MAXNV, true>(plan_row((n + W - 1) / W, MAXNV, 2, 16), [&]<int G, int NV>() {
      const dim3 grid(row_grid(m, G)), block(G < WAVE ? WAVE : G);
      if (note_plan(PLAN_LOOSE, G, NV, G < WAVE ? WAVE / G : 1, grid.x, block.x)) return;
      if (blend) softmax_rev_loose<T, W, G, NV, true><<<grid, block, 0, stream>>>(y, dy, dx, al, m, n);
      else softmax_rev_loose<T, W, G, NV, false><<<grid, block, 0, stream>>>(y, dy, dx, al, m, n);
    });
    if (!resident && !note_plan(PLAN_STREAM, STREAM_THREADS, 0, 1, stream_grid(m), STREAM_THREADS)) { /* rows beyond the registers of a workgroup */
      const dim3 grid(stream_grid(m)), block(STREAM_THREADS);
      if (blend) softmax_rev_stream<T, W, true, true><<<grid, block, 0, stream>>>(y, dy, dx, al, m, n);
      else softmax_rev_stream<T, W, false, true><<<grid, block, 0, stream>>>(y, dy, dx, al, m, n);
    }
    MP_CHECK_LAUNCH();
    return;
  }
  const size_t packs = (n + W - 1) / W;
  const int C = cluster_rev_size<T>(packs);
  const bool distinct = !ranges_overlap(dx, y, m * n * sizeof(T)) && !ranges_overlap(dx, dy, m * n * sizeof(T));
  if (C >= 1 && (C == 1 || (scratch != nullptr && distinct)) && m * (size_t)C < 0x7fffffffull) {
    const int ppb = cluster_chunk_packs(packs, C, (size_t)CLUSTER_THREADS * CLUSTER_REV_NV, CLUSTER_SKEW_MAX);
    require(ppb <= CLUSTER_THREADS * CLUSTER_REV_NV, "softmax reverse: cluster chunk exceeds the register tile");
    constexpr int WPS = share_parts<P>();
    share_word* callers = nullptr;
    long long region = 0;
    if (note_plan(PLAN_CLUSTER, CLUSTER_THREADS, CLUSTER_REV_NV, 1, m * C, CLUSTER_THREADS, C, ppb,
                  C > 1 ? m * (size_t)C * WPS * sizeof(share_word) : 0))
      return;
    if (C > 1) { /* as in the forward: the library's own words for this workspace and geometry, else the caller's, cleared */
      region = share_region(scratch, m, C, WPS);
      if (region < 0) {
        callers = static_cast<share_word*>(scratch);
        region = 0;
        const size_t words = m * (size_t)C * WPS;
        cluster_zero_slots<share_word><<<dim3((unsigned)((words + 255) / 256)), dim3(256), 0, stream>>>(callers, words);
      }
    }
    const dim3 grid((unsigned)(m * C)), block(CLUSTER_THREADS);
    if (blend) softmax_rev_cluster<T, W, true><<<grid, block, 0, stream>>>(y, dy, dx, al, callers, (size_t)region, m, n, C, ppb, cluster_tuning().spin_limit);
    else softmax_rev_cluster<T, W, false><<<grid, block, 0, stream>>>(y, dy, dx, al, callers, (size_t)region, m, n, C, ppb, cluster_tuning().spin_limit);
    MP_CHECK_LAUNCH();
    return;
  }
  const bool ragged = !(aligned16(y) && (n % W) == 0);
  constexpr int MAXNV = max_nv_for<T>(32);
  /* two packs a thread up to 256 packs a row, one from 512 on (interleaved repeats: r32 n = 2048
   * 512 x 1 6.25 TB/s against 256 x 2 5.95, r16 n = 4096 6.37 against 6.15, n = 8192 6.40 against 6.27) */
  const bool one_pack = sizeof(T) == 2 ? (packs > 400 && packs <= 512) || packs > 768 : packs >= (sizeof(T) == 4 ? 129 : 512);
  /* a pack a thread from 512 packs a row on (r32: from 129; interleaved repeats against two packs on
   * half the group: n = 576 5.90 -> 6.23 TB/s, 832 5.67 -> 6.16, 1152 5.93 -> 6.25, 1408 5.89 -> 6.31, 1536
   * 5.93 -> 6.20); r16 rows of 513 ... 768 packs stay at two on 512 threads
   * rather than one on a 1024-thread group they fill to three quarters or less (interleaved repeats:
   * n = 4608 5.23 -> 6.06 TB/s, 5120 5.51 -> 6.16, 5632 5.82 -> 6.16, 6144 and 6656 equal), and r16 rows of
   * 401 ... 512 packs take one pack on 512 threads (against two on 256: n = 3584 6.02 -> 6.25, 3840 5.98 ->
   * 6.46, 4096 6.10 -> 6.33; 3328 equal, 3072 better at two) */
  const RowPlan plan = row_regime_override() == REGIME_CLUSTER ? RowPlan{0, 0} : plan_row(packs, MAXNV, one_pack ? 1 : 2, 16);
  const unsigned rev_flags = rows_share_lines<T>(n);
  const bool resident = for_row_plan<MAXNV, true>(plan, [&]<int G, int NV>() {
    const dim3 grid(row_grid(m, G)), block(G < WAVE ? WAVE : G);
    if (note_plan(PLAN_RESIDENT, G, NV, G < WAVE ? WAVE / G : 1, grid.x, block.x)) return;
    if (ragged) {
      if (blend) softmax_rev_resident<T, W, G, NV, true, true><<<grid, block, 0, stream>>>(y, dy, dx, al, m, n, rev_flags);
      else softmax_rev_resident<T, W, G, NV, true, false><<<grid, block, 0, stream>>>(y, dy, dx, al, m, n, rev_flags);
    } else {
      if (blend) softmax_rev_resident<T, W, G, NV, false, true><<<grid, block, 0, stream>>>(y, dy, dx, al, m, n, rev_flags);
      else softmax_rev_resident<T, W, G, NV, false, false><<<grid, block, 0, stream>>>(y, dy, dx, al, m, n, rev_flags);
    }
  });
  if (!resident && !note_plan(PLAN_STREAM, STREAM_THREADS, 0, 1, stream_grid(m), STREAM_THREADS)) {
    const dim3 grid(stream_grid(m)), block(STREAM_THREADS);
    if (blend) softmax_rev_stream<T, W, true><<<grid, block, 0, stream>>>(y, dy, dx, al, m, n);
    else softmax_rev_stream<T, W, false><<<grid, block, 0, stream>>>(y, dy, dx, al, m, n);
  }
  MP_CHECK_LAUNCH();
}

}  // namespace mp

#endif
#endif
