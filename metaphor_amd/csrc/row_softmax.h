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
 * registers. Streaming kernels cover rows too long for registers with one online max/sum pass
 * (running maximum, running sum rescaled whenever the maximum moves) and one write pass.
 */
#ifndef MP_ROW_SOFTMAX_H
#define MP_ROW_SOFTMAX_H

#include "row_dispatch.h"

#if defined(__cplusplus) && defined(__HIPCC__)

namespace mp {

/* ------------------------------------------------------------------ resident forward */

template <class T, int W, int G, int NV, bool RAGGED>
__global__ __launch_bounds__(G) void softmax_fwd_resident(
    const T* x, T* y, size_t m, size_t n) {
  using P = typename precision<T>::type;
  __shared__ P slots[2][G / WAVE];

  const int lane = threadIdx.x; /* one row per workgroup of G threads */
  const size_t row = blockIdx.x;

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

  const P inv = (P)1 / s;
  t.each([&](P& e) { e *= inv; });
  t.store(y + row * n, g, lane);
}

/* ------------------------------------------------------------------ resident reverse */

template <class T, int W, int G, int NV, bool RAGGED, bool BLEND>
__global__ __launch_bounds__(G) void softmax_rev_resident(
    const T* y, const T* dy, T* dx, typename precision<T>::type alpha, size_t m, size_t n) {
  using P = typename precision<T>::type;
  __shared__ P slots[G / WAVE];

  const int lane = threadIdx.x;
  const size_t row = blockIdx.x;

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

/* ------------------------------------------------------------------ streaming forward */

/* Folds one value into a lane's running (max, sum of exp(x - max)). */
template <class P> __device__ __forceinline__ void online_rescale(P& run_max, P& run_sum, P chunk_max) {
  const P nm = chunk_max > run_max ? chunk_max : run_max;
  if (nm > run_max) { /* also taken on the first finite value: exp(-inf - nm) = 0 */
    run_sum *= exp_shifted(run_max, shift_of(nm));
    run_max = nm;
  }
}

template <class T, int W>
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
    P run_max = neg_inf<P>(), run_sum = (P)0;
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

    const P mx = group_allreduce<MaxOP, G>(run_max, slots[parity][0], lane);
    const P sh = shift_of(mx);
    const P scaled = run_max > neg_inf<P>() ? run_sum * exp_shifted(run_max, sh) : (P)0;
    const P s = group_allreduce<AddOP, G>(scaled, slots[parity][1], lane);
    const P inv = (P)1 / s;

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
          store_pack_nt<T, W>(ybody + (size_t)p * W, buf[u]);
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

/* ------------------------------------------------------------------ streaming reverse */

template <class T, int W, bool BLEND>
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
          load_pack<T, W>(gbody + (size_t)p * W, b[u]);
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
          load_pack_nt<T, W>(gbody + (size_t)p * W, b[u]);
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
            load_pack<T, W>(dbody + (size_t)p * W, old);
#pragma unroll
            for (int i = 0; i < W; ++i) out[i] += alpha * old[i];
          }
          store_pack_nt<T, W>(dbody + (size_t)p * W, out);
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

/* ------------------------------------------------------------------ host dispatch */

inline unsigned stream_grid(size_t m) {
  const size_t cap = (size_t)compute_units() * 2; /* two 1024-thread workgroups fit a CU */
  return (unsigned)(m < cap ? m : cap);
}

template <class T>
inline void softmax_forward(const T* x, T* y, size_t m, size_t n, hipStream_t stream) {
  if (m == 0 || n == 0) return;
  constexpr int W = PACK_BYTES / (int)sizeof(T);
  require(n <= 0x40000000ull, "softmax: row length must not exceed 2^30");
  if (misalign16(x) != misalign16(y)) { /* rows of x and y peel differently: element-wise */
    softmax_fwd_stream<T, 1><<<dim3(stream_grid(m)), dim3(STREAM_THREADS), 0, stream>>>(x, y, m, n);
    MP_CHECK_LAUNCH();
    return;
  }
  const bool ragged = !(aligned16(x) && (n % W) == 0);
  constexpr int MAXNV = max_nv_for<T>(64);
  const RowPlan plan = plan_row((n + W - 1) / W, MAXNV, 2);
  const bool resident = for_row_plan<MAXNV>(plan, [&]<int G, int NV>() {
    const dim3 grid(row_grid(m)), block(G);
    if (ragged) softmax_fwd_resident<T, W, G, NV, true><<<grid, block, 0, stream>>>(x, y, m, n);
    else softmax_fwd_resident<T, W, G, NV, false><<<grid, block, 0, stream>>>(x, y, m, n);
  });
  if (!resident)
    softmax_fwd_stream<T, W><<<dim3(stream_grid(m)), dim3(STREAM_THREADS), 0, stream>>>(x, y, m, n);
  MP_CHECK_LAUNCH();
}

template <class T>
inline void softmax_reverse(const T* y, const T* dy, T* dx, double alpha, size_t m, size_t n,
                            hipStream_t stream) {
  if (m == 0 || n == 0) return;
  using P = typename precision<T>::type;
  constexpr int W = PACK_BYTES / (int)sizeof(T);
  require(n <= 0x40000000ull, "softmax reverse: row length must not exceed 2^30");
  const P al = (P)alpha;
  const bool blend = alpha != 0.0;
  if (misalign16(y) != misalign16(dy) || misalign16(y) != misalign16(dx)) {
    const dim3 grid(stream_grid(m)), block(STREAM_THREADS);
    if (blend) softmax_rev_stream<T, 1, true><<<grid, block, 0, stream>>>(y, dy, dx, al, m, n);
    else softmax_rev_stream<T, 1, false><<<grid, block, 0, stream>>>(y, dy, dx, al, m, n);
    MP_CHECK_LAUNCH();
    return;
  }
  const bool ragged = !(aligned16(y) && (n % W) == 0);
  constexpr int MAXNV = max_nv_for<T>(32);
  const RowPlan plan = plan_row((n + W - 1) / W, MAXNV, 2);
  const bool resident = for_row_plan<MAXNV>(plan, [&]<int G, int NV>() {
    const dim3 grid(row_grid(m)), block(G);
    if (ragged) {
      if (blend) softmax_rev_resident<T, W, G, NV, true, true><<<grid, block, 0, stream>>>(y, dy, dx, al, m, n);
      else softmax_rev_resident<T, W, G, NV, true, false><<<grid, block, 0, stream>>>(y, dy, dx, al, m, n);
    } else {
      if (blend) softmax_rev_resident<T, W, G, NV, false, true><<<grid, block, 0, stream>>>(y, dy, dx, al, m, n);
      else softmax_rev_resident<T, W, G, NV, false, false><<<grid, block, 0, stream>>>(y, dy, dx, al, m, n);
    }
  });
  if (!resident) {
    const dim3 grid(stream_grid(m)), block(STREAM_THREADS);
    if (blend) softmax_rev_stream<T, W, true><<<grid, block, 0, stream>>>(y, dy, dx, al, m, n);
    else softmax_rev_stream<T, W, false><<<grid, block, 0, stream>>>(y, dy, dx, al, m, n);
  }
  MP_CHECK_LAUNCH();
}

}  // namespace mp

#endif
#endif
