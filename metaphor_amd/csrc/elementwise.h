/*
 * Flat elementwise engine: NIN read streams, NOUT write streams, one fused functor.
 *
 * The reference runs one thread per element with 4-byte accesses and a 32x over-sized grid
 * (src/cuda/nvcc_src/addition.cu:3-14 with GRID_1D, src/cuda/kernel_header.h:100), and its
 * 32-bit thread index wraps at 2^28 elements. Here every lane moves UNROLL 128-bit packs per
 * stream, all loads are issued before the first use, indices are 64-bit, and the grid is
 * exactly ceil(packs / (64*UNROLL)) single-wave workgroups.
 *
 * Aliasing: the reference's callers pass an output that aliases an input (c == b in
 * src/ops/addition.zig:67-73). Each lane reads all of its elements before it writes any of
 * them and no two lanes share an element, so any output may alias any input exactly.
 */
#ifndef MP_ELEMENTWISE_H
#define MP_ELEMENTWISE_H

#include "kernel_header.h"

#if defined(__cplusplus) && defined(__HIPCC__)

namespace mp {

template <int NIN, int NOUT> struct EwPtrs {
  const void* in[NIN > 0 ? NIN : 1]; /* generators (fill, sequence) have no input stream */
  void* out[NOUT];
};

/* A functor that declares `static constexpr bool needs_index = true` is also handed the
 * element's flat index: apply(in, out, index). */
template <class F, class P, int NIN, int NOUT>
__device__ __forceinline__ void ew_apply(const F& f, const P (&a)[NIN > 0 ? NIN : 1], P (&r)[NOUT], size_t index) {
  if constexpr (requires { F::needs_index; }) f.apply(a, r, index);
  else f.apply(a, r);
}

/* One wavefront per workgroup and one pack per stream per lane measured fastest on MI355X for
 * pure streaming (larger workgroups or deeper unrolling lose 3-8 % of HBM bandwidth). */
constexpr int EW_BLOCK = 64;
/* Kernels that only write (fill, sequence) want 256-thread workgroups: 4.6 -> 6.5 TB/s measured;
 * everything that also reads is fastest with single-wave workgroups. */
template <int NIN> constexpr int ew_block() { return NIN == 0 ? 256 : EW_BLOCK; }

/* F::apply(const P (&in)[NIN], P (&out)[NOUT]) computes one element. */
template <class T, int W, int NIN, int NOUT, int UNROLL, class F>
__global__ __launch_bounds__(ew_block<NIN>()) void ew_kernel(EwPtrs<NIN, NOUT> ptrs, size_t n, F f) {
  using P = typename precision<T>::type;
  constexpr int NA = NIN > 0 ? NIN : 1, EW_BLOCK = ew_block<NIN>();
  const size_t npacks = n / W;
  const size_t base = (size_t)blockIdx.x * (EW_BLOCK * UNROLL) + threadIdx.x;

  P in[UNROLL][NA][W];
#pragma unroll
  for (int u = 0; u < UNROLL; ++u) {
    const size_t p = base + (size_t)u * EW_BLOCK;
    if (p < npacks) {
#pragma unroll
      for (int s = 0; s < NIN; ++s)
        load_pack_nt<T, W>(static_cast<const T*>(ptrs.in[s]) + p * W, in[u][s]);
    }
  }
#pragma unroll
  for (int u = 0; u < UNROLL; ++u) {
    const size_t p = base + (size_t)u * EW_BLOCK;
    if (p < npacks) {
      P out[NOUT][W];
#pragma unroll
      for (int i = 0; i < W; ++i) {
        P a[NA], r[NOUT];
#pragma unroll
        for (int s = 0; s < NIN; ++s) a[s] = in[u][s][i];
        ew_apply<F, P, NIN, NOUT>(f, a, r, p * W + i);
#pragma unroll
        for (int s = 0; s < NOUT; ++s) out[s][i] = r[s];
      }
#pragma unroll
      for (int s = 0; s < NOUT; ++s)
        store_pack_nt<T, W>(static_cast<T*>(ptrs.out[s]) + p * W, out[s]);
    }
  }

  /* the n % W elements after the last whole pack */
  if (W > 1 && blockIdx.x == 0) {
    const size_t e = npacks * W + threadIdx.x;
    if (e < n) {
      P a[NA], r[NOUT];
#pragma unroll
      for (int s = 0; s < NIN; ++s) a[s] = (P) static_cast<const T*>(ptrs.in[s])[e];
      ew_apply<F, P, NIN, NOUT>(f, a, r, e);
#pragma unroll
      for (int s = 0; s < NOUT; ++s) static_cast<T*>(ptrs.out[s])[e] = (T)r[s];
    }
  }
}

/* Enqueue f over n elements. Operands that are all 16-byte aligned take the packed path;
 * anything else takes the same kernel with one-element packs. n == 0 enqueues nothing. */
template <class T, int NIN, int NOUT, int UNROLL, class F>
inline void ew_launch(const EwPtrs<NIN, NOUT>& ptrs, size_t n, F f, hipStream_t stream) {
  if (n == 0) return;
  constexpr int EW_BLOCK = ew_block<NIN>();
  require(n / EW_BLOCK < 0x7fffffffull, "elementwise launch: too many elements for one grid");
  bool packed = true;
  for (int s = 0; s < NIN; ++s) packed = packed && aligned16(ptrs.in[s]);
  for (int s = 0; s < NOUT; ++s) packed = packed && aligned16(ptrs.out[s]);
  constexpr int W = PACK_BYTES / (int)sizeof(T);
  if (packed) {
    const size_t npacks = n / W;
    const size_t per_block = (size_t)EW_BLOCK * UNROLL;
    size_t blocks = (npacks + per_block - 1) / per_block;
    if (blocks == 0) blocks = 1; /* only a scalar tail */
    ew_kernel<T, W, NIN, NOUT, UNROLL, F><<<dim3((unsigned)blocks), dim3(EW_BLOCK), 0, stream>>>(ptrs, n, f);
  } else {
    const size_t per_block = (size_t)EW_BLOCK * UNROLL;
    const size_t blocks = (n + per_block - 1) / per_block;
    ew_kernel<T, 1, NIN, NOUT, UNROLL, F><<<dim3((unsigned)blocks), dim3(EW_BLOCK), 0, stream>>>(ptrs, n, f);
  }
  MP_CHECK_LAUNCH();
}

}  // namespace mp

#endif
#endif
