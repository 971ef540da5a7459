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

/* How the operands of a launch lie in memory: all at the same place, other than its start, of a
 * 128-byte cache line, so that after the first `head` elements every
 * wavefront's kilobyte starts on a line again (a kilobyte that straddles lines costs 15 %,
 * whether its packs are 16-byte aligned or not: r32 with all operands shifted by one element 5.4
 * against 6.4 TB/s); all 16-byte aligned; or anything else, and the packs then start at any element (see loose_vec_of),
 * which costs a streaming kernel 5-15 % where one-element accesses cost half (r32) or three
 * quarters (r16) of the bandwidth. */
enum EwLayout { EW_ALIGNED, EW_PEELED, EW_LOOSE, EW_KEPT };
/* EW_KEPT is EW_ALIGNED with ordinary loads in place of non-temporal ones: the inputs stay in the
 * memory-side cache (256 MiB in front of the HBM stacks), where the reverse of the same expression,
 * which reads every input of its forward again (four of its nine streams for
 * selu(hadamard(add, add))), finds them. launch_fused_selu_hadamard_add_add_r32 and its reverse in
 * turn on operands that nothing touched for five steps, against the same with every operand one
 * element further (the peeled layout, whose loads stream): 8 MiB a tensor 23.3 -> 18.9 us a step,
 * 32 MiB 82.1 -> 74.1, 64 MiB 159.7 -> 145.3; the forward on its own pays for it from 16 MiB a
 * tensor up (32 MiB: 28.2 -> 30.8 us, 64 MiB: 55.6 -> 59.2) and gains below (8 MiB: 8.5 -> 7.8).
 * Taken by the forward launchers of fused chains whose inputs together are no larger than the
 * cache. */
constexpr size_t EW_KEEP_BYTES = 256u << 20;

/* F::apply(const P (&in)[NIN], P (&out)[NOUT]) computes one element. head: the elements before the
 * first pack (EW_PEELED only, less than a cache line of them). */
template <class T, int W, int LAYOUT, int NIN, int NOUT, int UNROLL, class F>
__device__ __forceinline__ void ew_body(const EwPtrs<NIN, NOUT>& ptrs, size_t n, unsigned head_arg, const F& f) {
  using P = typename precision<T>::type;
  constexpr int NA = NIN > 0 ? NIN : 1, EW_BLOCK = ew_block<NIN>();
  constexpr bool LOOSE = LAYOUT == EW_LOOSE, KEPT = LAYOUT == EW_KEPT;
  const size_t head = LAYOUT == EW_PEELED ? head_arg : 0;
  const size_t npacks = (n - head) / W;
  const size_t base = (size_t)blockIdx.x * (EW_BLOCK * UNROLL) + threadIdx.x;

  P in[UNROLL][NA][W];
#pragma unroll
  for (int u = 0; u < UNROLL; ++u) {
    const size_t p = base + (size_t)u * EW_BLOCK;
    if (p < npacks) {
#pragma unroll
      for (int s = 0; s < NIN; ++s) {
        if constexpr (LOOSE) load_pack_nt_loose<T, W>(static_cast<const T*>(ptrs.in[s]) + head + p * W, in[u][s]);
        else if constexpr (KEPT) load_pack<T, W>(static_cast<const T*>(ptrs.in[s]) + head + p * W, in[u][s]);
        else load_pack_nt<T, W>(static_cast<const T*>(ptrs.in[s]) + head + p * W, in[u][s]);
      }
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
        ew_apply<F, P, NIN, NOUT>(f, a, r, head + p * W + i);
#pragma unroll
        for (int s = 0; s < NOUT; ++s) out[s][i] = r[s];
      }
#pragma unroll
      for (int s = 0; s < NOUT; ++s) {
        if constexpr (LOOSE) store_pack_nt_loose<T, W>(static_cast<T*>(ptrs.out[s]) + head + p * W, out[s]);
        else store_pack_nt<T, W>(static_cast<T*>(ptrs.out[s]) + head + p * W, out[s]);
      }
    }
  }

  /* the elements before the first pack and after the last whole one */
  if (W > 1 && blockIdx.x == 0) {
    auto single = [&](size_t e) {
      P a[NA], r[NOUT];
#pragma unroll
      for (int s = 0; s < NIN; ++s) a[s] = (P) static_cast<const T*>(ptrs.in[s])[e];
      ew_apply<F, P, NIN, NOUT>(f, a, r, e);
#pragma unroll
      for (int s = 0; s < NOUT; ++s) static_cast<T*>(ptrs.out[s])[e] = (T)r[s];
    };
    const size_t after = head + npacks * W + threadIdx.x;
    if (after < n) single(after);
    if constexpr (LAYOUT == EW_PEELED)
      if (threadIdx.x < head) single(threadIdx.x); /* head < 128 / sizeof(T) <= 64 threads */
  }
}

template <class T, int W, int LAYOUT, int NIN, int NOUT, int UNROLL, class F>
__global__ __launch_bounds__(ew_block<NIN>()) void ew_kernel(EwPtrs<NIN, NOUT> ptrs, size_t n, unsigned head_arg, F f) {
  ew_body<T, W, LAYOUT, NIN, NOUT, UNROLL, F>(ptrs, n, head_arg, f);
}

/* How a launch over n elements is laid out: which kernel variant, how many elements come before
 * the first pack, how many workgroups. The one place that decides it, for the launchers compiled
 * into the library and for chains compiled at run time alike. */
struct EwPlan {
  int layout;
  unsigned head;
  unsigned blocks;
};
#ifdef MP_HOST_SIDE
inline EwPlan ew_plan(const void* const* in, int nin, void* const* out, int nout, size_t n, size_t elem_bytes,
                      int block_threads, int unroll, bool keepable = false) {
  const int W = PACK_BYTES / (int)elem_bytes;
  /* the place in a cache line that the operands share, or ~0u when they differ */
  auto in_line = [](const void* p) { return (unsigned)(reinterpret_cast<uintptr_t>(p) & 127u); };
  unsigned mis = nin > 0 ? in_line(in[0]) : in_line(out[0]);
  bool packed = true;
  for (int s = 0; s < nin; ++s) {
    mis = in_line(in[s]) == mis ? mis : ~0u;
    packed = packed && aligned16(in[s]);
  }
  for (int s = 0; s < nout; ++s) {
    mis = in_line(out[s]) == mis ? mis : ~0u;
    packed = packed && aligned16(out[s]);
  }
  const bool peel = mis != 0 && mis != ~0u && mis % elem_bytes == 0 && n >= (size_t)(128 / elem_bytes) + W;
  const unsigned head = peel ? (unsigned)((128 - mis) / elem_bytes) : 0;
  const size_t npacks = (n - head) / W;
  const size_t per_block = (size_t)block_threads * unroll;
  size_t blocks = (npacks + per_block - 1) / per_block;
  if (blocks == 0) blocks = 1; /* only single elements */
  const bool keep = keepable && !peel && packed && (size_t)nin * n * elem_bytes <= EW_KEEP_BYTES;
  return EwPlan{peel ? EW_PEELED : keep ? EW_KEPT : packed ? EW_ALIGNED : EW_LOOSE, head, (unsigned)blocks};
}

/* Enqueue f over n elements: one pack per stream per lane, laid out as EwLayout says.
 * n == 0 enqueues nothing. KEEPABLE: the launch is the forward of an expression whose reverse reads
 * its inputs again (see EW_KEPT). */
template <class T, int NIN, int NOUT, int UNROLL, bool KEEPABLE, class F>
inline void ew_launch_as(const EwPtrs<NIN, NOUT>& ptrs, size_t n, F f, hipStream_t stream) {
  if (n == 0) return;
  constexpr int EW_BLOCK = ew_block<NIN>();
  require(n / EW_BLOCK < 0x7fffffffull, "elementwise launch: too many elements for one grid");
  constexpr int W = PACK_BYTES / (int)sizeof(T);
  static_assert(128 / sizeof(T) <= 64, "the first workgroup's threads cover the head");
  const EwPlan plan = ew_plan(ptrs.in, NIN, ptrs.out, NOUT, n, sizeof(T), EW_BLOCK, UNROLL, KEEPABLE);
  const unsigned head = plan.head;
  const dim3 grid(plan.blocks), block(EW_BLOCK);
  if (plan.layout == EW_PEELED) ew_kernel<T, W, EW_PEELED, NIN, NOUT, UNROLL, F><<<grid, block, 0, stream>>>(ptrs, n, head, f);
  else if (plan.layout == EW_ALIGNED) ew_kernel<T, W, EW_ALIGNED, NIN, NOUT, UNROLL, F><<<grid, block, 0, stream>>>(ptrs, n, 0u, f);
  else if (plan.layout == EW_LOOSE) ew_kernel<T, W, EW_LOOSE, NIN, NOUT, UNROLL, F><<<grid, block, 0, stream>>>(ptrs, n, 0u, f);
  else if constexpr (KEEPABLE) ew_kernel<T, W, EW_KEPT, NIN, NOUT, UNROLL, F><<<grid, block, 0, stream>>>(ptrs, n, 0u, f);
  MP_CHECK_LAUNCH();
}
template <class T, int NIN, int NOUT, int UNROLL, class F>
inline void ew_launch(const EwPtrs<NIN, NOUT>& ptrs, size_t n, F f, hipStream_t stream) {
  ew_launch_as<T, NIN, NOUT, UNROLL, false, F>(ptrs, n, f, stream);
}
template <class T, int NIN, int NOUT, int UNROLL, class F>
inline void ew_launch_forward(const EwPtrs<NIN, NOUT>& ptrs, size_t n, F f, hipStream_t stream) {
  ew_launch_as<T, NIN, NOUT, UNROLL, true, F>(ptrs, n, f, stream);
}
#endif /* MP_HOST_SIDE */

}  // namespace mp

#endif
#endif
