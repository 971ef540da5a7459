/*
 * Shared device header of the gfx950 kernel library.
 *
 * Takes the place of the reference's src/cuda/kernel_header.h:1-267 for the HIP build:
 * the same roles (StreamContext access, error macros, DIMPAD, the up-cast `precision<T>`
 * rule of src/cuda/tensor_types.h:51-69, reduction helpers), re-designed for CDNA4:
 *   - wavefronts are 64 lanes; all-reduce is a DPP butterfly inside each 16-lane row
 *     followed by v_permlane16_swap / v_permlane32_swap across rows, no LDS traffic
 *     (the reference's warpReduce is a 32-lane __shfl_xor_sync loop, kernel_header.h:201-209);
 *   - workgroup reductions publish one value per wave in LDS and every thread folds them
 *     (the reference's blockReduce folds serially on thread 0, kernel_header.h:211-236);
 *   - every global access of the tuned paths is one 128-bit pack per lane.
 *
 * Kernel sources are written against the placeholder type `Scalar`; the generator
 * replicates each source for r16, r32 and r64 (reference: file_gen.zig:38,228-238).
 */
#ifndef MP_KERNEL_HEADER_H
#define MP_KERNEL_HEADER_H

#include "tensor_types.h"

/* placeholder for editors; the generator rewrites every `Scalar` token before compiling */
#define Scalar float

#define DIMPAD(M, N) (((M) + ((N) - 1)) / (N))

#if defined(__cplusplus) && defined(__HIPCC__)

/* A source compiled at run time (hiprtc defines __HIPCC_RTC__ and brings the device runtime with
 * it) sees the device side of this header only: no library headers exist there, and nothing of
 * the host side is needed. */
#ifndef __HIPCC_RTC__
#define MP_HOST_SIDE 1
#include <hip/hip_runtime.h>
#include <cmath>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#endif

#ifdef MP_HOST_SIDE
inline hipStream_t get_stream(StreamContext context) {
  return static_cast<hipStream_t>(context.hip_stream.ptr);
}

#define HIP_ASSERT(err) (mpHandleHipError((err), __FILE__, __LINE__))
inline void mpHandleHipError(hipError_t err, const char* file, int line) {
  if (err != hipSuccess) {
    fprintf(stderr, "%s in %s at line %d\n", hipGetErrorString(err), file, line);
    exit(EXIT_FAILURE);
  }
}

#ifdef MP_DIAGNOSTICS
/* Test build only: what a row launcher decided, recorded instead of launched. With `dry` set a
 * launcher runs its whole dispatch (with `cus` in place of the GPU's compute-unit count), notes the
 * kernel it would enqueue and returns before the launch, so the dispatch can be swept on a machine
 * without a GPU. kind: 0 short rows, 1 resident, 2 rows in pairs, 3 wavefront groups, 4 shared rows,
 * 5 shared rows pipelined, 6 two passes, 7 rows that peel differently. */
struct MpPlanNote {
  long long kind, group, packs_per_thread, rows_per_block, grid, block, cluster, chunk_packs, workspace_bytes;
  long long kept; /* 1: the forward's variant that leaves a tensor in the memory-side cache */
};
struct MpPlanProbe {
  bool dry = false, noted = false;
  int cus = 0;
  MpPlanNote note{};
};
inline MpPlanProbe& mp_plan_probe() {
  static thread_local MpPlanProbe probe;
  return probe;
}
/* a launch that the runtime rejects (bad grid, missing code object) must not pass silently */
#define MP_CHECK_LAUNCH() do { if (!mp_plan_probe().dry) HIP_ASSERT(hipGetLastError()); } while (0)
#else
/* a launch that the runtime rejects (bad grid, missing code object) must not pass silently */
#define MP_CHECK_LAUNCH() HIP_ASSERT(hipGetLastError())
#endif
#endif /* MP_HOST_SIDE */

namespace mp {

#ifdef MP_HOST_SIDE
/* argument checks of the launchers: same print-and-exit convention as a HIP error */
inline void require(bool ok, const char* what) {
  if (!ok) {
    fprintf(stderr, "metaphor kernels: %s\n", what);
    exit(EXIT_FAILURE);
  }
}
#endif

constexpr int WAVE = MP_WAVE_SIZE;
constexpr int PACK_BYTES = 16;

/* ---------------------------------------------------------------------------------------
 * numeric conventions
 * ------------------------------------------------------------------------------------- */

template <class T> struct precision { using type = float; };          /* r16, r32 -> fp32 */
template <> struct precision<double> { using type = double; };        /* r64 -> fp64 */

template <class T> constexpr int pack_width() { return PACK_BYTES / (int)sizeof(T); }

template <class P> __device__ __forceinline__ P neg_inf();
template <> __device__ __forceinline__ float neg_inf<float>() { return -__builtin_inff(); }
template <> __device__ __forceinline__ double neg_inf<double>() { return -__builtin_inf(); }

/* e^x. fp32: one v_exp_f32 on x*log2(e); fp64: library exp. */
__device__ __forceinline__ float fast_exp(float x) {
  return __builtin_amdgcn_exp2f(x * 1.44269504088896340736f);
}
__device__ __forceinline__ double fast_exp(double x) { return ::exp(x); }

/* e^(x - m) with one fused multiply-add in fp32: exp2(x*log2e - m*log2e). The rounding of
 * m*log2e is common to every element of a row, so it cancels in a normalised softmax. */
__device__ __forceinline__ float exp_shifted(float x, float m_log2e) {
  return __builtin_amdgcn_exp2f(__builtin_fmaf(x, 1.44269504088896340736f, -m_log2e));
}
__device__ __forceinline__ float shift_of(float m) { return m * 1.44269504088896340736f; }
__device__ __forceinline__ double exp_shifted(double x, double m) { return ::exp(x - m); }
__device__ __forceinline__ double shift_of(double m) { return m; }

/* 1 / sqrt(x) from the hardware's reciprocal square root (good to one ulp) instead of an IEEE
 * square root and an IEEE division, some forty instructions that every lane of a row would spend
 * on the same number. The instruction reads denormal arguments as zero: tiny ones are scaled
 * into range first (x = 0 still gives +inf). */
__device__ __forceinline__ float rsqrt_of(float x) {
  const bool tiny = x < 0x1p-100f;
  const float r = __builtin_amdgcn_rsqf(tiny ? x * 0x1p+100f : x);
  return tiny ? r * 0x1p+50f : r;
}
__device__ __forceinline__ double rsqrt_of(double x) { return 1.0 / ::sqrt(x); }

/* 1 / x for a row's sum (x >= 1 for a softmax row that has a finite element; 0 gives +inf as the
 * division does): the hardware's reciprocal, good to one ulp, instead of the ten instructions of
 * an IEEE division that every lane of the row would spend on the same number. */
__device__ __forceinline__ float reciprocal_of(float x) { return __builtin_amdgcn_rcpf(x); }
__device__ __forceinline__ double reciprocal_of(double x) { return 1.0 / x; }

/* e^x - 1 for x <= 0, accurate near 0: an 8-term series inside (-0.25, 0], exp-1 below. */
__device__ __forceinline__ float expm1_nonpos(float x) {
  float p = 1.0f / 40320.0f;
  p = __builtin_fmaf(p, x, 1.0f / 5040.0f);
  p = __builtin_fmaf(p, x, 1.0f / 720.0f);
  p = __builtin_fmaf(p, x, 1.0f / 120.0f);
  p = __builtin_fmaf(p, x, 1.0f / 24.0f);
  p = __builtin_fmaf(p, x, 1.0f / 6.0f);
  p = __builtin_fmaf(p, x, 0.5f);
  p = __builtin_fmaf(p * x, x, x);
  const float big = fast_exp(x) - 1.0f;
  return x > -0.25f ? p : big;
}
__device__ __forceinline__ double expm1_nonpos(double x) { return ::expm1(x); }

template <class P> __device__ __forceinline__ P selu_value(P x) {
  const P lam = (P)MP_SELU_SCALE, la = (P)(MP_SELU_SCALE * MP_SELU_ALPHA);
  const P neg = la * expm1_nonpos(x > (P)0 ? (P)0 : x);
  return x > (P)0 ? lam * x : neg;
}
template <class P> __device__ __forceinline__ P selu_slope(P x) {
  const P lam = (P)MP_SELU_SCALE, la = (P)(MP_SELU_SCALE * MP_SELU_ALPHA);
  const P neg = la * fast_exp(x > (P)0 ? (P)0 : x);
  return x > (P)0 ? lam : neg;
}

/* relu with the reference's convention: zero counts as positive (src/cuda/nvcc_src/relu.cu:12,
 * relu_reverse.cu:14) */
template <class P> __device__ __forceinline__ P relu_value(P x) { return x >= (P)0 ? x : (P)0; }
template <class P> __device__ __forceinline__ P relu_slope(P x) { return x >= (P)0 ? (P)1 : (P)0; }

/* ---------------------------------------------------------------------------------------
 * 128-bit packs
 * ------------------------------------------------------------------------------------- */

template <class T, int W> struct vec_of { typedef T type __attribute__((ext_vector_type(W))); };
/* The same pack behind a pointer that is only element-aligned. The hardware moves a misaligned
 * 128-bit global access as one instruction; measured on the MI355X with a 1 GiB copy, loads shifted
 * by 2 ... 14 bytes run at the aligned rate (6.2 TB/s) and shifted stores at 5.9. LDS accesses of
 * this type are split by the compiler. */
template <class T, int W> struct loose_vec_of { typedef T type __attribute__((ext_vector_type(W), aligned(sizeof(T)))); };

/* Load W consecutive elements (one pack when W > 1; p must be 16-byte aligned then). */
template <class T, int W, class P>
__device__ __forceinline__ void load_pack(const T* p, P (&out)[W]) {
  if constexpr (W == 1) {
    out[0] = (P)p[0];
  } else {
    using V = typename vec_of<T, W>::type;
    const V v = *reinterpret_cast<const V*>(p);
#pragma unroll
    for (int i = 0; i < W; ++i) out[i] = (P)v[i];
  }
}

/* Streaming variant: the data is not needed again by this kernel. */
template <class T, int W, class P>
__device__ __forceinline__ void load_pack_nt(const T* p, P (&out)[W]) {
  if constexpr (W == 1) {
    out[0] = (P)__builtin_nontemporal_load(p);
  } else {
    using V = typename vec_of<T, W>::type;
    const V v = __builtin_nontemporal_load(reinterpret_cast<const V*>(p));
#pragma unroll
    for (int i = 0; i < W; ++i) out[i] = (P)v[i];
  }
}

template <class T, int W, class P>
__device__ __forceinline__ void store_pack(T* p, const P (&in)[W]) {
  if constexpr (W == 1) {
    p[0] = (T)in[0];
  } else {
    using V = typename vec_of<T, W>::type;
    V v;
#pragma unroll
    for (int i = 0; i < W; ++i) v[i] = (T)in[i];
    *reinterpret_cast<V*>(p) = v;
  }
}

/* Write-once output: non-temporal so it does not evict what is still to be read. */
template <class T, int W, class P>
__device__ __forceinline__ void store_pack_nt(T* p, const P (&in)[W]) {
  if constexpr (W == 1) {
    __builtin_nontemporal_store((T)in[0], p);
  } else {
    using V = typename vec_of<T, W>::type;
    V v;
#pragma unroll
    for (int i = 0; i < W; ++i) v[i] = (T)in[i];
    __builtin_nontemporal_store(v, reinterpret_cast<V*>(p));
  }
}

/* An output that another kernel reads again soon (a forward's result, read by its reverse): an
 * ordinary store leaves it in the memory-side cache, a non-temporal one does not. A template
 * parameter and not a branch: the compiler merges two stores that differ in the hint alone, and
 * drops the hint. */
template <bool KEEP, class T, int W, class P>
__device__ __forceinline__ void store_pack_kept(T* p, const P (&in)[W]) {
  if constexpr (KEEP) store_pack<T, W>(p, in);
  else store_pack_nt<T, W>(p, in);
}

/* The four accessors above for packs that start at any element (see loose_vec_of). */
template <class T, int W, class P>
__device__ __forceinline__ void load_pack_loose(const T* p, P (&out)[W]) {
  const typename vec_of<T, W>::type v = *reinterpret_cast<const typename loose_vec_of<T, W>::type*>(p);
#pragma unroll
  for (int i = 0; i < W; ++i) out[i] = (P)v[i];
}
template <class T, int W, class P>
__device__ __forceinline__ void load_pack_nt_loose(const T* p, P (&out)[W]) {
  const typename vec_of<T, W>::type v =
      __builtin_nontemporal_load(reinterpret_cast<const typename loose_vec_of<T, W>::type*>(p));
#pragma unroll
  for (int i = 0; i < W; ++i) out[i] = (P)v[i];
}
template <class T, int W, class P>
__device__ __forceinline__ void store_pack_loose(T* p, const P (&in)[W]) {
  typename vec_of<T, W>::type v;
#pragma unroll
  for (int i = 0; i < W; ++i) v[i] = (T)in[i];
  *reinterpret_cast<typename loose_vec_of<T, W>::type*>(p) = v;
}
template <class T, int W, class P>
__device__ __forceinline__ void store_pack_nt_loose(T* p, const P (&in)[W]) {
  typename vec_of<T, W>::type v;
#pragma unroll
  for (int i = 0; i < W; ++i) v[i] = (T)in[i];
  __builtin_nontemporal_store(v, reinterpret_cast<typename loose_vec_of<T, W>::type*>(p));
}

/* The first c < W elements of a pack that starts at any element, moved as pieces of W/2, W/4 ... 1
 * elements picked by the bits of c: the end of a row that is not a whole number of packs long,
 * without touching the row behind it. c = n % W is the same for every row, so the branches are
 * uniform. The load leaves the elements from c on as they are. */
template <class T, int W, int OFF, int N, class P>
__device__ __forceinline__ void load_cut_pack_from(const T* p, P (&out)[W], unsigned c) {
  if constexpr (N >= 1) {
    if (c & N) {
      if constexpr (N == 1) {
        out[OFF] = (P)p[OFF];
      } else {
        P piece[N];
        load_pack_loose<T, N>(p + OFF, piece);
#pragma unroll
        for (int i = 0; i < N; ++i) out[OFF + i] = piece[i];
      }
      load_cut_pack_from<T, W, OFF + N, N / 2>(p, out, c);
    } else {
      load_cut_pack_from<T, W, OFF, N / 2>(p, out, c);
    }
  }
}
template <class T, int W, int OFF, int N, class P>
__device__ __forceinline__ void store_cut_pack_from(T* p, const P (&in)[W], unsigned c) {
  if constexpr (N >= 1) {
    if (c & N) {
      if constexpr (N == 1) {
        p[OFF] = (T)in[OFF];
      } else {
        P piece[N];
#pragma unroll
        for (int i = 0; i < N; ++i) piece[i] = in[OFF + i];
        store_pack_loose<T, N>(p + OFF, piece);
      }
      store_cut_pack_from<T, W, OFF + N, N / 2>(p, in, c);
    } else {
      store_cut_pack_from<T, W, OFF, N / 2>(p, in, c);
    }
  }
}
template <class T, int W, class P>
__device__ __forceinline__ void store_cut_pack(T* p, const P (&in)[W], unsigned c) {
  store_cut_pack_from<T, W, 0, W / 2>(p, in, c);
}

#ifdef MP_HOST_SIDE
inline bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }
inline unsigned misalign16(const void* p) { return (unsigned)(reinterpret_cast<uintptr_t>(p) & 15u); }
#endif

/* ---------------------------------------------------------------------------------------
 * cross-lane reductions (all 64 lanes must be active)
 * ------------------------------------------------------------------------------------- */

struct AddOP { template <class P> static __device__ __forceinline__ P apply(P a, P b) { return a + b; } };
struct MaxOP { template <class P> static __device__ __forceinline__ P apply(P a, P b) { return a > b ? a : b; } };

/* DPP controls: quad_perm [1,0,3,2], quad_perm [2,3,0,1], row_half_mirror, row_mirror */
constexpr int DPP_XOR1 = 0xB1, DPP_XOR2 = 0x4E, DPP_HALF_MIRROR = 0x141, DPP_MIRROR = 0x140;

template <int CTRL> __device__ __forceinline__ float dpp_move(float v) {
  return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xF, 0xF, true));
}
template <int CTRL> __device__ __forceinline__ double dpp_move(double v) {
  const unsigned long long b = __builtin_bit_cast(unsigned long long, v);
  const unsigned lo = (unsigned)__builtin_amdgcn_update_dpp(0, (int)(unsigned)b, CTRL, 0xF, 0xF, true);
  const unsigned hi = (unsigned)__builtin_amdgcn_update_dpp(0, (int)(unsigned)(b >> 32), CTRL, 0xF, 0xF, true);
  return __builtin_bit_cast(double, ((unsigned long long)hi << 32) | lo);
}

typedef unsigned uint2_t __attribute__((ext_vector_type(2)));

/* After the four DPP steps every lane of a 16-lane row holds that row's result. swap16 pairs
 * odd and even rows (lanes 0-31 and 32-63 then agree), swap32 pairs the wave halves; each
 * returns both values to fold. The two results are copied to scalars before the bit cast:
 * casting the vector element expression itself reads element 0 twice with this compiler. */
template <class OP> __device__ __forceinline__ float fold_swap16(float v) {
  const uint2_t r = __builtin_amdgcn_permlane16_swap(__builtin_bit_cast(unsigned, v), __builtin_bit_cast(unsigned, v), false, false);
  const unsigned kept = r[0], swapped = r[1];
  return OP::apply(__builtin_bit_cast(float, kept), __builtin_bit_cast(float, swapped));
}
template <class OP> __device__ __forceinline__ float fold_swap32(float v) {
  const uint2_t r = __builtin_amdgcn_permlane32_swap(__builtin_bit_cast(unsigned, v), __builtin_bit_cast(unsigned, v), false, false);
  const unsigned kept = r[0], swapped = r[1];
  return OP::apply(__builtin_bit_cast(float, kept), __builtin_bit_cast(float, swapped));
}
template <class OP> __device__ __forceinline__ double fold_swap16(double v) {
  const unsigned long long b = __builtin_bit_cast(unsigned long long, v);
  const uint2_t lo = __builtin_amdgcn_permlane16_swap((unsigned)b, (unsigned)b, false, false);
  const uint2_t hi = __builtin_amdgcn_permlane16_swap((unsigned)(b >> 32), (unsigned)(b >> 32), false, false);
  const unsigned lo0 = lo[0], lo1 = lo[1], hi0 = hi[0], hi1 = hi[1];
  return OP::apply(__builtin_bit_cast(double, ((unsigned long long)hi0 << 32) | lo0),
                   __builtin_bit_cast(double, ((unsigned long long)hi1 << 32) | lo1));
}
template <class OP> __device__ __forceinline__ double fold_swap32(double v) {
  const unsigned long long b = __builtin_bit_cast(unsigned long long, v);
  const uint2_t lo = __builtin_amdgcn_permlane32_swap((unsigned)b, (unsigned)b, false, false);
  const uint2_t hi = __builtin_amdgcn_permlane32_swap((unsigned)(b >> 32), (unsigned)(b >> 32), false, false);
  const unsigned lo0 = lo[0], lo1 = lo[1], hi0 = hi[0], hi1 = hi[1];
  return OP::apply(__builtin_bit_cast(double, ((unsigned long long)hi0 << 32) | lo0),
                   __builtin_bit_cast(double, ((unsigned long long)hi1 << 32) | lo1));
}

/* OP folded over the S = 8, 16, 32 or 64 lanes of an aligned sub-group of the wave; every lane of
 * the sub-group returns the result. All 64 lanes must execute it. */
template <class OP, int S, class P> __device__ __forceinline__ P lanes_allreduce(P v) {
  static_assert(S == 8 || S == 16 || S == 32 || S == 64, "sub-groups of 8, 16, 32 or 64 lanes");
  v = OP::apply(v, dpp_move<DPP_XOR1>(v));
  v = OP::apply(v, dpp_move<DPP_XOR2>(v));
  v = OP::apply(v, dpp_move<DPP_HALF_MIRROR>(v));
  if constexpr (S >= 16) v = OP::apply(v, dpp_move<DPP_MIRROR>(v));
  if constexpr (S >= 32) v = fold_swap16<OP>(v);
  if constexpr (S >= 64) v = fold_swap32<OP>(v);
  return v;
}

/* Every lane of the wave returns OP folded over all 64 lanes. */
template <class OP, class P> __device__ __forceinline__ P wave_allreduce(P v) {
  return lanes_allreduce<OP, WAVE>(v);
}

/* NW per-wave partials, one per lane with index lane % NW, folded so that every lane holds the
 * result: a DPP butterfly over NW <= 16 neighbouring lanes. Every lane applies OP over the same
 * tree with commuted operands, so all lanes agree bit for bit. */
template <class OP, int NW, class P> __device__ __forceinline__ P fold_partials(P v) {
  static_assert(NW >= 1 && NW <= 16 && (NW & (NW - 1)) == 0, "partials per group: a power of two up to 16");
  if constexpr (NW >= 2) v = OP::apply(v, dpp_move<DPP_XOR1>(v));
  if constexpr (NW >= 4) v = OP::apply(v, dpp_move<DPP_XOR2>(v));
  if constexpr (NW >= 8) v = OP::apply(v, dpp_move<DPP_HALF_MIRROR>(v));
  if constexpr (NW >= 16) v = OP::apply(v, dpp_move<DPP_MIRROR>(v));
  return v;
}

/* Every thread of a G-thread group (G/64 consecutive waves of the workgroup) returns OP
 * folded over the group. `slots` points at the group's G/64 LDS words for THIS reduction;
 * two reductions in flight must use different slots, and a loop that reuses slots must
 * alternate between two sets, which makes the single barrier below sufficient. After the
 * barrier each lane reads ONE partial (a conflict-free multicast) and the partials are folded
 * across lanes, instead of every lane reading and adding all of them. */
template <class OP, int G, class P>
__device__ __forceinline__ P group_allreduce(P v, P* slots, int lane_in_group) {
  if constexpr (G <= WAVE) { /* a wave or an aligned part of one: cross-lane only */
    return lanes_allreduce<OP, G>(v);
  } else {
    v = wave_allreduce<OP>(v);
    constexpr int NW = G / WAVE;
    if ((lane_in_group & (WAVE - 1)) == 0) slots[lane_in_group / WAVE] = v;
    __syncthreads();
    return fold_partials<OP, NW>(slots[lane_in_group & (NW - 1)]);
  }
}

/* A workgroup barrier that orders LDS traffic only. __syncthreads() also waits for every global
 * load and store of the wave (s_waitcnt vmcnt(0)), which ends a prefetch at the first reduction
 * that follows it; this one leaves global accesses in flight. For exchanges through LDS only:
 * it publishes nothing that was written to global memory. */
__device__ __forceinline__ void lds_barrier() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); }

/* Makes the compiler treat a register-held value as consumed and redefined here: everything that
 * produces it (a load in flight) is waited for at this point and not later. */
template <class V> __device__ __forceinline__ void settle(V& v) { asm volatile("" : "+v"(v)); }

/* ---------------------------------------------------------------------------------------
 * row geometry: [head scalars][nvec aligned packs][tail scalars]
 * ------------------------------------------------------------------------------------- */

template <class T, int W> struct RowGeom {
  int head;  /* elements before the first 16-byte boundary */
  int nvec;  /* whole packs */
  int tail;  /* elements after the last whole pack */
  __device__ __forceinline__ RowGeom(const T* row, size_t n, bool ragged) {
    if (W == 1 || !ragged) {
      head = 0;
      nvec = (int)(n / W);
      tail = (int)(n - (size_t)nvec * W);
    } else {
      const unsigned mis = (unsigned)(reinterpret_cast<uintptr_t>(row) & 15u);
      int h = (int)(((16u - mis) & 15u) / sizeof(T));
      if ((size_t)h > n) h = (int)n;
      head = h;
      nvec = (int)((n - h) / W);
      tail = (int)(n - h - (size_t)nvec * W);
    }
  }
};

/* A row held in registers by a group of G threads: NV packs per thread plus, for ragged
 * rows, one edge element on the group's first head+tail threads. */
template <class T, int W, int G, int NV, bool RAGGED> struct RowTile {
  using P = typename precision<T>::type;
  P v[NV][W];
  P edge;

  __device__ __forceinline__ void load(const T* row, const RowGeom<T, W>& g, int lane, P fill) {
    const T* body = row + g.head;
#pragma unroll
    for (int k = 0; k < NV; ++k) {
      const int p = k * G + lane;
      if (p < g.nvec) {
        load_pack_nt<T, W>(body + (size_t)p * W, v[k]); /* a resident row is read exactly once */
      } else {
#pragma unroll
        for (int i = 0; i < W; ++i) v[k][i] = fill;
      }
    }
    edge = fill;
    if constexpr (RAGGED) {
      if (lane < g.head) edge = (P)row[lane];
      else if (lane - g.head < g.tail) edge = (P)body[(size_t)g.nvec * W + (lane - g.head)];
    }
  }

  template <bool KEEP = false> __device__ __forceinline__ void store(T* row, const RowGeom<T, W>& g, int lane) const {
    T* body = row + g.head;
#pragma unroll
    for (int k = 0; k < NV; ++k) {
      const int p = k * G + lane;
      if (p < g.nvec) store_pack_kept<KEEP, T, W>(body + (size_t)p * W, v[k]);
    }
    if constexpr (RAGGED) {
      if (lane < g.head) row[lane] = (T)edge;
      else if (lane - g.head < g.tail) body[(size_t)g.nvec * W + (lane - g.head)] = (T)edge;
    }
  }

  /* f(value&, k, i) over pack elements; i == -1 marks the edge element */
  template <class F> __device__ __forceinline__ void each(F f) {
#pragma unroll
    for (int k = 0; k < NV; ++k) {
#pragma unroll
      for (int i = 0; i < W; ++i) f(v[k][i]);
    }
    if constexpr (RAGGED) f(edge);
  }
};

/* ---------------------------------------------------------------------------------------
 * row-regime selection shared by the softmax and RMSNorm launchers
 * ------------------------------------------------------------------------------------- */

#ifdef MP_HOST_SIDE
/* Before every launch of a row kernel: `if (note_plan(...)) return;`. Nothing in the library as
 * shipped; in the test build it records the decision and, on a dry run, says "do not launch". */
#ifdef MP_DIAGNOSTICS
inline bool note_plan(int kind, int group, int packs_per_thread, int rows_per_block, size_t grid, size_t block,
                      int cluster = 1, int chunk_packs = 0, size_t workspace_bytes = 0, bool kept = false) {
  MpPlanProbe& p = mp_plan_probe();
  if (!p.dry) return false;
  p.note = MpPlanNote{kind, group, packs_per_thread, rows_per_block, (long long)grid, (long long)block, cluster, chunk_packs,
                      (long long)workspace_bytes, kept ? 1 : 0};
  p.noted = true;
  return true;
}
inline bool plan_dry_run() { return mp_plan_probe().dry; }
#else
template <class... A> constexpr bool note_plan(A...) { return false; }
constexpr bool plan_dry_run() { return false; }
#endif
enum PlanKind { PLAN_SHORT = 0, PLAN_RESIDENT = 1, PLAN_PAIRED = 2, PLAN_ANY = 3, PLAN_CLUSTER = 4, PLAN_DEEP = 5,
                PLAN_STREAM = 6, PLAN_LOOSE = 7 };

/* Packs a thread must hold so that a G-thread group covers `packs` packs; 0 = too long. */
inline int packs_per_thread(size_t packs, int G, int max_nv) {
  for (int nv = 1; nv <= max_nv; nv *= 2)
    if ((size_t)nv * G >= packs) return nv;
  return 0;
}

/* The GPU's compute-unit count, read once per process. */
inline int compute_units() {
#ifdef MP_DIAGNOSTICS
  if (mp_plan_probe().dry && mp_plan_probe().cus > 0) return mp_plan_probe().cus;
#endif
  static int cus = [] {
    int dev = 0, n = 0;
    HIP_ASSERT(hipGetDevice(&dev));
    HIP_ASSERT(hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev));
    return n > 0 ? n : 256;
  }();
  return cus;
}
#endif /* MP_HOST_SIDE */

}  // namespace mp

#endif  /* __cplusplus && __HIPCC__ */
#endif  /* MP_KERNEL_HEADER_H */
