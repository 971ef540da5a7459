/*
 * What the kernels that share one long row between several workgroups have in common: the
 * scratch words the workgroups of a row publish their partial results in, the bounded wait for
 * the partners, the small kernel that clears the words before a launch, and the tuning knobs of
 * the tests. Used by the softmax and RMSNorm launchers; no counterpart in the reference, whose
 * row kernels give a row to one 32-lane warp (src/cuda/nvcc_src/reduce_ij_i.cu:3-33).
 */
#ifndef MP_ROW_CLUSTER_H
#define MP_ROW_CLUSTER_H

#include "row_dispatch.h"

#ifdef MP_HOST_SIDE
#include <mutex>
#endif

#if defined(__cplusplus) && defined(__HIPCC__)

namespace mp {

/* workgroup size of the shared-row kernels, and the most workgroups one row is split over (one
 * lane of the first wavefront polls each partner) */
constexpr int CLUSTER_THREADS = 1024, CLUSTER_MAX = WAVE;

/* Makes the compiler forget what it knows about a register-held pack, so that widened copies
 * of a whole chunk are not kept alive from one phase of a kernel to the next. */
template <class V> __device__ __forceinline__ void forget(V& v) {
  typedef unsigned words_t __attribute__((ext_vector_type(sizeof(V) / 4)));
  words_t w = __builtin_bit_cast(words_t, v);
  asm volatile("" : "+v"(w));
  v = __builtin_bit_cast(V, w);
}

/* Whether two operands of `bytes` bytes each share any byte. A row shared by several workgroups
 * may be read again by a workgroup that stopped waiting for its partners, after those have
 * written their chunks: the output must not touch an input at all, not only not equal it. */
inline bool ranges_overlap(const void* a, const void* b, size_t bytes) {
  const uintptr_t pa = reinterpret_cast<uintptr_t>(a), pb = reinterpret_cast<uintptr_t>(b);
  return pa < pb + bytes && pb < pa + bytes;
}

template <class P> struct slot_word { using type = unsigned; };
template <> struct slot_word<double> { using type = unsigned long long; };

template <class Word> __global__ __launch_bounds__(256) void cluster_zero_slots(Word* slots, size_t words) {
  const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
  if (i < words) slots[i] = 0;
}

/* Chunk size and poll limit of the cluster path. Constants in the library as shipped; the test
 * build (MP_DIAGNOSTICS) lets mpSetClusterTuning change them, to split short rows over several
 * workgroups and to drive the path of a workgroup that stops waiting. */
struct ClusterTuning {
  int packs_per_block = 0; /* 0: one pack per thread less than the register tile holds */
  unsigned spin_limit = 1u << 22;
  int deep = 0; /* the RMSNorm reverse's shared rows: 0 by the launcher's rule, 1 always the pipelined kernel, 2 never */
  int own_words = 1; /* stamped exchange words: 1 in the library's own memory where a region is to be had, 0 always in the caller's workspace */
  int keep_input = -1; /* what a forward leaves in the memory-side cache for its reverse (keep_input, keep_output): -1 by tensor size, 0 nothing, 1 always */
};
#ifdef MP_DIAGNOSTICS
inline ClusterTuning& cluster_tuning() {
  static ClusterTuning t;
  return t;
}
#else
constexpr ClusterTuning cluster_tuning() { return ClusterTuning{}; }
#endif

/* What a forward leaves in the memory-side cache (256 MiB in front of the HBM stacks, shared by the
 * eight XCDs) for the reverse that follows it. Streaming (non-temporal) accesses leave nothing
 * there, ordinary ones do, and a streaming load that finds its line there is served from it. So a
 * forward whose input the reverse reads again (RMSNorm: x) loads it with ordinary loads, a forward
 * whose output the reverse reads (softmax: y) stores it with ordinary stores, and everything else
 * stays streaming (ordinary stores of the rest push the kept tensor out again). Measured as steps
 * of a forward and its reverse on tensors not touched for several steps, against the same with
 * streaming accesses throughout, and the forward on its own:
 *   RMSNorm r32 [8192, 4096] (128 MiB a tensor): step 110.4 -> 103.4 us, forward 43.3 -> 44.2;
 *     [16384, 4096] (256 MiB): 214.8 -> 202.1, 85.8 -> 87.8; [32768, 4096] (512 MiB): 435.4 -> 418.9, 179.4 -> 182.1;
 *   softmax r32 [8192, 4096]: step 105.7 -> 96.9, forward 42.5 -> 43.8; [512, 151936] (296 MiB):
 *     246.6 -> 236.9, 99.0 -> 107.1; r16 [16384, 16384] (512 MiB): 424.7 -> 414.7, 173.2 -> 179.5.
 * A forward that no reverse follows pays for it, little for kept loads, more for kept stores of
 * tensors beyond the cache; the launchers cannot know what follows and keep by tensor size:
 * inputs up to the size of the cache, outputs up to half of it. */
constexpr size_t KEEP_INPUT_BYTES = 256u << 20;
constexpr size_t KEEP_OUTPUT_BYTES = 128u << 20;
inline bool keep_input(size_t tensor_bytes) {
  const int mode = cluster_tuning().keep_input;
  return mode < 0 ? tensor_bytes <= KEEP_INPUT_BYTES : mode != 0;
}
inline bool keep_output(size_t tensor_bytes) {
  const int mode = cluster_tuning().keep_input;
  return mode < 0 ? tensor_bytes <= KEEP_OUTPUT_BYTES : mode != 0;
}

/* Workgroups per row that a workspace must provide words for, given the number c the launcher
 * would use now. As shipped that is c itself (nothing can change it between the size query and
 * the launch). The test build sizes for the most workgroups any override can ask for, so a
 * workspace sized under one regime or tuning is never too small for a launch under another. */
inline size_t cluster_size_for_scratch(int c) {
#ifdef MP_DIAGNOSTICS
  (void)c;
  return (size_t)CLUSTER_MAX;
#else
  return c > 1 ? (size_t)c : 0;
#endif
}

/* A row whose first pack is not at the start of a 128-byte line moves every chunk boundary back
 * by the packs it is past one (at most 7), so that each wavefront's kilobyte covers eight whole
 * lines rather than parts of nine: the first workgroup's chunk is that much shorter and its first
 * lanes idle. Only when the C chunks still reach the end of the row; launchers size the chunks
 * for CLUSTER_SKEW_MAX packs more than the row has, so that they do unless the tile is full. */
constexpr int CLUSTER_SKEW_MAX = 7;
template <class T>
__device__ __forceinline__ int cluster_skew(const T* body, int C, int packs_per_block, int nvec) {
  const int skew = (int)((reinterpret_cast<uintptr_t>(body) >> 4) & 7u);
  return C * packs_per_block - nvec >= CLUSTER_SKEW_MAX ? skew : 0;
}

/* Packs of a row that each of its C workgroups takes: an even share, rounded up to whole
 * kilobytes (64 packs, what a wavefront reads at once) so that a chunk does not start in the
 * middle of a wavefront's access. Measured on the softmax forward: [512, 151936] r32 104.0 ->
 * 102.1 us, [2048, 50257] and [1000, 100000] equal within their scatter, never slower. Shares
 * below a pack a thread (only the test build's small chunks) stay as they are, so that those
 * tests still spread a short row over many workgroups. The last workgroups get what is left.
 * `spare` packs are added to the row before it is shared out when the register tile allows it. */
inline int cluster_chunk_packs(size_t packs, int C, size_t tile, size_t spare = 0) {
  if ((packs + spare + (size_t)C - 1) / (size_t)C <= tile) packs += spare;
  size_t share = (packs + (size_t)C - 1) / (size_t)C;
  if (share >= (size_t)CLUSTER_THREADS) {
    const size_t whole = (share + WAVE - 1) / WAVE * WAVE;
    if (whole <= tile && whole * (size_t)(C - 1) < packs) share = whole; /* no workgroup left empty */
  }
  return (int)share;
}

/* Sums over the C workgroups that share a row. Every workgroup calls this with its NVAL partial
 * sums; all threads return with the row totals in vals, and the result says whether every
 * partner was heard from. `mine` points at this row's C * NVAL scratch words, zero before the
 * kernel started; a published word is never zero (+0 is stored as -0), so non-zero means
 * published. Workgroups of a row publish before they wait, and the wait ends after spin_limit
 * polls whatever happens: a caller that gets `false` computes the totals some other way (it
 * re-reads the row), so every wave reaches the end of its kernel under any scheduling.
 * bc: NVAL + 1 words of LDS. Contains one barrier; all CLUSTER_THREADS threads must call it. */
template <int NVAL, class P>
__device__ __forceinline__ bool cluster_exchange_sums(typename slot_word<P>::type* mine, int C, int rank,
                                                      P (&vals)[NVAL], unsigned spin_limit, P* bc, int lane) {
  using Word = typename slot_word<P>::type;
  if (lane == 0) {
#pragma unroll
    for (int v = 0; v < NVAL; ++v) {
      const P part = vals[v] == (P)0 ? -(P)0 : vals[v];
      __hip_atomic_store(mine + (size_t)rank * NVAL + v, __builtin_bit_cast(Word, part), __ATOMIC_RELAXED,
                         __HIP_MEMORY_SCOPE_AGENT);
    }
  }
  if (lane < WAVE) { /* wave 0: lane r waits for workgroup r of this row */
    Word w[NVAL];
    bool heard = true;
    if (lane < C) {
      for (unsigned spins = 0;; ++spins) {
        heard = true;
#pragma unroll
        for (int v = 0; v < NVAL; ++v) {
          w[v] = __hip_atomic_load(mine + (size_t)lane * NVAL + v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
          heard = heard && w[v] != 0;
        }
        if (heard || spins >= spin_limit) break;
        __builtin_amdgcn_s_sleep(4);
      }
    }
    const P missing = wave_allreduce<AddOP>(heard ? (P)0 : (P)1); /* every lane takes part */
#pragma unroll
    for (int v = 0; v < NVAL; ++v) {
      const P total = wave_allreduce<AddOP>(lane < C && heard ? __builtin_bit_cast(P, w[v]) : (P)0);
      if (lane == 0) bc[v] = total;
    }
    if (lane == 0) bc[NVAL] = missing;
  }
  __syncthreads();
#pragma unroll
  for (int v = 0; v < NVAL; ++v) vals[v] = bc[v];
  return bc[NVAL] == (P)0;
}

/* ---------------------------------------------------------------------------------------
 * Stamped exchange words: the hand-over above without the clearing launch in front.
 *
 * A word is 64 bits: a stamp in the high half, 32 bits of a value in the low half (a value of
 * precision<T> takes one word for fp32, two for fp64). Workgroup `rank` of a row owns
 * WPS = values * parts consecutive words. At its start it reads the stamp its own first word
 * carries from the launch before (zero in memory nobody has written yet), adds one, and that is
 * the stamp of this launch: it publishes its values under it and takes a partner's words for
 * published when all of them carry it. Every workgroup of a row publishes exactly once per
 * launch, whether it later stops waiting or not, so the words of a row move from one stamp to
 * the next in step and a word left by an earlier launch can never carry the stamp being waited
 * for; nothing has to be cleared between launches, and launches recorded into a graph and
 * replayed are as good as fresh ones, since the stamp lives on the device.
 *
 * That needs words that only this protocol ever writes and that are tied to one launch geometry.
 * They live in device memory of the library (share_arena), handed out by share_region(): one
 * region per (caller's workspace address, rows, workgroups a row, words a workgroup), never taken
 * back. The caller's workspace is the key because launches that may overlap in time must have
 * different workspaces anyway, so they never meet in a region, while launches through one
 * workspace are ordered by the caller already. When the arena or the table is full, or a problem
 * needs more than the arena holds, the words are taken from the caller's workspace instead, which
 * the launcher then clears with cluster_zero_slots first (every stamp is 1 then): same kernels.
 * ------------------------------------------------------------------------------------- */

typedef unsigned long long share_word;
constexpr size_t SHARE_ARENA_WORDS = (size_t)(4u << 20) / sizeof(share_word);
constexpr int SHARE_REGIONS = 64;
static __device__ __align__(256) share_word share_arena[SHARE_ARENA_WORDS];

template <class P> constexpr int share_parts() { return (int)(sizeof(P) / 4); }

#ifdef MP_HOST_SIDE
struct ShareTable {
  struct Entry { uintptr_t workspace; size_t rows, offset; int per_row, wps; };
  std::mutex lock;
  Entry entries[SHARE_REGIONS];
  int count = 0;
  size_t used = 0;
};
static ShareTable share_table;

/* Offset (in words) of the region for this key inside share_arena; -1: none to be had, use the
 * caller's workspace. */
inline long long share_region(const void* workspace, size_t rows, int per_row, int wps) {
#ifdef MP_DIAGNOSTICS
  if (!cluster_tuning().own_words) return -1;
#endif
  const uintptr_t key = reinterpret_cast<uintptr_t>(workspace);
  const size_t need = rows * (size_t)per_row * (size_t)wps;
  std::lock_guard<std::mutex> hold(share_table.lock);
  for (int i = 0; i < share_table.count; ++i) {
    const ShareTable::Entry& e = share_table.entries[i];
    if (e.workspace == key && e.rows == rows && e.per_row == per_row && e.wps == wps) return (long long)e.offset;
  }
  const size_t start = (share_table.used + 31) / 32 * 32; /* regions start on 256-byte lines */
  if (share_table.count == SHARE_REGIONS || start + need > SHARE_ARENA_WORDS) return -1;
  share_table.entries[share_table.count++] = ShareTable::Entry{key, rows, start, per_row, wps};
  share_table.used = start + need;
  return (long long)start;
}
#endif

/* The words of the launch: the caller's (cleared by the launcher) when given, else the region at
 * `offset` of the library's arena. */
__device__ __forceinline__ share_word* share_words(share_word* callers, size_t offset) {
  return callers != nullptr ? callers : share_arena + offset;
}

/* The stamp of this launch for a workgroup whose first word is `mine`: asked for by the
 * workgroup's first lane before it loads its chunk, read (share_stamp_of) when it publishes.
 * Only wave 0 may use the result. */
__device__ __forceinline__ share_word share_peek(const share_word* mine, int lane) {
  share_word old = 0;
  if (lane == 0) old = __hip_atomic_load(mine, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  return old;
}
__device__ __forceinline__ unsigned share_stamp_of(share_word peeked) {
  const unsigned old = (unsigned)(peeked >> 32);
  return (unsigned)__builtin_amdgcn_readfirstlane((int)(old + 1u)); /* lane 0's, for every lane of wave 0 */
}

template <int NVAL, class P>
__device__ __forceinline__ void share_publish(share_word* mine, unsigned stamp, const P (&vals)[NVAL]) {
  constexpr int PARTS = share_parts<P>();
  typedef unsigned bits_t __attribute__((ext_vector_type(PARTS)));
#pragma unroll
  for (int v = 0; v < NVAL; ++v) {
    const bits_t b = __builtin_bit_cast(bits_t, vals[v]);
#pragma unroll
    for (int q = 0; q < PARTS; ++q)
      __hip_atomic_store(mine + v * PARTS + q, ((share_word)stamp << 32) | b[q], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  }
}

/* One look at a partner's words; true when every one carries the stamp (vals are then its values). */
template <int NVAL, class P>
__device__ __forceinline__ bool share_read(const share_word* theirs, unsigned stamp, P (&vals)[NVAL]) {
  constexpr int PARTS = share_parts<P>();
  typedef unsigned bits_t __attribute__((ext_vector_type(PARTS)));
  share_word w[NVAL * PARTS];
#pragma unroll
  for (int i = 0; i < NVAL * PARTS; ++i) w[i] = __hip_atomic_load(theirs + i, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  bool ok = true;
#pragma unroll
  for (int v = 0; v < NVAL; ++v) {
    bits_t b;
#pragma unroll
    for (int q = 0; q < PARTS; ++q) {
      ok = ok && (unsigned)(w[v * PARTS + q] >> 32) == stamp;
      b[q] = (unsigned)w[v * PARTS + q];
    }
    vals[v] = __builtin_bit_cast(P, b);
  }
  return ok;
}

/* cluster_exchange_sums on stamped words. `row_words` points at the row's C * NVAL * parts words,
 * `peeked` is share_peek() of this workgroup's first word, taken before the chunk was loaded. */
template <int NVAL, class P>
__device__ __forceinline__ bool share_exchange_sums(share_word* row_words, int C, int rank, share_word peeked,
                                                    P (&vals)[NVAL], unsigned spin_limit, P* bc, int lane) {
  constexpr int WPS = NVAL * share_parts<P>();
  if (lane < WAVE) { /* wave 0: lane r waits for workgroup r of this row */
    const unsigned stamp = share_stamp_of(peeked);
    if (lane == 0) share_publish<NVAL>(row_words + (size_t)rank * WPS, stamp, vals);
    P got[NVAL];
    bool heard = true;
    if (lane < C) {
      for (unsigned spins = 0;; ++spins) {
        heard = share_read<NVAL>(row_words + (size_t)lane * WPS, stamp, got);
        if (heard || spins >= spin_limit) break;
        __builtin_amdgcn_s_sleep(4);
      }
    }
    const P missing = wave_allreduce<AddOP>(heard ? (P)0 : (P)1); /* every lane takes part */
#pragma unroll
    for (int v = 0; v < NVAL; ++v) {
      const P total = wave_allreduce<AddOP>(lane < C && heard ? got[v] : (P)0);
      if (lane == 0) bc[v] = total;
    }
    if (lane == 0) bc[NVAL] = missing;
  }
  __syncthreads();
#pragma unroll
  for (int v = 0; v < NVAL; ++v) vals[v] = bc[v];
  return bc[NVAL] == (P)0;
}

}  // namespace mp

#endif
#endif
