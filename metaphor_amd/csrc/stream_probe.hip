/*
 * Measurement only: plain passes over memory with the stream mix of a workload and none of its
 * arithmetic, so that a kernel's rate can be put beside what this GPU gives a copy of the same
 * reads, writes and footprint. Built into lib/libmp_probe.so, which only bench.py loads; nothing
 * here is part of the kernel library or of the boundary. The reference has no counterpart (it
 * ships no timing code at all).
 */
#include "kernel_header.h"

namespace {

typedef float f4 __attribute__((ext_vector_type(4)));

struct ProbePtrs {
  const f4* in[5];
  f4* out[4];
};

/* NR streams read and NW written once, a 16-byte pack per lane and stream, one-shot workgroups
 * of B threads: the shape of the elementwise engine and, with B = 256, of a plain copy. */
template <int NR, int NW, int B>
__global__ __launch_bounds__(B) void probe_streams(ProbePtrs p, size_t packs) {
  const size_t i = (size_t)blockIdx.x * B + threadIdx.x;
  if (i >= packs) return;
  f4 v[NR];
#pragma unroll
  for (int s = 0; s < NR; ++s) v[s] = __builtin_nontemporal_load(p.in[s] + i);
  f4 t = v[0];
#pragma unroll
  for (int s = 1; s < NR; ++s) t += v[s];
#pragma unroll
  for (int s = 0; s < NW; ++s) __builtin_nontemporal_store(t + (float)s, p.out[s] + i);
}

/* The shape of the paired RMSNorm reverse without its arithmetic: 1024 threads hold a row of
 * 1024 packs, rows in pairs with the next row's loads in flight, one LDS-only barrier per row
 * between the loads and the store, NR streams read and one written. */
template <int NR>
__global__ __launch_bounds__(1024) void probe_row_pairs(ProbePtrs p, size_t m, size_t packs) {
  __shared__ float slots[2][16];
  const int tid = threadIdx.x;
  const size_t stride = gridDim.x, last = m - 1;
  size_t row = blockIdx.x;
  f4 a[NR], b[NR];
  auto fetch = [&](f4 (&v)[NR], size_t r) {
    r = r < last ? r : last;
#pragma unroll
    for (int s = 0; s < NR; ++s) v[s] = __builtin_nontemporal_load(p.in[s] + r * packs + tid);
  };
  auto finish = [&](const f4 (&v)[NR], size_t r, float* sl) {
    f4 t = v[0];
#pragma unroll
    for (int s = 1; s < NR; ++s) t += v[s];
    float w = mp::wave_allreduce<mp::AddOP>(t.x);
    if ((tid & 63) == 0) sl[tid >> 6] = w;
    mp::lds_barrier();
    w = mp::fold_partials<mp::AddOP, 16>(sl[tid & 15]);
    t.y += w == 12345.678f ? 1.0f : 0.0f; /* keeps the exchange alive */
    if (r < m) __builtin_nontemporal_store(t, p.out[0] + r * packs + tid);
  };
  fetch(a, row);
  for (; row < m; row += 2 * stride) {
    fetch(b, row + stride);
    __builtin_amdgcn_sched_barrier(0);
    finish(a, row, slots[0]);
    fetch(a, row + 2 * stride);
    __builtin_amdgcn_sched_barrier(0);
    finish(b, row + stride, slots[1]);
  }
}

template <int NR, int NW> void launch_streams(const ProbePtrs& p, size_t packs, int block, hipStream_t stream) {
  if (block == 64) probe_streams<NR, NW, 64><<<dim3((unsigned)((packs + 63) / 64)), dim3(64), 0, stream>>>(p, packs);
  else probe_streams<NR, NW, 256><<<dim3((unsigned)((packs + 255) / 256)), dim3(256), 0, stream>>>(p, packs);
}

}  // namespace

// in: nr device pointers, out: nw device pointers, each to `bytes` bytes (a multiple of 16, 16-byte
// aligned); block: 64 or 256 threads per workgroup. Mixes: 1R+1W, 2R+1W, 4R+1W, 5R+4W.
// Returns 0 after enqueueing, 1 for a mix or size it does not have.
extern "C" int mpProbeStreams(const void* const* in, void* const* out, int nr, int nw, len_t bytes, int block,
                              StreamContext stream) {
  if (bytes % 16 != 0 || (block != 64 && block != 256) || bytes / 16 / 64 >= 0x7fffffffull) return 1;
  ProbePtrs p{};
  for (int s = 0; s < nr && s < 5; ++s) p.in[s] = static_cast<const f4*>(in[s]);
  for (int s = 0; s < nw && s < 4; ++s) p.out[s] = static_cast<f4*>(out[s]);
  const size_t packs = bytes / 16;
  hipStream_t q = get_stream(stream);
  if (nr == 1 && nw == 1) launch_streams<1, 1>(p, packs, block, q);
  else if (nr == 2 && nw == 1) launch_streams<2, 1>(p, packs, block, q);
  else if (nr == 4 && nw == 1) launch_streams<4, 1>(p, packs, block, q);
  else if (nr == 5 && nw == 4) launch_streams<5, 4>(p, packs, block, q);
  else return 1;
  MP_CHECK_LAUNCH();
  return 0;
}

// nr (1 or 2) inputs and one output of m rows of 16 KiB each (4096 r32 values), on `workgroups`
// persistent workgroups of 1024 threads.
extern "C" int mpProbeRowPairs(const void* const* in, void* out, int nr, len_t m, len_t workgroups, StreamContext stream) {
  if (m == 0 || workgroups == 0 || workgroups > 0x7fffffffull) return 1;
  ProbePtrs p{};
  for (int s = 0; s < nr && s < 2; ++s) p.in[s] = static_cast<const f4*>(in[s]);
  p.out[0] = static_cast<f4*>(out);
  hipStream_t q = get_stream(stream);
  if (nr == 1) probe_row_pairs<1><<<dim3((unsigned)workgroups), dim3(1024), 0, q>>>(p, m, 1024);
  else if (nr == 2) probe_row_pairs<2><<<dim3((unsigned)workgroups), dim3(1024), 0, q>>>(p, m, 1024);
  else return 1;
  MP_CHECK_LAUNCH();
  return 0;
}
