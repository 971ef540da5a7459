/*
 * launch_rmsnorm_ij_j_reverse_r32 for callers that cannot allocate a workspace. No counterpart in
 * the reference, whose kernels get their workspace from the per-stream scratch of the host side
 * (src/core/utils.zig:20-36). Compiled once (no `Scalar` replication), into the shipped library only.
 */
#include "row_rmsnorm.h"

#include <atomic>

// ---------------------------------------------------------------------------------------------
// The entry point that brings its own workspace: launch_rmsnorm_ij_j_reverse_r32 for callers
// that cannot allocate one (code under HIP graph capture, serving loops, harnesses that forbid
// hipMalloc). The partial gain rows go into the file-scope device array below instead of a
// caller-owned buffer; nothing here allocates or frees.
//
// `scratch` as host code sees it is a stand-in for the symbol, not a device address: the address
// of the array on a device comes from hipGetSymbolAddress, asked once per device on the first call
// there (every GPU holds its own copy of the array at its own address, until the process ends),
// and that pointer is what the kernels get.
constexpr size_t MP_NOALLOC_SCRATCH_BYTES = (size_t)16 << 20;
static __device__ __align__(256) unsigned char scratch[MP_NOALLOC_SCRATCH_BYTES];

namespace {
constexpr int MP_NOALLOC_MAX_DEVICES = 64;
std::atomic<void*> scratch_on_device[MP_NOALLOC_MAX_DEVICES];
/* the stream of the last call on each device, and whether the warning below has been printed */
std::atomic<void*> last_stream[MP_NOALLOC_MAX_DEVICES];
std::atomic<bool> warned{false};

/* Calls on different streams of one device share the array and must not overlap in time, which
 * only the caller can see to. A change of stream is where that can go wrong: say so once. */
void note_stream(int dev, hipStream_t stream) {
  void* now = static_cast<void*>(stream);
  void* before = last_stream[dev].exchange(now, std::memory_order_relaxed);
  if (before != now && before != nullptr && !warned.exchange(true, std::memory_order_relaxed))
    fprintf(stderr,
            "mpRmsnormReverseR32NoAlloc: called on two streams of device %d; every call on a device uses the same "
            "built-in workspace, so calls on different streams must be ordered by the caller (an event or a "
            "synchronisation between them), or their gain gradients corrupt each other. Said once.\n", dev);
}

void* noalloc_scratch(hipStream_t stream) {
  int dev = 0;
  HIP_ASSERT(hipGetDevice(&dev));
  mp::require(dev >= 0 && dev < MP_NOALLOC_MAX_DEVICES, "mpRmsnormReverseR32NoAlloc: device index beyond 63");
  note_stream(dev, stream);
  void* ptr = scratch_on_device[dev].load(std::memory_order_acquire);
  if (ptr == nullptr) { /* two threads racing here both get the same answer */
    HIP_ASSERT(hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)));
    mp::require(ptr != nullptr, "mpRmsnormReverseR32NoAlloc: the workspace array has no device address");
    scratch_on_device[dev].store(ptr, std::memory_order_release);
  }
  return ptr;
}
}  // namespace

// Same computation and same kernels as launch_rmsnorm_ij_j_reverse_r32 (bit-identical results),
// without the scratch argument. Returns 0 after enqueueing, 1 (with a message on stderr, nothing
// enqueued) when [m, n] needs more workspace than the built-in 16 MiB. What a call needs is one
// row of n fp32 sums per workgroup of the row pass, at most two workgroups a compute unit:
// min(m, 2 * CUs) * n * 4 bytes, so rows of up to 4194304 / min(m, 2 * CUs) elements fit (8192 on
// the MI355X's 256 compute units, whatever m); rows shared by several workgroups add two words per
// row and workgroup. The array is shared by every call on a device and keeps the last call's
// contents; every word a launch reads it has written before (the partial rows by the row pass,
// the words of shared long rows by the clearing kernel), so nothing needs to start at zero, but
// two calls that overlap in time on one device (two streams, two threads) race on it.
extern "C" int mpRmsnormReverseR32NoAlloc(const void* src, const void* gain, const void* dst_grads,
                                          void* src_grads, void* gain_grads, double eps, double alpha,
                                          len_t m, len_t n, StreamContext stream) {
  const size_t need = mp::rmsnorm_reverse_scratch_bytes<r32>(m, n);
  if (need > MP_NOALLOC_SCRATCH_BYTES) {
    fprintf(stderr,
            "mpRmsnormReverseR32NoAlloc: [%lu, %lu] needs %zu bytes of workspace, the built-in array holds %zu; "
            "call launch_rmsnorm_ij_j_reverse_r32 with a caller-owned workspace instead\n",
            (unsigned long)m, (unsigned long)n, need, MP_NOALLOC_SCRATCH_BYTES);
    return 1;
  }
  void* ptr = noalloc_scratch(get_stream(stream));
  mp::rmsnorm_reverse<r32>(static_cast<const r32*>(src), static_cast<const r32*>(gain),
                           static_cast<const r32*>(dst_grads), static_cast<r32*>(src_grads),
                           static_cast<r32*>(gain_grads), ptr, eps, alpha, m, n, get_stream(stream));
  return 0;
}
