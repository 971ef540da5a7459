#include "../row_rmsnorm.h"

// dst[i,j] = src[i,j] * gain[j] / sqrt(mean_j src[i,:]^2 + eps). No reference kernel exists;
// scalars cross the boundary as double and sizes as len_t like every reference launcher
// (src/cuda/nvcc_src/reduce_ij_i.cu:35-42). dst may be src. scratch: mpRmsnormScratchBytes(dtype, m, n)
// bytes owned by the caller (0 for rows one workgroup holds), or NULL: rows longer than that are
// then read twice.
// An input of up to 256 MiB is read so that it stays in the GPU's memory-side cache, where the
// reverse that reads it again finds it (a step of forward and reverse gains 6 %, a forward on its
// own pays 2 %); larger inputs stream past the cache.
extern "C" void launch_rmsnorm_ij_j_Scalar(
  const void* src,
  const void* gain,
  void* dst,
  void* scratch,
  double eps,
  len_t m,
  len_t n,
  StreamContext stream
) {
  mp::rmsnorm_forward<Scalar>(static_cast<const Scalar*>(src), static_cast<const Scalar*>(gain),
                              static_cast<Scalar*>(dst), scratch, eps, m, n, get_stream(stream));
}
