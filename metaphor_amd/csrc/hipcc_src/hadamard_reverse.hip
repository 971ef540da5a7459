#include "../elementwise.h"

struct HadamardReverseFn_Scalar {
  template <class P> __device__ __forceinline__ void apply(const P (&in)[3], P (&out)[1]) const {
    out[0] = in[2] + in[0] * in[1];
  }
};

// c += a * b. Replaces src/cuda/nvcc_src/hadamard_reverse.cu:3-29; called twice per
// hadamard reverse with the operands swapped (src/ops/hadamard.zig:65-79).
extern "C" void launch_hadamard_reverse_Scalar(
  const void* a,
  const void* b,
  void* c,
  len_t N,
  StreamContext stream
) {
  const mp::EwPtrs<3, 1> ptrs{{a, b, c}, {c}};
  mp::ew_launch<Scalar, 3, 1, 1>(ptrs, N, HadamardReverseFn_Scalar{}, get_stream(stream));
}
