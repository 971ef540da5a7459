#include "../elementwise.h"

struct NegateFn_Scalar {
  template <class P> __device__ __forceinline__ void apply(const P (&in)[1], P (&out)[1]) const {
    out[0] = -in[0];
  }
};

// b = -a. Replaces src/cuda/nvcc_src/negate.cu:3-26.
extern "C" void launch_negate_Scalar(
  const void* a,
  void* b,
  len_t N,
  StreamContext stream
) {
  const mp::EwPtrs<1, 1> ptrs{{a}, {b}};
  mp::ew_launch<Scalar, 1, 1, 1>(ptrs, N, NegateFn_Scalar{}, get_stream(stream));
}
