#include "../elementwise.h"

struct ReluFn_Scalar {
  template <class P> __device__ __forceinline__ void apply(const P (&in)[1], P (&out)[1]) const {
    out[0] = in[0] >= (P)0 ? in[0] : (P)0;
  }
};

// b = (a >= 0) ? a : 0. Replaces src/cuda/nvcc_src/relu.cu:3-27.
extern "C" void launch_relu_Scalar(
  const void* a,
  void* b,
  len_t n,
  StreamContext stream
) {
  const mp::EwPtrs<1, 1> ptrs{{a}, {b}};
  mp::ew_launch<Scalar, 1, 1, 1>(ptrs, n, ReluFn_Scalar{}, get_stream(stream));
}
