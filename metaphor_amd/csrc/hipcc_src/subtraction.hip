#include "../elementwise.h"

struct SubtractionFn_Scalar {
  template <class P> __device__ __forceinline__ void apply(const P (&in)[2], P (&out)[1]) const {
    out[0] = in[0] - in[1];
  }
};

// c = a - b. Replaces src/cuda/nvcc_src/subtraction.cu:3-29.
extern "C" void launch_subtraction_Scalar(
  const void* a,
  const void* b,
  void* c,
  len_t N,
  StreamContext stream
) {
  const mp::EwPtrs<2, 1> ptrs{{a, b}, {c}};
  mp::ew_launch<Scalar, 2, 1, 1>(ptrs, N, SubtractionFn_Scalar{}, get_stream(stream));
}
