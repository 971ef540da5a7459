#include "../elementwise.h"

struct DilateReverseFn_Scalar {
  double value;
  template <class P> __device__ __forceinline__ void apply(const P (&in)[2], P (&out)[1]) const {
    out[0] = in[1] + in[0] * (P)value;
  }
};

// b += a * value. Replaces src/cuda/nvcc_src/dilate_reverse.cu:3-29.
extern "C" void launch_dilate_reverse_Scalar(
  const void* a,
  double value,
  void* b,
  len_t N,
  StreamContext stream
) {
  const mp::EwPtrs<2, 1> ptrs{{a, b}, {b}};
  mp::ew_launch<Scalar, 2, 1, 1>(ptrs, N, DilateReverseFn_Scalar{(double)static_cast<Scalar>(value)}, get_stream(stream));
}
