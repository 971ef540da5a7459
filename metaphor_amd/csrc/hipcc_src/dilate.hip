#include "../elementwise.h"

struct DilateFn_Scalar {
  double value;
  template <class P> __device__ __forceinline__ void apply(const P (&in)[1], P (&out)[1]) const {
    out[0] = in[0] * (P)value;
  }
};

// c = a * value. Replaces src/cuda/nvcc_src/dilate.cu:3-29; the scalar crosses as double and is
// narrowed to the storage type in the launcher, as there (:24).
extern "C" void launch_dilate_Scalar(
  const void* a,
  double value,
  void* c,
  len_t N,
  StreamContext stream
) {
  const mp::EwPtrs<1, 1> ptrs{{a}, {c}};
  mp::ew_launch<Scalar, 1, 1, 1>(ptrs, N, DilateFn_Scalar{(double)static_cast<Scalar>(value)}, get_stream(stream));
}
