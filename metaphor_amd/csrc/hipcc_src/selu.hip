#include "../elementwise.h"

struct SeluFn_Scalar {
  template <class P> __device__ __forceinline__ void apply(const P (&in)[1], P (&out)[1]) const {
    out[0] = mp::selu_value(in[0]);
  }
};

// b = selu(a) = scale*a for a > 0, scale*alpha*expm1(a) otherwise. The reference names
// mp.ops.selu (README.md:97) but ships no kernel; the signature is that of its activation
// launchers (src/cuda/nvcc_src/relu.cu:16-21).
extern "C" void launch_selu_Scalar(
  const void* a,
  void* b,
  len_t N,
  StreamContext stream
) {
  const mp::EwPtrs<1, 1> ptrs{{a}, {b}};
  mp::ew_launch<Scalar, 1, 1, 1>(ptrs, N, SeluFn_Scalar{}, get_stream(stream));
}
