#include "../elementwise.h"

struct ReluReverseFn_Scalar {
  template <class P> __device__ __forceinline__ void apply(const P (&in)[3], P (&out)[1]) const {
    out[0] = in[1] + in[2] * (in[0] >= (P)0 ? (P)1 : (P)0);
  }
};

// a_grads += b_grads * ((a_value >= 0) ? 1 : 0). Replaces src/cuda/nvcc_src/relu_reverse.cu:3-31.
extern "C" void launch_relu_reverse_Scalar(
  const void* a_value,
  void* a_grads,
  const void* b_grads,
  len_t N,
  StreamContext stream
) {
  const mp::EwPtrs<3, 1> ptrs{{a_value, a_grads, b_grads}, {a_grads}};
  mp::ew_launch<Scalar, 3, 1, 1>(ptrs, N, ReluReverseFn_Scalar{}, get_stream(stream));
}
