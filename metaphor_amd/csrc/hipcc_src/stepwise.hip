#include "../elementwise.h"

struct StepwiseFn_Scalar {
  template <class P> __device__ __forceinline__ void apply(const P (&in)[1], P (&out)[1]) const {
    out[0] = in[0] >= (P)0 ? (P)1 : (P)0;
  }
};

// b = (a >= 0) ? 1 : 0, the derivative of relu that src/ops/relu.zig:54-57 asks this launcher
// for. The reference body (src/cuda/nvcc_src/stepwise.cu:11-12) is a verbatim copy of relu and
// returns a itself for a >= 0; the step function is what its caller needs.
extern "C" void launch_stepwise_Scalar(
  const void* a,
  void* b,
  len_t n,
  StreamContext stream
) {
  const mp::EwPtrs<1, 1> ptrs{{a}, {b}};
  mp::ew_launch<Scalar, 1, 1, 1>(ptrs, n, StepwiseFn_Scalar{}, get_stream(stream));
}
