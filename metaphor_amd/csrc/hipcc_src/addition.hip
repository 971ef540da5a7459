#include "../elementwise.h"

struct AdditionFn_Scalar {
  template <class P> __device__ __forceinline__ void apply(const P (&in)[2], P (&out)[1]) const {
    out[0] = in[0] + in[1];
  }
};

// c = a + b. Replaces src/cuda/nvcc_src/addition.cu:3-29. The reference also calls this
// launcher in place as the reverse of add (c aliasing b, src/ops/addition.zig:67-81).
extern "C" void launch_addition_Scalar(
  const void* a,
  const void* b,
  void* c,
  len_t N,
  StreamContext stream
) {
  const mp::EwPtrs<2, 1> ptrs{{a, b}, {c}};
  mp::ew_launch<Scalar, 2, 1, 1>(ptrs, N, AdditionFn_Scalar{}, get_stream(stream));
}
