#include "../elementwise.h"

struct FusedSeluHadamardAddAddFn_Scalar {
  template <class P> __device__ __forceinline__ void apply(const P (&in)[4], P (&out)[1]) const {
    out[0] = mp::selu_value((in[0] + in[1]) * (in[2] + in[3]));
  }
};

// e = selu((a + b) * (c + d)) in one pass: 4 reads and 1 write per element, where the
// reference's composition (README.md:89-97) takes four launches and three temporaries
// (src/cuda/nvcc_src/addition.cu:12 twice, hadamard.cu:12, then the activation).
extern "C" void launch_fused_selu_hadamard_add_add_Scalar(
  const void* a,
  const void* b,
  const void* c,
  const void* d,
  void* e,
  len_t N,
  StreamContext stream
) {
  const mp::EwPtrs<4, 1> ptrs{{a, b, c, d}, {e}};
  mp::ew_launch<Scalar, 4, 1, 1>(ptrs, N, FusedSeluHadamardAddAddFn_Scalar{}, get_stream(stream));
}
