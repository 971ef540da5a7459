#include "../elementwise.h"

struct FusedReverseBlendFn_Scalar {
  double alpha;
  template <class P> __device__ __forceinline__ void apply(const P (&in)[9], P (&out)[4]) const {
    const P u = in[0] + in[1], v = in[2] + in[3];
    const P g = in[4] * mp::selu_slope(u * v);
    const P al = (P)alpha;
    out[0] = g * v + al * in[5];
    out[1] = g * v + al * in[6];
    out[2] = g * u + al * in[7];
    out[3] = g * u + al * in[8];
  }
};

// Reverse of e = selu((a + b) * (c + d)) in one pass. With u = a+b, v = c+d, w = u*v and
// g = de * selu'(w):  da = db = g*v,  dc = dd = g*u, each written as val + alpha*old
// (the blend convention of src/cuda/nvcc_src/permutate_ij_ji.cu:37-38). alpha == 0 never
// reads the old gradients: 5 reads and 4 writes per element, against the reference's seven
// read-modify-write launches (src/ops/hadamard.zig:65-79, src/ops/addition.zig:67-81).
struct FusedReverseOverwriteFn_Scalar {
  template <class P> __device__ __forceinline__ void apply(const P (&in)[5], P (&out)[4]) const {
    const P u = in[0] + in[1], v = in[2] + in[3];
    const P g = in[4] * mp::selu_slope(u * v);
    out[0] = out[1] = g * v;
    out[2] = out[3] = g * u;
  }
};

extern "C" void launch_fused_selu_hadamard_add_add_reverse_Scalar(
  const void* a,
  const void* b,
  const void* c,
  const void* d,
  const void* e_grads,
  void* a_grads,
  void* b_grads,
  void* c_grads,
  void* d_grads,
  double alpha,
  len_t N,
  StreamContext stream
) {
  if (alpha == 0.0) {
    const mp::EwPtrs<5, 4> ptrs{{a, b, c, d, e_grads}, {a_grads, b_grads, c_grads, d_grads}};
    mp::ew_launch<Scalar, 5, 4, 1>(ptrs, N, FusedReverseOverwriteFn_Scalar{}, get_stream(stream));
  } else {
    const mp::EwPtrs<9, 4> ptrs{{a, b, c, d, e_grads, a_grads, b_grads, c_grads, d_grads},
                                {a_grads, b_grads, c_grads, d_grads}};
    mp::ew_launch<Scalar, 9, 4, 1>(ptrs, N, FusedReverseBlendFn_Scalar{alpha}, get_stream(stream));
  }
}
