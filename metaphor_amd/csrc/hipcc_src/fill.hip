#include "../elementwise.h"

struct FillFn_Scalar {
  double value;
  template <class P> __device__ __forceinline__ void apply(const P (&)[1], P (&out)[1]) const {
    out[0] = (P)value;
  }
};

// dev_a = value. Replaces src/cuda/nvcc_src/fill.cu:4-27; seeds dL/dz = 1 on the reverse path
// (src/core/graph.zig:116).
extern "C" void launch_fill_Scalar(
  void* dev_a,
  double value,
  len_t N,
  StreamContext stream
) {
  const mp::EwPtrs<0, 1> ptrs{{nullptr}, {dev_a}};
  mp::ew_launch<Scalar, 0, 1, 1>(ptrs, N, FillFn_Scalar{(double)static_cast<Scalar>(value)}, get_stream(stream));
}
