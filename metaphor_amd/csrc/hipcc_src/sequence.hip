#include "../elementwise.h"

struct SequenceFn_Scalar {
  static constexpr bool needs_index = true;
  double init, step;
  template <class P> __device__ __forceinline__ void apply(const P (&)[1], P (&out)[1], size_t index) const {
    out[0] = (P)init + (P)step * (P)index;
  }
};

// dev_a[i] = init + step * i. Replaces src/cuda/nvcc_src/sequence.cu:5-32; evaluated in
// precision<T>, so r16 does not lose the index above 2048 as Scalar(tid) does there.
extern "C" void launch_sequence_Scalar(
  void* dev_a,
  double init,
  double step,
  len_t N,
  StreamContext stream
) {
  const mp::EwPtrs<0, 1> ptrs{{nullptr}, {dev_a}};
  mp::ew_launch<Scalar, 0, 1, 1>(ptrs, N, SequenceFn_Scalar{(double)static_cast<Scalar>(init), (double)static_cast<Scalar>(step)}, get_stream(stream));
}
