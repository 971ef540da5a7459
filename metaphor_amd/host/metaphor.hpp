/*
 * Host side of the hot path, in C++ above the C-ABI boundary.
 *
 * Mirrors the reference's public surface for this path (src/metaphor.zig:13-56) with the same
 * names, argument meaning and error behaviour, so a program written against the Zig library
 * reads the same here:
 *   mp::device::{init, sync, check, total_memory}       src/metaphor.zig:13-18
 *   mp::stream::{init, deinit, sync}, 16 slots          src/core/utils.zig:39-111
 *   mp::Graph / mp::Tensor / GraphConfig / TensorClass  src/core/graph.zig:28-121, 256-363, 500-631
 *   mp::ops::{add, sub, hadamard, translate, dilate, relu, reduce, broadcast, inner_product,
 *             inner_product_scaled, permutate}           src/metaphor.zig:44-56, src/ops/*.zig
 *   mp::ops::{selu, softmax, rmsnorm}                   new ops in the same shape
 *   mp::io::{save_tensor, load_tensor}, Graph::{save, load}   src/core/tensor_file.zig
 *   mp::algo::{fill, copy, sequence}, mp::util::{to_device, from_device}, mp::stream::Group<N>
 * Errors follow the reference: an impossible request panics (prints and aborts), nothing returns
 * a status.
 *
 * What is new here is where the kernels come from. add / sub / hadamard / selu / relu / dilate /
 * translate do not launch:
 * they record a pending node. A pending node is materialised when something needs its bytes (a
 * non-elementwise op, data_ptr(), native(), reverse()). At that point the recorded expression is
 * written out with its leaves numbered in order of first appearance and looked up in the table
 * of generated fused chains (chains.hpp, from chains.json): selu(hadamard(add(a,b), add(c,d)))
 * becomes ONE launch of launch_fused_selu_hadamard_add_add and, in reverse, one launch of its
 * _reverse twin. An expression that is not in the table runs one launch per op exactly as the
 * reference does (src/ops/addition.zig:27-58, src/ops/hadamard.zig:25-56), each of its operands
 * getting the same chance first -- unless the graph was made with Fusion::any, which has such an
 * expression compiled at run time (mpChainForward / mpChainReverse) and runs it as one kernel too.
 */
#ifndef MP_HOST_METAPHOR_HPP
#define MP_HOST_METAPHOR_HPP

#include <cstddef>
#include <cstdint>
#include <string>
#include <unordered_map>
#include <vector>

#include "chain_fusion.h"
#include "device_utils.h"
#include "kernel_decls.h"

namespace mp {

[[noreturn]] void panic(const char* what);

/* src/core/scalar.zig:35-66 */
enum class Tag : int { r16 = 0, r32 = 1, r64 = 2 };
inline size_t tag_size(Tag t) { return t == Tag::r16 ? 2 : t == Tag::r32 ? 4 : 8; }

/* src/core/graph.zig:28-32 */
enum class TensorClass : int { inp = 0, wgt = 1, hid = 2 };
enum class Mode { train, eval };
enum class ReverseCleanup { keep, free };

/* src/core/utils.zig:8-37 */
struct StreamEntry {
  size_t ID = 0;
  StreamContext context{};
  void* scratch_head = nullptr;
  size_t scratch_bytes = 0;
  /* grows on demand; the previous block is released in stream order */
  void* get_scratch(size_t bytes);
};
using Stream = StreamEntry*;
constexpr size_t MAX_STREAMS = 16;

namespace device {
void init(uint32_t device_number);
void sync();
void check();
size_t total_memory(uint32_t device_number);
}  // namespace device

namespace stream {
Stream init();
void deinit(Stream s);
void sync(Stream s);
/* N streams made, synchronised and released together (src/core/utils.zig:47-71). */
template <size_t N> struct Group {
  static_assert(N <= MAX_STREAMS, "Stream group is larger than max streams.");
  Stream items[N];
  static Group init() {
    Group g;
    for (size_t i = 0; i < N; ++i) g.items[i] = stream::init();
    return g;
  }
  void synchronize() const {
    for (size_t i = 0; i < N; ++i) stream::sync(items[i]);
  }
  void deinit() const {
    for (size_t i = 0; i < N; ++i) stream::deinit(items[i]);
  }
};
}  // namespace stream

class Graph;

struct TensorData {
  void* ptr = nullptr;
  size_t len = 0; /* elements; 0 after free */
  Tag dtype = Tag::r32;
};

/* src/core/graph.zig:34-183 */
struct Tensor {
  Graph* ptr = nullptr;
  size_t idx = 0;
  TensorClass cls = TensorClass::inp;

  bool same(const Tensor& o) const { return ptr == o.ptr && idx == o.idx && cls == o.cls; }
  Tag dtype() const;
  const std::vector<size_t>& sizes() const;
  size_t len() const;   /* 0 once freed */
  size_t rank() const { return sizes().size(); }
  void* data_ptr() const;   /* materialises a pending node */
  void* grad_ptr() const;   /* nullptr when no gradient exists */
  bool has_grad() const { return grad_ptr() != nullptr; }
  Stream stream() const;
  StreamContext context() const;
  void detach() const;
  void free() const;
  void reverse(ReverseCleanup cleanup) const;
  /* host copies (blocking); grad is empty when no gradient exists */
  template <class T> std::vector<T> native() const { return native_bytes<T>(false); }
  template <class T> std::vector<T> native_grad() const { return native_bytes<T>(true); }

 private:
  void copy_out(void* dst, size_t bytes, bool grad) const;
  template <class T> std::vector<T> native_bytes(bool grad) const {
    if (sizeof(T) != tag_size(dtype())) panic("Tensor.native: element type does not match dtype");
    if (grad && !has_grad()) return {};
    std::vector<T> out(len());
    copy_out(out.data(), out.size() * sizeof(T), grad);
    return out;
  }
};

/* src/core/graph.zig:776-829: a tensor, a scalar or an index expression such as "ij,jk->ik" */
struct OpDatum {
  enum Kind { tensor, scalar, expr } kind = tensor;
  Tensor t{};
  double s = 0.0;
  std::string e;
  OpDatum(Tensor x) : kind(tensor), t(x) {}
  OpDatum(double v) : kind(scalar), s(v) {}
  OpDatum(const char* x) : kind(expr), e(x) {}
  OpDatum(const std::string& x) : kind(expr), e(x) {}
};

/* src/core/graph.zig:776-829: reverse through a table of functions, arguments stored by value */
struct OpInterface {
  void (*reverse)(const std::vector<OpDatum>&) = nullptr;
  std::vector<OpDatum> args;
  bool live = false;
};

/* Which pending elementwise expressions become one kernel per direction: the ones the build
 * listed (the generated table of chains.hpp), or any expression, compiled when it is first met
 * (chain_fusion.h). With `any` the tensors inside an expression never exist, so they have neither
 * values nor gradients of their own unless somebody asks for their bytes; `listed` keeps every
 * expression outside the table exactly as the reference runs it, one launch and one tensor per op. */
enum class Fusion { listed, any };

struct GraphConfig {
  Stream stream = nullptr;
  Mode mode = Mode::train;
  Fusion fusion = Fusion::listed;
};

/* Exact-byte-size free-list cache over the stream-ordered allocator
 * (src/core/tensor_allocator.zig:95-141). */
class TensorAllocator {
 public:
  TensorData alloc(Tag dtype, size_t n, Stream s);
  void free(TensorData d, Stream s);
  void deinit(Stream s);

 private:
  std::unordered_map<size_t, std::vector<void*>> cache_;
};

enum class Pending : int { none = 0, add, sub, hadamard, selu, relu, dilate, translate };

/* deferred elementwise nodes: record, query, compute; value is the constant of dilate / translate */
Tensor defer(Graph* g, Pending op, Tensor x, Tensor y, double value = 0.0);
bool is_pending(Tensor t);
void materialise(Tensor t);

class Graph {
 public:
  static Graph* init(GraphConfig config);
  void deinit();

  /* src/core/graph.zig:500-520 */
  Tensor tensor(TensorClass cls, Tag dtype, const std::vector<size_t>& sizes);

  enum class ResetGroup { node, leaf };
  enum class ResetComponent { all, grd };
  void reset(ResetGroup group, ResetComponent component);

  Mode mode = Mode::train;
  Stream stream = nullptr;
  Fusion fusion = Fusion::listed;
  /* the shapes of the expressions this graph had compiled at run time (constants spelled "#": a value
   * that changes from call to call is an argument of the same kernel) */
  std::vector<std::string> runtime_chains_;

  /* kernels enqueued through this graph so far (fusion is observable through it) */
  size_t launches = 0;

  /* materialise every pending node; called before anything mutates tensor bytes in place */
  void flush();

  /* Checkpoints in the reference's format (src/core/tensor_file.zig:25-86 and the save / load
   * walk of src/core/graph.zig:633-702): the raw bytes of every weight leaf, one file per
   * weight named <prefix>_<n> with n counting the weights in creation order. */
  void save(const std::string& dir, const std::string& prefix);
  void load(const std::string& dir, const std::string& prefix);

  /* core internals, public to the op modules as src/core/root.zig exports them */
  struct Leaf {
    TensorData data, grad;
    std::vector<size_t> sizes;
    TensorClass cls;
  };
  struct Node {
    TensorData data, grad;
    std::vector<size_t> sizes;
    OpInterface op;
    int deps = 0;
    bool attached = true;
    Pending pending = Pending::none; /* recorded, not yet computed */
    Tensor in0{}, in1{};
    double value = 0.0; /* dilate, translate: the constant */
  };
  std::vector<Leaf> leaves_;
  std::vector<Node> nodes_;
  TensorAllocator allocator_;

  void reverse(size_t idx, ReverseCleanup cleanup);
  void free_tensor(Tensor t);
  void free_gradient(Tensor t);
  TensorData& data_of(Tensor t);
  TensorData& grad_of(Tensor t);

 private:
  Graph() = default;
};

/* src/core/graph.zig:205-209, 710-757 */
inline size_t dkey(Tensor t) { return (size_t)t.dtype(); }
void enable_gradient(Tensor t); /* allocates AND zeroes: every reverse kernel accumulates */
void attach_op(Tensor t, void (*rev)(const std::vector<OpDatum>&), std::vector<OpDatum> args);

namespace ops {
Tensor add(Tensor x, Tensor y);
Tensor sub(Tensor x, Tensor y);
Tensor hadamard(Tensor x, Tensor y);
Tensor selu(Tensor x);
Tensor relu(Tensor x);
Tensor translate(Tensor x, double value); /* src/ops/translate.zig */
Tensor dilate(Tensor x, double value);    /* src/ops/dilate.zig */
/* src/ops/reduce.zig: "ij->i", "ij->j"; src/ops/broadcast.zig: "i->ij", "j->ij" */
Tensor reduce(Tensor x, const char* expr);
Tensor broadcast(Tensor x, const std::vector<size_t>& sizes, const char* expr);
/* src/ops/permutate.zig: "ij->ji" */
Tensor permutate(Tensor x, const char* expr);
/* src/ops/inner_product.zig: "ij,jk->ik", "ij,kj->ik", "ji,jk->ik", "ij,j->i", "i,ij->j".
 * Transposed operands go to the matrix-product launchers as flags: nothing is transposed into
 * scratch first, forward or reverse. */
Tensor inner_product(Tensor x, Tensor y, const char* expr);
Tensor inner_product_scaled(Tensor x, Tensor y, double scale, const char* expr);
/* expr names the axis in the reference's notation; "ij|j" (rows over the last dim) is supported */
Tensor softmax(Tensor x, const char* expr = "ij|j");
Tensor rmsnorm(Tensor x, Tensor gain, double eps);
}  // namespace ops

namespace algo {
void fill(Tensor t, double value);
void copy(Tensor src, Tensor dst);
void sequence(Tensor t, double init, double step);
}  // namespace algo

/* src/core/tensor_file.zig:88-149: one tensor to / from a named file of raw bytes */
namespace io {
void save_tensor(const std::string& dir, const std::string& filename, Tensor x);
void load_tensor(const std::string& dir, const std::string& filename, Tensor x);
}  // namespace io

namespace util {
void to_device(const void* src, Tensor dst, size_t bytes);
void from_device(Tensor src, void* dst, size_t bytes);
}  // namespace util

}  // namespace mp

#endif
