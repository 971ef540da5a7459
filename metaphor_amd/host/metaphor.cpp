/*
 * Host side of the hot path: stream registry, tensor allocator, graph / autograd walk, op
 * modules and the deferred-elementwise fusion. See metaphor.hpp for the map to the reference.
 * Everything device-side goes through the C-ABI (mp* utilities and launch_* kernels); no HIP
 * header is needed to build this file.
 */
#include "metaphor.hpp"

#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <mutex>
#include <string>

#include "chains.hpp"
#include "kernels.hpp"

namespace mp {

void panic(const char* what) {
  fprintf(stderr, "metaphor: %s\n", what);
  abort();
}

/* ------------------------------------------------------------------ streams / device */

static std::mutex stream_mutex;
static StreamEntry stream_array[MAX_STREAMS];
static bool stream_used[MAX_STREAMS];

void* StreamEntry::get_scratch(size_t bytes) {
  if (scratch_bytes < bytes) {
    if (scratch_head) mpMemFree(scratch_head, context);
    scratch_head = mpMemAlloc(bytes, context);
    if (!scratch_head) panic("get_scratch: device allocation failed");
    scratch_bytes = bytes;
  }
  return scratch_head;
}

namespace device {
void init(uint32_t device_number) { mpInitDevice(device_number); }
void sync() { mpDeviceSynchronize(); }
void check() { mpCheckLastError(); }
size_t total_memory(uint32_t device_number) { return mpDeviceTotalMemory(device_number); }
}  // namespace device

namespace stream {
Stream init() {
  std::lock_guard<std::mutex> lock(stream_mutex);
  for (size_t i = 0; i < MAX_STREAMS; ++i) {
    if (!stream_used[i]) {
      stream_used[i] = true;
      stream_array[i] = StreamEntry{};
      stream_array[i].ID = i;
      stream_array[i].context = mpInitStream();
      return &stream_array[i];
    }
  }
  panic("stream limit reached - increase streams");
}

void deinit(Stream s) {
  if (s->scratch_head) {
    mpMemFree(s->scratch_head, s->context);
    mpStreamSynchronize(s->context);
  }
  mpDeinitStream(s->context);
  mpDeviceSynchronize();
  std::lock_guard<std::mutex> lock(stream_mutex);
  stream_used[s->ID] = false;
}

void sync(Stream s) { mpStreamSynchronize(s->context); }
}  // namespace stream

/* ------------------------------------------------------------------ tensor allocator */

TensorData TensorAllocator::alloc(Tag dtype, size_t n, Stream s) {
  const size_t bytes = n * tag_size(dtype);
  auto it = cache_.find(bytes);
  void* p = nullptr;
  if (it != cache_.end() && !it->second.empty()) {
    p = it->second.back();
    it->second.pop_back();
  } else {
    p = mpMemAlloc(bytes, s->context);
    if (!p) panic("TensorAllocator.alloc: device allocation failed");
  }
  return TensorData{p, n, dtype};
}

void TensorAllocator::free(TensorData d, Stream) {
  if (!d.ptr) return;
  cache_[d.len * tag_size(d.dtype)].push_back(d.ptr);
}

void TensorAllocator::deinit(Stream s) {
  for (auto& kv : cache_)
    for (void* p : kv.second) mpMemFree(p, s->context);
  cache_.clear();
}

/* ------------------------------------------------------------------ graph */

Graph* Graph::init(GraphConfig config) {
  if (!config.stream) panic("Graph.init: a stream is required");
  Graph* g = new Graph();
  g->stream = config.stream;
  g->mode = config.mode;
  g->fusion = config.fusion;
  return g;
}

void Graph::deinit() {
  reset(ResetGroup::node, ResetComponent::all);
  reset(ResetGroup::leaf, ResetComponent::all);
  allocator_.deinit(stream);
  mpStreamSynchronize(stream->context);
  delete this;
}

TensorData& Graph::data_of(Tensor t) {
  return t.cls == TensorClass::hid ? nodes_[t.idx].data : leaves_[t.idx].data;
}
TensorData& Graph::grad_of(Tensor t) {
  return t.cls == TensorClass::hid ? nodes_[t.idx].grad : leaves_[t.idx].grad;
}

Tensor Graph::tensor(TensorClass cls, Tag dtype, const std::vector<size_t>& sizes) {
  if (sizes.empty()) panic("Graph.tensor: sizes must not be empty");
  size_t n = 1;
  for (size_t s : sizes) n *= s;
  if (n == 0) panic("Graph.tensor: every size must be positive");
  if (cls == TensorClass::hid) {
    Node node;
    node.data = allocator_.alloc(dtype, n, stream);
    node.sizes = sizes;
    nodes_.push_back(std::move(node));
    return Tensor{this, nodes_.size() - 1, cls};
  }
  Leaf leaf;
  leaf.data = allocator_.alloc(dtype, n, stream);
  leaf.sizes = sizes;
  leaf.cls = cls;
  leaves_.push_back(std::move(leaf));
  return Tensor{this, leaves_.size() - 1, cls};
}

void Graph::free_gradient(Tensor t) {
  TensorData& g = grad_of(t);
  if (g.ptr) {
    allocator_.free(g, stream);
    g = TensorData{};
  }
}

void Graph::free_tensor(Tensor t) {
  TensorData& d = data_of(t);
  if (d.len == 0) return;
  if (d.ptr) allocator_.free(d, stream);
  d.ptr = nullptr;
  d.len = 0;
  if (t.cls == TensorClass::hid) nodes_[t.idx].pending = Pending::none;
  free_gradient(t);
}

void Graph::reset(ResetGroup group, ResetComponent component) {
  if (group == ResetGroup::leaf) {
    for (size_t i = 0; i < leaves_.size(); ++i) {
      Tensor t{this, i, leaves_[i].cls};
      if (component == ResetComponent::grd) free_gradient(t);
      else free_tensor(t);
    }
    if (component == ResetComponent::all) leaves_.clear();
  } else {
    for (size_t i = 0; i < nodes_.size(); ++i) {
      Tensor t{this, i, TensorClass::hid};
      if (component == ResetComponent::grd) {
        free_gradient(t);
        nodes_[i].deps = 0;
      } else {
        free_tensor(t);
      }
    }
    if (component == ResetComponent::all) nodes_.clear();
  }
}

void enable_gradient(Tensor t) {
  Graph* g = t.ptr;
  TensorData& grd = g->grad_of(t);
  if (!grd.ptr) {
    grd = g->allocator_.alloc(t.dtype(), t.len(), g->stream);
    /* the reference leaves new gradient storage unwritten (src/core/graph.zig:710-722) although
     * every reverse kernel accumulates into it; here it starts at zero */
    kernels::fill(dkey(t), grd.ptr, 0.0, (len_t)grd.len, g->stream->context);
    g->launches++;
  }
}

void attach_op(Tensor t, void (*rev)(const std::vector<OpDatum>&), std::vector<OpDatum> args) {
  if (t.cls != TensorClass::hid) panic("attach_op: only computed tensors carry an op");
  Graph* g = t.ptr;
  for (size_t i = 0; i + 1 < args.size(); ++i) { /* the last argument is the output itself */
    const OpDatum& a = args[i];
    if (a.kind == OpDatum::tensor && a.t.cls == TensorClass::hid) g->nodes_[a.t.idx].deps += 1;
  }
  OpInterface& op = g->nodes_[t.idx].op;
  op.reverse = rev;
  op.args = std::move(args);
  op.live = true;
}

/* src/core/graph.zig:552-631 */
void Graph::reverse(size_t idx, ReverseCleanup cleanup) {
  if (mode == Mode::eval) panic("Graph.reverse: graph is in eval mode");
  if (nodes_.empty()) return;
  std::vector<size_t> node_stack{idx}, free_stack;
  while (!node_stack.empty()) {
    const size_t last = node_stack.back();
    node_stack.pop_back();
    OpInterface& op = nodes_[last].op;
    if (!op.live) continue;
    if (cleanup == ReverseCleanup::free) free_stack.push_back(last);
    op.reverse(op.args);
    for (const OpDatum& arg : op.args) {
      if (arg.kind != OpDatum::tensor) continue;
      if (arg.t.cls != TensorClass::hid || arg.t.idx == last) continue;
      if (!nodes_[arg.t.idx].attached) continue;
      if (--nodes_[arg.t.idx].deps == 0) node_stack.push_back(arg.t.idx);
    }
    op.args.clear();
    op.live = false;
  }
  if (cleanup == ReverseCleanup::free) {
    mpStreamSynchronize(stream->context);
    for (size_t node : free_stack) free_tensor(Tensor{this, node, TensorClass::hid});
  }
}

/* ------------------------------------------------------------------ tensor */

Tag Tensor::dtype() const { return ptr->data_of(*this).dtype; }
const std::vector<size_t>& Tensor::sizes() const {
  return cls == TensorClass::hid ? ptr->nodes_[idx].sizes : ptr->leaves_[idx].sizes;
}
size_t Tensor::len() const { return ptr->data_of(*this).len; }
Stream Tensor::stream() const { return ptr->stream; }
StreamContext Tensor::context() const { return ptr->stream->context; }
void* Tensor::grad_ptr() const { return ptr->grad_of(*this).ptr; }
void Tensor::detach() const {
  if (cls == TensorClass::hid) ptr->nodes_[idx].attached = false;
}
void Tensor::free() const { ptr->free_tensor(*this); }

void* Tensor::data_ptr() const {
  materialise(*this);
  return ptr->data_of(*this).ptr;
}

void Tensor::reverse(ReverseCleanup cleanup) const {
  materialise(*this);
  if (!has_grad()) {
    /* no loss applied: d self / d self = 1 (src/core/graph.zig:112-117) */
    ptr->grad_of(*this) = ptr->allocator_.alloc(dtype(), len(), ptr->stream);
    kernels::fill(dkey(*this), grad_ptr(), 1.0, (len_t)len(), context());
    ptr->launches++;
  }
  if (cls != TensorClass::hid) return;
  ptr->reverse(idx, cleanup);
}

void Tensor::copy_out(void* dst, size_t bytes, bool grad) const {
  const void* src = grad ? grad_ptr() : data_ptr();
  mpMemcpyDtoH(dst, src, bytes, context()); /* returns with the bytes on the host */
}

/* ------------------------------------------------------------------ deferred elementwise */

bool is_pending(Tensor t) {
  return t.cls == TensorClass::hid && t.ptr->nodes_[t.idx].pending != Pending::none;
}

/* A pending node owns no bytes yet: its buffer is taken from the allocator when it is computed. */
Tensor defer(Graph* g, Pending op, Tensor x, Tensor y, double value) {
  Graph::Node node;
  node.value = value;
  node.data = TensorData{nullptr, x.len(), x.dtype()};
  node.sizes = x.sizes();
  node.pending = op;
  node.in0 = x;
  node.in1 = y;
  g->nodes_.push_back(std::move(node));
  return Tensor{g, g->nodes_.size() - 1, TensorClass::hid};
}

static void addition_reverse(const std::vector<OpDatum>& a);
static void subtraction_reverse(const std::vector<OpDatum>& a);
static void hadamard_reverse(const std::vector<OpDatum>& a);
static void selu_reverse(const std::vector<OpDatum>& a);
static void relu_reverse(const std::vector<OpDatum>& a);
static void translate_reverse(const std::vector<OpDatum>& a);
static void dilate_reverse(const std::vector<OpDatum>& a);
static void chain_reverse(const std::vector<OpDatum>& a);
static void runtime_chain_reverse(const std::vector<OpDatum>& a);

static const char* pending_name(Pending op) {
  switch (op) {
    case Pending::add: return "add";
    case Pending::sub: return "sub";
    case Pending::hadamard: return "mul";
    case Pending::selu: return "selu";
    case Pending::relu: return "relu";
    case Pending::dilate: return "scale";
    case Pending::translate: return "shift";
    default: return "?";
  }
}

/* The expression below t, as the chain table spells it: pending nodes of this graph become
 * op(...), everything else a leaf numbered in order of first appearance (the same tensor keeps
 * its number). Gives up (returns false) beyond eight leaves or 64 nodes. shape_only: the constants of
 * dilate and translate are spelled "#" (expressions that differ in them only are one kernel). */
static bool spell(Graph* g, Tensor t, std::string& out, std::vector<Tensor>& leaves, int& budget, bool shape_only = false) {
  if (--budget < 0) return false;
  if (is_pending(t) && t.ptr == g) {
    const Graph::Node& node = g->nodes_[t.idx];
    out += pending_name(node.pending);
    out += '(';
    if (!spell(g, node.in0, out, leaves, budget, shape_only)) return false;
    if (node.pending == Pending::dilate || node.pending == Pending::translate) {
      char text[40]; /* the constant as every generator of chains spells it; "#" when only the shape is asked for */
      snprintf(text, sizeof text, ",%.17g", node.value);
      out += shape_only ? ",#" : text;
    } else if (node.pending != Pending::selu && node.pending != Pending::relu) {
      out += ',';
      if (!spell(g, node.in1, out, leaves, budget, shape_only)) return false;
    }
    out += ')';
    return true;
  }
  size_t k = 0;
  while (k < leaves.size() && !leaves[k].same(t)) ++k;
  if (k == leaves.size()) {
    if (leaves.size() == 8) return false;
    leaves.push_back(t);
  }
  out += std::to_string(k);
  return true;
}

static const FusedChain* find_chain(const std::string& signature) {
  for (const FusedChain& c : fused_chains)
    if (signature == c.signature) return &c;
  return nullptr;
}

/* The pending nodes of this graph inside the expression below t (t itself included when pending). */
static void pending_below(Graph* g, Tensor t, std::vector<size_t>& out, int& budget) {
  if (--budget < 0 || !(is_pending(t) && t.ptr == g)) return;
  out.push_back(t.idx);
  const Graph::Node& node = g->nodes_[t.idx];
  pending_below(g, node.in0, out, budget);
  if (node.pending != Pending::selu && node.pending != Pending::relu && node.pending != Pending::dilate &&
      node.pending != Pending::translate)
    pending_below(g, node.in1, out, budget);
}

/* Several results in one kernel: other pending results of this graph (pending nodes that no pending
 * node consumes) whose expressions share a pending subexpression with t's are computed with it, as
 * one forward launch with as many output streams (mpChainForwardMany), so that what they share is
 * read and computed once: u = a + b; e1 = selu(u * c); e2 = relu(u - d) is one launch. Each result
 * keeps a reverse of its own (its own expression, one launch each): the graph's reverse walk
 * reaches the results one at a time. True when t was computed this way. */
static bool materialise_with_siblings(Graph* g, Tensor t, const std::string& signature, const std::vector<Tensor>& leaves) {
  int budget = 64;
  std::vector<size_t> mine;
  pending_below(g, t, mine, budget);
  if (mine.size() < 2) return false; /* nothing below t that another result could share */
  std::vector<char> consumed(g->nodes_.size(), 0), shared(g->nodes_.size(), 0);
  size_t first = g->nodes_.size();
  for (size_t i = 0; i < g->nodes_.size(); ++i) {
    const Graph::Node& node = g->nodes_[i];
    if (node.pending == Pending::none) continue;
    for (const Tensor& in : {node.in0, node.in1})
      if (in.ptr == g && in.cls == TensorClass::hid && in.idx < consumed.size()) consumed[in.idx] = 1;
  }
  for (size_t i : mine)
    if (i != t.idx) {
      shared[i] = 1;
      first = i < first ? i : first;
    }
  struct Root { Tensor t; std::string own; std::vector<Tensor> own_leaves; };
  std::vector<Root> roots{{t, signature, leaves}};
  std::string combined = signature;
  std::vector<Tensor> all = leaves;
  for (size_t i = first + 1; i < g->nodes_.size() && roots.size() < 4; ++i) {
    const Graph::Node& node = g->nodes_[i];
    if (i == t.idx || node.pending == Pending::none || consumed[i]) continue;
    if (node.data.len != g->nodes_[t.idx].data.len || node.data.dtype != g->nodes_[t.idx].data.dtype) continue;
    const Tensor other{g, i, TensorClass::hid};
    std::vector<size_t> theirs;
    int room = 64;
    pending_below(g, other, theirs, room);
    bool overlap = false;
    for (size_t j : theirs) overlap = overlap || shared[j];
    if (!overlap) continue;
    std::string text, own;
    std::vector<Tensor> together = all, own_leaves;
    int b1 = 64, b2 = 64;
    if (!spell(g, other, text, together, b1) || !spell(g, other, own, own_leaves, b2)) continue; /* too many leaves: it stays by itself */
    combined += ";" + text;
    all = together;
    roots.push_back({other, own, own_leaves});
  }
  if (roots.size() < 2 || mpChainCompile(combined.c_str(), (int)t.dtype()) != 0) return false;
  void* x[8];
  void* outs[4];
  for (size_t i = 0; i < all.size(); ++i) {
    if (all[i].len() == 0) panic("materialise: an input of a pending node was freed");
    x[i] = all[i].data_ptr();
  }
  { /* the shape this graph had compiled */
    std::string shape;
    std::vector<Tensor> again;
    int room = 64;
    for (size_t r = 0; r < roots.size(); ++r) {
      if (r) shape += ';';
      room = 64;
      spell(g, roots[r].t, shape, again, room, true);
    }
    size_t idx = 0;
    while (idx < g->runtime_chains_.size() && g->runtime_chains_[idx] != shape) ++idx;
    if (idx == g->runtime_chains_.size()) g->runtime_chains_.push_back(shape);
  }
  const size_t n = g->nodes_[t.idx].data.len;
  const Tag dt = g->nodes_[t.idx].data.dtype;
  for (size_t r = 0; r < roots.size(); ++r) {
    TensorData d = g->allocator_.alloc(dt, n, g->stream);
    g->nodes_[roots[r].t.idx].data = d;
    g->nodes_[roots[r].t.idx].pending = Pending::none;
    outs[r] = d.ptr;
  }
  if (mpChainForwardMany(combined.c_str(), (int)dt, x, outs, (len_t)n, g->stream->context) != 0) panic(mpChainError());
  g->launches++;
  if (g->mode == Mode::train)
    for (const Root& root : roots) {
      std::vector<OpDatum> args(root.own_leaves.begin(), root.own_leaves.end());
      args.push_back(OpDatum(root.own));
      args.push_back(root.t);
      attach_op(root.t, runtime_chain_reverse, std::move(args));
    }
  return true;
}

void materialise(Tensor t) {
  if (!is_pending(t)) return;
  Graph* g = t.ptr;
  const Pending op = g->nodes_[t.idx].pending;
  const Tensor in0 = g->nodes_[t.idx].in0, in1 = g->nodes_[t.idx].in1;
  const double value = g->nodes_[t.idx].value;
  const size_t n = g->nodes_[t.idx].data.len;
  const Tag dt = g->nodes_[t.idx].data.dtype;
  const size_t key = (size_t)dt;
  const StreamContext ctx = g->stream->context;

  auto take_buffer = [&]() {
    TensorData d = g->allocator_.alloc(dt, n, g->stream);
    g->nodes_[t.idx].data = d;
    g->nodes_[t.idx].pending = Pending::none;
    return d.ptr;
  };

  /* the whole pending expression as one generated kernel, if the table has it; the inner
   * pending nodes then stay unmaterialised */
  {
    std::string signature;
    std::vector<Tensor> leaves;
    int budget = 64;
    const bool spelled = spell(g, t, signature, leaves, budget);
    const FusedChain* chain = spelled ? find_chain(signature) : nullptr;
    if (chain) {
      void* x[8];
      for (size_t i = 0; i < leaves.size(); ++i) {
        if (leaves[i].len() == 0) panic("materialise: an input of a pending node was freed");
        x[i] = leaves[i].data_ptr();
      }
      void* out = take_buffer();
      chain->forward(key, x, out, (len_t)n, ctx);
      g->launches++;
      if (g->mode == Mode::train) {
        std::vector<OpDatum> args(leaves.begin(), leaves.end());
        args.push_back(OpDatum((double)(chain - fused_chains)));
        args.push_back(t);
        attach_op(t, chain_reverse, std::move(args));
      }
      return;
    }
    /* not listed: compiled now if the graph asks for that and the expression has more than one op
     * (a single op is already one kernel). A refusal (too many leaves, a compile failure) falls
     * through to one launch per op. */
    const bool several = signature.find('(') != signature.rfind('(');
    if (g->fusion == Fusion::any && spelled && materialise_with_siblings(g, t, signature, leaves)) return;
    if (g->fusion == Fusion::any && spelled && several &&
        mpChainCompile(signature.c_str(), (int)key) == 0) {
      void* x[8];
      for (size_t i = 0; i < leaves.size(); ++i) {
        if (leaves[i].len() == 0) panic("materialise: an input of a pending node was freed");
        x[i] = leaves[i].data_ptr();
      }
      { /* the shapes this graph had compiled: a constant that changes from call to call adds nothing */
        std::string shape;
        std::vector<Tensor> again;
        int room = 64;
        spell(g, t, shape, again, room, true);
        size_t idx = 0;
        while (idx < g->runtime_chains_.size() && g->runtime_chains_[idx] != shape) ++idx;
        if (idx == g->runtime_chains_.size()) g->runtime_chains_.push_back(shape);
      }
      void* out = take_buffer();
      if (mpChainForward(signature.c_str(), (int)key, x, out, (len_t)n, ctx) != 0) panic(mpChainError());
      g->launches++;
      if (g->mode == Mode::train) { /* the reverse gets the text itself, constants included */
        std::vector<OpDatum> args(leaves.begin(), leaves.end());
        args.push_back(OpDatum(signature));
        args.push_back(t);
        attach_op(t, runtime_chain_reverse, std::move(args));
      }
      return;
    }
  }

  /* anything else: one launch per op, as the reference's forward_impl does */
  const bool with_constant = op == Pending::dilate || op == Pending::translate;
  if (in0.len() == 0 || (!with_constant && in1.len() == 0)) panic("materialise: an input of a pending node was freed");
  void* p0 = in0.data_ptr();
  if (with_constant) { /* src/ops/dilate.zig, src/ops/translate.zig */
    void* pz = take_buffer();
    if (op == Pending::dilate) kernels::dilate(key, p0, value, pz, (len_t)n, ctx);
    else kernels::translate(key, p0, value, pz, (len_t)n, ctx);
    g->launches++;
    if (g->mode == Mode::train) attach_op(t, op == Pending::dilate ? dilate_reverse : translate_reverse, {in0, value, t});
    return;
  }
  if (op == Pending::selu || op == Pending::relu) {
    void* pz = take_buffer();
    if (op == Pending::selu) kernels::selu(key, p0, pz, (len_t)n, ctx);
    else kernels::relu(key, p0, pz, (len_t)n, ctx);
    g->launches++;
    if (g->mode == Mode::train) attach_op(t, op == Pending::selu ? selu_reverse : relu_reverse, {in0, t});
    return;
  }
  void* p1 = in1.data_ptr();
  void* pz = take_buffer();
  if (op == Pending::add) {
    kernels::addition(key, p0, p1, pz, (len_t)n, ctx);
    if (g->mode == Mode::train) attach_op(t, addition_reverse, {in0, in1, t});
  } else if (op == Pending::sub) {
    kernels::subtraction(key, p0, p1, pz, (len_t)n, ctx);
    if (g->mode == Mode::train) attach_op(t, subtraction_reverse, {in0, in1, t});
  } else {
    kernels::hadamard(key, p0, p1, pz, (len_t)n, ctx);
    if (g->mode == Mode::train) attach_op(t, hadamard_reverse, {in0, in1, t});
  }
  g->launches++;
}

void Graph::flush() {
  for (size_t i = 0; i < nodes_.size(); ++i) materialise(Tensor{this, i, TensorClass::hid});
}

/* ------------------------------------------------------------------ op modules */

static void check_pair(Tensor x, Tensor y, const char* what) {
  if (x.dtype() != y.dtype()) panic(what);
  if (x.sizes() != y.sizes()) panic(what);
}

/* src/ops/addition.zig:60-82: gx = gz + gx, gy = gz + gy, in place */
static void addition_reverse(const std::vector<OpDatum>& a) {
  const Tensor x = a[0].t, y = a[1].t, z = a[2].t;
  enable_gradient(x);
  enable_gradient(y);
  const size_t key = dkey(z);
  kernels::addition(key, z.grad_ptr(), x.grad_ptr(), x.grad_ptr(), (len_t)x.len(), x.context());
  kernels::addition(key, z.grad_ptr(), y.grad_ptr(), y.grad_ptr(), (len_t)y.len(), y.context());
  z.ptr->launches += 2;
}

/* src/ops/subtraction.zig:60-82 with the sign its second launch means: gx = gz + gx, gy = gy - gz
 * (the reference passes (gz, gy) to the subtraction kernel, which yields gz - gy) */
static void subtraction_reverse(const std::vector<OpDatum>& a) {
  const Tensor x = a[0].t, y = a[1].t, z = a[2].t;
  enable_gradient(x);
  enable_gradient(y);
  const size_t key = dkey(z);
  kernels::addition(key, z.grad_ptr(), x.grad_ptr(), x.grad_ptr(), (len_t)x.len(), x.context());
  kernels::subtraction(key, y.grad_ptr(), z.grad_ptr(), y.grad_ptr(), (len_t)y.len(), y.context());
  z.ptr->launches += 2;
}

/* src/ops/hadamard.zig:58-80 */
static void hadamard_reverse(const std::vector<OpDatum>& a) {
  const Tensor x = a[0].t, y = a[1].t, z = a[2].t;
  enable_gradient(x);
  enable_gradient(y);
  const size_t key = dkey(z);
  kernels::hadamard_reverse(key, z.grad_ptr(), y.data_ptr(), x.grad_ptr(), (len_t)x.len(), x.context());
  kernels::hadamard_reverse(key, z.grad_ptr(), x.data_ptr(), y.grad_ptr(), (len_t)y.len(), y.context());
  z.ptr->launches += 2;
}

/* the shape of src/ops/relu.zig:39-52 */
static void selu_reverse(const std::vector<OpDatum>& a) {
  const Tensor x = a[0].t, z = a[1].t;
  enable_gradient(x);
  kernels::selu_reverse(dkey(z), x.data_ptr(), x.grad_ptr(), z.grad_ptr(), (len_t)x.len(), x.context());
  z.ptr->launches++;
}

static void relu_reverse(const std::vector<OpDatum>& a) {
  const Tensor x = a[0].t, z = a[1].t;
  enable_gradient(x);
  kernels::relu_reverse(dkey(z), x.data_ptr(), x.grad_ptr(), z.grad_ptr(), (len_t)x.len(), x.context());
  z.ptr->launches++;
}

/* One launch writes every leaf gradient of a generated chain. args = leaves..., chain index,
 * output. If no leaf has a gradient yet the launch creates them (alpha = 0 overwrites);
 * otherwise the missing ones are zero-filled and all are blended (alpha = 1). A tensor that
 * appears more than once in the expression is one leaf whose contributions the kernel adds. */
static void chain_reverse(const std::vector<OpDatum>& a) {
  const size_t k = a.size() - 2;
  const FusedChain& chain = fused_chains[(size_t)a[k].s];
  const Tensor out = a[k + 1].t;
  Graph* g = out.ptr;
  bool any = false;
  for (size_t i = 0; i < k; ++i) any = any || a[i].t.has_grad();
  void* x[8];
  void* grads[8];
  for (size_t i = 0; i < k; ++i) {
    const Tensor t = a[i].t;
    if (any) enable_gradient(t);
    else t.ptr->grad_of(t) = t.ptr->allocator_.alloc(t.dtype(), t.len(), t.ptr->stream);
    x[i] = t.data_ptr();
    grads[i] = t.grad_ptr();
  }
  chain.reverse(dkey(out), x, out.grad_ptr(), grads, any ? 1.0 : 0.0, (len_t)out.len(), out.context());
  g->launches++;
}

/* The same for an expression compiled at run time: args = leaves..., the expression's text, output. */
static void runtime_chain_reverse(const std::vector<OpDatum>& a) {
  const size_t k = a.size() - 2;
  const Tensor out = a[k + 1].t;
  Graph* g = out.ptr;
  const std::string& signature = a[k].e;
  bool any = false;
  for (size_t i = 0; i < k; ++i) any = any || a[i].t.has_grad();
  void* x[8];
  void* grads[8];
  for (size_t i = 0; i < k; ++i) {
    const Tensor t = a[i].t;
    if (any) enable_gradient(t);
    else t.ptr->grad_of(t) = t.ptr->allocator_.alloc(t.dtype(), t.len(), t.ptr->stream);
    x[i] = t.data_ptr();
    grads[i] = t.grad_ptr();
  }
  if (mpChainReverse(signature.c_str(), (int)dkey(out), x, out.grad_ptr(), grads, any ? 1.0 : 0.0, (len_t)out.len(),
                     out.context()) != 0)
    panic(mpChainError());
  g->launches++;
}

static void softmax_reverse(const std::vector<OpDatum>& a) {
  const Tensor x = a[0].t, z = a[1].t;
  const bool fresh = !x.has_grad();
  if (fresh) {
    TensorData& grd = x.ptr->grad_of(x);
    grd = x.ptr->allocator_.alloc(x.dtype(), x.len(), x.ptr->stream);
  }
  const size_t n = z.sizes().back(), m = z.len() / n;
  const len_t bytes = mpSoftmaxReverseScratchBytes((len_t)dkey(z), (len_t)m, (len_t)n);
  void* scratch = bytes ? z.stream()->get_scratch(bytes) : nullptr;
  kernels::softmax_ij_j_reverse(dkey(z), z.data_ptr(), z.grad_ptr(), x.grad_ptr(), scratch, fresh ? 0.0 : 1.0,
                                (len_t)m, (len_t)n, z.context());
  z.ptr->launches++;
}

static void rmsnorm_reverse(const std::vector<OpDatum>& a) {
  const Tensor x = a[0].t, gain = a[1].t, z = a[3].t;
  const double eps = a[2].s;
  const bool fresh = !x.has_grad() && !gain.has_grad();
  if (fresh) {
    x.ptr->grad_of(x) = x.ptr->allocator_.alloc(x.dtype(), x.len(), x.ptr->stream);
    gain.ptr->grad_of(gain) = gain.ptr->allocator_.alloc(gain.dtype(), gain.len(), gain.ptr->stream);
  } else {
    enable_gradient(x);
    enable_gradient(gain);
  }
  const size_t n = z.sizes().back(), m = z.len() / n;
  void* scratch = z.stream()->get_scratch(mpRmsnormReverseScratchBytes((len_t)dkey(z), (len_t)m, (len_t)n));
  kernels::rmsnorm_ij_j_reverse(dkey(z), x.data_ptr(), gain.data_ptr(), z.grad_ptr(), x.grad_ptr(),
                                gain.grad_ptr(), scratch, eps, fresh ? 0.0 : 1.0, (len_t)m, (len_t)n,
                                z.context());
  z.ptr->launches += 2;
}

/* Gradient storage on first touch. Returns the blend factor for the launcher that writes it:
 * 0 for storage just allocated (the first write overwrites, nothing is zero-filled or read
 * back), 1 for a gradient that already holds a sum. */
static double first_touch(Tensor t) {
  if (t.has_grad()) return 1.0;
  t.ptr->grad_of(t) = t.ptr->allocator_.alloc(t.dtype(), t.len(), t.ptr->stream);
  return 0.0;
}

/* column sums with the workspace that lets tall, narrow matrices use the whole GPU */
static void column_sums(Graph* g, size_t key, const void* src, void* dst, double alpha, size_t m, size_t n) {
  const len_t bytes = mpReduceScratchBytes((len_t)key, (len_t)m, (len_t)n);
  void* scratch = bytes ? g->stream->get_scratch(bytes) : nullptr;
  kernels::reduce_ij_j_scratch(key, src, dst, scratch, alpha, (len_t)m, (len_t)n, g->stream->context);
  g->launches += bytes ? 2 : 1;
}

/* src/ops/translate.zig: gx = gz + gx */
static void translate_reverse(const std::vector<OpDatum>& a) {
  const Tensor x = a[0].t, z = a[2].t;
  if (first_touch(x) == 0.0) kernels::copy(dkey(z), z.grad_ptr(), x.grad_ptr(), (len_t)x.len(), x.context());
  else kernels::addition(dkey(z), z.grad_ptr(), x.grad_ptr(), x.grad_ptr(), (len_t)x.len(), x.context());
  z.ptr->launches++;
}

/* src/ops/dilate.zig:46-58: gx += gz * value */
static void dilate_reverse(const std::vector<OpDatum>& a) {
  const Tensor x = a[0].t, z = a[2].t;
  const double value = a[1].s;
  if (first_touch(x) == 0.0) kernels::dilate(dkey(z), z.grad_ptr(), value, x.grad_ptr(), (len_t)x.len(), x.context());
  else kernels::dilate_reverse(dkey(z), z.grad_ptr(), value, x.grad_ptr(), (len_t)x.len(), x.context());
  z.ptr->launches++;
}

/* src/ops/reduce.zig:104-121,148-165: the reverse of a sum is a broadcast of its gradient */
static void reduce_reverse(const std::vector<OpDatum>& a) {
  const Tensor x = a[0].t, y = a[2].t;
  const double beta = first_touch(x);
  const len_t m = (len_t)x.sizes()[0], n = (len_t)x.sizes()[1];
  if (a[1].e == "ij->i") kernels::broadcast_i_ij(dkey(y), y.grad_ptr(), x.grad_ptr(), beta, m, n, x.context());
  else kernels::broadcast_j_ij(dkey(y), y.grad_ptr(), x.grad_ptr(), beta, m, n, x.context());
  y.ptr->launches++;
}

/* src/ops/broadcast.zig:109-125,153-169 with the sizes of the broadcast OUTPUT (the reference
 * reads them from the rank-1 input and would trip its own rank assertion) */
static void broadcast_reverse(const std::vector<OpDatum>& a) {
  const Tensor x = a[0].t, y = a[2].t;
  const double beta = first_touch(x);
  const len_t m = (len_t)y.sizes()[0], n = (len_t)y.sizes()[1];
  if (a[1].e == "i->ij") kernels::reduce_ij_i(dkey(y), y.grad_ptr(), x.grad_ptr(), beta, m, n, x.context());
  else { column_sums(y.ptr, dkey(y), y.grad_ptr(), x.grad_ptr(), beta, m, n); return; }
  y.ptr->launches++;
}

/* src/ops/permutate.zig:58-69: the gradient comes back transposed and accumulates */
static void permutate_reverse(const std::vector<OpDatum>& a) {
  const Tensor x = a[0].t, y = a[2].t;
  const double beta = first_touch(x);
  kernels::permutate_ij_ji(dkey(y), y.grad_ptr(), x.grad_ptr(), beta, (len_t)y.sizes()[0], (len_t)y.sizes()[1],
                           x.context());
  y.ptr->launches++;
}

/* The three operand forms of the matrix product, c[m,k] = alpha * op(a) . op(b) + beta * c over n. */
enum class Product { ij_jk, ij_kj, ji_jk };

static void product(Graph* g, size_t key, Product form, const void* a, const void* b, double alpha, void* c,
                    double beta, size_t m, size_t n, size_t k) {
  const StreamContext ctx = g->stream->context;
  switch (form) {
    case Product::ij_jk: kernels::inner_product_ij_jk_ik(key, a, b, alpha, c, beta, (len_t)m, (len_t)n, (len_t)k, ctx); break;
    case Product::ij_kj: kernels::inner_product_ij_kj_ik(key, a, b, alpha, c, beta, (len_t)m, (len_t)n, (len_t)k, ctx); break;
    case Product::ji_jk: kernels::inner_product_ji_jk_ik(key, a, b, alpha, c, beta, (len_t)m, (len_t)n, (len_t)k, ctx); break;
  }
  g->launches++;
}

struct ProductPlan {
  Product form;
  size_t m, n, k;            /* output rows, contraction, output columns */
  std::vector<size_t> sizes; /* of the output tensor */
};

/* src/ops/inner_product.zig:124-133 (the expression map) and :150-260 (vectors as matrices with
 * one unit dimension). */
static ProductPlan plan_product(Tensor x, Tensor y, const std::string& expr) {
  const std::vector<size_t>&xs = x.sizes(), &ys = y.sizes();
  auto need = [](bool ok) { if (!ok) panic("inner_product: operand sizes do not fit the expression"); };
  if (expr == "ij,jk->ik") { need(xs.size() == 2 && ys.size() == 2 && xs[1] == ys[0]); return {Product::ij_jk, xs[0], xs[1], ys[1], {xs[0], ys[1]}}; }
  if (expr == "ij,kj->ik") { need(xs.size() == 2 && ys.size() == 2 && xs[1] == ys[1]); return {Product::ij_kj, xs[0], xs[1], ys[0], {xs[0], ys[0]}}; }
  if (expr == "ji,jk->ik") { need(xs.size() == 2 && ys.size() == 2 && xs[0] == ys[0]); return {Product::ji_jk, xs[1], xs[0], ys[1], {xs[1], ys[1]}}; }
  if (expr == "ij,j->i") { need(xs.size() == 2 && ys.size() == 1 && xs[1] == ys[0]); return {Product::ij_jk, xs[0], xs[1], 1, {xs[0]}}; }
  if (expr == "i,ij->j") { need(xs.size() == 1 && ys.size() == 2 && xs[0] == ys[0]); return {Product::ij_jk, 1, xs[0], ys[1], {ys[1]}}; }
  panic("Invalid expression for inner product.");
}

/* The reverse products of src/ops/inner_product.zig:200-421, one launch each: with G = grad(z),
 *   z = x.y     : gx += s G.T(y)   gy += s T(x).G
 *   z = x.T(y)  : gx += s G.y      gy += s T(G).x
 *   z = T(x).y  : gx += s y.T(G)   gy += s x.G                                              */
static void inner_product_reverse(const std::vector<OpDatum>& a) {
  const Tensor x = a[0].t, y = a[1].t, z = a[4].t;
  const double s = a[2].s;
  const ProductPlan p = plan_product(x, y, a[3].e);
  Graph* g = z.ptr;
  const size_t key = dkey(z);
  const double bx = first_touch(x);
  switch (p.form) {
    case Product::ij_jk: product(g, key, Product::ij_kj, z.grad_ptr(), y.data_ptr(), s, x.grad_ptr(), bx, p.m, p.k, p.n); break;
    case Product::ij_kj: product(g, key, Product::ij_jk, z.grad_ptr(), y.data_ptr(), s, x.grad_ptr(), bx, p.m, p.k, p.n); break;
    case Product::ji_jk: product(g, key, Product::ij_kj, y.data_ptr(), z.grad_ptr(), s, x.grad_ptr(), bx, p.n, p.k, p.m); break;
  }
  const double by = first_touch(y); /* after x: when x and y are one tensor the second product accumulates */
  switch (p.form) {
    case Product::ij_jk: product(g, key, Product::ji_jk, x.data_ptr(), z.grad_ptr(), s, y.grad_ptr(), by, p.n, p.m, p.k); break;
    case Product::ij_kj: product(g, key, Product::ji_jk, z.grad_ptr(), x.data_ptr(), s, y.grad_ptr(), by, p.k, p.m, p.n); break;
    case Product::ji_jk: product(g, key, Product::ij_jk, x.data_ptr(), z.grad_ptr(), s, y.grad_ptr(), by, p.n, p.m, p.k); break;
  }
}

namespace ops {

Tensor add(Tensor x, Tensor y) {
  check_pair(x, y, "add: operands must agree in dtype and sizes");
  return defer(x.ptr, Pending::add, x, y);
}

Tensor sub(Tensor x, Tensor y) {
  check_pair(x, y, "sub: operands must agree in dtype and sizes");
  return defer(x.ptr, Pending::sub, x, y);
}

Tensor hadamard(Tensor x, Tensor y) {
  check_pair(x, y, "hadamard: operands must agree in dtype and sizes");
  return defer(x.ptr, Pending::hadamard, x, y);
}

Tensor selu(Tensor x) { return defer(x.ptr, Pending::selu, x, x); }

/* src/ops/relu.zig:13-37, deferred like the other elementwise ops */
Tensor relu(Tensor x) { return defer(x.ptr, Pending::relu, x, x); }

Tensor softmax(Tensor x, const char* expr) {
  if (std::strcmp(expr, "ij|j") != 0) panic("softmax: only the row form \"ij|j\" exists");
  if (x.rank() < 1) panic("softmax: tensor has no axis");
  Graph* g = x.ptr;
  void* px = x.data_ptr();
  Tensor z = g->tensor(TensorClass::hid, x.dtype(), x.sizes());
  const size_t n = x.sizes().back(), m = x.len() / n;
  const len_t bytes = mpSoftmaxScratchBytes((len_t)dkey(z), (len_t)m, (len_t)n);
  void* scratch = bytes ? z.stream()->get_scratch(bytes) : nullptr;
  kernels::softmax_ij_j(dkey(z), px, z.data_ptr(), scratch, (len_t)m, (len_t)n, z.context());
  g->launches++;
  if (g->mode == Mode::train) attach_op(z, softmax_reverse, {x, z});
  return z;
}

Tensor rmsnorm(Tensor x, Tensor gain, double eps) {
  if (x.dtype() != gain.dtype()) panic("rmsnorm: x and gain must agree in dtype");
  if (gain.len() != x.sizes().back()) panic("rmsnorm: gain must have one entry per column");
  Graph* g = x.ptr;
  void* px = x.data_ptr();
  void* pg = gain.data_ptr();
  Tensor z = g->tensor(TensorClass::hid, x.dtype(), x.sizes());
  const size_t n = x.sizes().back(), m = x.len() / n;
  const len_t bytes = mpRmsnormScratchBytes((len_t)dkey(z), (len_t)m, (len_t)n);
  void* scratch = bytes ? z.stream()->get_scratch(bytes) : nullptr;
  kernels::rmsnorm_ij_j(dkey(z), px, pg, z.data_ptr(), scratch, eps, (len_t)m, (len_t)n, z.context());
  g->launches++;
  if (g->mode == Mode::train) attach_op(z, rmsnorm_reverse, {x, gain, eps, z});
  return z;
}

Tensor translate(Tensor x, double value) { return defer(x.ptr, Pending::translate, x, x, value); }

Tensor dilate(Tensor x, double value) { return defer(x.ptr, Pending::dilate, x, x, value); }

Tensor reduce(Tensor x, const char* expr) {
  const std::string e = expr;
  if (e != "ij->i" && e != "ij->j") panic("Invalid expression for reduction.");
  if (x.rank() != 2) panic("reduce: tensor must have rank 2");
  Graph* g = x.ptr;
  void* px = x.data_ptr();
  const len_t m = (len_t)x.sizes()[0], n = (len_t)x.sizes()[1];
  Tensor y = g->tensor(TensorClass::hid, x.dtype(), {e == "ij->i" ? (size_t)m : (size_t)n});
  if (e == "ij->i") kernels::reduce_ij_i(dkey(y), px, y.data_ptr(), 0.0, m, n, y.context());
  else column_sums(g, dkey(y), px, y.data_ptr(), 0.0, m, n);
  if (e == "ij->i") g->launches++;
  if (g->mode == Mode::train) attach_op(y, reduce_reverse, {x, e, y});
  return y;
}

Tensor broadcast(Tensor x, const std::vector<size_t>& sizes, const char* expr) {
  const std::string e = expr;
  if (e != "i->ij" && e != "j->ij") panic("Invalid expression for broadcast.");
  if (x.rank() != 1 || sizes.size() != 2) panic("broadcast: a rank-1 tensor broadcasts to rank 2");
  if (x.len() != (e == "i->ij" ? sizes[0] : sizes[1])) panic("broadcast: sizes do not fit the expression");
  Graph* g = x.ptr;
  void* px = x.data_ptr();
  Tensor y = g->tensor(TensorClass::hid, x.dtype(), sizes);
  if (e == "i->ij") kernels::broadcast_i_ij(dkey(y), px, y.data_ptr(), 0.0, (len_t)sizes[0], (len_t)sizes[1], y.context());
  else kernels::broadcast_j_ij(dkey(y), px, y.data_ptr(), 0.0, (len_t)sizes[0], (len_t)sizes[1], y.context());
  g->launches++;
  if (g->mode == Mode::train) attach_op(y, broadcast_reverse, {x, e, y});
  return y;
}

Tensor permutate(Tensor x, const char* expr) {
  if (std::strcmp(expr, "ij->ji") != 0) panic("Invalid expression for permutate.");
  if (x.rank() != 2) panic("permutate: tensor must have rank 2");
  Graph* g = x.ptr;
  void* px = x.data_ptr();
  Tensor y = g->tensor(TensorClass::hid, x.dtype(), {x.sizes()[1], x.sizes()[0]});
  kernels::permutate_ij_ji(dkey(y), px, y.data_ptr(), 0.0, (len_t)x.sizes()[0], (len_t)x.sizes()[1], y.context());
  g->launches++;
  if (g->mode == Mode::train) attach_op(y, permutate_reverse, {x, std::string(expr), y});
  return y;
}

Tensor inner_product_scaled(Tensor x, Tensor y, double scale, const char* expr) {
  if (x.dtype() != y.dtype()) panic("inner_product: operands must agree in dtype");
  const ProductPlan p = plan_product(x, y, expr);
  Graph* g = x.ptr;
  void* px = x.data_ptr();
  void* py = y.data_ptr();
  Tensor z = g->tensor(TensorClass::hid, x.dtype(), p.sizes);
  product(g, dkey(z), p.form, px, py, scale, z.data_ptr(), 0.0, p.m, p.n, p.k);
  if (g->mode == Mode::train) attach_op(z, inner_product_reverse, {x, y, scale, std::string(expr), z});
  return z;
}

Tensor inner_product(Tensor x, Tensor y, const char* expr) { return inner_product_scaled(x, y, 1.0, expr); }

}  // namespace ops

namespace algo {

void fill(Tensor t, double value) {
  t.ptr->flush(); /* pending nodes may read these bytes */
  kernels::fill(dkey(t), t.data_ptr(), value, (len_t)t.len(), t.context());
  t.ptr->launches++;
}

void copy(Tensor src, Tensor dst) {
  check_pair(src, dst, "copy: operands must agree in dtype and sizes");
  dst.ptr->flush();
  kernels::copy(dkey(src), src.data_ptr(), dst.data_ptr(), (len_t)src.len(), src.context());
  dst.ptr->launches++;
}

void sequence(Tensor t, double init, double step) {
  t.ptr->flush();
  kernels::sequence(dkey(t), t.data_ptr(), init, step, (len_t)t.len(), t.context());
  t.ptr->launches++;
}

}  // namespace algo

/* ------------------------------------------------------------------ tensor files */

static std::string join_path(const std::string& dir, const std::string& name) {
  if (dir.empty()) return name;
  return dir.back() == '/' ? dir + name : dir + "/" + name;
}

static void write_bytes(const std::string& path, const void* dev, size_t bytes, Stream s) {
  std::vector<unsigned char> host(bytes);
  mpMemcpyDtoH(host.data(), dev, bytes, s->context); /* returns with the bytes landed */
  FILE* f = std::fopen(path.c_str(), "wb");
  if (!f) panic("Failed to create save file");
  const size_t done = std::fwrite(host.data(), 1, bytes, f);
  if (std::fclose(f) != 0 || done != bytes) panic("Failed to write to save file");
}

static void read_bytes(const std::string& path, void* dev, size_t bytes, Stream s) {
  FILE* f = std::fopen(path.c_str(), "rb");
  if (!f) panic("Failed to open load file.");
  std::vector<unsigned char> host(bytes + 1);
  const size_t got = std::fread(host.data(), 1, bytes + 1, f); /* one more byte than fits shows a longer file */
  std::fclose(f);
  if (got != bytes) panic("Byte count loaded does not match provided tensor size.");
  mpMemcpyHtoD(dev, host.data(), bytes, s->context);
  mpStreamSynchronize(s->context);
}

namespace io {

void save_tensor(const std::string& dir, const std::string& filename, Tensor x) {
  const size_t bytes = x.len() * tag_size(x.dtype());
  if (bytes == 0) panic("save_tensor: tensor holds no bytes");
  write_bytes(join_path(dir, filename), x.data_ptr(), bytes, x.stream());
}

void load_tensor(const std::string& dir, const std::string& filename, Tensor x) {
  const size_t bytes = x.len() * tag_size(x.dtype());
  if (bytes == 0) panic("load_tensor: tensor holds no bytes");
  x.ptr->flush(); /* pending nodes may still read the bytes about to be replaced */
  read_bytes(join_path(dir, filename), x.data_ptr(), bytes, x.stream());
}

}  // namespace io

void Graph::save(const std::string& dir, const std::string& prefix) {
  size_t wgt_idx = 0;
  for (const Leaf& leaf : leaves_) {
    if (leaf.cls != TensorClass::wgt) continue;
    const size_t bytes = leaf.data.len * tag_size(leaf.data.dtype);
    if (bytes == 0) panic("Graph.save: a weight has no storage");
    write_bytes(join_path(dir, prefix + "_" + std::to_string(wgt_idx)), leaf.data.ptr, bytes, stream);
    ++wgt_idx;
  }
}

void Graph::load(const std::string& dir, const std::string& prefix) {
  flush();
  size_t wgt_idx = 0;
  for (const Leaf& leaf : leaves_) {
    if (leaf.cls != TensorClass::wgt) continue;
    const size_t bytes = leaf.data.len * tag_size(leaf.data.dtype);
    if (bytes == 0) panic("Graph.load: a weight has no storage");
    read_bytes(join_path(dir, prefix + "_" + std::to_string(wgt_idx)), leaf.data.ptr, bytes, stream);
    ++wgt_idx;
  }
}

namespace util {

void to_device(const void* src, Tensor dst, size_t bytes) {
  if (bytes != dst.len() * tag_size(dst.dtype())) panic("to_device: byte count does not match the tensor");
  dst.ptr->flush();
  mpMemcpyHtoD(dst.data_ptr(), src, bytes, dst.context());
  mpStreamSynchronize(dst.context()); /* the host buffer may go away right after this call */
}

void from_device(Tensor src, void* dst, size_t bytes) {
  if (bytes != src.len() * tag_size(src.dtype())) panic("from_device: byte count does not match the tensor");
  mpMemcpyDtoH(dst, src.data_ptr(), bytes, src.context());
}

}  // namespace util

}  // namespace mp
