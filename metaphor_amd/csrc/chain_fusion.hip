/*
 * Elementwise expressions fused at run time: mpChainForward / mpChainReverse take an expression
 * over add, sub, mul, neg, relu, selu, scale(x, c) and shift(x, c) as text, and run it as ONE kernel of the flat elementwise
 * engine (elementwise.h) and its reverse as ONE kernel that writes every leaf gradient. The constants
 * of scale and shift are kernel arguments, so an expression is compiled once whatever their values. The first
 * call for an (expression, dtype) writes the three functors (forward, reverse that overwrites,
 * reverse that blends), compiles them with hiprtc against the very headers this library is built
 * from (their text is embedded at build time) and keeps the code object for the life of the
 * process; each device loads it once. Later calls are a map lookup and a launch.
 *
 * The reference has no counterpart: its generator replicates fixed kernel sources at build time
 * (file_gen.zig:200-328) and each op launches its own kernel through its own temporary
 * (src/ops/addition.zig:37-47, src/ops/hadamard.zig:35-45). The expressions listed in
 * chains.json take the same route at build time (chaingen.py); this file is the same generator,
 * line for line, for expressions nobody listed. tests/test_chain_fusion.py holds the two to the
 * same text.
 *
 * Errors: unlike the launchers (print and exit, src/cuda/kernel_header.h:64-98) these entry points
 * return non-zero and enqueue nothing, because the caller has a fallback (one launch per op);
 * mpChainError() gives the reason.
 *
 * Several results over the same leaves ("selu(mul(add(0,1),2));relu(sub(add(0,1),3))") are one
 * kernel with as many output streams (mpChainForwardMany) and one reverse kernel that takes every
 * result's upstream gradient (mpChainReverseMany): what two results share is read once.
 */
#include "elementwise.h"

#include <hip/hiprtc.h>

#include <atomic>
#include <map>
#include <memory>
#include <mutex>
#include <string>
#include <vector>

#include "chain_fusion.h"
#include "chain_headers.inc" /* CHAIN_HEADER_NAMES, CHAIN_HEADER_TEXT, CHAIN_HEADER_COUNT: written by the build */

#ifndef MP_GPU_ARCH
#define MP_GPU_ARCH "gfx950"
#endif

namespace {

constexpr int MAX_LEAVES = 8, MAX_NODES = 64, MAX_CONSTANTS = 8, MAX_ROOTS = 4, MAX_DEVICES = 64;

enum Op { LEAF, ADD, SUB, MUL, NEG, RELU, SELU, SCALE, SHIFT };

struct Node {
  Op op;
  int leaf;    /* LEAF: its number */
  int arg[2];  /* indices into Expr::nodes */
  std::string name; /* the forward value's spelling in the generated code */
  int constant;     /* SCALE, SHIFT: which of the call's constants; -1 for the other ops */
};

/* The constants of an expression are not part of the kernel: the generated code reads them from its
 * functor (c[0], c[1], ... in the order their ops close in the text), which every launch fills from
 * the text it was given. One compilation serves every value. */
struct Expr {
  std::vector<Node> nodes;
  std::vector<double> constants;
  std::vector<int> roots; /* one per result: "e1;e2" has two, over the same leaves */
  int leaves = 0;
};

/* What a chain's kernels take as their last argument: the generated functors begin with these members. */
struct FunctorArgs {
  double alpha;
  double c[MAX_CONSTANTS];
};

thread_local std::string last_error;

int fail(const std::string& what) {
  last_error = what;
  return 1;
}

/* ---------------------------------------------------------------- text -> tree */

struct Parser {
  const char* p;
  Expr& e;
  std::string err;
  int next_leaf = 0; /* leaves must appear as 0, 1, 2, ... in order of first appearance */
  int depth = 0;

  void skip() {
    while (*p == ' ' || *p == '\t') ++p;
  }
  bool take(char c) {
    skip();
    if (*p != c) {
      err = std::string("expected '") + c + "' at \"" + p + "\"";
      return false;
    }
    ++p;
    return true;
  }
  bool room() { /* before every node is added, and on the way down: a nest of unary ops adds none until it turns back */
    if ((int)e.nodes.size() >= MAX_NODES || depth > MAX_NODES) {
      err = "more than 64 nodes";
      return false;
    }
    return true;
  }
  int node() {
    ++depth;
    const int made = node_here();
    --depth;
    return made;
  }
  int node_here() {
    skip();
    if (!room()) return -1;
    const char* q = p;
    if (*q == 'x') ++q;
    if (*q >= '0' && *q <= '9') { /* a leaf: 3 or x3 */
      int v = 0;
      while (*q >= '0' && *q <= '9' && v < 1000) v = v * 10 + (*q++ - '0');
      p = q;
      if (v > next_leaf) {
        err = "number the leaves in order of first appearance";
        return -1;
      }
      if (v == next_leaf) ++next_leaf;
      if (next_leaf > MAX_LEAVES) {
        err = "more than 8 leaves";
        return -1;
      }
      e.nodes.push_back(Node{LEAF, v, {-1, -1}, "in[" + std::to_string(v) + "]", -1});
      return (int)e.nodes.size() - 1;
    }
    std::string word;
    while ((*p >= 'a' && *p <= 'z') || *p == '_') word += *p++;
    Op op;
    if (word == "add") op = ADD;
    else if (word == "sub") op = SUB;
    else if (word == "mul") op = MUL;
    else if (word == "neg") op = NEG;
    else if (word == "relu") op = RELU;
    else if (word == "selu") op = SELU;
    else if (word == "scale") op = SCALE;
    else if (word == "shift") op = SHIFT;
    else {
      err = "unknown op \"" + word + "\"";
      return -1;
    }
    if (!take('(')) return -1;
    int a = node(), b = -1;
    if (a < 0) return -1;
    if (op == ADD || op == SUB || op == MUL) {
      if (!take(',')) return -1;
      b = node();
      if (b < 0) return -1;
    }
    int constant = -1;
    if (op == SCALE || op == SHIFT) { /* a literal second argument: scale(0,0.5) */
      if (!take(',')) return -1;
      skip();
      char* end = nullptr;
      const double value = strtod(p, &end);
      if (end == p || !(value == value) || value - value != 0.0) {
        err = std::string("expected a finite number at \"") + p + "\"";
        return -1;
      }
      p = end;
      if ((int)e.constants.size() >= MAX_CONSTANTS) {
        err = "more than 8 constants";
        return -1;
      }
      constant = (int)e.constants.size();
      e.constants.push_back(value);
    }
    if (!take(')')) return -1;
    if (!room()) return -1;
    e.nodes.push_back(Node{op, -1, {a, b}, "", constant});
    return (int)e.nodes.size() - 1;
  }
};

bool parse(const char* text, Expr& e, std::string& err) {
  if (text == nullptr) {
    err = "no expression";
    return false;
  }
  Parser ps{text, e, "", 0, 0};
  for (;;) { /* results separated by ';', leaves numbered across all of them */
    const int root = ps.node();
    if (root < 0) {
      err = ps.err;
      return false;
    }
    if (e.nodes[root].op == LEAF) {
      err = "a bare leaf is not a chain";
      return false;
    }
    e.roots.push_back(root);
    ps.skip();
    if (*ps.p != ';') break;
    ++ps.p;
    if ((int)e.roots.size() >= MAX_ROOTS) {
      err = "more than 4 results";
      return false;
    }
  }
  if (*ps.p != '\0') {
    err = std::string("trailing text \"") + ps.p + "\"";
    return false;
  }
  e.leaves = ps.next_leaf;
  return true;
}

/* The expression as the cache spells it: bare leaf numbers, no blanks, "#" for a constant
 * ("scale(add(x0, x1), 0.5)" -> "scale(add(0,1),#)"). */
void spell(const Expr& e, int n, std::string& out) {
  static const char* const names[] = {"", "add", "sub", "mul", "neg", "relu", "selu", "scale", "shift"};
  const Node& node = e.nodes[n];
  if (node.op == LEAF) {
    out += std::to_string(node.leaf);
    return;
  }
  out += names[node.op];
  out += '(';
  spell(e, node.arg[0], out);
  if (node.arg[1] >= 0) {
    out += ',';
    spell(e, node.arg[1], out);
  }
  if (node.constant >= 0) out += ",#";
  out += ')';
}

/* ---------------------------------------------------------------- tree -> functor bodies
 * The same lines, names and order as chaingen.py writes (_forward_lines, _reverse_lines). */

void forward_lines(Expr& e, int n, int& counter, std::vector<std::string>& lines) {
  Node& node = e.nodes[n];
  if (node.op == LEAF) return;
  forward_lines(e, node.arg[0], counter, lines);
  if (node.arg[1] >= 0) forward_lines(e, node.arg[1], counter, lines);
  const std::string& a = e.nodes[node.arg[0]].name;
  const std::string b = node.arg[1] >= 0 ? e.nodes[node.arg[1]].name : "";
  std::string rhs;
  switch (node.op) {
    case ADD: rhs = a + " + " + b; break;
    case SUB: rhs = a + " - " + b; break;
    case MUL: rhs = a + " * " + b; break;
    case NEG: rhs = "-" + a; break;
    case RELU: rhs = "mp::relu_value(" + a + ")"; break;
    case SELU: rhs = "mp::selu_value(" + a + ")"; break;
    case SCALE: rhs = a + " * (P)c[" + std::to_string(node.constant) + "]"; break;
    case SHIFT: rhs = a + " + (P)c[" + std::to_string(node.constant) + "]"; break;
    default: break;
  }
  node.name = "t" + std::to_string(counter++);
  lines.push_back("    const P " + node.name + " = " + rhs + ";");
}

void sweep(const Expr& e, int n, const std::string& adjoint, int& counter, std::vector<std::string>& lines,
           std::vector<std::vector<std::string>>& leaf_terms) {
  const Node& node = e.nodes[n];
  if (node.op == LEAF) {
    leaf_terms[node.leaf].push_back(adjoint);
    return;
  }
  auto fresh = [&](const std::string& expr) {
    const std::string name = "a" + std::to_string(counter++);
    lines.push_back("    const P " + name + " = " + expr + ";");
    return name;
  };
  const std::string& v0 = e.nodes[node.arg[0]].name;
  switch (node.op) {
    case ADD:
      sweep(e, node.arg[0], adjoint, counter, lines, leaf_terms);
      sweep(e, node.arg[1], adjoint, counter, lines, leaf_terms);
      break;
    case SUB:
      sweep(e, node.arg[0], adjoint, counter, lines, leaf_terms);
      sweep(e, node.arg[1], fresh("-" + adjoint), counter, lines, leaf_terms);
      break;
    case MUL: {
      const std::string& v1 = e.nodes[node.arg[1]].name;
      sweep(e, node.arg[0], fresh(adjoint + " * " + v1), counter, lines, leaf_terms);
      sweep(e, node.arg[1], fresh(adjoint + " * " + v0), counter, lines, leaf_terms);
      break;
    }
    case NEG: sweep(e, node.arg[0], fresh("-" + adjoint), counter, lines, leaf_terms); break;
    case RELU: sweep(e, node.arg[0], fresh(adjoint + " * mp::relu_slope(" + v0 + ")"), counter, lines, leaf_terms); break;
    case SELU: sweep(e, node.arg[0], fresh(adjoint + " * mp::selu_slope(" + v0 + ")"), counter, lines, leaf_terms); break;
    case SCALE: sweep(e, node.arg[0], fresh(adjoint + " * (P)c[" + std::to_string(node.constant) + "]"), counter, lines, leaf_terms); break;
    case SHIFT: sweep(e, node.arg[0], adjoint, counter, lines, leaf_terms); break;
    default: break;
  }
}

std::string join(const std::vector<std::string>& v, const char* sep) {
  std::string out;
  for (size_t i = 0; i < v.size(); ++i) out += (i ? sep : "") + v[i];
  return out;
}

const char* storage_type(int dtype) { return dtype == MP_R16 ? "_Float16" : dtype == MP_R32 ? "float" : "double"; }

std::string functor(const char* name, int nin, int nout, const std::string& body) {
  return std::string("struct ") + name + " {\n  double alpha;\n  double c[" + std::to_string(MAX_CONSTANTS) + "];\n  template <class P> __device__ __forceinline__ void apply(const P (&in)[" +
         std::to_string(nin) + "], P (&out)[" + std::to_string(nout) + "]) const {\n" + body + "  }\n};\n\n";
}

/* The whole source of one (expression, dtype): three functors, nine kernels (each functor in the
 * three operand layouts of the engine). With R results the forward writes out[0..R), the reverse
 * reads their upstream gradients as in[k..k+R) and adds every result's contribution to a leaf; a
 * subexpression that two results share is spelled twice and merged by the compiler. */
std::string chain_source(Expr& e, int dtype) {
  const int k = e.leaves, R = (int)e.roots.size();
  int counter = 0;
  std::vector<std::string> fwd, rev;
  std::vector<std::string> values;
  for (int root : e.roots) {
    const size_t before = fwd.size();
    forward_lines(e, root, counter, fwd);
    values.push_back(e.nodes[root].name);
    rev.insert(rev.end(), fwd.begin() + (long)before, fwd.end() - 1); /* no adjoint rule needs a result's own value */
  }
  std::vector<std::vector<std::string>> leaf_terms(k);
  counter = 0;
  for (int r = 0; r < R; ++r) sweep(e, e.roots[r], "in[" + std::to_string(k + r) + "]", counter, rev, leaf_terms);

  std::string fwd_body = join(fwd, "\n") + "\n";
  for (int r = 0; r < R; ++r) fwd_body += "    out[" + std::to_string(r) + "] = " + values[r] + ";\n";
  std::string rev_body = rev.empty() ? "" : join(rev, "\n") + "\n";
  std::string over = rev_body, blend = "    const P al = (P)alpha;\n" + rev_body;
  for (int i = 0; i < k; ++i) {
    const std::string g = leaf_terms[i].empty() ? "(P)0" : join(leaf_terms[i], " + ");
    over += "    out[" + std::to_string(i) + "] = " + g + ";\n";
    blend += "    out[" + std::to_string(i) + "] = " + g + " + al * in[" + std::to_string(k + R + i) + "];\n";
  }

  std::string s = "#include \"elementwise.h\"\n\nnamespace {\n\n";
  s += functor("ChainForward", k, R, fwd_body);
  s += functor("ChainReverseOverwrite", k + R, k, over);
  s += functor("ChainReverseBlend", 2 * k + R, k, blend);
  s += "}  // namespace\n\n";
  s += std::string("typedef ") + storage_type(dtype) + " ChainT;\n";
  s += "#define MP_CHAIN_KERNEL(NAME, LAYOUT, NIN, NOUT, F) \\\n"
       "  extern \"C\" __global__ __launch_bounds__(mp::EW_BLOCK) void NAME(mp::EwPtrs<NIN, NOUT> ptrs, size_t n, unsigned head, F f) { \\\n"
       "    mp::ew_body<ChainT, mp::PACK_BYTES / (int)sizeof(ChainT), LAYOUT, NIN, NOUT, 1, F>(ptrs, n, head, f); \\\n"
       "  }\n";
  const char* layouts[3] = {"mp::EW_ALIGNED", "mp::EW_PEELED", "mp::EW_LOOSE"};
  const struct { const char* stem; const char* fn; int nin, nout; } kinds[3] = {
      {"chain_forward", "ChainForward", k, R},
      {"chain_reverse_overwrite", "ChainReverseOverwrite", k + R, k},
      {"chain_reverse_blend", "ChainReverseBlend", 2 * k + R, k}};
  for (const auto& kind : kinds)
    for (int l = 0; l < 3; ++l)
      s += std::string("MP_CHAIN_KERNEL(") + kind.stem + "_" + std::to_string(l) + ", " + layouts[l] + ", " +
           std::to_string(kind.nin) + ", " + std::to_string(kind.nout) + ", " + kind.fn + ")\n";
  /* the forward once more with loads that leave the inputs in the memory-side cache for the reverse */
  s += std::string("MP_CHAIN_KERNEL(chain_forward_3, mp::EW_KEPT, ") + std::to_string(k) + ", " + std::to_string(R) + ", ChainForward)\n";
  return s;
}

/* ---------------------------------------------------------------- source -> code object */

std::atomic<unsigned long> compilations{0}; /* hiprtc compilations this process has started */

bool compile(const std::string& generated, std::vector<char>& code, std::string& err) {
  compilations.fetch_add(1, std::memory_order_relaxed);
  /* test hook: with MP_CHAIN_BREAK_COMPILE set in the environment every compilation fails, which no
   * expression that parses can bring about by itself */
  const std::string source = getenv("MP_CHAIN_BREAK_COMPILE") ? generated + "\n#error MP_CHAIN_BREAK_COMPILE is set\n" : generated;
  hiprtcProgram prog;
  hiprtcResult r = hiprtcCreateProgram(&prog, source.c_str(), "chain.hip", CHAIN_HEADER_COUNT, CHAIN_HEADER_TEXT, CHAIN_HEADER_NAMES);
  if (r != HIPRTC_SUCCESS) {
    err = std::string("hiprtcCreateProgram: ") + hiprtcGetErrorString(r);
    return false;
  }
  /* the flags the library's own device objects are built with; packed fp32 arithmetic stays off */
  const char* options[] = {"--offload-arch=" MP_GPU_ARCH, "-O3", "-std=c++20", "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"};
  r = hiprtcCompileProgram(prog, (int)(sizeof(options) / sizeof(options[0])), options);
  if (r != HIPRTC_SUCCESS) {
    size_t n = 0;
    hiprtcGetProgramLogSize(prog, &n);
    std::string log(n, '\0');
    if (n) hiprtcGetProgramLog(prog, log.data());
    err = std::string("hiprtcCompileProgram: ") + hiprtcGetErrorString(r) + "\n" + log;
    hiprtcDestroyProgram(&prog);
    return false;
  }
  size_t n = 0;
  r = hiprtcGetCodeSize(prog, &n);
  if (r == HIPRTC_SUCCESS) {
    code.resize(n);
    r = hiprtcGetCode(prog, code.data());
  }
  hiprtcDestroyProgram(&prog);
  if (r != HIPRTC_SUCCESS) {
    err = std::string("hiprtcGetCode: ") + hiprtcGetErrorString(r);
    return false;
  }
  return true;
}

/* ---------------------------------------------------------------- the process-wide cache */

struct Loaded {
  std::atomic<bool> ready{false}; /* set after module and fn are written, read before they are used */
  hipModule_t module = nullptr;
  hipFunction_t fn[12] = {}; /* three kinds x (three layouts, and for the forward the one that keeps its inputs) */
};

/* `build` is held while this chain is compiled or loaded on a device, so that neither holds up
 * calls for other chains; `compiled` and Loaded::ready let calls for a chain that is ready pass
 * without taking it. */
struct Chain {
  int leaves = 0, roots = 1;
  std::string source;
  std::mutex build;
  std::atomic<bool> compiled{false};
  std::atomic<bool> failed{false}; /* a compilation that failed is not tried again: `failure` says why */
  std::string failure;
  std::vector<char> code;
  Loaded on_device[MAX_DEVICES];
};

std::mutex cache_lock; /* the map only: held for a lookup or an insertion, never for a compilation */
std::map<std::pair<std::string, int>, std::unique_ptr<Chain>> cache; /* entries are never removed */

/* The chain of (signature, dtype): its source on first sight, its code object when `compiled` is
 * asked for. NULL with last_error set when it cannot be had. Text that does not parse is not
 * cached (it is as cheap to find wrong again as to look up); a compilation that failed is, with its
 * log, so that a caller who falls back to one launch per op does not pay for it on every call.
 * constants: the values of this call's text, for the launch. */
Chain* chain_for(const char* signature, int dtype, bool compiled, std::vector<double>* constants = nullptr) {
  if (dtype != MP_R16 && dtype != MP_R32 && dtype != MP_R64) {
    fail("dtype must be 0 (r16), 1 (r32) or 2 (r64)");
    return nullptr;
  }
  /* parsing costs a microsecond; it also gives the text the cache is keyed by */
  Expr e;
  std::string err;
  if (!parse(signature, e, err)) {
    fail(std::string("chain \"") + (signature ? signature : "") + "\": " + err);
    return nullptr;
  }
  std::string canonical;
  for (size_t r = 0; r < e.roots.size(); ++r) {
    if (r) canonical += ';';
    spell(e, e.roots[r], canonical);
  }
  if (constants) *constants = e.constants;
  Chain* c = nullptr;
  {
    std::lock_guard<std::mutex> hold(cache_lock);
    auto key = std::make_pair(canonical, dtype);
    auto it = cache.find(key);
    if (it == cache.end()) {
      auto fresh = std::make_unique<Chain>();
      fresh->leaves = e.leaves;
      fresh->roots = (int)e.roots.size();
      fresh->source = chain_source(e, dtype);
      it = cache.emplace(std::move(key), std::move(fresh)).first;
    }
    c = it->second.get();
  }
  if (compiled && !c->compiled.load(std::memory_order_acquire)) {
    std::lock_guard<std::mutex> hold(c->build);
    if (c->failed.load(std::memory_order_relaxed)) {
      fail(c->failure);
      return nullptr;
    }
    if (!c->compiled.load(std::memory_order_relaxed)) {
      std::vector<char> code;
      if (!compile(c->source, code, err)) {
        c->failure = std::string("chain \"") + canonical + "\": " + err;
        c->failed.store(true, std::memory_order_release);
        fail(c->failure);
        return nullptr;
      }
      c->code = std::move(code);
      c->compiled.store(true, std::memory_order_release);
    }
  }
  return c;
}

/* The nine kernels of a chain on the current device, loading the code object there on first use. */
const Loaded* loaded_here(Chain* c) {
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= MAX_DEVICES) {
    fail("no current device");
    return nullptr;
  }
  Loaded& l = c->on_device[dev];
  if (l.ready.load(std::memory_order_acquire)) return &l;
  std::lock_guard<std::mutex> hold(c->build);
  if (l.ready.load(std::memory_order_relaxed)) return &l;
  hipModule_t module = nullptr;
  hipError_t r = hipModuleLoadData(&module, c->code.data());
  if (r != hipSuccess) {
    fail(std::string("hipModuleLoadData: ") + hipGetErrorString(r));
    return nullptr;
  }
  const char* stems[3] = {"chain_forward_", "chain_reverse_overwrite_", "chain_reverse_blend_"};
  for (int k = 0; k < 3; ++k)
    for (int layout = 0; layout < (k == 0 ? 4 : 3); ++layout) { /* only the forward has the variant that keeps its inputs */
      const std::string name = stems[k] + std::to_string(layout);
      r = hipModuleGetFunction(&l.fn[k * 4 + layout], module, name.c_str());
      if (r != hipSuccess) {
        fail("hipModuleGetFunction(" + name + "): " + hipGetErrorString(r));
        (void)hipModuleUnload(module);
        return nullptr;
      }
    }
  l.module = module;
  l.ready.store(true, std::memory_order_release);
  return &l;
}

int layout_index(int layout) { return layout == mp::EW_ALIGNED ? 0 : layout == mp::EW_PEELED ? 1 : layout == mp::EW_LOOSE ? 2 : 3; }

/* One launch: kind 0 forward, 1 reverse that overwrites, 2 reverse that blends. */
int enqueue(Chain* c, int kind, int dtype, const void* const* in, int nin, void* const* out, int nout, double alpha,
            const std::vector<double>& constants, size_t n, hipStream_t stream) {
  if (n == 0) return 0;
  for (int s = 0; s < nin; ++s)
    if (in[s] == nullptr) return fail("a NULL operand");
  for (int s = 0; s < nout; ++s)
    if (out[s] == nullptr) return fail("a NULL output");
  if (n / mp::EW_BLOCK >= 0x7fffffffull) return fail("too many elements for one grid");
  const Loaded* l = loaded_here(c);
  if (l == nullptr) return 1;
  const size_t elem = dtype == MP_R16 ? 2 : dtype == MP_R32 ? 4 : 8;
  const mp::EwPlan plan = mp::ew_plan(in, nin, out, nout, n, elem, mp::EW_BLOCK, 1, kind == 0);
  /* the kernel's first parameter is EwPtrs<nin, nout> by value: the inputs, then the outputs */
  const void* ptrs[2 * MAX_LEAVES + MAX_ROOTS + MAX_LEAVES];
  for (int s = 0; s < nin; ++s) ptrs[s] = in[s];
  for (int s = 0; s < nout; ++s) ptrs[nin + s] = out[s];
  unsigned head = plan.head;
  FunctorArgs args{};
  args.alpha = alpha;
  for (size_t i = 0; i < constants.size() && i < (size_t)MAX_CONSTANTS; ++i) args.c[i] = constants[i];
  void* params[4] = {ptrs, &n, &head, &args};
  const hipError_t r = hipModuleLaunchKernel(l->fn[kind * 4 + layout_index(plan.layout)], plan.blocks, 1, 1, mp::EW_BLOCK, 1, 1,
                                             0, stream, params, nullptr);
  if (r != hipSuccess) return fail(std::string("hipModuleLaunchKernel: ") + hipGetErrorString(r));
  return 0;
}

}  // namespace

extern "C" int mpChainCompile(const char* signature, int dtype) { return chain_for(signature, dtype, true) ? 0 : 1; }

extern "C" int mpChainLeaves(const char* signature) {
  Expr e;
  std::string err;
  if (!parse(signature, e, err)) {
    fail(std::string("chain \"") + (signature ? signature : "") + "\": " + err);
    return -1;
  }
  return e.leaves;
}

extern "C" const char* mpChainSource(const char* signature, int dtype) {
  Chain* c = chain_for(signature, dtype, false);
  return c ? c->source.c_str() : nullptr;
}

extern "C" const void* mpChainCodeObject(const char* signature, int dtype, len_t* bytes) {
  Chain* c = chain_for(signature, dtype, true);
  if (bytes) *bytes = c ? (len_t)c->code.size() : 0;
  return c ? c->code.data() : nullptr;
}

extern "C" int mpChainRoots(const char* signature) {
  Expr e;
  std::string err;
  if (!parse(signature, e, err)) {
    fail(std::string("chain \"") + (signature ? signature : "") + "\": " + err);
    return -1;
  }
  return (int)e.roots.size();
}

extern "C" int mpChainForwardMany(const char* signature, int dtype, const void* const* x, void* const* outs, len_t n,
                                  StreamContext stream) {
  if (x == nullptr || outs == nullptr) return fail("no operand array");
  std::vector<double> constants;
  Chain* c = chain_for(signature, dtype, true, &constants);
  if (c == nullptr) return 1;
  return enqueue(c, 0, dtype, x, c->leaves, outs, c->roots, 0.0, constants, (size_t)n, get_stream(stream));
}

extern "C" int mpChainForward(const char* signature, int dtype, const void* const* x, void* out, len_t n, StreamContext stream) {
  if (x == nullptr) return fail("no operand array");
  const int roots = mpChainRoots(signature);
  if (roots < 0) return 1;
  if (roots != 1) return fail("an expression with several results goes through mpChainForwardMany");
  void* outs[1] = {out};
  return mpChainForwardMany(signature, dtype, x, outs, n, stream);
}

extern "C" int mpChainReverseMany(const char* signature, int dtype, const void* const* x, const void* const* out_grads,
                                  void* const* g, double alpha, len_t n, StreamContext stream) {
  if (x == nullptr || g == nullptr || out_grads == nullptr) return fail("no operand array");
  std::vector<double> constants;
  Chain* c = chain_for(signature, dtype, true, &constants);
  if (c == nullptr) return 1;
  const int k = c->leaves, R = c->roots;
  const void* in[2 * MAX_LEAVES + MAX_ROOTS];
  for (int i = 0; i < k; ++i) in[i] = x[i];
  for (int r = 0; r < R; ++r) in[k + r] = out_grads[r];
  if (alpha == 0.0) return enqueue(c, 1, dtype, in, k + R, g, k, 0.0, constants, (size_t)n, get_stream(stream));
  for (int i = 0; i < k; ++i) in[k + R + i] = g[i];
  return enqueue(c, 2, dtype, in, 2 * k + R, g, k, alpha, constants, (size_t)n, get_stream(stream));
}

extern "C" int mpChainReverse(const char* signature, int dtype, const void* const* x, const void* out_grads, void* const* g,
                              double alpha, len_t n, StreamContext stream) {
  if (x == nullptr || g == nullptr) return fail("no operand array");
  const int roots = mpChainRoots(signature);
  if (roots < 0) return 1;
  if (roots != 1) return fail("an expression with several results goes through mpChainReverseMany");
  const void* ups[1] = {out_grads};
  return mpChainReverseMany(signature, dtype, x, ups, g, alpha, n, stream);
}

extern "C" len_t mpChainCacheSize(void) {
  std::lock_guard<std::mutex> hold(cache_lock);
  len_t n = 0;
  for (const auto& kv : cache) n += kv.second->compiled.load(std::memory_order_acquire) ? 1 : 0;
  return n;
}

extern "C" len_t mpChainCompilations(void) { return (len_t)compilations.load(std::memory_order_relaxed); }

extern "C" const char* mpChainError(void) { return last_error.c_str(); }
