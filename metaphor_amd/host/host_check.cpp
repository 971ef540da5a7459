/*
 * Check program of the C++ host side. Runs on a GPU.
 *
 *   host_check <output directory>
 *
 * Part 1 replays the reference's own example (src/examples/subgraphs.zig:8-133) with the same
 * assertions: two relu(add) blocks, detach, reverse(.free) then reverse(.keep).
 * Part 2 builds e = selu(hadamard(add(a,b), add(c,d))) through mp::ops, checks that forward and
 * reverse are one kernel each, and writes inputs, outputs and gradients as raw little-endian
 * files for the Python test to compare with the CPU oracle; the same for softmax and RMSNorm
 * through the graph, and for an expression that must NOT fuse (a repeated input).
 * Part 3 is the matrix side: the reference's src/examples/experimental.zig, every inner-product
 * expression, permutate, reduce / broadcast, and checkpoint files.
 */
#include <chrono>
#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <string>
#include <vector>

#include "metaphor.hpp"

#define CHECK(cond)                                                          \
  do {                                                                       \
    if (!(cond)) {                                                           \
      fprintf(stderr, "host_check: %s failed at line %d\n", #cond, __LINE__); \
      return 1;                                                              \
    }                                                                        \
  } while (0)

static std::string out_dir;

template <class T> static void dump(const std::string& name, const std::vector<T>& v) {
  const std::string path = out_dir + "/" + name + ".bin";
  FILE* f = fopen(path.c_str(), "wb");
  if (!f || fwrite(v.data(), sizeof(T), v.size(), f) != v.size()) {
    fprintf(stderr, "host_check: cannot write %s\n", path.c_str());
    exit(2);
  }
  fclose(f);
}

/* SplitMix64 -> uniform in [lo, hi) */
struct Rng {
  uint64_t s;
  double next() {
    uint64_t z = (s += 0x9e3779b97f4a7c15ull);
    z = (z ^ (z >> 30)) * 0xbf58476d1ce4e5b9ull;
    z = (z ^ (z >> 27)) * 0x94d049bb133111ebull;
    z ^= z >> 31;
    return (double)(z >> 11) / 9007199254740992.0;
  }
  std::vector<float> uniform(size_t n, double lo, double hi) {
    std::vector<float> v(n);
    for (auto& x : v) x = (float)(lo + (hi - lo) * next());
    return v;
  }
  std::vector<float> normal(size_t n, double mu, double sd) {
    std::vector<float> v(n);
    for (auto& x : v) {
      const double u1 = next() + 1e-300, u2 = next();
      x = (float)(mu + sd * std::sqrt(-2.0 * std::log(u1)) * std::cos(6.283185307179586 * u2));
    }
    return v;
  }
};

/* upload an upstream gradient, as a loss would have left it (reverse seeds ones only when none exists) */
static void set_grad(mp::Tensor t, const std::vector<float>& host) {
  mp::enable_gradient(t);
  mpMemcpyHtoD(t.grad_ptr(), host.data(), host.size() * sizeof(float), t.context());
  mpStreamSynchronize(t.context());
}

static mp::Tensor leaf(mp::Graph* G, mp::TensorClass cls, const std::vector<size_t>& sizes,
                       const std::vector<float>& host) {
  mp::Tensor t = G->tensor(cls, mp::Tag::r32, sizes);
  mp::util::to_device(host.data(), t, host.size() * sizeof(float));
  return t;
}

static int subgraphs_example(mp::Stream stream) {
  mp::Graph* G = mp::Graph::init({stream, mp::Mode::train});
  const size_t M = 32;
  mp::Tensor x = G->tensor(mp::TensorClass::inp, mp::Tag::r32, {M});
  mp::Tensor w1 = G->tensor(mp::TensorClass::wgt, mp::Tag::r32, {M});
  mp::Tensor w2 = G->tensor(mp::TensorClass::wgt, mp::Tag::r32, {M});
  mp::algo::fill(x, 1.0);
  mp::algo::fill(w1, 1.0);
  mp::algo::fill(w2, 1.0);

  mp::Tensor z1 = mp::ops::add(x, w1);
  mp::Tensor z2 = mp::ops::relu(z1);
  mp::Tensor z3 = mp::ops::add(z2, w2);
  mp::Tensor z4 = mp::ops::relu(z3);
  for (float v : z4.native<float>()) CHECK(v == 3.0f);

  z2.detach();
  z4.reverse(mp::ReverseCleanup::free);
  CHECK(z4.len() == 0);
  CHECK(z3.len() == 0);
  CHECK(!z4.has_grad());
  CHECK(!z3.has_grad());
  CHECK(z2.len() != 0);
  CHECK(w2.len() != 0);
  CHECK(z2.has_grad());
  CHECK(w2.has_grad());
  CHECK(z1.len() != 0);
  CHECK(w1.len() != 0);
  CHECK(!z1.has_grad());
  CHECK(!w1.has_grad());
  for (float v : w2.native_grad<float>()) CHECK(v == 1.0f);

  z2.reverse(mp::ReverseCleanup::keep);
  CHECK(x.len() != 0);
  CHECK(z1.len() != 0);
  CHECK(w1.len() != 0);
  CHECK(z1.has_grad());
  CHECK(w1.has_grad());
  CHECK(x.has_grad());
  for (float v : w1.native_grad<float>()) CHECK(v == 1.0f);
  for (float v : x.native_grad<float>()) CHECK(v == 1.0f);
  G->deinit();
  return 0;
}

static int fused_chain(mp::Stream stream) {
  mp::Graph* G = mp::Graph::init({stream, mp::Mode::train});
  const size_t n = 100003;
  Rng r{7};
  const auto ha = r.uniform(n, -2, 2), hb = r.uniform(n, -2, 2), hc = r.uniform(n, -2, 2), hd = r.uniform(n, -2, 2);
  mp::Tensor a = leaf(G, mp::TensorClass::wgt, {n}, ha), b = leaf(G, mp::TensorClass::wgt, {n}, hb);
  mp::Tensor c = leaf(G, mp::TensorClass::wgt, {n}, hc), d = leaf(G, mp::TensorClass::inp, {n}, hd);
  dump("fused_a", ha); dump("fused_b", hb); dump("fused_c", hc); dump("fused_d", hd);

  const size_t before = G->launches;
  mp::Tensor e = mp::ops::selu(mp::ops::hadamard(mp::ops::add(a, b), mp::ops::add(c, d)));
  CHECK(G->launches == before);                 /* nothing ran yet */
  dump("fused_e", e.native<float>());
  CHECK(G->launches == before + 1);             /* the whole chain was one kernel */

  const size_t before_rev = G->launches;
  e.reverse(mp::ReverseCleanup::keep);          /* seeds de = 1 */
  CHECK(G->launches == before_rev + 1 + 1);     /* the seed fill of de, then ONE reverse kernel */
  dump("fused_da", a.native_grad<float>()); dump("fused_db", b.native_grad<float>());
  dump("fused_dc", c.native_grad<float>()); dump("fused_dd", d.native_grad<float>());

  /* second pass over the same leaves: gradients accumulate (alpha = 1 path) */
  mp::Tensor e2 = mp::ops::selu(mp::ops::hadamard(mp::ops::add(a, b), mp::ops::add(c, d)));
  e2.reverse(mp::ReverseCleanup::free);
  CHECK(e2.len() == 0);
  dump("fused_da2", a.native_grad<float>());

  /* a repeated input must not fuse: selu((a+a)*(c+d)) runs per op and still differentiates right */
  G->reset(mp::Graph::ResetGroup::leaf, mp::Graph::ResetComponent::grd);
  const size_t l0 = G->launches;
  mp::Tensor f = mp::ops::selu(mp::ops::hadamard(mp::ops::add(a, a), mp::ops::add(c, d)));
  dump("rep_f", f.native<float>());
  CHECK(G->launches == l0 + 4);
  f.reverse(mp::ReverseCleanup::keep);
  dump("rep_da", a.native_grad<float>()); dump("rep_dc", c.native_grad<float>());

  /* other entries of the generated chain table: one kernel forward, one kernel reverse each */
  G->reset(mp::Graph::ResetGroup::leaf, mp::Graph::ResetComponent::grd);
  {
    size_t l = G->launches;
    mp::Tensor p = mp::ops::hadamard(mp::ops::add(a, b), mp::ops::add(c, d));
    dump("chain_mul_add_add", p.native<float>());
    CHECK(G->launches == l + 1);
    l = G->launches;
    p.reverse(mp::ReverseCleanup::free);
    CHECK(G->launches == l + 2);
    dump("chain_mul_add_add_da", a.native_grad<float>()); dump("chain_mul_add_add_dd", d.native_grad<float>());

    G->reset(mp::Graph::ResetGroup::leaf, mp::Graph::ResetComponent::grd);
    l = G->launches;
    mp::Tensor q = mp::ops::selu(mp::ops::hadamard(mp::ops::sub(a, b), c));
    dump("chain_selu_mul_sub", q.native<float>());
    CHECK(G->launches == l + 1);
    q.reverse(mp::ReverseCleanup::free);
    dump("chain_selu_mul_sub_da", a.native_grad<float>()); dump("chain_selu_mul_sub_db", b.native_grad<float>());
    dump("chain_selu_mul_sub_dc", c.native_grad<float>());

    /* not in the table as a whole: relu takes its own kernel, its operand selu(add(a,b)) is a chain */
    G->reset(mp::Graph::ResetGroup::leaf, mp::Graph::ResetComponent::grd);
    l = G->launches;
    mp::Tensor r2 = mp::ops::relu(mp::ops::selu(mp::ops::add(a, b)));
    dump("chain_relu_selu_add", r2.native<float>());
    CHECK(G->launches == l + 2);
    r2.reverse(mp::ReverseCleanup::free);
    dump("chain_relu_selu_add_da", a.native_grad<float>());

    /* relu defers like the other elementwise ops: relu(hadamard(add, add)) is one kernel each way */
    G->reset(mp::Graph::ResetGroup::leaf, mp::Graph::ResetComponent::grd);
    l = G->launches;
    mp::Tensor r3 = mp::ops::relu(mp::ops::hadamard(mp::ops::add(a, b), mp::ops::add(c, d)));
    dump("chain_relu_mul_add_add", r3.native<float>());
    CHECK(G->launches == l + 1);
    l = G->launches;
    r3.reverse(mp::ReverseCleanup::free);
    CHECK(G->launches == l + 2); /* the seed fill and one reverse kernel */
    dump("chain_relu_mul_add_add_da", a.native_grad<float>()); dump("chain_relu_mul_add_add_dc", c.native_grad<float>());

    /* sub alone is not a chain: per-op kernel and the per-op reverse (gx += gz, gy -= gz) */
    G->reset(mp::Graph::ResetGroup::leaf, mp::Graph::ResetComponent::grd);
    mp::Tensor s2 = mp::ops::sub(a, b);
    dump("plain_sub", s2.native<float>());
    s2.reverse(mp::ReverseCleanup::free);
    dump("plain_sub_da", a.native_grad<float>()); dump("plain_sub_db", b.native_grad<float>());
  }

  /* a graph that fuses whatever it meets: the repeated-input expression above, which no table
   * lists, is compiled at run time into one kernel per direction; a is ONE leaf whose two
   * contributions the reverse kernel adds */
  {
    mp::Graph* R = mp::Graph::init({stream, mp::Mode::train, mp::Fusion::any});
    mp::Tensor ra = leaf(R, mp::TensorClass::wgt, {n}, ha), rc = leaf(R, mp::TensorClass::wgt, {n}, hc);
    mp::Tensor rd = leaf(R, mp::TensorClass::wgt, {n}, hd);
    size_t l = R->launches;
    mp::Tensor f2 = mp::ops::selu(mp::ops::hadamard(mp::ops::add(ra, ra), mp::ops::sub(rc, rd)));
    dump("any_f", f2.native<float>());
    CHECK(R->launches == l + 1);
    l = R->launches;
    f2.reverse(mp::ReverseCleanup::keep);
    CHECK(R->launches == l + 2); /* the seed fill and one reverse kernel */
    dump("any_da", ra.native_grad<float>()); dump("any_dc", rc.native_grad<float>()); dump("any_dd", rd.native_grad<float>());
    /* a second pass accumulates into the existing gradients (alpha = 1) */
    mp::Tensor f3 = mp::ops::selu(mp::ops::hadamard(mp::ops::add(ra, ra), mp::ops::sub(rc, rd)));
    f3.reverse(mp::ReverseCleanup::free);
    dump("any_da2", ra.native_grad<float>());
    CHECK(R->runtime_chains_.size() == 1);
    /* dilate and translate defer like the other elementwise ops and carry their constants into the
     * expression: relu(0.125 * (a * c) + 0.5) is one kernel each way */
    R->reset(mp::Graph::ResetGroup::leaf, mp::Graph::ResetComponent::grd);
    l = R->launches;
    mp::Tensor f4 = mp::ops::relu(mp::ops::translate(mp::ops::dilate(mp::ops::hadamard(ra, rc), 0.125), 0.5));
    dump("any_affine", f4.native<float>());
    CHECK(R->launches == l + 1);
    l = R->launches;
    f4.reverse(mp::ReverseCleanup::free);
    CHECK(R->launches == l + 2);
    dump("any_affine_da", ra.native_grad<float>()); dump("any_affine_dc", rc.native_grad<float>());
    CHECK(R->runtime_chains_.size() == 2);
    /* the same expression with other constants (a step size that changes every step) is the same kernel
     * with other arguments: nothing is compiled, no new shape is recorded */
    {
      const len_t compiled = mpChainCacheSize(), started = mpChainCompilations();
      R->reset(mp::Graph::ResetGroup::leaf, mp::Graph::ResetComponent::grd);
      l = R->launches;
      mp::Tensor f5 = mp::ops::relu(mp::ops::translate(mp::ops::dilate(mp::ops::hadamard(ra, rc), -0.75), 0.25));
      dump("any_affine2", f5.native<float>());
      CHECK(R->launches == l + 1);
      f5.reverse(mp::ReverseCleanup::free);
      dump("any_affine2_da", ra.native_grad<float>()); dump("any_affine2_dc", rc.native_grad<float>());
      CHECK(R->runtime_chains_.size() == 2);
      CHECK(mpChainCacheSize() == compiled);
      CHECK(mpChainCompilations() == started);
    }
    /* two results that share a subexpression are one forward kernel with two output streams:
     * u = a + b; e1 = selu(u * c); e2 = relu(u - d). Each keeps a reverse of its own. */
    {
      mp::Tensor rb = leaf(R, mp::TensorClass::wgt, {n}, hb);
      R->reset(mp::Graph::ResetGroup::leaf, mp::Graph::ResetComponent::grd);
      const size_t shapes = R->runtime_chains_.size();
      l = R->launches;
      mp::Tensor u = mp::ops::add(ra, rb);
      mp::Tensor e1 = mp::ops::selu(mp::ops::hadamard(u, rc));
      mp::Tensor e2 = mp::ops::relu(mp::ops::sub(u, rd));
      dump("two_e1", e1.native<float>());
      CHECK(R->launches == l + 1); /* both results came out of that one launch */
      dump("two_e2", e2.native<float>());
      CHECK(R->launches == l + 1);
      CHECK(R->runtime_chains_.size() == shapes + 1);
      l = R->launches;
      e1.reverse(mp::ReverseCleanup::keep);
      e2.reverse(mp::ReverseCleanup::keep);
      CHECK(R->launches == l + 5); /* a seed fill and one reverse kernel per result, and the zero fill of d's new
                                      gradient beside the existing ones of a and b in the second reverse */
      dump("two_da", ra.native_grad<float>()); dump("two_db", rb.native_grad<float>());
      dump("two_dc", rc.native_grad<float>()); dump("two_dd", rd.native_grad<float>());
    }
    /* a single op stays the op's own kernel and keeps its own reverse */
    l = R->launches;
    mp::Tensor s3 = mp::ops::sub(rc, rd);
    dump("any_sub", s3.native<float>());
    CHECK(R->launches == l + 1);
    R->deinit();
  }

  /* eval mode attaches nothing and reverse is refused by construction: only forward here */
  mp::Graph* E = mp::Graph::init({stream, mp::Mode::eval});
  mp::Tensor ea = leaf(E, mp::TensorClass::inp, {n}, ha), eb = leaf(E, mp::TensorClass::inp, {n}, hb);
  mp::Tensor ec = leaf(E, mp::TensorClass::inp, {n}, hc), ed = leaf(E, mp::TensorClass::inp, {n}, hd);
  mp::Tensor ee = mp::ops::selu(mp::ops::hadamard(mp::ops::add(ea, eb), mp::ops::add(ec, ed)));
  dump("eval_e", ee.native<float>());
  E->deinit();
  G->deinit();
  return 0;
}

static int row_ops(mp::Stream stream) {
  mp::Graph* G = mp::Graph::init({stream, mp::Mode::train});
  const size_t m = 37, n = 1000;
  Rng r{11};
  const auto hx = r.normal(m * n, 0, 1), hg = r.normal(n, 1, 0.02), hs = r.normal(m * n, 0, 2);
  mp::Tensor x = leaf(G, mp::TensorClass::inp, {m, n}, hx);
  mp::Tensor g = leaf(G, mp::TensorClass::wgt, {n}, hg);
  mp::Tensor s = leaf(G, mp::TensorClass::inp, {m, n}, hs);
  dump("row_x", hx); dump("row_g", hg); dump("row_s", hs);

  const auto hdy = r.normal(m * n, 0, 1), hdp = r.normal(m * n, 0, 1);
  dump("row_dy", hdy); dump("row_dp", hdp);

  mp::Tensor y = mp::ops::rmsnorm(x, g, 1e-6);
  dump("row_y", y.native<float>());
  set_grad(y, hdy);
  y.reverse(mp::ReverseCleanup::keep);
  dump("row_dx", x.native_grad<float>()); dump("row_dg", g.native_grad<float>());

  /* p = softmax(s + s) exercises a pending add feeding a row op */
  mp::Tensor p = mp::ops::softmax(mp::ops::add(s, s));
  dump("row_p", p.native<float>());
  set_grad(p, hdp);
  p.reverse(mp::ReverseCleanup::keep);
  dump("row_ds", s.native_grad<float>());
  G->deinit();
  return 0;
}

/* Part 3: the matrix side of the surface. First the reference's own example with its hand-computable
 * answers (src/examples/experimental.zig:19-62), then every inner-product expression, permutate,
 * reduce / broadcast, dilate and translate on random operands, dumped for the oracle check, and a
 * checkpoint round trip in the reference's file format. */
static int matrix_ops(mp::Stream stream) {
  mp::Graph* G = mp::Graph::init({stream, mp::Mode::train});
  {
    mp::Tensor x = G->tensor(mp::TensorClass::wgt, mp::Tag::r32, {3, 2});
    mp::Tensor y = G->tensor(mp::TensorClass::wgt, mp::Tag::r32, {2, 2});
    mp::algo::sequence(x, 1.0, 1.0);
    mp::algo::sequence(y, 1.0, 1.0);
    mp::Tensor z = mp::ops::inner_product(x, y, "ij,jk->ik");
    mp::Tensor a = mp::ops::reduce(y, "ij->i");
    mp::Tensor b = mp::ops::broadcast(a, x.sizes(), "j->ij");
    mp::Tensor c = mp::ops::reduce(x, "ij->j");
    mp::Tensor d = mp::ops::broadcast(c, y.sizes(), "i->ij");
    CHECK((z.native<float>() == std::vector<float>{7, 10, 15, 22, 23, 34}));
    CHECK((b.native<float>() == std::vector<float>{3, 7, 3, 7, 3, 7}));
    CHECK((d.native<float>() == std::vector<float>{9, 9, 12, 12}));
    z.reverse(mp::ReverseCleanup::keep);
    CHECK(x.native_grad<float>() == b.native<float>()); /* reverse mode agrees with the forward-mode check */
    CHECK(y.native_grad<float>() == d.native<float>());
    G->reset(mp::Graph::ResetGroup::node, mp::Graph::ResetComponent::all);
    G->reset(mp::Graph::ResetGroup::leaf, mp::Graph::ResetComponent::grd);
  }
  Rng r{99};
  const size_t m = 37, n = 53, k = 29;
  const auto ha = r.normal(m * n, 0, 1), hb = r.normal(n * k, 0, 1), hbt = r.normal(k * n, 0, 1);
  const auto hat = r.normal(n * m, 0, 1), hv = r.normal(n, 0, 1), hu = r.normal(m, 0, 1);
  const auto hg = r.normal(m * k, 0, 1), hgi = r.normal(m, 0, 1), hgn = r.normal(n, 0, 1), hgmn = r.normal(m * n, 0, 1);
  dump("mx_a", ha); dump("mx_b", hb); dump("mx_bt", hbt); dump("mx_at", hat); dump("mx_v", hv); dump("mx_u", hu);
  dump("mx_g", hg); dump("mx_gi", hgi); dump("mx_gn", hgn); dump("mx_gmn", hgmn);
  mp::Tensor a = leaf(G, mp::TensorClass::wgt, {m, n}, ha);
  mp::Tensor b = leaf(G, mp::TensorClass::wgt, {n, k}, hb);
  mp::Tensor bt = leaf(G, mp::TensorClass::wgt, {k, n}, hbt);
  mp::Tensor at = leaf(G, mp::TensorClass::wgt, {n, m}, hat);
  mp::Tensor v = leaf(G, mp::TensorClass::wgt, {n}, hv);
  mp::Tensor u = leaf(G, mp::TensorClass::wgt, {m}, hu);
  struct Case { const char* name; const char* expr; mp::Tensor x, y; const std::vector<float>* seed; double scale; };
  const Case cases[] = {
      {"nn", "ij,jk->ik", a, b, &hg, 1.0},   {"nt", "ij,kj->ik", a, bt, &hg, 0.5}, {"tn", "ji,jk->ik", at, b, &hg, -2.0},
      {"mv", "ij,j->i", a, v, &hgi, 1.0},    {"vm", "i,ij->j", u, a, &hgn, 1.5},
  };
  for (const Case& c : cases) {
    const size_t before = G->launches;
    mp::Tensor z = mp::ops::inner_product_scaled(c.x, c.y, c.scale, c.expr);
    CHECK(G->launches == before + 1); /* transposed operands cost no extra kernel */
    dump(std::string("mx_") + c.name + "_z", z.native<float>());
    set_grad(z, *c.seed);
    const size_t mid = G->launches;
    z.reverse(mp::ReverseCleanup::keep);
    CHECK(G->launches == mid + 2); /* one product per operand gradient, no zero fills, no transposes */
    dump(std::string("mx_") + c.name + "_dx", c.x.native_grad<float>());
    dump(std::string("mx_") + c.name + "_dy", c.y.native_grad<float>());
    G->reset(mp::Graph::ResetGroup::node, mp::Graph::ResetComponent::all);
    G->reset(mp::Graph::ResetGroup::leaf, mp::Graph::ResetComponent::grd);
  }
  { /* a gradient that already exists is accumulated into: the same product twice */
    mp::Tensor z1 = mp::ops::inner_product(a, b, "ij,jk->ik"), z2 = mp::ops::inner_product(a, b, "ij,jk->ik");
    set_grad(z1, hg); set_grad(z2, hg);
    z1.reverse(mp::ReverseCleanup::keep);
    z2.reverse(mp::ReverseCleanup::keep);
    dump("mx_nn_dx2", a.native_grad<float>());
    G->reset(mp::Graph::ResetGroup::node, mp::Graph::ResetComponent::all);
    G->reset(mp::Graph::ResetGroup::leaf, mp::Graph::ResetComponent::grd);
  }
  { /* t = permutate(dilate(translate(a, 0.25), 3.0)) with an upstream gradient */
    mp::Tensor t = mp::ops::permutate(mp::ops::dilate(mp::ops::translate(a, 0.25), 3.0), "ij->ji");
    CHECK((t.sizes() == std::vector<size_t>{n, m}));
    dump("mx_perm", t.native<float>());
    set_grad(t, hat); /* any [n, m] values */
    t.reverse(mp::ReverseCleanup::keep);
    dump("mx_perm_da", a.native_grad<float>());
    G->reset(mp::Graph::ResetGroup::node, mp::Graph::ResetComponent::all);
    G->reset(mp::Graph::ResetGroup::leaf, mp::Graph::ResetComponent::grd);
  }
  { /* reduce and broadcast with upstream gradients */
    mp::Tensor ri = mp::ops::reduce(a, "ij->i");
    set_grad(ri, hgi);
    ri.reverse(mp::ReverseCleanup::keep);
    dump("mx_reduce_i", ri.native<float>()); dump("mx_reduce_i_da", a.native_grad<float>());
    G->reset(mp::Graph::ResetGroup::node, mp::Graph::ResetComponent::all);
    G->reset(mp::Graph::ResetGroup::leaf, mp::Graph::ResetComponent::grd);
    mp::Tensor bj = mp::ops::broadcast(v, {m, n}, "j->ij");
    set_grad(bj, hgmn);
    bj.reverse(mp::ReverseCleanup::keep);
    dump("mx_bcast_j", bj.native<float>()); dump("mx_bcast_j_dv", v.native_grad<float>());
    G->reset(mp::Graph::ResetGroup::node, mp::Graph::ResetComponent::all);
    G->reset(mp::Graph::ResetGroup::leaf, mp::Graph::ResetComponent::grd);
  }
  { /* checkpoint round trip: every weight of the graph -> ckpt_0, ckpt_1, ..., overwrite, load, compare */
    G->save(out_dir, "ckpt");
    mp::io::save_tensor(out_dir, "single_a", a);
    for (mp::Tensor t : {a, b, bt, at, v, u}) mp::algo::fill(t, -1.0);
    G->load(out_dir, "ckpt");
    CHECK(a.native<float>() == ha && b.native<float>() == hb && bt.native<float>() == hbt);
    CHECK(at.native<float>() == hat && v.native<float>() == hv && u.native<float>() == hu);
    mp::algo::fill(a, 0.0);
    mp::io::load_tensor(out_dir, "single_a", a);
    CHECK(a.native<float>() == ha);
  }
  G->deinit();
  return 0;
}

/* What one launch costs a native caller: `launches` calls of launch_softmax_ij_j_r32 on
 * [256, 1024] (the smallest benchmark configuration, a 2.7 us kernel) enqueued back to back on
 * one stream of this library, no interpreter in between. enqueue_us is the host time per call,
 * back_to_back_us the time per launch until the stream has drained. */
static int launch_cost(int launches) {
  mp::device::init(0);
  mp::Stream s = mp::stream::init();
  const size_t m = 256, n = 1024, bytes = m * n * sizeof(float);
  void* x = mpMemAlloc(bytes, s->context);
  void* y = mpMemAlloc(bytes, s->context);
  std::vector<float> h(m * n, 0.25f);
  mpMemcpyHtoD(x, h.data(), bytes, s->context);
  for (int i = 0; i < 200; ++i) launch_softmax_ij_j_r32(x, y, nullptr, m, n, s->context);
  mpStreamSynchronize(s->context);
  const auto t0 = std::chrono::steady_clock::now();
  for (int i = 0; i < launches; ++i) launch_softmax_ij_j_r32(x, y, nullptr, m, n, s->context);
  const auto t1 = std::chrono::steady_clock::now();
  mpStreamSynchronize(s->context);
  const auto t2 = std::chrono::steady_clock::now();
  mpCheckLastError();
  const double enq = std::chrono::duration<double, std::micro>(t1 - t0).count() / launches;
  const double all = std::chrono::duration<double, std::micro>(t2 - t0).count() / launches;
  printf("{\"launches\": %d, \"enqueue_us\": %.3f, \"back_to_back_us\": %.3f}\n", launches, enq, all);
  mpMemFree(x, s->context);
  mpMemFree(y, s->context);
  mp::stream::deinit(s);
  return 0;
}

int main(int argc, char** argv) {
  if (argc == 3 && std::string(argv[1]) == "--launch-cost") return launch_cost(atoi(argv[2]) > 0 ? atoi(argv[2]) : 2000);
  if (argc != 2) {
    fprintf(stderr, "usage: host_check <output directory> | host_check --launch-cost <launches>\n");
    return 2;
  }
  out_dir = argv[1];
  mp::device::init(0);
  CHECK(mp::device::total_memory(0) > 0);
  mp::Stream stream = mp::stream::init();
  mp::Stream second = mp::stream::init();
  CHECK(stream->ID == 0 && second->ID == 1);
  mp::stream::deinit(second);

  if (subgraphs_example(stream)) return 1;
  printf("host_check: subgraphs example ok\n");
  if (fused_chain(stream)) return 1;
  printf("host_check: fused chain ok (one kernel forward, one kernel reverse)\n");
  if (row_ops(stream)) return 1;
  printf("host_check: softmax / rmsnorm through the graph ok\n");
  if (matrix_ops(stream)) return 1;
  printf("host_check: inner products, permutate, reduce / broadcast, checkpoint files ok\n");

  { /* a group of streams: slots 1..3 beside the stream above, the same graph code on each of them */
    auto group = mp::stream::Group<3>::init();
    CHECK(group.items[0]->ID == 1 && group.items[2]->ID == 3);
    for (mp::Stream s : group.items)
      if (subgraphs_example(s)) return 1;
    group.synchronize();
    group.deinit();
    mp::Stream again = mp::stream::init();
    CHECK(again->ID == 1); /* released slots are handed out again */
    mp::stream::deinit(again);
  }
  printf("host_check: stream group ok\n");

  mp::stream::sync(stream);
  mp::stream::deinit(stream);
  mp::device::check();
  printf("host_check: done\n");
  return 0;
}
