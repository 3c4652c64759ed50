// The reference's node tests (tests/test-rnn.cc, tests/test-nodes.cc) replayed in C++ through
// the adapter above the C-ABI: same inputs, same expected values, same tolerances
// (BOOST_CHECK_CLOSE's 0.001 percent; gradient checks by central differences as
// dynet/grad-check.cc does).  The numbers are the reference tests' fixtures.
//
//   test_adapter            run every case on GPU 0, exit status = number of failed checks
//   test_adapter --no-gpu   expect device creation to fail with cuda_exception (CPU-only box)
#include <cmath>
#include <cstdio>
#include <cstring>
#include <functional>
#include <string>
#include <vector>

#include "dynet_hip_adapter.h"

using namespace dynet_hip;
using std::vector;

static int g_failed = 0, g_checks = 0;
static const char* g_case = "";

#define CHECK(cond)                                                          \
  do {                                                                       \
    ++g_checks;                                                              \
    if (!(cond)) {                                                           \
      ++g_failed;                                                            \
      std::printf("FAIL %s: %s (line %d)\n", g_case, #cond, __LINE__);       \
    }                                                                        \
  } while (0)

// BOOST_CHECK_CLOSE(a, b, pct): |a-b| within pct percent of both
static void check_close(double a, double b, double pct, int line) {
  ++g_checks;
  const double d = std::fabs(a - b), tol = pct / 100.0;
  if (!(d <= tol * std::fabs(a) && d <= tol * std::fabs(b))) {
    ++g_failed;
    std::printf("FAIL %s: %.9g vs %.9g (line %d)\n", g_case, a, b, line);
  }
}
static void check_small(double a, double tol, int line) {
  ++g_checks;
  if (!(std::fabs(a) < tol)) {
    ++g_failed;
    std::printf("FAIL %s: |%.9g| >= %g (line %d)\n", g_case, a, tol, line);
  }
}
#define CHECK_CLOSE(a, b, pct) check_close((a), (b), (pct), __LINE__)
#define CHECK_SMALL(a, tol) check_small((a), (tol), __LINE__)

struct Fixture {
  Device_GPU dev;
  Fixture() : dev(0, 64, 64, 64, 64) {}
  Tensor input(const Dim& d, const vector<float>& vals, DeviceMempool mp = DeviceMempool::FXS) {
    Tensor t = dev.allocate_tensor(mp, d);
    TensorTools::set_elements(t, vals);
    return t;
  }
  Tensor zeros(const Dim& d, DeviceMempool mp = DeviceMempool::DEDFS) {
    Tensor t = dev.allocate_tensor(mp, d);
    TensorTools::zero(t);
    return t;
  }
  void reset() {
    for (int k : {0, 1, 3}) dev.pools[k]->free();
  }
};

// Central-difference check of every argument's gradient of z = sum_j w_j * fx_j, with the step
// and the acceptance rule of dynet/grad-check.cc:20-87 (alpha = 5e-4; |g - g_act| > 0.1 and
// relative difference > 0.1 is a failure).
static bool check_grad(Fixture& F, const Node& node, vector<Tensor>& args, const Dim& out_dim,
                       const vector<bool>& differentiable) {
  vector<const Tensor*> xs;
  for (Tensor& a : args) xs.push_back(&a);
  Tensor fx = F.dev.allocate_tensor(DeviceMempool::FXS, out_dim);
  vector<float> w(out_dim.size());
  for (size_t j = 0; j < w.size(); ++j) w[j] = 0.3f + 0.1f * float(j % 7) - 0.05f * float(j % 3);
  auto loss = [&]() {
    node.forward_dev_impl(F.dev, xs, fx);
    const vector<float> y = as_vector(fx);
    double z = 0;
    for (size_t j = 0; j < y.size(); ++j) z += double(w[j]) * y[j];
    return z;
  };
  loss();
  Tensor dEdf = F.input(out_dim, w, DeviceMempool::DEDFS);
  bool ok = true;
  const float alpha = 5e-4f;
  for (unsigned i = 0; i < args.size(); ++i) {
    if (!differentiable[i]) continue;
    Tensor dEdxi = F.zeros(args[i].d);
    node.forward_dev_impl(F.dev, xs, fx);
    node.backward_dev_impl(F.dev, xs, fx, dEdf, i, dEdxi);
    const vector<float> g = as_vector(dEdxi);
    vector<float> vals = as_vector(args[i]);
    for (size_t e = 0; e < vals.size(); ++e) {
      const float old = vals[e];
      vals[e] = old - alpha;
      TensorTools::set_elements(args[i], vals);
      const double el = loss();
      vals[e] = old + alpha;
      TensorTools::set_elements(args[i], vals);
      const double er = loss();
      vals[e] = old;
      const double gn = (er - el) / (2 * alpha);
      const double f = std::fabs(gn - g[e]), m = std::fmax(std::fabs(gn), std::fabs(g[e]));
      if (f > 0.01 && m > 0.0 && f / m > 0.01) {  // ten times tighter than the reference's rule
        ok = false;
        std::printf("  grad mismatch %s arg %u elem %zu: numeric %.6g analytic %.6g\n", g_case, i, e, gn, double(g[e]));
      }
    }
    TensorTools::set_elements(args[i], vals);
  }
  return ok;
}

static vector<float> cycle(size_t n, std::initializer_list<float> pattern) {
  vector<float> p(pattern), out(n);
  for (size_t i = 0; i < n; ++i) out[i] = p[i % p.size()];
  return out;
}

// ---- tests/test-rnn.cc:245-259 ----
static void lstm_node_h_fwd(Fixture& F) {
  g_case = "lstm_node_h_fwd";
  const unsigned hidden_dim = 3, batch_size = 2;
  Tensor c_t = F.input(Dim({hidden_dim}, batch_size), {0.f, 0.1f, 0.2f, 0.3f, 0.4f, 0.7f});
  Tensor gates_t = F.input(Dim({hidden_dim * 4}, batch_size),
                           {0.f, 0.1f, 0.2f, 0.3f, 0.4f, 0.5f, 0.f, -0.1f, -0.2f, -0.3f, -0.4f, -0.5f,
                            0.01f, 0.11f, 0.21f, 0.31f, 0.41f, 0.51f, -0.01f, -0.11f, -0.21f, -0.31f, -0.41f, -0.51f});
  Tensor h_t = F.dev.allocate_tensor(DeviceMempool::FXS, Dim({hidden_dim}, batch_size));
  VanillaLSTMH().forward_dev_impl(F.dev, {&c_t, &gates_t}, h_t);
  const vector<float> h = as_vector(h_t);
  CHECK_SMALL(h[0], 1.0e-6);
  CHECK_CLOSE(h[1], -0.009966799462, 0.001);
  CHECK_CLOSE(h[2], -0.03947506404, 0.001);
  CHECK_CLOSE(h[3], -0.002913126125, 0.001);
  CHECK_CLOSE(h[4], -0.04179438585, 0.001);
  CHECK_CLOSE(h[5], -0.1269172332, 0.001);
}

// ---- tests/test-rnn.cc:285-300 ----
static void lstm_node_c_fwd(Fixture& F) {
  g_case = "lstm_node_c_fwd";
  const unsigned hidden_dim = 3, batch_size = 2;
  Tensor c_tm1 = F.input(Dim({hidden_dim}, batch_size), {0.f, 0.1f, 0.2f, 0.3f, 0.4f, 0.5f});
  Tensor gates_t = F.input(Dim({hidden_dim * 4}, batch_size),
                           {0.f, 0.1f, 0.2f, 0.3f, 0.4f, 0.5f, 0.f, -0.1f, -0.2f, -0.3f, -0.4f, -0.5f,
                            0.01f, 0.11f, 0.21f, 0.31f, 0.41f, 0.51f, -0.01f, -0.11f, -0.21f, -0.31f, -0.41f, -0.51f});
  Tensor c_t = F.dev.allocate_tensor(DeviceMempool::FXS, Dim({hidden_dim}, batch_size));
  VanillaLSTMC().forward_dev_impl(F.dev, {&c_tm1, &gates_t}, c_t);
  const vector<float> c = as_vector(c_t);
  CHECK_SMALL(c[0], 1.0e-6);
  CHECK_SMALL(c[1], 1.0e-6);
  CHECK_SMALL(c[2], 1.0e-6);
  CHECK_CLOSE(c[3], 0.0899, 0.001);
  CHECK_CLOSE(c[4], 0.1189, 0.001);
  CHECK_CLOSE(c[5], 0.1479, 0.001);
}

// ---- tests/test-rnn.cc:301-339 ----
static void lstm_node_gates_fwd(Fixture& F) {
  g_case = "lstm_node_gates_fwd";
  const unsigned input_dim = 2, hidden_dim = 2, batch_size = 2;
  Tensor x_t = F.input(Dim({input_dim}, batch_size), {0.f, 0.1f, 0.2f, 0.3f});
  Tensor h_tm1 = F.input(Dim({input_dim}, batch_size), {0.f, -0.1f, 0.2f, -0.3f});
  Tensor Wx = F.input(Dim({hidden_dim * 4, input_dim}, 1), cycle(16, {0.f, 1.1f, 2.2f, 3.3f}));
  Tensor Wh = F.input(Dim({hidden_dim * 4, hidden_dim}, 1), cycle(16, {0.1f, 1.2f, 2.3f, 3.4f}));
  Tensor b = F.input(Dim({hidden_dim * 4}, 1), cycle(8, {0.f, 0.1f}));
  Tensor gates = F.dev.allocate_tensor(DeviceMempool::FXS, Dim({hidden_dim * 4}, batch_size));
  VanillaLSTMGates(false, 0.f).forward_dev_impl(F.dev, {&x_t, &h_tm1, &Wx, &Wh, &b}, gates);
  const vector<float> g = as_vector(gates);
  const double want[16] = {0.497500021, 0.522484825, 0.729087922, 0.748381722, 0.497500021, 0.522484825,
                           -0.009999656681, 0.08975778475, 0.497500021, 0.629483112, 0.866458277, 0.917586682,
                           0.497500021, 0.629483112, 0.7013741309, 0.8874941329};
  for (int i = 0; i < 16; ++i) CHECK_CLOSE(g[i], want[i], 0.001);
}

// ---- gradient checks: tests/test-rnn.cc:261-284 (H, C), :341-357 (gates), :402-460 (dropout) ----
static void lstm_node_gradients(Fixture& F) {
  const unsigned hidden_dim = 3, batch_size = 2, input_dim = 5;
  const vector<float> param_6 = {0.f, 0.1f, 0.2f, 0.3f, 0.4f, 0.5f};
  const vector<float> param_24 = cycle(24, {0.f, 0.1f, 0.2f, 0.3f, 0.4f, 0.5f});
  g_case = "lstm_node_h_gradient";
  {
    vector<Tensor> a = {F.input(Dim({hidden_dim}, batch_size), param_6), F.input(Dim({hidden_dim * 4}, batch_size), param_24)};
    CHECK(check_grad(F, VanillaLSTMH(), a, Dim({hidden_dim}, batch_size), {true, true}));
  }
  g_case = "lstm_node_c_gradient";
  {
    vector<Tensor> a = {F.input(Dim({hidden_dim}, batch_size), param_6), F.input(Dim({hidden_dim * 4}, batch_size), param_24)};
    CHECK(check_grad(F, VanillaLSTMC(), a, Dim({hidden_dim}, batch_size), {true, true}));
  }
  const vector<float> x10 = {0.1f, 0.2f, 0.3f, 0.4f, 0.5f, 0.4f, 0.5f, 0.3f, 0.4f, 0.5f};
  const vector<float> Wx60 = cycle(60, {0.1f, 0.2f, 0.3f, 0.4f, 0.5f, 0.4f, 0.5f, 0.3f, 0.4f, 0.5f});
  vector<float> Wh36 = cycle(36, {0.1f, 0.2f, 0.3f, 0.4f, 0.5f, 0.f});
  Wh36[35] = -0.5f;
  const vector<float> b12 = {0.f, 0.1f, 0.2f, 0.3f, 0.4f, 0.5f, 0.f, 0.4f, 0.5f, 0.3f, 0.4f, 0.5f};
  g_case = "lstm_node_gates_bwd";
  {
    vector<Tensor> a = {F.input(Dim({input_dim}, batch_size), x10), F.input(Dim({hidden_dim}, batch_size), param_6),
                        F.input(Dim({hidden_dim * 4, input_dim}), Wx60), F.input(Dim({hidden_dim * 4, hidden_dim}), Wh36),
                        F.input(Dim({hidden_dim * 4}), b12)};
    CHECK(check_grad(F, VanillaLSTMGates(false, 0.f), a, Dim({hidden_dim * 4}, batch_size), {true, true, true, true, true}));
  }
  g_case = "lstm_node_gates_dropout_bwd";
  {
    vector<Tensor> a = {F.input(Dim({input_dim}, batch_size), x10), F.input(Dim({hidden_dim}, batch_size), param_6),
                        F.input(Dim({hidden_dim * 4, input_dim}), Wx60), F.input(Dim({hidden_dim * 4, hidden_dim}), Wh36),
                        F.input(Dim({hidden_dim * 4}), b12),
                        F.input(Dim({input_dim}, batch_size), {0.f, 0.f, 1.f, 0.f, 0.f, 1.f, 1.f, 1.f, 1.f, 1.f}),
                        F.input(Dim({hidden_dim}, batch_size), {0.f, 1.f, 1.f, 1.f, 1.f, 0.f})};
    CHECK(check_grad(F, VanillaLSTMGates(true, 0.f), a, Dim({hidden_dim * 4}, batch_size),
                     {true, true, true, true, true, false, false}));
  }
  g_case = "lstm_node_gates_multi_input_bwd";  // tests/test-rnn.cc:433-460: two inputs of 2 and 3 rows
  {
    vector<Tensor> a = {F.input(Dim({2}, batch_size), {0.1f, 0.2f, 0.4f, 0.5f}),
                        F.input(Dim({3}, batch_size), {0.3f, 0.4f, 0.5f, 0.3f, 0.4f, 0.5f}),
                        F.input(Dim({hidden_dim}, batch_size), param_6), F.input(Dim({hidden_dim * 4, input_dim}), Wx60),
                        F.input(Dim({hidden_dim * 4, hidden_dim}), Wh36), F.input(Dim({hidden_dim * 4}), b12)};
    CHECK(check_grad(F, VanillaLSTMGates(false, 0.f), a, Dim({hidden_dim * 4}, batch_size),
                     {true, true, true, true, true, true}));
  }
}

// ---- tests/test-nodes.cc:854-860 (tanh), :944-960 (rectify, logistic), :1408-1484 (cmult) on {1.1,-2.2,3.3} ----
static void elementwise_gradients(Fixture& F) {
  const vector<float> param_vals = {1.1f, -2.2f, 3.3f}, param2_vals = {2.2f, 3.4f, -1.2f};
  g_case = "tanh_gradient";
  { vector<Tensor> a = {F.input(Dim({3}), param_vals)}; CHECK(check_grad(F, Tanh(), a, Dim({3}), {true})); }
  g_case = "logistic_gradient";
  { vector<Tensor> a = {F.input(Dim({3}), param_vals)}; CHECK(check_grad(F, LogisticSigmoid(), a, Dim({3}), {true})); }
  g_case = "rectify_gradient";
  { vector<Tensor> a = {F.input(Dim({3}), param_vals)}; CHECK(check_grad(F, Rectify(), a, Dim({3}), {true})); }
  g_case = "cmult_gradient";
  {
    vector<Tensor> a = {F.input(Dim({3}), param_vals), F.input(Dim({3}), param2_vals)};
    CHECK(check_grad(F, CwiseMultiply(), a, Dim({3}), {true, true}));
  }
  g_case = "cmult_batch_gradient";  // one side with batch size 1: its gradient is summed over the batch
  {
    vector<Tensor> a = {F.input(Dim({3}, 2), {1.1f, -2.2f, 3.3f, 0.5f, 0.25f, -1.5f}), F.input(Dim({3}), param2_vals)};
    CHECK(check_grad(F, CwiseMultiply(), a, Dim({3}, 2), {true, true}));
  }
  g_case = "sum_batches_gradient";  // tests/test-nodes.cc:2229-2236
  {
    vector<Tensor> a = {F.input(Dim({3}, 2), {1.1f, -2.2f, 3.3f, 0.5f, 0.25f, -1.5f})};
    CHECK(check_grad(F, SumBatches(), a, Dim({3}), {true}));
    Tensor y = F.dev.allocate_tensor(DeviceMempool::FXS, Dim({3}));
    SumBatches().forward_dev_impl(F.dev, {&a[0]}, y);
    const vector<float> v = as_vector(y);
    CHECK_CLOSE(v[0], 1.6, 0.001);
    CHECK_CLOSE(v[1], -1.95, 0.001);
    CHECK_CLOSE(v[2], 1.8, 0.001);
  }
}

// ---- tests/test-nodes.cc:2404-2426 ----
static void layer_norm(Fixture& F) {
  g_case = "layer_norm_forward";
  {
    Tensor x = F.input(Dim({3}), {1.1f, -2.2f, 3.3f}), g = F.input(Dim({3}), {1.f, 1.f, 1.f}), b = F.input(Dim({3}), {0.f, 0.f, 0.f});
    Tensor y = F.dev.allocate_tensor(DeviceMempool::FXS, Dim({3}));
    LayerNorm().forward_dev_impl(F.dev, {&x, &g, &b}, y);
    const vector<float> v = as_vector(y);
    const double mu = (v[0] + v[1] + v[2]) / 3.0;
    const double std = std::sqrt(((v[0] - mu) * (v[0] - mu) + (v[1] - mu) * (v[1] - mu) + (v[2] - mu) * (v[2] - mu)) / 3.0);
    CHECK_SMALL(mu, 1e-6);
    CHECK_CLOSE(std, 1.0, 0.01);
  }
  g_case = "layer_norm_backward";
  {
    vector<Tensor> a = {F.input(Dim({3}), {1.1f, -2.2f, 3.3f}), F.input(Dim({3}), {2.2f, 3.4f, -1.2f}),
                        F.input(Dim({3}), {1.1f, 2.2f, 3.3f})};
    CHECK(check_grad(F, LayerNorm(), a, Dim({3}), {true, true, true}));
  }
  g_case = "layer_norm_batch_backward";
  {
    vector<Tensor> a = {F.input(Dim({4}, 3), {1.1f, -2.2f, 3.3f, 0.4f, 0.5f, 0.25f, -1.5f, 2.f, -0.3f, 0.7f, 1.9f, -2.4f}),
                        F.input(Dim({4}), {2.2f, 3.4f, -1.2f, 0.8f}), F.input(Dim({4}), {1.1f, 2.2f, 3.3f, -0.4f})};
    CHECK(check_grad(F, LayerNorm(), a, Dim({4}, 3), {true, true, true}));
  }
}

// ---- lookup (tests/test-nodes.cc:2485-2541) and PickNegLogSoftmax / LogSoftmax (:337-383, :1083-1130, :2088-2105) ----
static void lookup_and_softmax(Fixture& F) {
  g_case = "lookup_forward_bit_exact";
  const unsigned D = 3, V = 5;
  vector<float> table(D * V);
  for (size_t i = 0; i < table.size(); ++i) table[i] = 0.1f * float(i) - 0.45f;
  Tensor all_values = F.input(Dim({D}, V), table, DeviceMempool::PS);
  Tensor all_grads = F.zeros(Dim({D}, V), DeviceMempool::PS);
  const vector<unsigned> ids = {2, 0, 2, 4, 2};
  LookupNode lookup(&all_values, &all_grads, &ids);
  lookup.aux_mem = F.dev.pools[0]->allocate(lookup.aux_storage_size());
  Tensor fx = F.dev.allocate_tensor(DeviceMempool::FXS, Dim({D}, (unsigned)ids.size()));
  lookup.forward_dev_impl(F.dev, {}, fx);
  const vector<float> got = as_vector(fx);
  for (size_t b = 0; b < ids.size(); ++b)
    for (unsigned j = 0; j < D; ++j) CHECK(std::memcmp(&got[b * D + j], &table[ids[b] * D + j], sizeof(float)) == 0);
  g_case = "lookup_accumulate_grad";
  vector<float> gv(D * ids.size());
  for (size_t i = 0; i < gv.size(); ++i) gv[i] = 0.5f + 0.25f * float(i);
  Tensor g = F.input(Dim({D}, (unsigned)ids.size()), gv, DeviceMempool::DEDFS);
  lookup.accumulate_grad(F.dev, fx, g);
  const vector<float> acc = as_vector(all_grads);
  for (unsigned r = 0; r < V; ++r)
    for (unsigned j = 0; j < D; ++j) {
      float want = 0.f;
      for (size_t b = 0; b < ids.size(); ++b)
        if (ids[b] == r) want += gv[b * D + j];  // ascending b: the CPU path's order
      CHECK_CLOSE(acc[r * D + j] + 1.0, want + 1.0, 0.001);
    }
  g_case = "lookup_out_of_range";
  {
    const vector<unsigned> bad = {1, 7};
    LookupNode l2(&all_values, &all_grads, &bad);
    l2.aux_mem = F.dev.pools[0]->allocate(l2.aux_storage_size());
    Tensor f2 = F.dev.allocate_tensor(DeviceMempool::FXS, Dim({D}, 2));
    bool threw = false;
    try { l2.forward_dev_impl(F.dev, {}, f2); } catch (const std::invalid_argument&) { threw = true; }
    CHECK(threw);
  }
  g_case = "pickneglogsoftmax_batch_gradient";
  {
    const vector<unsigned> idx = {1, 2};
    PickNegLogSoftmax pnls(&idx);
    pnls.aux_mem = F.dev.pools[0]->allocate(pnls.aux_storage_size());
    vector<Tensor> a = {F.input(Dim({3}, 2), {1.1f, -2.2f, 3.3f, 2.1f, -1.2f, 4.3f})};
    CHECK(check_grad(F, pnls, a, Dim({1}, 2), {true}));
    // value: -log softmax(x)[idx]
    Tensor y = F.dev.allocate_tensor(DeviceMempool::FXS, Dim({1}, 2));
    pnls.forward_dev_impl(F.dev, {&a[0]}, y);
    const vector<float> v = as_vector(y);
    const double z0 = std::log(std::exp(1.1) + std::exp(-2.2) + std::exp(3.3));
    const double z1 = std::log(std::exp(2.1) + std::exp(-1.2) + std::exp(4.3));
    CHECK_CLOSE(v[0], z0 - (-2.2), 0.001);
    CHECK_CLOSE(v[1], z1 - 4.3, 0.001);
    const vector<unsigned> bad = {1, 3};
    PickNegLogSoftmax p2(&bad);
    p2.aux_mem = pnls.aux_mem;
    bool threw = false;
    try { p2.forward_dev_impl(F.dev, {&a[0]}, y); } catch (const std::invalid_argument&) { threw = true; }
    CHECK(threw);
  }
  g_case = "log_softmax_gradient";
  {
    const Dim d({3}, 2);
    LogSoftmax ls(d);
    ls.aux_mem = F.dev.pools[0]->allocate(ls.aux_storage_size());
    vector<Tensor> a = {F.input(d, {1.1f, -2.2f, 3.3f, 2.1f, -1.2f, 4.3f})};
    CHECK(check_grad(F, ls, a, d, {true}));
  }
  g_case = "affine_gradient";  // tests/test-nodes.cc:384-416
  {
    vector<Tensor> a = {F.input(Dim({3}), {1.1f, -2.2f, 3.3f}),
                        F.input(Dim({3, 2}), {0.1f, 0.2f, 0.3f, -0.4f, 0.5f, 0.6f}),
                        F.input(Dim({2}, 2), {1.f, -0.5f, 0.25f, 2.f})};
    CHECK(check_grad(F, AffineTransform(), a, Dim({3}, 2), {true, true, true}));
  }
}

// tests/test-nodes.cc:1236-1272 only run these nodes ("noise is random, so it cannot be tested
// simply"); here the values are checked against what the node's definition fixes.
static void random_nodes(Fixture& F) {
  g_case = "dropout_forward";
  {
    F.dev.reset_rng(3);
    const Dim d({64}, 8);
    vector<float> xv(d.size());
    for (size_t i = 0; i < xv.size(); ++i) xv[i] = 0.25f + 0.01f * float(i);
    Tensor x = F.input(d, xv);
    Dropout node(d, 0.5f);
    node.aux_mem = F.dev.pools[0]->allocate(node.aux_storage_size());
    Tensor fx = F.dev.allocate_tensor(DeviceMempool::FXS, d);
    node.forward_dev_impl(F.dev, {&x}, fx);
    const vector<float> y = as_vector(fx);
    Tensor mask(d, static_cast<float*>(node.aux_mem), &F.dev, DeviceMempool::FXS);
    const vector<float> m = as_vector(mask);
    size_t kept = 0;
    for (size_t i = 0; i < y.size(); ++i) {
      CHECK(m[i] == 0.f || m[i] == 2.f);  // bernoulli(1 - p) * 1 / (1 - p)
      CHECK(y[i] == xv[i] * m[i]);
      kept += m[i] != 0.f;
    }
    CHECK(kept > y.size() * 2 / 5 && kept < y.size() * 3 / 5);
    // backward accumulates dEdf (.) mask
    vector<float> gv(d.size(), 1.5f);
    Tensor dEdf = F.input(d, gv, DeviceMempool::DEDFS);
    Tensor dEdx = F.zeros(d);
    TensorTools::constant(dEdx, 1.f);
    node.backward_dev_impl(F.dev, {&x}, fx, dEdf, 0, dEdx);
    const vector<float> g = as_vector(dEdx);
    for (size_t i = 0; i < g.size(); ++i) CHECK(g[i] == 1.f + 1.5f * m[i]);
    // the same seed gives the same mask again; the next draw differs
    F.dev.reset_rng(3);
    node.forward_dev_impl(F.dev, {&x}, fx);
    CHECK(as_vector(mask) == m);
    node.forward_dev_impl(F.dev, {&x}, fx);
    CHECK(as_vector(mask) != m);
  }
  g_case = "random_nodes";
  {
    F.dev.reset_rng(1);
    const Dim d({1000}, 4);
    Tensor fx = F.dev.allocate_tensor(DeviceMempool::FXS, d);
    RandomNormal(2.f, 0.5f).forward_dev_impl(F.dev, {}, fx);
    vector<float> v = as_vector(fx);
    double s = 0, ss = 0;
    for (float e : v) { s += e; ss += double(e) * e; }
    const double mean = s / v.size(), var = ss / v.size() - mean * mean;
    CHECK_SMALL(mean - 2.0, 0.05);
    CHECK_SMALL(std::sqrt(var) - 0.5, 0.05);
    RandomUniform(-1.f, 3.f).forward_dev_impl(F.dev, {}, fx);
    v = as_vector(fx);
    s = 0;
    for (float e : v) { CHECK(e > -1.f && e <= 3.f); s += e; }
    CHECK_SMALL(s / v.size() - 1.0, 0.1);
    RandomBernoulli(0.25f, 4.f).forward_dev_impl(F.dev, {}, fx);
    v = as_vector(fx);
    size_t ones = 0;
    for (float e : v) { CHECK(e == 0.f || e == 4.f); ones += e != 0.f; }
    CHECK_SMALL(double(ones) / v.size() - 0.25, 0.03);
    bool threw = false;
    try { RandomBernoulli(1.5f).forward_dev_impl(F.dev, {}, fx); } catch (const std::invalid_argument&) { threw = true; }
    CHECK(threw);
  }
}

int main(int argc, char** argv) {
  if (argc > 1 && std::strcmp(argv[1], "--no-gpu") == 0) {
    try {
      Device_GPU dev(0, 1, 1, 1, 1);
    } catch (const cuda_exception& e) {
      std::printf("device creation failed as expected: %s\n", e.what());
      return 0;
    }
    std::printf("a GPU is present: nothing to check in --no-gpu mode\n");
    return 0;
  }
  Fixture F;
  const std::vector<std::function<void(Fixture&)>> cases = {lstm_node_h_fwd,      lstm_node_c_fwd, lstm_node_gates_fwd,
                                                             lstm_node_gradients,  elementwise_gradients, layer_norm,
                                                             lookup_and_softmax,   random_nodes};
  for (const auto& c : cases) {
    c(F);
    F.reset();
  }
  std::printf("%d checks, %d failed\n", g_checks, g_failed);
  return g_failed > 255 ? 255 : g_failed;
}
