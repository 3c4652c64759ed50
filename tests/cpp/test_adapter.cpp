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
    // the same with the activation derivative cached in aux_mem across the five backward calls
    g_case = "lstm_node_gates_bwd_cached_dpre";
    const Dim gd({hidden_dim * 4}, batch_size);
    VanillaLSTMGates cached(false, 0.f, gd);
    CHECK(cached.aux_storage_size() == gd.size() * sizeof(float));
    Tensor aux = F.dev.allocate_tensor(DeviceMempool::FXS, gd);
    cached.aux_mem = aux.v;
    CHECK(check_grad(F, cached, a, gd, {true, true, true, true, true}));
    // and call by call against the uncached node, bit for bit
    VanillaLSTMGates plain(false, 0.f);
    vector<const Tensor*> xs;
    for (Tensor& t : a) xs.push_back(&t);
    Tensor fx = F.dev.allocate_tensor(DeviceMempool::FXS, gd), dEdf = F.input(gd, cycle(gd.size(), {0.3f, -0.2f, 0.5f, 0.1f, -0.4f}), DeviceMempool::DEDFS);
    plain.forward_dev_impl(F.dev, xs, fx);
    cached.forward_dev_impl(F.dev, xs, fx);
    for (unsigned i = 0; i < 5; ++i) {
      Tensor g0 = F.zeros(a[i].d), g1 = F.zeros(a[i].d);
      plain.backward_dev_impl(F.dev, xs, fx, dEdf, i, g0);
      cached.backward_dev_impl(F.dev, xs, fx, dEdf, i, g1);
      CHECK(as_vector(g0) == as_vector(g1));
    }
    // a second backward pass on the same forward: the executor refills pools[DEDFS], so the same dEdf address
    // comes back with other contents (dynet/exec.cc:178-208); the cached derivative must not be reused
    g_case = "lstm_node_gates_bwd_second_pass_same_dEdf_address";
    TensorTools::set_elements(dEdf, cycle(gd.size(), {-0.7f, 0.4f, 0.2f, -0.1f, 0.6f, 0.3f, -0.5f}));
    for (unsigned i = 0; i < 5; ++i) {
      Tensor g0 = F.zeros(a[i].d), g1 = F.zeros(a[i].d);
      plain.backward_dev_impl(F.dev, xs, fx, dEdf, i, g0);
      cached.backward_dev_impl(F.dev, xs, fx, dEdf, i, g1);
      CHECK(as_vector(g0) == as_vector(g1));
    }
    // a pass that asks for some of the arguments only (needs_derivative), then a new one starting at a later index
    TensorTools::set_elements(dEdf, cycle(gd.size(), {0.9f, -0.3f, 0.1f}));
    for (unsigned i : {1u, 3u, 2u, 4u}) {  // 1, 3 = one pass; 2, 4 = the next (2 <= 3)
      if (i == 2u) TensorTools::set_elements(dEdf, cycle(gd.size(), {0.2f, 0.8f, -0.6f, 0.5f}));
      Tensor g0 = F.zeros(a[i].d), g1 = F.zeros(a[i].d);
      plain.backward_dev_impl(F.dev, xs, fx, dEdf, i, g0);
      cached.backward_dev_impl(F.dev, xs, fx, dEdf, i, g1);
      CHECK(as_vector(g0) == as_vector(g1));
    }
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

// ---- the executor's accumulation of a parameter gradient over the timesteps of an unrolled LSTM
// (dynet/exec.cc:247-280): T gates nodes add their products into the dEdf of the same ParameterNode.  With the
// gradients of the parameter nodes registered as deferrable, the nodes record, and the gradient is formed as one
// product when it is first read -- which every way of reading it through this adapter does.
static void deferred_parameter_gradients(Fixture& F) {
  g_case = "deferred_parameter_gradients";
  const unsigned H = 8, I = 12, B = 16, T = 3;
  auto ramp = [](size_t n, float a, float b) {
    vector<float> v(n);
    for (size_t k = 0; k < n; ++k) v[k] = a * std::sin(0.37f * float(k) + b);
    return v;
  };
  ParameterStorage pWx, pWh, pb;
  pWx.values = F.input(Dim({4 * H, I}), ramp(4 * H * I, 0.3f, 0.1f), DeviceMempool::PS);
  pWh.values = F.input(Dim({4 * H, H}), ramp(4 * H * H, 0.3f, 0.7f), DeviceMempool::PS);
  pb.values = F.input(Dim({4 * H}), ramp(4 * H, 0.1f, 0.3f), DeviceMempool::PS);
  for (ParameterStorage* ps : {&pWx, &pWh, &pb}) ps->g = F.zeros(ps->values.d, DeviceMempool::PS);
  ParameterNode nWx(&pWx), nWh(&pWh, 0.5f), nb(&pb);
  Tensor Wx = F.dev.allocate_tensor(DeviceMempool::FXS, pWx.values.d), Wh = F.dev.allocate_tensor(DeviceMempool::FXS, pWh.values.d),
         b = F.dev.allocate_tensor(DeviceMempool::FXS, pb.values.d);
  nWx.forward_dev_impl(F.dev, {}, Wx);
  nWh.forward_dev_impl(F.dev, {}, Wh);
  nb.forward_dev_impl(F.dev, {}, b);
  {  // forward = values * weight decay
    const vector<float> v = as_vector(pWh.values), w = as_vector(Wh);
    bool ok = true;
    for (size_t k = 0; k < v.size(); ++k) ok = ok && w[k] == 0.5f * v[k];
    CHECK(ok);
  }
  bool threw = false;
  try {
    Tensor dummy;
    nWx.backward_dev_impl(F.dev, {}, Wx, Wx, 0, dummy);
  } catch (const std::runtime_error&) {
    threw = true;
  }
  CHECK(threw);
  const Dim gd({4 * H}, B);
  vector<Tensor> x, h, fx, dEdf, aux;
  vector<VanillaLSTMGates> nodes;
  for (unsigned t = 0; t < T; ++t) {
    x.push_back(F.input(Dim({I}, B), ramp(I * B, 0.8f, 0.2f * t)));
    h.push_back(F.input(Dim({H}, B), ramp(H * B, 0.6f, 1.0f + 0.3f * t)));
    fx.push_back(F.dev.allocate_tensor(DeviceMempool::FXS, gd));
    aux.push_back(F.dev.allocate_tensor(DeviceMempool::FXS, gd));
    dEdf.push_back(F.input(gd, ramp(gd.size(), 0.5f, 2.0f + t), DeviceMempool::DEDFS));
    nodes.emplace_back(false, 0.f, gd);
  }
  auto run_backward = [&](Tensor& dWx, Tensor& dWh, Tensor& db) {
    for (int t = int(T) - 1; t >= 0; --t) {  // reverse topological order
      vector<const Tensor*> xs = {&x[t], &h[t], &Wx, &Wh, &b};
      nodes[t].aux_mem = aux[t].v;
      nodes[t].forward_dev_impl(F.dev, xs, fx[t]);
      nodes[t].backward_dev_impl(F.dev, xs, fx[t], dEdf[t], 2, dWx);
      nodes[t].backward_dev_impl(F.dev, xs, fx[t], dEdf[t], 3, dWh);
      nodes[t].backward_dev_impl(F.dev, xs, fx[t], dEdf[t], 4, db);
    }
  };
  // node by node, as without the registry
  F.dev.deferred->clear();
  Tensor eWx = F.zeros(Wx.d), eWh = F.zeros(Wh.d), eb = F.zeros(b.d);
  run_backward(eWx, eWh, eb);
  CHECK(!F.dev.deferred->pending(eWx.v) && !F.dev.deferred->pending(eWh.v) && !F.dev.deferred->pending(eb.v));
  const vector<float> wantWx = as_vector(eWx), wantWh = as_vector(eWh), wantb = as_vector(eb);
  // recorded: the executor registers the parameter nodes' gradients at the start of backward
  Tensor dWx = F.zeros(Wx.d), dWh = F.zeros(Wh.d), db = F.zeros(b.d);
  F.dev.deferred->clear();
  for (Tensor* g : {&dWx, &dWh, &db}) F.dev.deferred->allow(g->v);
  run_backward(dWx, dWh, db);
  CHECK(F.dev.deferred->pending(dWx.v) && F.dev.deferred->pending(dWh.v) && F.dev.deferred->pending(db.v));
  auto close = [](const vector<float>& a, const vector<float>& w) {
    if (a.size() != w.size()) return false;
    double scale = 0;
    for (float v : w) scale = std::fmax(scale, std::fabs(v));
    for (size_t k = 0; k < a.size(); ++k)
      if (std::fabs(double(a[k]) - w[k]) > 1e-5 * scale) return false;
    return scale > 0;
  };
  // (1) as_vector: whoever looks at the gradient sees all of it
  CHECK(close(as_vector(dWx), wantWx));
  CHECK(!F.dev.deferred->pending(dWx.v));
  // (2) the executor's hand-over to the parameter
  nWh.accumulate_grad(dWh);
  CHECK(!F.dev.deferred->pending(dWh.v) && pWh.nonzero_grad);
  CHECK(close(as_vector(pWh.g), wantWh));
  // (3) everything that is left
  F.dev.deferred->flush_all();
  CHECK(!F.dev.deferred->pending(db.v));
  CHECK(close(as_vector(db), wantb));
  // a second backward pass records afresh and adds to what the gradient holds
  F.dev.deferred->clear();
  F.dev.deferred->allow(dWx.v);
  Tensor d2Wh = F.zeros(Wh.d), d2b = F.zeros(b.d);
  run_backward(dWx, d2Wh, d2b);  // dWh and db not registered: formed at once
  CHECK(!F.dev.deferred->pending(d2Wh.v) && close(as_vector(d2Wh), wantWh));
  vector<float> twice = wantWx;
  for (float& v : twice) v *= 2.f;
  CHECK(close(as_vector(dWx), twice));
  F.dev.deferred->clear();
}

// ---- tests/test-nodes.cc:1277-1321: argmax_forward, argmax_backward, straight_through_backward ----
static void argmax_node(Fixture& F) {
  g_case = "argmax_node";
  const vector<float> batch_vals = {1.1f, 2.6f, 3.3f, 4.0f, 5.1f, 6.6f};
  const Dim xd({3}, 2);
  Tensor x = F.input(xd, batch_vals);
  vector<const Tensor*> xs = {&x};
  for (bool st : {false, true}) {
    Argmax node(xd, 0, st);
    CHECK(node.aux_storage_size() == 2 * sizeof(long long));
    Tensor aux = F.dev.allocate_tensor(DeviceMempool::FXS, Dim({4}));  // 16 bytes
    node.aux_mem = aux.v;
    Tensor fx = F.dev.allocate_tensor(DeviceMempool::FXS, xd);
    node.forward_dev_impl(F.dev, xs, fx);
    CHECK(as_vector(fx) == (vector<float>{0.f, 0.f, 1.f, 0.f, 0.f, 1.f}));
    // z = sum_batches(dot_product(y, x_)) with x_ = batch_vals: dz/dy = batch_vals
    Tensor dEdf = F.input(xd, batch_vals, DeviceMempool::DEDFS), dx = F.zeros(xd);
    node.backward_dev_impl(F.dev, xs, fx, dEdf, 0, dx);
    CHECK(as_vector(dx) == (st ? batch_vals : vector<float>(6, 0.f)));
  }
  bool threw = false;
  try {
    Argmax bad(Dim({3, 2}), 0, false);
  } catch (const std::invalid_argument&) {
    threw = true;
  }
  CHECK(threw);
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

// ---- tests/test-nodes.cc:297-372 (sum, logsumexp) and :1984-2000 (pick_range): the node-level part of each ----
static void sum_logsumexp_pick_range(Fixture& F) {
  const vector<float> param_vals = {1.1f, -2.2f, 3.3f}, param2_vals = {2.2f, 3.4f, -1.2f};
  const vector<float> batch_vals = {1.f, 2.f, 3.f, 4.f, 5.f, 6.f};
  g_case = "sum_gradient";
  {
    vector<Tensor> a = {F.input(Dim({3}), param2_vals), F.input(Dim({3}), param_vals), F.input(Dim({3}), param2_vals)};
    CHECK(check_grad(F, Sum(), a, Dim({3}), {true, true, true}));
    Tensor y = F.dev.allocate_tensor(DeviceMempool::FXS, Dim({3}));
    Sum().forward_dev_impl(F.dev, {&a[0], &a[1], &a[2]}, y);
    const vector<float> v = as_vector(y);
    for (int j = 0; j < 3; ++j) CHECK_CLOSE(v[j], 2.0 * param2_vals[j] + param_vals[j], 0.001);
  }
  g_case = "sum_batch_gradient";  // arguments of batch size 2 and 1: the latter's gradient is summed over the batch
  {
    vector<Tensor> a = {F.input(Dim({3}, 2), batch_vals), F.input(Dim({3}), param_vals), F.input(Dim({3}, 2), batch_vals)};
    CHECK(check_grad(F, Sum(), a, Dim({3}, 2), {true, true, true}));
  }
  g_case = "empty_sum";
  {
    bool thrown = false;
    Tensor y = F.dev.allocate_tensor(DeviceMempool::FXS, Dim({3}));
    try {
      Sum().forward_dev_impl(F.dev, {}, y);
    } catch (const std::invalid_argument&) {
      thrown = true;
    }
    CHECK(thrown);
  }
  g_case = "logsumexp_gradient";
  {
    vector<Tensor> a = {F.input(Dim({1}), {2.2f}), F.input(Dim({1}), {1.1f})};
    CHECK(check_grad(F, LogSumExp(), a, Dim({1}), {true, true}));
    Tensor y = F.dev.allocate_tensor(DeviceMempool::FXS, Dim({1}));
    LogSumExp().forward_dev_impl(F.dev, {&a[0], &a[1]}, y);
    CHECK_CLOSE(as_vector(y)[0], std::log(std::exp(2.2) + std::exp(1.1)), 0.001);
  }
  g_case = "logsumexp_vector_gradient";
  {
    vector<Tensor> a = {F.input(Dim({3}), param_vals), F.input(Dim({3}), param2_vals)};
    CHECK(check_grad(F, LogSumExp(), a, Dim({3}), {true, true}));
  }
  g_case = "logsumexp_singleelem_batch_gradient";
  {
    vector<Tensor> a = {F.input(Dim({1}, 3), param_vals)};
    CHECK(check_grad(F, LogSumExp(), a, Dim({1}, 3), {true}));
  }
  g_case = "logsumexp_inequal_batch_gradient";
  {
    vector<float> x3(6);
    for (int j = 0; j < 6; ++j) x3[j] = param_vals[j % 3] + batch_vals[j];
    vector<Tensor> a = {F.input(Dim({3}), param_vals), F.input(Dim({3}, 2), x3)};
    CHECK(check_grad(F, LogSumExp(), a, Dim({3}, 2), {true, true}));
  }
  g_case = "logsumexp_forty_arguments";  // more than one launch takes: chained through the result
  {
    vector<Tensor> a;
    vector<const Tensor*> xs;
    double want = 0;
    for (int k = 0; k < 40; ++k) {
      a.push_back(F.input(Dim({1}), {0.1f * float(k) - 2.f}));
      want += std::exp(0.1 * k - 2.0);
    }
    for (Tensor& t : a) xs.push_back(&t);
    Tensor y = F.dev.allocate_tensor(DeviceMempool::FXS, Dim({1}));
    LogSumExp().forward_dev_impl(F.dev, xs, y);
    CHECK_CLOSE(as_vector(y)[0], std::log(want), 0.001);
  }
  g_case = "pick_range_gradient";
  {
    vector<Tensor> a = {F.input(Dim({3}), param_vals)};
    CHECK(check_grad(F, PickRange(0, 2), a, Dim({2}), {true}));
    Tensor y = F.dev.allocate_tensor(DeviceMempool::FXS, Dim({2}));
    PickRange(0, 2).forward_dev_impl(F.dev, {&a[0]}, y);
    const vector<float> v = as_vector(y);
    CHECK(v[0] == param_vals[0] && v[1] == param_vals[1]);
  }
  g_case = "pick_range_dim_gradient";
  {
    const vector<float> sq = {1.1f, 2.2f, 3.3f, 1.2f, 2.1f, 3.4f, 1.3f, 2.3f, 3.5f};  // 3 x 3, column-major
    vector<Tensor> a = {F.input(Dim({3, 3}), sq)};
    CHECK(check_grad(F, PickRange(0, 2, 1), a, Dim({3, 2}), {true}));
    Tensor y = F.dev.allocate_tensor(DeviceMempool::FXS, Dim({3, 2}));
    PickRange(1, 3, 1).forward_dev_impl(F.dev, {&a[0]}, y);
    const vector<float> v = as_vector(y);
    for (int j = 0; j < 6; ++j) CHECK(v[j] == sq[3 + j]);
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

// ---- component-wise nodes with dimension broadcast (tests/test-nodes.cc:177-212, 583-608, 1457-1484, 384-391) ----
static void cwise_broadcast(Fixture& F) {
  const vector<float> param1 = {1.1f, -2.2f, 3.3f}, param4 = {1.1f, 2.2f, 3.3f, -1.2f, 2.1f, 3.4f};
  const vector<float> cube1 = {.051f, .062f, .073f, .052f, .062f, .072f, .053f, .063f, .073f,
                               .111f, -.122f, -.033f, -.112f, -.022f, -.132f, -.113f, -.123f, -.133f,
                               .211f, .222f, .233f, .212f, .222f, .232f, .213f, .223f, .233f};
  const Dim two[] = {Dim({3, 1}, 2), Dim({3, 2}, 1)};
  const Dim three[] = {Dim({3, 3, 3}, 1), Dim({3, 3, 1}, 3), Dim({1, 3, 3}, 3), Dim({9, 3, 1}, 1), Dim({1, 3, 9}, 1),
                       Dim({1, 3, 1}, 9)};
  auto both_orders = [&](const Node& node, const Dim& d1, const vector<float>& v1, const Dim& d2,
                         const vector<float>& v2, bool swap_too) {
    { vector<Tensor> a = {F.input(d1, v1), F.input(d2, v2)}; CHECK(check_grad(F, node, a, d2, {true, true})); }
    if (swap_too) { vector<Tensor> a = {F.input(d2, v2), F.input(d1, v1)}; CHECK(check_grad(F, node, a, d2, {true, true})); }
    F.reset();
  };
  for (const Dim& d : two) {
    g_case = "cadd_broadcast2_gradient";
    both_orders(CwiseSum(), Dim({3, 1}), param1, d, param4, true);
    g_case = "cmult_broadcast2_gradient";
    both_orders(CwiseMultiply(), Dim({3, 1}), param1, d, param4, true);
    g_case = "cdiv_broadcast2_gradient";  // cdiv(x2, x1): the denominator is the broadcast side
    { vector<Tensor> a = {F.input(d, param4), F.input(Dim({3, 1}), param1)}; CHECK(check_grad(F, CwiseQuotient(), a, d, {true, true})); }
    F.reset();
  }
  for (const Dim& d : three) {
    g_case = "cadd_broadcast3_gradient";
    both_orders(CwiseSum(), Dim({1, 3, 1}), param1, d, cube1, true);
    g_case = "cmult_broadcast3_gradient";
    both_orders(CwiseMultiply(), Dim({1, 3, 1}), param1, d, cube1, true);
    g_case = "cdiv_broadcast3_gradient";
    { vector<Tensor> a = {F.input(d, cube1), F.input(Dim({1, 3, 1}), param1)}; CHECK(check_grad(F, CwiseQuotient(), a, d, {true, true})); }
    F.reset();
  }
  g_case = "cadd_broadcast2_neg_val";  // tests/test-nodes.cc:206-213: sum of x1 - x2 is -6.5
  {
    Tensor x1 = F.input(Dim({3, 1}), param1), x2 = F.input(Dim({3, 1}, 2), param4);
    Tensor nx2 = F.dev.allocate_tensor(DeviceMempool::FXS, x2.d), y = F.dev.allocate_tensor(DeviceMempool::FXS, x2.d);
    Negate().forward_dev_impl(F.dev, {&x2}, nx2);
    CwiseSum().forward_dev_impl(F.dev, {&x1, &nx2}, y);
    double z = 0;
    for (float e : as_vector(y)) z += e;
    CHECK_CLOSE(z, -6.5, 0.001);
  }
  g_case = "softmax_logsumexp_dims_gradient";  // tests/test-nodes.cc: softmax_cols_gradient, logsumexp_dim_gradient
  for (unsigned dim : {0u, 1u}) {
    const vector<float> sq = {1.1f, 2.2f, 3.4f, 1.2f, 2.5f, 3.2f, 5.3f, 2.3f, 3.3f, -0.4f, 0.6f, 1.7f};
    { vector<Tensor> a = {F.input(Dim({3, 2}, 2), sq)}; CHECK(check_grad(F, Softmax(dim), a, Dim({3, 2}, 2), {true})); }
    { vector<Tensor> a = {F.input(Dim({3, 2}, 2), sq)};
      CHECK(check_grad(F, LogSumExpDimension(dim), a, dim == 0 ? Dim({2}, 2) : Dim({3}, 2), {true})); }
    F.reset();
  }
  g_case = "matmul_batched_left_gradient";  // MatrixMultiply with a batched left operand, all three shims
  {
    struct MatMul : public Node {
      void forward_dev_impl(const Device_GPU& dev, const std::vector<const Tensor*>& xs, Tensor& fx) const override {
        MatrixMultiply(dev, *xs[0], *xs[1], fx, dev.kSCALAR_ZERO);
      }
      void backward_dev_impl(const Device_GPU& dev, const std::vector<const Tensor*>& xs, const Tensor&, const Tensor& dEdf,
                             unsigned i, Tensor& dEdxi) const override {
        if (i == 0) MatrixMultiplyTranspAcc(dev, dEdf, *xs[1], dEdxi);
        else MatrixTranspMultiplyAcc(dev, *xs[0], dEdf, dEdxi);
      }
    };
    const vector<float> lv = {1.1f, -2.2f, 3.3f, 0.4f, 0.5f, -0.6f, 0.7f, 0.8f, -0.9f, 1.0f, 1.2f, -1.3f};
    const vector<float> rv = {0.3f, -0.2f, 0.5f, 0.7f, -1.1f, 0.9f, 0.2f, 0.4f};
    { vector<Tensor> a = {F.input(Dim({3, 2}, 2), lv), F.input(Dim({2, 2}, 2), rv)};
      CHECK(check_grad(F, MatMul(), a, Dim({3, 2}, 2), {true, true})); }
    { vector<Tensor> a = {F.input(Dim({3, 2}, 2), lv), F.input(Dim({2, 2}), {0.3f, -0.2f, 0.5f, 0.7f})};
      CHECK(check_grad(F, MatMul(), a, Dim({3, 2}, 2), {true, false})); }
    F.reset();
  }
  g_case = "addscalar_gradient";
  { vector<Tensor> a = {F.input(Dim({3}), param1)}; CHECK(check_grad(F, ConstantPlusX(2.0f), a, Dim({3}), {true})); }
  g_case = "scalarsubtract_gradient";
  { vector<Tensor> a = {F.input(Dim({3}), param1)}; CHECK(check_grad(F, ConstantMinusX(2.0f), a, Dim({3}), {true})); }
  g_case = "mean_std_elems_gradient";
  {
    vector<Tensor> a = {F.input(Dim({3}, 2), param4)};
    CHECK(check_grad(F, MeanElements(), a, Dim({1}, 2), {true}));
    CHECK(check_grad(F, StdElements(), a, Dim({1}, 2), {true}));
  }
}

// ---- layer_norm as the reference composes it from eight nodes (dynet/expr.cc:248-253) against the fused node ----
static void layer_norm_composite(Fixture& F) {
  g_case = "layer_norm_composite";
  const unsigned n = 64, bd = 5;
  vector<float> xv(n * bd), gv(n), bv(n), wv(n * bd);
  for (size_t k = 0; k < xv.size(); ++k) xv[k] = std::sin(0.37f * float(k)) * 2.f + 0.01f * float(k % 11);
  for (size_t k = 0; k < n; ++k) { gv[k] = 0.5f + 0.01f * float(k); bv[k] = 0.1f * std::cos(float(k)); }
  for (size_t k = 0; k < wv.size(); ++k) wv[k] = 0.3f + 0.1f * float(k % 7) - 0.05f * float(k % 3);
  const Dim dx({n}, bd), dp({n}), ds({1}, bd);
  Tensor x = F.input(dx, xv), g = F.input(dp, gv), b = F.input(dp, bv), dEdf = F.input(dx, wv, DeviceMempool::DEDFS);
  auto fx = [&](const Dim& d) { return F.dev.allocate_tensor(DeviceMempool::FXS, d); };
  Tensor mu = fx(ds), nmu = fx(ds), xc = fx(dx), sigma = fx(ds), se = fx(ds), q = fx(dx), gq = fx(dx), y = fx(dx), fused = fx(dx);
  const MeanElements mean_n; const Negate neg_n; const CwiseSum sum_n; const StdElements std_n;
  const ConstantPlusX eps_n(1e-8f); const CwiseQuotient div_n; const CwiseMultiply mul_n;
  mean_n.forward_dev_impl(F.dev, {&x}, mu);
  neg_n.forward_dev_impl(F.dev, {&mu}, nmu);
  sum_n.forward_dev_impl(F.dev, {&x, &nmu}, xc);
  std_n.forward_dev_impl(F.dev, {&x}, sigma);
  eps_n.forward_dev_impl(F.dev, {&sigma}, se);
  div_n.forward_dev_impl(F.dev, {&xc, &se}, q);
  mul_n.forward_dev_impl(F.dev, {&g, &q}, gq);
  sum_n.forward_dev_impl(F.dev, {&gq, &b}, y);
  LayerNorm().forward_dev_impl(F.dev, {&x, &g, &b}, fused);
  const vector<float> yc = as_vector(y), yf = as_vector(fused);
  for (size_t k = 0; k < yc.size(); ++k) CHECK_SMALL(yc[k] - yf[k], 2e-6 * (1.0 + std::fabs(yf[k])));
  // backward through the eight nodes in reverse order
  Tensor d_gq = F.zeros(dx), d_b = F.zeros(dp), d_g = F.zeros(dp), d_q = F.zeros(dx), d_xc = F.zeros(dx), d_se = F.zeros(ds),
         d_sigma = F.zeros(ds), d_x = F.zeros(dx), d_nmu = F.zeros(ds), d_mu = F.zeros(ds);
  sum_n.backward_dev_impl(F.dev, {&gq, &b}, y, dEdf, 0, d_gq);
  sum_n.backward_dev_impl(F.dev, {&gq, &b}, y, dEdf, 1, d_b);
  mul_n.backward_dev_impl(F.dev, {&g, &q}, gq, d_gq, 0, d_g);
  mul_n.backward_dev_impl(F.dev, {&g, &q}, gq, d_gq, 1, d_q);
  div_n.backward_dev_impl(F.dev, {&xc, &se}, q, d_q, 0, d_xc);
  div_n.backward_dev_impl(F.dev, {&xc, &se}, q, d_q, 1, d_se);
  eps_n.backward_dev_impl(F.dev, {&sigma}, se, d_se, 0, d_sigma);
  std_n.backward_dev_impl(F.dev, {&x}, sigma, d_sigma, 0, d_x);
  sum_n.backward_dev_impl(F.dev, {&x, &nmu}, xc, d_xc, 0, d_x);
  sum_n.backward_dev_impl(F.dev, {&x, &nmu}, xc, d_xc, 1, d_nmu);
  neg_n.backward_dev_impl(F.dev, {&mu}, nmu, d_nmu, 0, d_mu);
  mean_n.backward_dev_impl(F.dev, {&x}, mu, d_mu, 0, d_x);
  Tensor f_x = F.zeros(dx), f_g = F.zeros(dp), f_b = F.zeros(dp);
  const LayerNorm ln;
  ln.forward_dev_impl(F.dev, {&x, &g, &b}, fused);
  ln.backward_dev_impl(F.dev, {&x, &g, &b}, fused, dEdf, 0, f_x);
  ln.backward_dev_impl(F.dev, {&x, &g, &b}, fused, dEdf, 1, f_g);
  ln.backward_dev_impl(F.dev, {&x, &g, &b}, fused, dEdf, 2, f_b);
  const vector<float> cx = as_vector(d_x), cg = as_vector(d_g), cb = as_vector(d_b), rx = as_vector(f_x), rg = as_vector(f_g),
                      rb = as_vector(f_b);
  for (size_t k = 0; k < cx.size(); ++k) CHECK_SMALL(cx[k] - rx[k], 1e-5 * (1.0 + std::fabs(rx[k])));
  for (size_t k = 0; k < n; ++k) {
    CHECK_SMALL(cg[k] - rg[k], 1e-5 * (1.0 + std::fabs(rg[k])));
    CHECK_SMALL(cb[k] - rb[k], 1e-5 * (1.0 + std::fabs(rb[k])));
  }
}

// ---- BatchedExecutionEngine::combine_tensors / accumulate_tensors (dynet/exec.cc:298-409) ----
static void combine_and_accumulate(Fixture& F) {
  g_case = "combine_tensors";
  // 128 nodes of 1024 floats, then a ragged tail (sizes 1, 7, 1000, 3)
  vector<unsigned> sizes(128, 1024);
  for (unsigned s : {1u, 7u, 1000u, 3u}) sizes.push_back(s);
  vector<Tensor> parts;
  vector<vector<float>> host;
  vector<float> expect;
  unsigned seed = 1;
  for (unsigned sz : sizes) {
    vector<float> v(sz);
    for (float& e : v) { seed = seed * 1664525u + 1013904223u; e = float(seed >> 8) * (1.f / 16777216.f) - 0.5f; }
    expect.insert(expect.end(), v.begin(), v.end());
    parts.push_back(F.input(Dim({sz}), v));
    host.push_back(v);
  }
  vector<const Tensor*> ptrs;
  for (const Tensor& t : parts) ptrs.push_back(&t);
  for (int rep = 0; rep < 3; ++rep) {  // repeated calls walk the staging ring
    Tensor tout;
    combine_tensors(F.dev, ptrs, tout);
    CHECK(tout.d.size() == expect.size());
    CHECK(as_vector(tout) == expect);
  }
  g_case = "accumulate_tensors";
  vector<Tensor> grads;
  for (size_t k = 0; k < sizes.size(); ++k) {
    vector<float> init(sizes[k]);
    for (size_t e = 0; e < init.size(); ++e) init[e] = 0.25f * float((k + e) % 5);
    grads.push_back(F.input(Dim({sizes[k]}), init, DeviceMempool::DEDFS));
  }
  Tensor tin = F.input(Dim({static_cast<unsigned>(expect.size())}), expect, DeviceMempool::DEDFS);
  vector<Tensor*> gp;
  for (Tensor& t : grads) gp.push_back(&t);
  accumulate_tensors(F.dev, tin, gp);
  accumulate_tensors(F.dev, tin, gp);
  for (size_t k = 0; k < sizes.size(); ++k) {
    const vector<float> got = as_vector(grads[k]);
    bool same = true;
    for (size_t e = 0; e < got.size(); ++e) same = same && got[e] == (0.25f * float((k + e) % 5) + host[k][e]) + host[k][e];
    CHECK(same);
  }
  bool threw = false;
  gp.pop_back();
  try { accumulate_tensors(F.dev, tin, gp); } catch (const std::invalid_argument&) { threw = true; }
  CHECK(threw);
  g_case = "staging_ring_wraps";  // more staged bytes than the ring holds: the wrap must not corrupt earlier tables
  {
    vector<const Tensor*> two = {&parts[0], &parts[1]};
    vector<float> want(host[0]);
    want.insert(want.end(), host[1].begin(), host[1].end());
    bool ok = true;
    for (int rep = 0; rep < 6000; ++rep) {  // 6000 x 64 bytes > 256 KiB
      const size_t used = F.dev.pools[0]->used();
      Tensor tout;
      combine_tensors(F.dev, two, tout);
      if (rep % 1500 == 0) ok = ok && as_vector(tout) == want;
      F.dev.pools[0]->set_used(used);
    }
    CHECK(ok);
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
                                                             lookup_and_softmax,   random_nodes,    cwise_broadcast,       layer_norm_composite,
                                                             combine_and_accumulate, argmax_node, deferred_parameter_gradients,
                                                             sum_logsumexp_pick_range};
  for (const auto& c : cases) {
    c(F);
    F.reset();
  }
  std::printf("%d checks, %d failed\n", g_checks, g_failed);
  return g_failed > 255 ? 255 : g_failed;
}
