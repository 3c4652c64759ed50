// C++ host side above the C-ABI: the operator interface DyNet's nodes expose on their GPU
// path, with the same names, argument meaning and error behaviour, forwarding to
// libdynet_hip.so.  In a DyNet build these bodies become the Device_GPU instantiations
// of forward_dev_impl / backward_dev_impl (dynet/nodes-def-macros.h:44-62,
// dynet/nodes-impl-macros.h:13-61); here they stand on a minimal Dim / Tensor / Device_GPU
// of their own, because DyNet's headers pull in Eigen, so that the library can be driven
// and tested from C++ the way the reference's tests drive its nodes.
//
//   xs      arguments in the node's own order (dynet/nodes-lstm.cc:101-112 etc.)
//   fx      forward overwrites it
//   dEdxi   backward accumulates into it (dynet/exec.cc:207-208 zeroes it once)
//   errors  std::invalid_argument for bad arguments (DYNET_ARG_CHECK, dynet/except.h:41-46),
//           dynet_hip::cuda_exception for runtime failures (dynet/cuda.h:20-52),
//           dynet_hip::out_of_memory (dynet/except.h:11-14)
#pragma once

#include <cstddef>
#include <initializer_list>
#include <map>
#include <stdexcept>
#include <string>
#include <vector>

#include "dynet_hip.h"

namespace dynet_hip {

typedef float real;  // dynet/tensor.h:36

struct cuda_exception : public std::runtime_error {
  explicit cuda_exception(const std::string& what) : std::runtime_error(what) {}
};
struct out_of_memory : public std::runtime_error {
  explicit out_of_memory(const std::string& what) : std::runtime_error(what) {}
};

inline void abi_check(int status) {
  if (status == DYHIP_OK) return;
  const std::string msg = dyhip_last_error();
  if (status == DYHIP_ERR_INVALID_ARG) throw std::invalid_argument(msg);
  if (status == DYHIP_ERR_OUT_OF_MEMORY) throw out_of_memory(msg);
  throw cuda_exception(msg);
}

// dynet/dim.h:34-304, the part the nodes use
struct Dim {
  unsigned d[7];
  unsigned nd;
  unsigned bd;
  Dim() : nd(0), bd(1) {}
  Dim(std::initializer_list<unsigned> x, unsigned b = 1) : nd(0), bd(b) {
    for (unsigned v : x) d[nd++] = v;
  }
  unsigned batch_size() const {
    unsigned p = 1;
    for (unsigned i = 0; i < nd; ++i) p *= d[i];
    return p;
  }
  unsigned size() const { return batch_size() * bd; }
  unsigned rows() const { return nd ? d[0] : 1; }
  unsigned cols() const { return nd > 1 ? d[1] : 1; }
  unsigned batch_elems() const { return bd; }
  unsigned operator[](unsigned i) const { return i < nd ? d[i] : 1; }
};

enum class DeviceMempool { FXS = 0, DEDFS = 1, PS = 2, SCS = 3, NONE = 4 };  // dynet/device-structs.h:15

// dynet/aligned-mem-pool.h:47-69 over the library's pool
class AlignedMemoryPool {
 public:
  explicit AlignedMemoryPool(dyhip_pool* p) : p_(p) {}
  void* allocate(size_t n) {
    void* out = nullptr;
    abi_check(dyhip_pool_allocate(p_, n, &out));
    return out;
  }
  void free() { abi_check(dyhip_pool_free(p_)); }
  void zero_allocated_memory() { abi_check(dyhip_pool_zero_allocated(p_)); }
  size_t used() {
    size_t u = 0;
    abi_check(dyhip_pool_used(p_, &u));
    return u;
  }
  void set_used(size_t s) { abi_check(dyhip_pool_set_used(p_, s)); }

 private:
  dyhip_pool* p_;
};

struct Device_GPU;

// dynet/tensor.h:46-120, the fields the nodes touch
struct Tensor {
  Dim d;
  float* v;
  Device_GPU* device;
  DeviceMempool mem_pool;
  Tensor() : v(nullptr), device(nullptr), mem_pool(DeviceMempool::NONE) {}
  Tensor(const Dim& d, float* v, Device_GPU* dev, DeviceMempool mp) : d(d), v(v), device(dev), mem_pool(mp) {}
};

// dynet/devices.h:46-61, dynet/devices.cc:91-121
// Page-locked staging ring for the small host tables a call hands to the GPU (pointer / length tables of the
// batched executor, dynet/exec.cc:319-355).  A copy from it is asynchronous, so a slice may only be reused once
// the copies issued from it have run: the ring synchronises the device when it wraps, which with 24-byte entries
// is once per ~10^4 staged tensors, and never otherwise.
class PinnedStaging {
 public:
  explicit PinnedStaging(dyhip_device* dev, size_t bytes = size_t(256) << 10) : dev_(dev), cap_(0), cur_(0), base_(nullptr) {
    grow(bytes);
  }
  ~PinnedStaging() {
    if (base_) {
      dyhip_device_sync(dev_);
      dyhip_host_free(base_);
    }
  }
  PinnedStaging(const PinnedStaging&) = delete;
  PinnedStaging& operator=(const PinnedStaging&) = delete;
  void* take(size_t bytes) {
    bytes = (bytes + 63) & ~size_t(63);
    if (bytes > cap_) grow(2 * bytes);
    if (cur_ + bytes > cap_) {
      abi_check(dyhip_device_sync(dev_));
      cur_ = 0;
    }
    void* out = static_cast<char*>(base_) + cur_;
    cur_ += bytes;
    return out;
  }

 private:
  void grow(size_t bytes) {
    if (base_) {
      abi_check(dyhip_device_sync(dev_));
      abi_check(dyhip_host_free(base_));
      base_ = nullptr;
    }
    abi_check(dyhip_host_alloc(bytes, &base_));
    cap_ = bytes;
    cur_ = 0;
  }
  dyhip_device* dev_;
  size_t cap_, cur_;
  void* base_;
};

// Products that nodes add into the gradient of an arity-0 node (a parameter or a lookup), recorded instead of
// formed.  The executor visits a node's arguments one at a time (dynet/exec.cc:247-262), so the T gates nodes of an
// unrolled LSTM add T products of depth B (the batch) into the same dEdf of the ParameterNode of Wx: T launches that
// each read and rewrite the whole gradient for a product too shallow to fill the matrix cores.  Nobody reads such a
// gradient before the executor hands it to the parameter (ParameterNode::accumulate_grad, dynet/exec.cc:274-280),
// and the operands (node outputs in pools[FXS], the cached activation derivative in the node's aux_mem) stay alive
// until the graph is freed.  So a node may record (operands, shape) here, and the recorded products of one gradient
// are formed as ONE product over the gathered operands when the gradient is first read: by accumulate_grad, by
// as_vector / TensorTools of this adapter, or by flush_all.
//
// The executor's part (three lines in ExecutionEngine::backward): after ndEdfs is allocated, call clear() and then
// allow(ndEdfs[i].v) for every i in cg.parameter_nodes; gradients of other nodes are never deferred, because the
// executor reads them (as dEdf of that node's own backward) right after its consumers have run.
class DeferredGrads {
 public:
  explicit DeferredGrads(dyhip_device* dev, std::vector<AlignedMemoryPool*>* pools) : dev_(dev), pools_(pools) {}
  void clear() {
    allowed_.clear();
    pending_.clear();
  }
  void allow(const float* dst) { allowed_[dst] = true; }
  bool allowed(const float* dst) const { return allowed_.count(dst) != 0; }
  bool pending(const float* dst) const {
    auto it = pending_.find(dst);
    return it != pending_.end() && !it->second.empty();
  }
  // dst[M x N] += l[M x K] * r[N x K]^T (MatrixMultiplyTranspAcc); with r == nullptr: dst[M] += sum of l's K columns
  void record(float* dst, unsigned M, unsigned N, unsigned K, const float* l, const float* r) {
    pending_[dst].push_back(Product{M, N, K, l, r});
  }
  void flush(const float* dst) {
    auto it = pending_.find(dst);
    if (it == pending_.end() || it->second.empty()) return;
    std::vector<Product> list;
    list.swap(it->second);
    float* out = const_cast<float*>(dst);
    bool same = true;
    for (const Product& p : list) same = same && p.M == list[0].M && p.N == list[0].N && p.K == list[0].K && (p.r == nullptr) == (list[0].r == nullptr);
    AlignedMemoryPool* scs = (*pools_)[static_cast<int>(DeviceMempool::SCS)];
    if (!same || list.size() == 1) {  // nothing to merge: form them one by one
      for (const Product& p : list) form(out, p.M, p.N, p.K, p.l, p.r, scs);
      scs->free();
      return;
    }
    const unsigned n = static_cast<unsigned>(list.size()), M = list[0].M, N = list[0].N, K = list[0].K;
    std::vector<const float*> ls, rs;
    for (const Product& p : list) {
      ls.push_back(p.l);
      rs.push_back(p.r);
    }
    float* gl = static_cast<float*>(scs->allocate(sizeof(float) * size_t(M) * K * n));
    abi_check(dyhip_gather_segments(dev_, n, size_t(M) * K, ls.data(), gl));
    float* gr = nullptr;
    if (list[0].r != nullptr) {
      gr = static_cast<float*>(scs->allocate(sizeof(float) * size_t(N) * K * n));
      abi_check(dyhip_gather_segments(dev_, n, size_t(N) * K, rs.data(), gr));
    }
    form(out, M, N, K * n, gl, gr, scs);
    scs->free();
  }
  void flush_all() {
    std::vector<const float*> keys;
    for (auto& kv : pending_) keys.push_back(kv.first);
    for (const float* k : keys) flush(k);
  }

 private:
  struct Product {
    unsigned M, N, K;
    const float *l, *r;
  };
  void form(float* out, unsigned M, unsigned N, unsigned K, const float* l, const float* r, AlignedMemoryPool* scs) {
    if (r != nullptr) {
      abi_check(dyhip_gemm_nt_acc(dev_, M, N, K, l, r, out));
    } else {
      size_t need = 0;
      abi_check(dyhip_batch_reduce_workspace(M, K, &need));
      void* ws = need ? scs->allocate(need) : nullptr;
      abi_check(dyhip_csum_backward(dev_, M, 1, K, l, 0, out, ws, need));
    }
  }
  dyhip_device* dev_;
  std::vector<AlignedMemoryPool*>* pools_;
  std::map<const float*, bool> allowed_;
  std::map<const float*, std::vector<Product>> pending_;
};

struct Device_GPU {
  dyhip_device* hip;
  float *kSCALAR_MINUSONE, *kSCALAR_ONE, *kSCALAR_ZERO;
  std::vector<AlignedMemoryPool*> pools;
  PinnedStaging* staging;
  DeferredGrads* deferred;

  Device_GPU(int device_id, size_t fxs_mb, size_t dedfs_mb, size_t ps_mb, size_t scs_mb)
      : hip(nullptr), staging(nullptr), deferred(nullptr) {
    const size_t mb[4] = {fxs_mb, dedfs_mb, ps_mb, scs_mb};
    abi_check(dyhip_device_create(device_id, mb, &hip));
    const float* s[3];
    for (int k = 0; k < 3; ++k) abi_check(dyhip_device_scalar(hip, k, &s[k]));
    kSCALAR_MINUSONE = const_cast<float*>(s[DYHIP_SCALAR_MINUSONE]);
    kSCALAR_ONE = const_cast<float*>(s[DYHIP_SCALAR_ONE]);
    kSCALAR_ZERO = const_cast<float*>(s[DYHIP_SCALAR_ZERO]);
    for (int k = 0; k < 4; ++k) {
      dyhip_pool* p = nullptr;
      abi_check(dyhip_device_pool(hip, k, &p));
      pools.push_back(new AlignedMemoryPool(p));
    }
    staging = new PinnedStaging(hip);
    deferred = new DeferredGrads(hip, &pools);
  }
  ~Device_GPU() {
    delete deferred;
    delete staging;
    for (AlignedMemoryPool* p : pools) delete p;
    if (hip) dyhip_device_destroy(hip);
  }
  Device_GPU(const Device_GPU&) = delete;
  Device_GPU& operator=(const Device_GPU&) = delete;

  // Device_GPU::reset_rng (dynet/devices.cc:130-135)
  void reset_rng(unsigned seed) { abi_check(dyhip_reset_rng(hip, seed)); }

  // Device::allocate_tensor (dynet/devices.cc:82-88)
  Tensor allocate_tensor(DeviceMempool mp, const Dim& d) {
    float* v = static_cast<float*>(pools[static_cast<int>(mp)]->allocate(sizeof(float) * d.size()));
    return Tensor(d, v, this, mp);
  }
};

// dynet/tensor.h TensorTools, the calls the tests use (dynet/tensor.cc:66-229)
struct TensorTools {
  static void set_elements(Tensor& t, const std::vector<float>& vals) {
    if (vals.size() != t.d.size()) throw std::invalid_argument("set_elements: size mismatch");
    abi_check(dyhip_memcpy_h2d(t.device->hip, t.v, vals.data(), sizeof(float) * vals.size()));
    abi_check(dyhip_device_sync(t.device->hip));
  }
  static void zero(Tensor& t) { abi_check(dyhip_zero(t.device->hip, t.v, sizeof(float) * t.d.size())); }
  static void constant(Tensor& t, float c) { abi_check(dyhip_constant(t.device->hip, t.d.size(), c, t.v)); }
  static void accumulate(Tensor& t, const Tensor& src) {
    src.device->deferred->flush(src.v);
    abi_check(dyhip_accumulate(t.device->hip, t.d.size(), src.v, t.v));
  }
  // dynet/tensor.cc:261-303 (GPU branches)
  static void randomize_bernoulli(Tensor& t, real p, real scale = 1.f) {
    abi_check(dyhip_randomize_bernoulli(t.device->hip, t.d.size(), p, scale, t.v));
  }
  static void randomize_normal(Tensor& t, real mean = 0.f, real stddev = 1.f) {
    abi_check(dyhip_randomize_normal(t.device->hip, t.d.size(), mean, stddev, t.v));
  }
  static void randomize_uniform(Tensor& t, real left = 0.f, real right = 1.f) {
    abi_check(dyhip_randomize_uniform(t.device->hip, t.d.size(), left, right, t.v));
  }
};
inline std::vector<real> as_vector(const Tensor& t) {  // blocking copy, dynet/tensor.cc:66-93
  t.device->deferred->flush(t.v);  // a gradient with recorded products is complete before anyone sees it
  std::vector<real> out(t.d.size());
  abi_check(dyhip_memcpy_d2h(t.device->hip, out.data(), t.v, sizeof(float) * out.size()));
  return out;
}

// ---- nodes ---------------------------------------------------------------------------------
struct Node {
  virtual ~Node() {}
  mutable void* aux_mem = nullptr;  // assigned by the executor before forward (dynet/exec.cc:138-147)
  virtual size_t aux_storage_size() const { return 0; }
  virtual void forward_dev_impl(const Device_GPU& dev, const std::vector<const Tensor*>& xs, Tensor& fx) const = 0;
  virtual void backward_dev_impl(const Device_GPU& dev, const std::vector<const Tensor*>& xs, const Tensor& fx,
                                 const Tensor& dEdf, unsigned i, Tensor& dEdxi) const = 0;

 protected:
  static AlignedMemoryPool* scratch(const Tensor& fx) { return fx.device->pools[static_cast<int>(DeviceMempool::SCS)]; }
};

// dynet/nodes-lstm.h:9-26, nodes-lstm.cc:101-527.  xs = {x_t[0..k), h_tm1, Wx, Wh, b [, mask_x, mask_h]}
//
// The executor calls backward once per differentiable argument with the same dEdf; the activation
// derivative dpre = dEdf * act'(fx) (dynet/nodes-lstm.cc:358-361) is the same for all of them.  When the
// node was given aux_mem (aux_storage_size() = one fx-sized tensor, requested by passing the output
// dimension to the constructor), the first backward call of a backward pass stores dpre there and the
// others reuse it.  A pass is recognised by the executor's own order: it visits the arguments of a node
// in ascending order (dynet/exec.cc:247-262), so a call whose argument index does not exceed the last
// one served starts a new pass -- the executor frees and refills pools[DEDFS] at the start of every
// backward (dynet/exec.cc:178), so a second backward on the same forward can present the same dEdf
// address with other contents.  forward invalidates the cache too.  Without aux_mem every call
// recomputes dpre.
struct VanillaLSTMGates : public Node {
  VanillaLSTMGates(bool dropout, real weightnoise_std, const Dim& dim = Dim())
      : dropout(dropout), weightnoise_std(weightnoise_std), dim(dim) {}
  bool dropout;
  real weightnoise_std;
  Dim dim;  // the node's output dimension ({4H}, B) when the dpre cache is wanted
  size_t aux_storage_size() const override { return dim.nd ? dim.size() * sizeof(float) : 0; }

  void forward_dev_impl(const Device_GPU& dev, const std::vector<const Tensor*>& xs, Tensor& fx) const override {
    dpre_of_ = nullptr;
    last_i_ = -1;
    Args a = unpack(xs);
    size_t need = 0;
    abi_check(dyhip_lstm_gates_workspace(a.k, a.I, a.H, a.B, dropout, &need));
    void* ws = need ? scratch(fx)->allocate(need) : nullptr;
    abi_check(dyhip_lstm_gates_forward(dev.hip, a.k, a.x.data(), a.xd.data(), a.H, a.B, xs[a.k]->v, xs[a.k + 1]->v,
                                       xs[a.k + 2]->v, xs[a.k + 3]->v, a.mx, a.mx_bd, a.mh, a.mh_bd,
                                       DYHIP_LOGISTIC_PACKET, fx.v, ws, need));
    scratch(fx)->free();
  }
  void backward_dev_impl(const Device_GPU& dev, const std::vector<const Tensor*>& xs, const Tensor& fx,
                         const Tensor& dEdf, unsigned i, Tensor& dEdxi) const override {
    Args a = unpack(xs);
    if (i > a.k + 3) return;  // the dropout masks get no gradient (dynet/nodes-lstm.cc:522)
    size_t need = 0;
    abi_check(dyhip_lstm_gates_backward_workspace(a.k, a.I, a.H, a.B, dropout, &need));
    void* ws = scratch(fx)->allocate(need);
    const float* dpre = nullptr;
    if (aux_mem != nullptr && dim.nd && dim.size() == fx.d.size()) {
      if (dpre_of_ != dEdf.v || int(i) <= last_i_) {
        abi_check(dyhip_lstm_gates_dpre(dev.hip, a.H, a.B, fx.v, dEdf.v, static_cast<float*>(aux_mem)));
        dpre_of_ = dEdf.v;
      }
      last_i_ = int(i);
      dpre = static_cast<const float*>(aux_mem);
    }
    // Wx (one input, no dropout), Wh and b of a node whose activation derivative is cached: when the destination is
    // the gradient of an arity-0 node, the product is recorded and formed together with those of the other timesteps
    // (dynet/nodes-lstm.cc:472-500: dWx += dpre x^T, dWh += dpre h_tm1^T, db += sum of dpre's columns)
    if (dpre != nullptr && !dropout && a.k == 1 && i >= a.k + 1 && dev.deferred->allowed(dEdxi.v)) {
      const float* r = i == a.k + 1 ? xs[0]->v : i == a.k + 2 ? xs[a.k]->v : nullptr;
      const unsigned N = i == a.k + 1 ? a.I : i == a.k + 2 ? a.H : 1;
      dev.deferred->record(dEdxi.v, 4 * a.H, N, a.B, dpre, r);
      scratch(fx)->free();
      return;
    }
    abi_check(dyhip_lstm_gates_backward(dev.hip, a.k, a.x.data(), a.xd.data(), a.H, a.B, xs[a.k]->v, xs[a.k + 1]->v,
                                        xs[a.k + 2]->v, a.mx, a.mx_bd, a.mh, a.mh_bd, fx.v, dEdf.v, dpre, i,
                                        dEdxi.v, ws, need));
    scratch(fx)->free();
  }

 private:
  mutable const float* dpre_of_ = nullptr;  // the dEdf whose dpre sits in aux_mem
  mutable int last_i_ = -1;                 // the argument served by the latest backward call
  struct Args {
    unsigned k, I, H, B, mx_bd, mh_bd;
    std::vector<const float*> x;
    std::vector<unsigned> xd;
    const float *mx, *mh;
  };
  Args unpack(const std::vector<const Tensor*>& xs) const {
    if (weightnoise_std != 0.f) throw std::invalid_argument("VanillaLSTMGates: weight noise is not supported");
    if (xs.size() < (dropout ? 7u : 5u)) throw std::invalid_argument("Failed input count check in VanillaLSTMGates");
    Args a;
    a.k = static_cast<unsigned>(dropout ? xs.size() - 6 : xs.size() - 4);
    a.H = xs[a.k]->d[0];
    a.B = xs[0]->d.bd;
    a.I = 0;
    for (unsigned j = 0; j < a.k; ++j) {
      a.x.push_back(xs[j]->v);
      a.xd.push_back(xs[j]->d[0]);
      a.I += xs[j]->d[0];
    }
    a.mx = dropout ? xs[a.k + 4]->v : nullptr;
    a.mh = dropout ? xs[a.k + 5]->v : nullptr;
    a.mx_bd = dropout ? xs[a.k + 4]->d.bd : 0;
    a.mh_bd = dropout ? xs[a.k + 5]->d.bd : 0;
    return a;
  }
};

// dynet/nodes-lstm.cc:562-615.  xs = {c_tm1, gates_t}
struct VanillaLSTMC : public Node {
  void forward_dev_impl(const Device_GPU& dev, const std::vector<const Tensor*>& xs, Tensor& fx) const override {
    abi_check(dyhip_lstm_c_forward(dev.hip, xs[0]->d[0], xs[0]->d.bd, xs[0]->v, xs[1]->v, fx.v));
  }
  void backward_dev_impl(const Device_GPU& dev, const std::vector<const Tensor*>& xs, const Tensor&,
                         const Tensor& dEdf, unsigned i, Tensor& dEdxi) const override {
    abi_check(dyhip_lstm_c_backward(dev.hip, xs[0]->d[0], xs[0]->d.bd, xs[0]->v, xs[1]->v, dEdf.v, i, dEdxi.v));
  }
};

// dynet/nodes-lstm.cc:650-703.  xs = {c_t, gates_t}
struct VanillaLSTMH : public Node {
  void forward_dev_impl(const Device_GPU& dev, const std::vector<const Tensor*>& xs, Tensor& fx) const override {
    abi_check(dyhip_lstm_h_forward(dev.hip, xs[0]->d[0], xs[0]->d.bd, xs[0]->v, xs[1]->v, fx.v));
  }
  void backward_dev_impl(const Device_GPU& dev, const std::vector<const Tensor*>& xs, const Tensor&,
                         const Tensor& dEdf, unsigned i, Tensor& dEdxi) const override {
    abi_check(dyhip_lstm_h_backward(dev.hip, xs[0]->d[0], xs[0]->d.bd, xs[0]->v, xs[1]->v, dEdf.v, i, dEdxi.v));
  }
};

// Tanh (dynet/nodes-trig.cc:312-326), LogisticSigmoid (dynet/nodes-activations.cc:65-78), Rectify (:31-44)
template <int OP>
struct UnaryNode : public Node {
  void forward_dev_impl(const Device_GPU& dev, const std::vector<const Tensor*>& xs, Tensor& fx) const override {
    abi_check(dyhip_unary_forward(dev.hip, OP, DYHIP_LOGISTIC_PACKET, fx.d.size(), xs[0]->v, fx.v));
  }
  void backward_dev_impl(const Device_GPU& dev, const std::vector<const Tensor*>&, const Tensor& fx,
                         const Tensor& dEdf, unsigned, Tensor& dEdxi) const override {
    abi_check(dyhip_unary_backward(dev.hip, OP, fx.d.size(), fx.v, dEdf.v, dEdxi.v));
  }
};
typedef UnaryNode<DYHIP_OP_TANH> Tanh;
typedef UnaryNode<DYHIP_OP_LOGISTIC> LogisticSigmoid;
typedef UnaryNode<DYHIP_OP_RECTIFY> Rectify;
typedef UnaryNode<DYHIP_OP_NEGATE> Negate;

// CwiseSum / CwiseMultiply / CwiseQuotient (dynet/nodes-arith-cwise.cc:51-126, 197-306, 339-419): every
// dimension and the batch of either argument may be 1 against the other's size (the reference's
// get_broadcasting_bits rule); backward sums over the dimensions argument i was broadcast over.
inline void dims5(const Dim& d, unsigned out[5]) {
  if (d.nd > 4) throw std::invalid_argument("component-wise nodes take tensors of at most 4 dimensions");
  for (unsigned k = 0; k < 4; ++k) out[k] = d[k];
  out[4] = d.bd;
}
template <int OP>
struct CwiseNode : public Node {
  void forward_dev_impl(const Device_GPU& dev, const std::vector<const Tensor*>& xs, Tensor& fx) const override {
    unsigned da[5], db[5];
    dims5(xs[0]->d, da);
    dims5(xs[1]->d, db);
    abi_check(dyhip_cwise_forward(dev.hip, OP, da, db, xs[0]->v, xs[1]->v, fx.v));
  }
  void backward_dev_impl(const Device_GPU& dev, const std::vector<const Tensor*>& xs, const Tensor& fx,
                         const Tensor& dEdf, unsigned i, Tensor& dEdxi) const override {
    unsigned da[5], db[5];
    dims5(xs[0]->d, da);
    dims5(xs[1]->d, db);
    size_t need = 0;
    abi_check(dyhip_cwise_backward_workspace(da, db, i, &need));
    void* ws = need ? scratch(fx)->allocate(need) : nullptr;
    abi_check(dyhip_cwise_backward(dev.hip, OP, da, db, xs[0]->v, xs[1]->v, dEdf.v, i, dEdxi.v, ws, need));
    scratch(fx)->free();
  }
};
typedef CwiseNode<DYHIP_CWISE_SUM> CwiseSum;
typedef CwiseNode<DYHIP_CWISE_MULT> CwiseMultiply;
typedef CwiseNode<DYHIP_CWISE_QUOTIENT> CwiseQuotient;

// ConstantPlusX / ConstantMinusX (dynet/nodes-arith-const.cc:30-44, 63-77)
struct ConstantPlusX : public Node {
  explicit ConstantPlusX(real c) : c(c) {}
  real c;
  void forward_dev_impl(const Device_GPU& dev, const std::vector<const Tensor*>& xs, Tensor& fx) const override {
    abi_check(dyhip_const_plus_x_forward(dev.hip, fx.d.size(), c, xs[0]->v, fx.v));
  }
  void backward_dev_impl(const Device_GPU& dev, const std::vector<const Tensor*>&, const Tensor&, const Tensor& dEdf,
                         unsigned, Tensor& dEdxi) const override {
    abi_check(dyhip_accumulate(dev.hip, dEdf.d.size(), dEdf.v, dEdxi.v));
  }
};
struct ConstantMinusX : public Node {
  explicit ConstantMinusX(real c) : c(c) {}
  real c;
  void forward_dev_impl(const Device_GPU& dev, const std::vector<const Tensor*>& xs, Tensor& fx) const override {
    abi_check(dyhip_const_minus_x_forward(dev.hip, fx.d.size(), c, xs[0]->v, fx.v));
  }
  void backward_dev_impl(const Device_GPU& dev, const std::vector<const Tensor*>&, const Tensor& fx, const Tensor& dEdf,
                         unsigned, Tensor& dEdxi) const override {
    abi_check(dyhip_unary_backward(dev.hip, DYHIP_OP_NEGATE, fx.d.size(), fx.v, dEdf.v, dEdxi.v));
  }
};

// mean_elems / std_elems: MomentElements with order 1 and StdElements (dynet/nodes-moments.cc:121-148, 380-400)
struct MeanElements : public Node {
  void forward_dev_impl(const Device_GPU& dev, const std::vector<const Tensor*>& xs, Tensor& fx) const override {
    abi_check(dyhip_mean_elems_forward(dev.hip, xs[0]->d.batch_size(), xs[0]->d.bd, xs[0]->v, fx.v));
  }
  void backward_dev_impl(const Device_GPU& dev, const std::vector<const Tensor*>& xs, const Tensor&, const Tensor& dEdf,
                         unsigned, Tensor& dEdxi) const override {
    abi_check(dyhip_mean_elems_backward(dev.hip, xs[0]->d.batch_size(), xs[0]->d.bd, dEdf.v, dEdxi.v));
  }
};
struct StdElements : public Node {
  void forward_dev_impl(const Device_GPU& dev, const std::vector<const Tensor*>& xs, Tensor& fx) const override {
    abi_check(dyhip_std_elems_forward(dev.hip, xs[0]->d.batch_size(), xs[0]->d.bd, xs[0]->v, fx.v));
  }
  void backward_dev_impl(const Device_GPU& dev, const std::vector<const Tensor*>& xs, const Tensor& fx,
                         const Tensor& dEdf, unsigned, Tensor& dEdxi) const override {
    abi_check(dyhip_std_elems_backward(dev.hip, xs[0]->d.batch_size(), xs[0]->d.bd, xs[0]->v, fx.v, dEdf.v, dEdxi.v));
  }
};

// dynet/nodes-dropout.cc:25-47: the mask lives in aux_mem (dim.size() floats)
struct Dropout : public Node {
  Dropout(const Dim& dim, real p) : dim(dim), p(p) {}
  Dim dim;
  real p;
  size_t aux_storage_size() const override { return dim.size() * sizeof(float); }
  void forward_dev_impl(const Device_GPU& dev, const std::vector<const Tensor*>& xs, Tensor& fx) const override {
    abi_check(dyhip_dropout_forward(dev.hip, fx.d.size(), p, xs[0]->v, static_cast<float*>(aux_mem), fx.v));
  }
  void backward_dev_impl(const Device_GPU& dev, const std::vector<const Tensor*>&, const Tensor& fx, const Tensor& dEdf,
                         unsigned, Tensor& dEdxi) const override {
    abi_check(dyhip_dropout_backward(dev.hip, fx.d.size(), static_cast<const float*>(aux_mem), dEdf.v, dEdxi.v));
  }
};

// dynet/nodes-random.cc:68-137: nodes without arguments whose forward fills fx
struct RandomBernoulli : public Node {
  RandomBernoulli(real p, real scale = 1.f) : p(p), scale(scale) {}
  real p, scale;
  void forward_dev_impl(const Device_GPU&, const std::vector<const Tensor*>&, Tensor& fx) const override {
    TensorTools::randomize_bernoulli(fx, p, scale);
  }
  void backward_dev_impl(const Device_GPU&, const std::vector<const Tensor*>&, const Tensor&, const Tensor&, unsigned,
                         Tensor&) const override {
    throw std::runtime_error("Called backward() on an arity 0 node");
  }
};
struct RandomNormal : public RandomBernoulli {
  RandomNormal(real mean = 0.f, real stddev = 1.f) : RandomBernoulli(mean, stddev) {}
  void forward_dev_impl(const Device_GPU&, const std::vector<const Tensor*>&, Tensor& fx) const override {
    TensorTools::randomize_normal(fx, p, scale);
  }
};
struct RandomUniform : public RandomBernoulli {
  RandomUniform(real left, real right) : RandomBernoulli(left, right) {}
  void forward_dev_impl(const Device_GPU&, const std::vector<const Tensor*>&, Tensor& fx) const override {
    TensorTools::randomize_uniform(fx, p, scale);
  }
};

// sum_batches = SumDimension({}, include_batch_dim) (dynet/nodes-arith-sum.cc:197-248, dynet/expr.cc:218)
struct SumBatches : public Node {
  void forward_dev_impl(const Device_GPU& dev, const std::vector<const Tensor*>& xs, Tensor& fx) const override {
    size_t need = 0;
    abi_check(dyhip_batch_reduce_workspace(fx.d.batch_size(), xs[0]->d.bd, &need));
    void* ws = need ? scratch(fx)->allocate(need) : nullptr;
    abi_check(dyhip_sum_batches_forward(dev.hip, fx.d.batch_size(), xs[0]->d.bd, xs[0]->v, fx.v, ws, need));
    scratch(fx)->free();
  }
  void backward_dev_impl(const Device_GPU& dev, const std::vector<const Tensor*>& xs, const Tensor& fx,
                         const Tensor& dEdf, unsigned, Tensor& dEdxi) const override {
    abi_check(dyhip_sum_batches_backward(dev.hip, fx.d.batch_size(), xs[0]->d.bd, dEdf.v, dEdxi.v));
  }
};

// layer_norm(x, g, b) as one node instead of the 8-node composite of dynet/expr.cc:248-253.  xs = {x, g, b}
struct LayerNorm : public Node {
  void forward_dev_impl(const Device_GPU& dev, const std::vector<const Tensor*>& xs, Tensor& fx) const override {
    abi_check(dyhip_layer_norm_forward(dev.hip, xs[0]->d.batch_size(), xs[0]->d.bd, xs[0]->v, xs[1]->v, xs[2]->v, fx.v));
  }
  void backward_dev_impl(const Device_GPU& dev, const std::vector<const Tensor*>& xs, const Tensor& fx,
                         const Tensor& dEdf, unsigned i, Tensor& dEdxi) const override {
    const size_t n = xs[0]->d.batch_size();
    const unsigned bd = xs[0]->d.bd;
    size_t need = 0;
    abi_check(dyhip_layer_norm_backward_workspace(n, bd, &need));
    void* ws = scratch(fx)->allocate(need);
    abi_check(dyhip_layer_norm_backward(dev.hip, n, bd, xs[0]->v, xs[1]->v, dEdf.v, i == 0 ? dEdxi.v : nullptr,
                                        i == 1 ? dEdxi.v : nullptr, i == 2 ? dEdxi.v : nullptr, ws, need));
    scratch(fx)->free();
  }
};

// LookupNode (dynet/param-nodes.cc:304-329) over a table Dim({D}, V) stored as V contiguous rows
// (dynet/model.cc:130-159); accumulate_grads = LookupParameterStorage::accumulate_grads_dev (:728-743)
struct LookupNode : public Node {
  LookupNode(const Tensor* all_values, Tensor* all_grads, const std::vector<unsigned>* pindices)
      : all_values(all_values), all_grads(all_grads), pindices(pindices) {}
  const Tensor* all_values;
  Tensor* all_grads;
  const std::vector<unsigned>* pindices;
  // aux_mem = [ids | sorted (id, position) plan].  The reference keeps only the ids there (:154-156); the
  // plan depends on nothing but the ids, so forward builds it and the backward pass starts at the reduction.
  static size_t ids_bytes(size_t n) { return (sizeof(unsigned) * n + 255) / 256 * 256; }
  size_t aux_storage_size() const override {
    size_t plan = 0;
    abi_check(dyhip_lookup_plan_bytes(static_cast<unsigned>(pindices->size()), &plan));
    return ids_bytes(pindices->size()) + plan;
  }

  void forward_dev_impl(const Device_GPU& dev, const std::vector<const Tensor*>&, Tensor& fx) const override {
    const unsigned n = static_cast<unsigned>(pindices->size());
    unsigned* ids_dev = static_cast<unsigned*>(aux_mem);
    abi_check(dyhip_lookup_forward(dev.hip, n, pindices->data(), ids_dev, all_values->d.batch_size(), all_values->d.bd,
                                   all_values->v, 1.0f, fx.v));
    size_t plan = 0, need = 0;
    abi_check(dyhip_lookup_plan_bytes(n, &plan));
    abi_check(dyhip_lookup_plan_workspace(n, all_values->d.bd, &need));
    void* ws = need ? scratch(fx)->allocate(need) : nullptr;
    abi_check(dyhip_lookup_build_plan(dev.hip, n, ids_dev, all_values->d.bd, static_cast<char*>(aux_mem) + ids_bytes(n),
                                      plan, ws, need));
    scratch(fx)->free();
  }
  void backward_dev_impl(const Device_GPU&, const std::vector<const Tensor*>&, const Tensor&, const Tensor&, unsigned,
                         Tensor&) const override {
    throw std::runtime_error("called backward() on arity 0 node: i = 0");  // dynet/param-nodes.cc:331-337
  }
  void accumulate_grad(const Device_GPU& dev, const Tensor& fx, const Tensor& g) const {
    const unsigned n = static_cast<unsigned>(pindices->size());
    const size_t D = all_values->d.batch_size();
    size_t need = 0;
    abi_check(dyhip_lookup_accumulate_grads_planned_workspace(n, D, &need));
    void* ws = need ? scratch(fx)->allocate(need) : nullptr;
    abi_check(dyhip_lookup_accumulate_grads_planned(dev.hip, n, static_cast<const char*>(aux_mem) + ids_bytes(n), D,
                                                    all_values->d.bd, g.v, all_grads->v, ws, need));
    scratch(fx)->free();
  }
};

// PickNegLogSoftmax (dynet/nodes-pickneglogsoftmax.cc:72-145); aux_mem = [z | m | ids]
struct PickNegLogSoftmax : public Node {
  explicit PickNegLogSoftmax(const std::vector<unsigned>* pvals) : pvals(pvals) {}
  const std::vector<unsigned>* pvals;
  size_t aux_storage_size() const override { return 2 * sizeof(float) * pvals->size() + sizeof(unsigned) * pvals->size(); }
  void forward_dev_impl(const Device_GPU& dev, const std::vector<const Tensor*>& xs, Tensor& fx) const override {
    if (xs[0]->d.cols() != 1) throw std::invalid_argument("PickNegLogSoftmax::forward not yet implemented for multiple columns");
    if (pvals->size() != xs[0]->d.bd) throw std::invalid_argument("PickNegLogSoftmax: one index per batch element expected");
    abi_check(dyhip_pnls_forward(dev.hip, xs[0]->d.rows(), xs[0]->d.bd, xs[0]->v, pvals->data(), aux_mem, fx.v));
  }
  void backward_dev_impl(const Device_GPU& dev, const std::vector<const Tensor*>& xs, const Tensor&, const Tensor& dEdf,
                         unsigned, Tensor& dEdxi) const override {
    abi_check(dyhip_pnls_backward(dev.hip, xs[0]->d.rows(), xs[0]->d.bd, xs[0]->v, aux_mem, dEdf.v, dEdxi.v));
  }
};

// ParameterStorage reduced to what the node needs (dynet/model.h:76-118): values and gradient on the device
struct ParameterStorage {
  Tensor values, g;
  bool nonzero_grad = false;
  // ParameterStorage::accumulate_grad (dynet/model.cc:556-571): g += d
  void accumulate_grad(const Tensor& d) {
    nonzero_grad = true;
    abi_check(dyhip_accumulate(values.device->hip, g.d.size(), d.v, g.v));
  }
};

// ParameterNode over a dense parameter (dynet/param-nodes.h:40-58, dynet/param-nodes.cc:43-50,201-225): forward copies
// the values times the current weight decay; backward must never be called (arity 0); accumulate_grad is where the
// executor hands the node's gradient to the parameter (dynet/exec.cc:274-280) -- and where the products recorded into
// that gradient are formed.
struct ParameterNode : public Node {
  ParameterNode(ParameterStorage* params, real weight_decay = 1.f) : params(params), weight_decay(weight_decay) {}
  ParameterStorage* params;
  real weight_decay;
  void forward_dev_impl(const Device_GPU& dev, const std::vector<const Tensor*>& xs, Tensor& fx) const override {
    if (!xs.empty()) throw std::invalid_argument("Failed dimension check in ParameterNode");
    abi_check(dyhip_scale_copy(dev.hip, fx.d.size(), params->values.v, weight_decay, fx.v));
  }
  void backward_dev_impl(const Device_GPU&, const std::vector<const Tensor*>&, const Tensor&, const Tensor&, unsigned i,
                         Tensor&) const override {
    throw std::runtime_error("called backward() on arity 0 node: i = " + std::to_string(i));
  }
  void accumulate_grad(const Tensor& g) const {
    g.device->deferred->flush(g.v);
    params->accumulate_grad(g);
  }
};

// Argmax over a vector per batch element (dynet/nodes-argmax.h, dynet/nodes-argmax.cc:26-68); aux_mem = one 64-bit
// index per batch element (:37-39).  fx is one-hot; backward copies the gradient through when straight_through is set
// and contributes nothing otherwise.
struct Argmax : public Node {
  Argmax(const Dim& dim, unsigned d, bool straight_through) : dim(dim), d(d), straight_through(straight_through) {
    if (dim.nd != 1) throw std::invalid_argument("Argmax only supports vectors for now");
    if (d >= dim.nd) throw std::invalid_argument("Cannot compute argmax along that dimension");
  }
  Dim dim;
  unsigned d;
  bool straight_through;
  size_t aux_storage_size() const override { return dim.size() / dim[d] * sizeof(long long); }
  void forward_dev_impl(const Device_GPU& dev, const std::vector<const Tensor*>& xs, Tensor& fx) const override {
    abi_check(dyhip_argmax_onehot_forward(dev.hip, xs[0]->d[d], xs[0]->d.bd, xs[0]->v, static_cast<long long*>(aux_mem),
                                          fx.v));
  }
  void backward_dev_impl(const Device_GPU& dev, const std::vector<const Tensor*>&, const Tensor&, const Tensor& dEdf,
                         unsigned, Tensor& dEdxi) const override {
    if (straight_through) abi_check(dyhip_accumulate(dev.hip, dEdf.d.size(), dEdf.v, dEdxi.v));
  }
};

// LogSoftmax (dynet/nodes-softmaxes.cc:127-214); aux_mem = [z | m]
struct LogSoftmax : public Node {
  explicit LogSoftmax(const Dim& dim) : dim(dim) {}
  Dim dim;
  size_t aux_storage_size() const override { return 2 * dim.size() / dim.rows() * sizeof(float); }
  void forward_dev_impl(const Device_GPU& dev, const std::vector<const Tensor*>& xs, Tensor& fx) const override {
    abi_check(dyhip_log_softmax_forward(dev.hip, xs[0]->d.rows(), xs[0]->d.cols() * xs[0]->d.bd, xs[0]->v, aux_mem, fx.v));
  }
  void backward_dev_impl(const Device_GPU& dev, const std::vector<const Tensor*>& xs, const Tensor& fx,
                         const Tensor& dEdf, unsigned, Tensor& dEdxi) const override {
    abi_check(dyhip_log_softmax_backward(dev.hip, xs[0]->d.rows(), xs[0]->d.cols() * xs[0]->d.bd, fx.v, dEdf.v, aux_mem,
                                         dEdxi.v));
  }
};

// Softmax along dimension 0 or 1 (dynet/nodes-softmaxes.cc:40-125)
struct Softmax : public Node {
  explicit Softmax(unsigned dimension = 0) : dimension(dimension) {}
  unsigned dimension;
  void forward_dev_impl(const Device_GPU& dev, const std::vector<const Tensor*>& xs, Tensor& fx) const override {
    const Dim& d = xs[0]->d;
    if (dimension == 0) {
      const unsigned cols = d.cols() * d.bd;
      void* ws = scratch(fx)->allocate(2 * sizeof(float) * cols);
      abi_check(dyhip_softmax_forward(dev.hip, d.rows(), cols, xs[0]->v, fx.v, ws, 2 * sizeof(float) * cols));
      scratch(fx)->free();
    } else {
      abi_check(dyhip_softmax_rows_forward(dev.hip, d.rows(), d.cols(), d.bd, xs[0]->v, fx.v));
    }
  }
  void backward_dev_impl(const Device_GPU& dev, const std::vector<const Tensor*>& xs, const Tensor& fx,
                         const Tensor& dEdf, unsigned, Tensor& dEdxi) const override {
    const Dim& d = xs[0]->d;
    if (dimension == 0) {
      const unsigned cols = d.cols() * d.bd;
      void* ws = scratch(fx)->allocate(sizeof(float) * cols);
      abi_check(dyhip_softmax_backward(dev.hip, d.rows(), cols, fx.v, dEdf.v, dEdxi.v, ws, sizeof(float) * cols));
      scratch(fx)->free();
    } else {
      abi_check(dyhip_softmax_rows_backward(dev.hip, d.rows(), d.cols(), d.bd, fx.v, dEdf.v, dEdxi.v));
    }
  }
};

// LogSumExpDimension (dynet/nodes-logsumexp.cc:126-145); the maxima go to scratch as in the reference
struct LogSumExpDimension : public Node {
  explicit LogSumExpDimension(unsigned dimension = 0) : dimension(dimension) {}
  unsigned dimension;
  void forward_dev_impl(const Device_GPU& dev, const std::vector<const Tensor*>& xs, Tensor& fx) const override {
    const Dim& d = xs[0]->d;
    if (d.nd > 2) throw std::invalid_argument("LogSumExpDimension supports tensors of dimension <= 2");
    float* ms = static_cast<float*>(scratch(fx)->allocate(sizeof(float) * fx.d.size()));
    abi_check(dyhip_logsumexp_dim_forward(dev.hip, d.rows(), d.cols(), d.bd, xs[0]->v, dimension, ms, fx.v));
    scratch(fx)->free();
  }
  void backward_dev_impl(const Device_GPU& dev, const std::vector<const Tensor*>& xs, const Tensor& fx,
                         const Tensor& dEdf, unsigned, Tensor& dEdxi) const override {
    const Dim& d = xs[0]->d;
    abi_check(dyhip_logsumexp_dim_backward(dev.hip, d.rows(), d.cols(), d.bd, xs[0]->v, fx.v, dEdf.v, dimension, dEdxi.v));
  }
};

// LogSumExp over its arguments (dynet/nodes-logsumexp.cc:38-124): same shape, each with the result's batch size or 1
struct LogSumExp : public Node {
  static void gather(const std::vector<const Tensor*>& xs, std::vector<const float*>& p, std::vector<unsigned>& b) {
    for (const Tensor* x : xs) {
      p.push_back(x->v);
      b.push_back(x->d.bd);
    }
  }
  void forward_dev_impl(const Device_GPU& dev, const std::vector<const Tensor*>& xs, Tensor& fx) const override {
    std::vector<const float*> p;
    std::vector<unsigned> b;
    gather(xs, p, b);
    abi_check(dyhip_logsumexp_node_forward(dev.hip, static_cast<unsigned>(xs.size()), fx.d.batch_size(), fx.d.bd, p.data(),
                                           b.data(), fx.v));
  }
  void backward_dev_impl(const Device_GPU& dev, const std::vector<const Tensor*>& xs, const Tensor& fx,
                         const Tensor& dEdf, unsigned i, Tensor& dEdxi) const override {
    std::vector<const float*> p;
    std::vector<unsigned> b;
    gather(xs, p, b);
    // an argument broadcast over the batch: its terms are formed in scratch and summed over the batch from there
    size_t need = 0;
    if (xs[i]->d.bd != fx.d.bd) {
      abi_check(dyhip_batch_reduce_workspace(fx.d.batch_size(), fx.d.bd, &need));
      need += (sizeof(float) * fx.d.size() + 255) / 256 * 256;
    }
    void* ws = need ? scratch(fx)->allocate(need) : nullptr;
    abi_check(dyhip_logsumexp_node_backward(dev.hip, static_cast<unsigned>(xs.size()), fx.d.batch_size(), fx.d.bd, p.data(),
                                            b.data(), fx.v, dEdf.v, i, dEdxi.v, ws, need));
    scratch(fx)->free();
  }
};

// Sum / esum (dynet/nodes-arith-sum.cc:65-129): any number of same-shaped arguments with the result's batch size or 1
struct Sum : public Node {
  void forward_dev_impl(const Device_GPU& dev, const std::vector<const Tensor*>& xs, Tensor& fx) const override {
    if (xs.empty()) throw std::invalid_argument("Sum needs at least one argument");  // nodes-arith-sum.cc:39
    std::vector<const float*> p;
    std::vector<unsigned> b;
    LogSumExp::gather(xs, p, b);
    abi_check(dyhip_sum_forward(dev.hip, static_cast<unsigned>(xs.size()), fx.d.batch_size(), fx.d.bd, p.data(), b.data(),
                                fx.v));
  }
  void backward_dev_impl(const Device_GPU& dev, const std::vector<const Tensor*>& xs, const Tensor& fx,
                         const Tensor& dEdf, unsigned i, Tensor& dEdxi) const override {
    size_t need = 0;
    abi_check(dyhip_batch_reduce_workspace(fx.d.batch_size(), fx.d.bd, &need));
    void* ws = need ? scratch(fx)->allocate(need) : nullptr;
    // dEdxi += dEdf, summed over the batch for an argument of batch size 1 (:115-128)
    abi_check(dyhip_csum_backward(dev.hip, fx.d.batch_size(), xs[i]->d.bd, fx.d.bd, dEdf.v, 0, dEdxi.v, ws, need));
    scratch(fx)->free();
  }
};

// PickRange (dynet/nodes-select.cc:216-259): the slice [start, end) of dimension `dim`
struct PickRange : public Node {
  PickRange(unsigned start, unsigned end, unsigned dim = 0) : start(start), end(end), dim(dim) {}
  unsigned start, end, dim;
  void split(const Dim& d, size_t& inner, size_t& len, size_t& outer) const {
    inner = 1;
    outer = d.bd;
    for (unsigned j = 0; j < d.nd; ++j) (j < dim ? inner : outer) *= j == dim ? 1 : d[j];
    len = d[dim];
  }
  void forward_dev_impl(const Device_GPU& dev, const std::vector<const Tensor*>& xs, Tensor& fx) const override {
    size_t inner, len, outer;
    split(xs[0]->d, inner, len, outer);
    abi_check(dyhip_pick_range_forward(dev.hip, inner, len, outer, start, end, xs[0]->v, fx.v));
  }
  void backward_dev_impl(const Device_GPU& dev, const std::vector<const Tensor*>& xs, const Tensor&, const Tensor& dEdf,
                         unsigned, Tensor& dEdxi) const override {
    size_t inner, len, outer;
    split(xs[0]->d, inner, len, outer);
    abi_check(dyhip_pick_range_backward(dev.hip, inner, len, outer, start, end, dEdf.v, dEdxi.v));
  }
};

// AffineTransform with one (W, x) pair (dynet/nodes-affinetransform.cc:77-156).  xs = {bias, W, x}
struct AffineTransform : public Node {
  void forward_dev_impl(const Device_GPU& dev, const std::vector<const Tensor*>& xs, Tensor& fx) const override {
    if (xs.size() != 3) throw std::invalid_argument("AffineTransform: this device path takes one (W, x) pair");
    abi_check(dyhip_affine_forward(dev.hip, xs[1]->d.rows(), xs[2]->d.cols() * xs[2]->d.bd, xs[1]->d.cols(), xs[0]->v,
                                   xs[1]->v, xs[2]->v, fx.v));
  }
  void backward_dev_impl(const Device_GPU& dev, const std::vector<const Tensor*>& xs, const Tensor& fx,
                         const Tensor& dEdf, unsigned i, Tensor& dEdxi) const override {
    const size_t M = xs[1]->d.rows(), K = xs[1]->d.cols(), N = size_t(xs[2]->d.cols()) * xs[2]->d.bd;
    if (i == 0) {
      size_t need = 0;
      abi_check(dyhip_batch_reduce_workspace(M, static_cast<unsigned>(N), &need));
      void* ws = need ? scratch(fx)->allocate(need) : nullptr;
      abi_check(dyhip_csum_backward(dev.hip, M, 1, static_cast<unsigned>(N), dEdf.v, 0, dEdxi.v, ws, need));
      scratch(fx)->free();
    } else if (i == 1) {
      abi_check(dyhip_gemm_nt_acc(dev.hip, M, K, N, dEdf.v, xs[2]->v, dEdxi.v));  // MatrixMultiplyTranspAcc
    } else {
      abi_check(dyhip_gemm_tn_acc(dev.hip, K, N, M, xs[1]->v, dEdf.v, dEdxi.v));  // MatrixTranspMultiplyAcc
    }
  }
};

// dynet/matrix-multiply.h:16-37,97-117,162-180 on Device_GPU: one GEMM over all columns when the left operand
// is shared by the batch, the strided-batched form otherwise (same branch conditions as the reference)
inline size_t batch_stride(const Tensor& t) { return t.d.bd > 1 ? t.d.batch_size() : 0; }
inline void MatrixMultiply(const Device_GPU& dev, const Tensor& l, const Tensor& r, Tensor& y, const float* acc_scalar) {
  const float beta = acc_scalar == dev.kSCALAR_ONE ? 1.0f : 0.0f;
  if (l.d.bd == 1 && r.d.bd == y.d.bd)
    abi_check(dyhip_gemm_nn(dev.hip, y.d.rows(), size_t(y.d.cols()) * y.d.bd, l.d.cols(), l.v, r.v, beta, y.v));
  else
    abi_check(dyhip_gemm_strided_batched(dev.hip, 0, 0, y.d.rows(), y.d.cols(), l.d.cols(), l.v, batch_stride(l), r.v,
                                         batch_stride(r), beta, y.v, y.d.batch_size(), y.d.bd));
}
inline void MatrixTranspMultiplyAcc(const Device_GPU& dev, const Tensor& l, const Tensor& r, Tensor& y) {
  const unsigned max_b = l.d.bd > r.d.bd ? l.d.bd : r.d.bd;
  if (l.d.bd == 1 && y.d.bd == r.d.bd)
    abi_check(dyhip_gemm_tn_acc(dev.hip, y.d.rows(), size_t(y.d.cols()) * y.d.bd, l.d.rows(), l.v, r.v, y.v));
  else
    abi_check(dyhip_gemm_strided_batched(dev.hip, 1, 0, y.d.rows(), y.d.cols(), l.d.rows(), l.v, batch_stride(l), r.v,
                                         batch_stride(r), 1.0f, y.v, y.d.batch_size(), max_b));
}
inline void MatrixMultiplyTranspAcc(const Device_GPU& dev, const Tensor& l, const Tensor& r, Tensor& y) {
  const unsigned max_b = l.d.bd > r.d.bd ? l.d.bd : r.d.bd;
  if (y.d.bd == 1 && l.d.bd == r.d.bd)
    abi_check(dyhip_gemm_nt_acc(dev.hip, y.d.rows(), y.d.cols(), size_t(l.d.cols()) * l.d.bd, l.v, r.v, y.v));
  else
    abi_check(dyhip_gemm_strided_batched(dev.hip, 0, 1, y.d.rows(), y.d.cols(), l.d.cols(), l.v, batch_stride(l), r.v,
                                         batch_stride(r), 1.0f, y.v, y.d.batch_size(), max_b));
}

// dynet::gpu::* (dynet/gpu-ops.h:9-15): same argument lists behind the device
namespace gpu {
inline void dense_to_sparse_assign(const Device_GPU& dev, int n, const unsigned* ids, float* src, float* trg) {
  abi_check(dyhip_dense_to_sparse_assign(dev.hip, n, ids, src, trg));
}
inline void sparse_to_dense_assign(const Device_GPU& dev, int n, const unsigned* ids, float* src, float* trg) {
  abi_check(dyhip_sparse_to_dense_assign(dev.hip, n, ids, src, trg));
}
inline void dense_to_sparse_subtract(const Device_GPU& dev, int n, const unsigned* ids, float* src, float* trg) {
  abi_check(dyhip_dense_to_sparse_subtract(dev.hip, n, ids, src, trg));
}
inline void sparse_to_dense_block_assign_and_multiply(const Device_GPU& dev, int n, const unsigned* idx, int bsize,
                                                      float mult, float* src, float* trg) {
  abi_check(dyhip_sparse_to_dense_block_assign_and_multiply(dev.hip, n, idx, bsize, mult, src, trg));
}
inline void dense_to_sparse_block_add(const Device_GPU& dev, int n, const unsigned* ids, int bsize, float* src, float* trg) {
  abi_check(dyhip_dense_to_sparse_block_add(dev.hip, n, ids, bsize, src, trg));
}
inline void parallel_memcpy(const Device_GPU& dev, int num_seqs, int max_len, float** src, float** trg, size_t* len) {
  abi_check(dyhip_parallel_memcpy(dev.hip, num_seqs, max_len, src, trg, len));
}
inline void parallel_accumulate(const Device_GPU& dev, int num_seqs, int max_len, float** src, float** trg, size_t* len) {
  abi_check(dyhip_parallel_accumulate(dev.hip, num_seqs, max_len, src, trg, len));
}
}  // namespace gpu

// The GPU branches of BatchedExecutionEngine::combine_tensors / accumulate_tensors (dynet/exec.cc:298-361,
// 363-409) without the executor around them: the caller names the tensors.  The [src | trg | len] table is
// written into page-locked staging memory, so its copy to the device queues behind earlier work instead of
// stalling the host the way the reference's copy from a pageable std::vector does.
namespace detail {
inline void stage_and_move(Device_GPU& dev, DeviceMempool table_pool, const std::vector<float*>& srcs,
                           const std::vector<float*>& trgs, const std::vector<size_t>& lens, bool accumulate) {
  const size_t n = srcs.size();
  if (n == 0) return;
  static_assert(sizeof(float*) == sizeof(size_t), "pointer and length entries share one table");
  size_t* host = static_cast<size_t*>(dev.staging->take(3 * n * sizeof(size_t)));
  size_t max_len = 0;
  for (size_t k = 0; k < n; ++k) {
    host[k] = reinterpret_cast<size_t>(srcs[k]);
    host[n + k] = reinterpret_cast<size_t>(trgs[k]);
    host[2 * n + k] = lens[k];
    if (lens[k] > max_len) max_len = lens[k];
  }
  void* table = dev.pools[static_cast<int>(table_pool)]->allocate(3 * n * sizeof(size_t));
  abi_check(dyhip_memcpy_h2d(dev.hip, table, host, 3 * n * sizeof(size_t)));
  float** d_src = static_cast<float**>(table);
  float** d_trg = d_src + n;
  size_t* d_len = static_cast<size_t*>(table) + 2 * n;
  if (accumulate) gpu::parallel_accumulate(dev, static_cast<int>(n), static_cast<int>(max_len), d_src, d_trg, d_len);
  else gpu::parallel_memcpy(dev, static_cast<int>(n), static_cast<int>(max_len), d_src, d_trg, d_len);
}
}  // namespace detail

// tout becomes one contiguous tensor Dim({sum of sizes}) allocated from pools[FXS], holding the tensors of
// `parts` back to back (dynet/exec.cc:298-361)
inline void combine_tensors(Device_GPU& dev, const std::vector<const Tensor*>& parts, Tensor& tout) {
  size_t total = 0;
  for (const Tensor* t : parts) total += t->d.size();
  if (total > 0xffffffffu) throw std::invalid_argument("combine_tensors: more than 2^32 - 1 elements");
  tout.d = Dim({static_cast<unsigned>(total)});
  tout.device = &dev;
  tout.mem_pool = DeviceMempool::FXS;
  tout.v = static_cast<float*>(dev.pools[static_cast<int>(DeviceMempool::FXS)]->allocate(total * sizeof(float)));
  std::vector<float*> srcs, trgs;
  std::vector<size_t> lens;
  float* dest = tout.v;
  for (const Tensor* t : parts) {
    srcs.push_back(t->v);
    trgs.push_back(dest);
    lens.push_back(t->d.size());
    dest += t->d.size();
  }
  detail::stage_and_move(dev, DeviceMempool::FXS, srcs, trgs, lens, false);
}

// every tensor of `grads` += its slice of tin, slices back to back in the order given (dynet/exec.cc:363-409);
// two entries must not name the same memory, as the reference's one-thread-per-element kernel assumes
inline void accumulate_tensors(Device_GPU& dev, const Tensor& tin, const std::vector<Tensor*>& grads) {
  std::vector<float*> srcs, trgs;
  std::vector<size_t> lens;
  float* src = tin.v;
  size_t total = 0;
  for (Tensor* t : grads) {
    srcs.push_back(src);
    trgs.push_back(t->v);
    lens.push_back(t->d.size());
    src += t->d.size();
    total += t->d.size();
  }
  if (total != tin.d.size()) throw std::invalid_argument("accumulate_tensors: the slices do not cover the input tensor");
  detail::stage_and_move(dev, DeviceMempool::DEDFS, srcs, trgs, lens, true);
}

}  // namespace dynet_hip
