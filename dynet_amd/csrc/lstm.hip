// Fused LSTM nodes: VanillaLSTMGates, VanillaLSTMC, VanillaLSTMH
// (dynet/nodes-lstm.cc:101-235, 237-527, 562-615, 650-703).
//
// Gates forward is ONE GEMM launch over two K segments ([Wx | Wh] * [x ; h])
// whose epilogue adds the bias and the +1 forget bias and applies logistic to
// rows [0,3H) and tanh to rows [3H,4H) -- the reference issues a broadcast, a
// slice add, two cuBLAS calls and six slice/activation launches for the same
// result.  Backward computes dpre = dEdf * act'(fx) once per call (or takes it
// precomputed) and feeds the transposed GEMM forms; the bias gradient is a
// batch reduction.  C and H are single elementwise kernels each way (the
// reference copies gate slices to scratch first).
//
// Layout: gates is 4H x B column-major, gate order i, f, o, g; c, h are H x B.
#include <initializer_list>

#include "gemm.h"

namespace dyhip {

int batch_reduce(dyhip_device* dev, size_t n, unsigned bd, const float* in0, const float* in1, float* out,
                 bool accumulate, void* ws, size_t ws_bytes);

static size_t align256(size_t n) { return (n + 255) / 256 * 256; }

// blocks along the grid's second dimension for B batch elements (kernels stride over the rest)
static unsigned grid_y(unsigned B) { return B < 65535u ? B : 65535u; }

// dst[b*dst_ld + off + r] = src[b*rows + r] * (mask ? mask[(mask_b ? b : 0)*dst_ld + off + r] : 1)
__global__ __launch_bounds__(256) void rows_copy_mask_kernel(unsigned rows, unsigned dst_ld, unsigned off,
                                                             const float* __restrict__ src,
                                                             const float* __restrict__ mask, int mask_b,
                                                             float* __restrict__ dst, unsigned B) {
  const unsigned r = blockIdx.x * 256 + threadIdx.x;
  if (r >= rows) return;
  for (unsigned b = blockIdx.y; b < B; b += gridDim.y) {  // the grid's second dimension holds at most 65535 blocks
    float v = src[size_t(b) * rows + r];
    if (mask) v *= mask[size_t(mask_b ? b : 0) * dst_ld + off + r];
    dst[size_t(b) * dst_ld + off + r] = v;
  }
}

// out[b*rows + r] += tmp[b*rows + r] * mask[(mask_b ? b : 0)*mask_ld + off + r]
__global__ __launch_bounds__(256) void acc_mul_mask_kernel(unsigned rows, unsigned mask_ld, unsigned off,
                                                           const float* __restrict__ tmp,
                                                           const float* __restrict__ mask, int mask_b,
                                                           float* __restrict__ out, unsigned B) {
  const unsigned r = blockIdx.x * 256 + threadIdx.x;
  if (r >= rows) return;
  for (unsigned b = blockIdx.y; b < B; b += gridDim.y)
    out[size_t(b) * rows + r] += tmp[size_t(b) * rows + r] * mask[size_t(mask_b ? b : 0) * mask_ld + off + r];
}

// dpre[i, b] = i < 3H ? d*f*(1-f) : d*(1-f*f)      (dynet/nodes-lstm.cc:358-361)
__global__ __launch_bounds__(256) void lstm_dpre_kernel(unsigned H, const float* __restrict__ fx,
                                                        const float* __restrict__ dEdf, float* __restrict__ dpre,
                                                        unsigned B) {
  const unsigned i = blockIdx.x * 256 + threadIdx.x;
  if (i >= 4 * H) return;
  for (unsigned b = blockIdx.y; b < B; b += gridDim.y) {
    const size_t e = size_t(b) * 4 * H + i;
    const float f = fx[e], d = dEdf[e];
    dpre[e] = i < 3 * H ? d * f * (1.f - f) : d * (1.f - f * f);
  }
}

// mode 0: c = i*g + f*c_prev                                   (C forward, :562-589)
// mode 1: dc_prev += dc*f                                      (C backward i=0, :605-606)
// mode 2: di += dc*g; df += dc*c_prev; dg += dc*i              (C backward i=1, :607-614)
// mode 3: h = o*tanh(c)                                        (H forward, :650-668)
// mode 4: dc += dh*o*(1 - tanh(c)^2)                           (H backward i=0, :684-694)
// mode 5: do += dh*tanh(c)                                     (H backward i=1, :695-701)
// `state` is c_prev (modes 0-2) or c (modes 3-5); `d` is dEdf for the backward modes.
template <int MODE>
__global__ __launch_bounds__(256) void lstm_pointwise_kernel(unsigned H, const float* __restrict__ state,
                                                             const float* __restrict__ gates,
                                                             const float* __restrict__ d, float* __restrict__ out,
                                                             unsigned B) {
  const unsigned r = blockIdx.x * 256 + threadIdx.x;
  if (r >= H) return;
  for (unsigned b = blockIdx.y; b < B; b += gridDim.y) {
  const size_t s = size_t(b) * H + r;
  const float* gt = gates + size_t(b) * 4 * H;
  if (MODE == 0) {
    out[s] = gt[r] * gt[3 * H + r] + gt[H + r] * state[s];
  } else if (MODE == 1) {
    out[s] += d[s] * gt[H + r];
  } else if (MODE == 2) {
    float* dg = out + size_t(b) * 4 * H;
    const float dc = d[s];
    dg[r] += dc * gt[3 * H + r];
    dg[H + r] += dc * state[s];
    dg[3 * H + r] += dc * gt[r];
  } else if (MODE == 3) {
    out[s] = gt[2 * H + r] * tanh_accurate(state[s]);
  } else if (MODE == 4) {
    const float t = tanh_accurate(state[s]);
    out[s] += d[s] * gt[2 * H + r] * (1.f - t * t);
  } else {
    out[size_t(b) * 4 * H + 2 * H + r] += d[s] * tanh_accurate(state[s]);
  }
}
}

template <int MODE>
static int launch_pointwise(dyhip_device* dev, unsigned H, unsigned B, const float* state, const float* gates,
                            const float* d, float* out) {
  if (H == 0 || B == 0) return DYHIP_OK;
  hipLaunchKernelGGL(lstm_pointwise_kernel<MODE>, dim3(cdiv<unsigned>(H, 256), grid_y(B)), dim3(256), 0, dev->stream, H,
                     state, gates, d, out, B);
  DYHIP_CHECK_LAUNCH();
  return DYHIP_OK;
}


// ---- fused cell step: gates + C + H in one kernel around the recurrent GEMM ----------
// The input projection Wx*x of every timestep is one large GEMM up front; a timestep is
// then (1) the split-K GEMM Wh*h_tm1 whose unreduced slices stay in a workspace and
// (2) this kernel, which adds the slices, the input projection, the bias and the forget
// bias, applies the activations and forms c and h.  One thread owns V consecutive hidden
// units of one batch column and touches the four gate rows j, H+j, 2H+j, 3H+j.
template <int V>
struct Pack;
template <>
struct Pack<1> {
  float v[1];
  __device__ __forceinline__ void load(const float* p) { v[0] = *p; }
  __device__ __forceinline__ void store(float* p) const { *p = v[0]; }
};
template <>
struct Pack<4> {
  float v[4];
  __device__ __forceinline__ void load(const float* p) {
    const float4 t = *reinterpret_cast<const float4*>(p);
    v[0] = t.x; v[1] = t.y; v[2] = t.z; v[3] = t.w;
  }
  __device__ __forceinline__ void store(float* p) const { *reinterpret_cast<float4*>(p) = make_float4(v[0], v[1], v[2], v[3]); }
};

constexpr int kCellThreads = 64;

template <int V>
__global__ __launch_bounds__(kCellThreads) void lstm_cell_fwd_kernel(unsigned H, unsigned splits, size_t slice,
                                                                     const float* xproj, const float* __restrict__ rec,
                                                                     const float* __restrict__ bias,
                                                                     const float* __restrict__ c_prev, int mode,
                                                                     float* gates, float* __restrict__ c,
                                                                     float* __restrict__ h, unsigned b_first) {
  const unsigned j = (blockIdx.x * kCellThreads + threadIdx.x) * V, b = b_first + blockIdx.y;
  if (j >= H) return;
  const size_t g0 = size_t(b) * 4 * H + j, s0 = size_t(b) * H + j;
  Pack<V> pre[4], cp;
#pragma unroll
  for (int q = 0; q < 4; ++q) {
    Pack<V> bq, xq;
    bq.load(bias + q * H + j);
    xq.load(xproj + g0 + size_t(q) * H);
#pragma unroll
    for (int e = 0; e < V; ++e) pre[q].v[e] = (q == 1 ? bq.v[e] + 1.0f : bq.v[e]) + xq.v[e];
  }
  for (unsigned k = 0; k < splits; ++k) {
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      Pack<V> r;
      r.load(rec + size_t(k) * slice + g0 + size_t(q) * H);
#pragma unroll
      for (int e = 0; e < V; ++e) pre[q].v[e] += r.v[e];
    }
  }
  if (c_prev) cp.load(c_prev + s0);
  Pack<V> cn, hn;
#pragma unroll
  for (int e = 0; e < V; ++e) {
    const float gi = logistic(mode, pre[0].v[e]), gf = logistic(mode, pre[1].v[e]), go = logistic(mode, pre[2].v[e]);
    const float gg = tanh_accurate(pre[3].v[e]);
    pre[0].v[e] = gi; pre[1].v[e] = gf; pre[2].v[e] = go; pre[3].v[e] = gg;
    const float cv = c_prev ? gi * gg + gf * cp.v[e] : gi * gg;
    cn.v[e] = cv;
    hn.v[e] = go * tanh_accurate(cv);
  }
#pragma unroll
  for (int q = 0; q < 4; ++q) pre[q].store(gates + g0 + size_t(q) * H);
  cn.store(c + s0);
  hn.store(h + s0);
}

// Backward of the same step.  dh = dh_in + sum of the slices of Wh^T * dpre_{t+1}; then the
// H, C and gate-activation backward formulas of dynet/nodes-lstm.cc:358-361,605-614,684-701
// in one pass: writes dpre (4H x B) and dc_tm1.
template <int V>
__global__ __launch_bounds__(kCellThreads) void lstm_cell_bwd_kernel(unsigned H, unsigned splits, size_t slice,
                                                                     const float* __restrict__ gates,
                                                                     const float* __restrict__ c,
                                                                     const float* __restrict__ c_prev,
                                                                     const float* __restrict__ dh_in,
                                                                     const float* __restrict__ rec,
                                                                     const float* dc_in, float* __restrict__ dpre,
                                                                     float* dc_prev, unsigned b_first) {
  const unsigned j = (blockIdx.x * kCellThreads + threadIdx.x) * V, b = b_first + blockIdx.y;
  if (j >= H) return;
  const size_t g0 = size_t(b) * 4 * H + j, s0 = size_t(b) * H + j;
  Pack<V> gt[4], cv, cp, dh, dc;
#pragma unroll
  for (int q = 0; q < 4; ++q) gt[q].load(gates + g0 + size_t(q) * H);
  cv.load(c + s0);
  dh.load(dh_in + s0);
  if (c_prev) cp.load(c_prev + s0);
  if (dc_in) dc.load(dc_in + s0);
  for (unsigned k = 0; k < splits; ++k) {
    Pack<V> r;
    r.load(rec + size_t(k) * slice + s0);
#pragma unroll
    for (int e = 0; e < V; ++e) dh.v[e] += r.v[e];
  }
  Pack<V> out[4], dcp;
#pragma unroll
  for (int e = 0; e < V; ++e) {
    const float gi = gt[0].v[e], gf = gt[1].v[e], go = gt[2].v[e], gg = gt[3].v[e];
    const float t = tanh_accurate(cv.v[e]);
    const float dcv = (dc_in ? dc.v[e] : 0.f) + dh.v[e] * go * (1.f - t * t);
    const float d_o = dh.v[e] * t;
    const float d_i = dcv * gg, d_f = c_prev ? dcv * cp.v[e] : 0.f, d_g = dcv * gi;
    dcp.v[e] = dcv * gf;
    out[0].v[e] = d_i * gi * (1.f - gi);
    out[1].v[e] = d_f * gf * (1.f - gf);
    out[2].v[e] = d_o * go * (1.f - go);
    out[3].v[e] = d_g * (1.f - gg * gg);
  }
#pragma unroll
  for (int q = 0; q < 4; ++q) out[q].store(dpre + g0 + size_t(q) * H);
  if (dc_prev) dcp.store(dc_prev + s0);
}

// ---- single-launch forward step: recurrent product and cell update in one kernel -------
// A block owns 8 hidden units x 32 batch columns.  Its 32 weight rows are the four gate
// rows (i, f, o, g) of those 8 units, so after the product all four pre-activations of a
// hidden unit sit in the same block and the cell update runs in the epilogue: the 4H x B
// product never goes to memory.  The four waves split the H-deep sum in quarters, each
// streaming its quarter through a private double-buffered LDS stage into 32x32x2 MFMAs,
// and the quarters meet in LDS.
//
// The weights are read from a packed copy Wp[H/8][H][32]: tile rt, column k holds the 32
// rows {g*H + rt*8 + u : g < 4, u < 8} at index g*8 + u, which makes a wave's stage one
// contiguous 4 KiB run.  Blocks of one row tile are H/8 apart in launch order, so with
// H/8 a multiple of 8 they land on the same XCD and share that L2's copy of the tile.
constexpr int kStepBK = 32;                 // k depth of one LDS stage
constexpr int kStepPitchB = 34;             // B stage: [k][col], 2-way conflicts at most on the transposing write
constexpr int kStepPitchR = 33;             // quarter-sum exchange: [row][col]
constexpr int kStepWaveFloats = 2 * 32 * kStepBK + 2 * kStepBK * kStepPitchB;  // per-wave A + B stages
typedef float stepx16 __attribute__((ext_vector_type(16)));

// W is 4H x K (Wh: K = H, Wx: K = the input size)
__global__ __launch_bounds__(256) void lstm_pack_recurrent_kernel(unsigned H, unsigned K, const float* __restrict__ W,
                                                                  float* __restrict__ Wp) {
  const size_t o = size_t(blockIdx.x) * 256 + threadIdx.x;  // output index, (rt*K + k)*32 + g*8 + u
  if (o >= size_t(4) * H * K) return;
  const unsigned r = o % 32, g = r / 8, u = r % 8;
  const size_t tk = o / 32;
  const unsigned k = tk % K, rt = tk / K;
  Wp[o] = W[size_t(g) * H + rt * 8 + u + size_t(k) * 4 * H];
}

// orders a wave's LDS writes before the reads its other lanes issue afterwards
__device__ __forceinline__ void step_wave_sync() {
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

// Up to two products feed the pre-activations: Wx * x (packed Wx, depth I) and Wh * h_tm1 (packed Wh,
// depth H); either may be absent (null), and Wx * x may instead arrive precomputed in xproj.
struct StepOperand {
  const float* Wp;  // packed weights [H/8][K][32]
  const float* v;   // K x B, column-major
  unsigned K;
};

__global__ __launch_bounds__(256, 2) void lstm_step_fwd_kernel(unsigned H, unsigned B, StepOperand op0, StepOperand op1,
                                                               const float* xproj,
                                                               const float* __restrict__ bias,
                                                               const float* __restrict__ c_prev, int mode,
                                                               float* gates, float* __restrict__ c,
                                                               float* __restrict__ h) {
  __shared__ __attribute__((aligned(16))) float lds[4 * kStepWaveFloats];
  const unsigned RT = H / 8;
  const unsigned rt = blockIdx.x % RT, ct = blockIdx.x / RT;
  const unsigned wave = threadIdx.x / 64, lane = threadIdx.x % 64;
  const unsigned l32 = lane % 32, lhi = lane / 32;
  float* la = lds + wave * kStepWaveFloats;
  float* lb = la + 2 * 32 * kStepBK;
  const unsigned bk = 4 * (lane % 8), bc = lane / 8;

  // the epilogue's thread owns hidden unit eu of batch column ecc; its operands are fetched
  // now so that their latency hides behind the product
  const unsigned eu = threadIdx.x % 8, ecc = threadIdx.x / 8;
  const unsigned ecol = ct * 32 + ecc, ej = rt * 8 + eu;
  float pre[4] = {0.f, 0.f, 0.f, 0.f}, cp = 0.f;
  if (ecol < B) {
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      const float bq = bias[q * H + ej];
      pre[q] = q == 1 ? bq + 1.0f : bq;
      if (xproj != nullptr) pre[q] += xproj[size_t(ecol) * 4 * H + ej + size_t(q) * H];
    }
    if (c_prev != nullptr) cp = c_prev[size_t(ecol) * H + ej];
  }

  float4 ra0, ra1, ra2, ra3, rb0, rb1, rb2, rb3;
#define STEP_LOAD1(i, st)                                                                  \
  ra##i = *reinterpret_cast<const float4*>(ga + size_t(st) * 32 * kStepBK + i * 256);      \
  rb##i = *reinterpret_cast<const float4*>(gb##i + (st) * kStepBK);
#define STEP_LOAD(st) STEP_LOAD1(0, st) STEP_LOAD1(1, st) STEP_LOAD1(2, st) STEP_LOAD1(3, st)
#define STEP_STORE1(i)                                                                     \
  *reinterpret_cast<float4*>(a_ + i * 256) = ra##i;                                        \
  b_[0 * kStepPitchB + 8 * i] = rb##i.x;                                                   \
  b_[1 * kStepPitchB + 8 * i] = rb##i.y;                                                   \
  b_[2 * kStepPitchB + 8 * i] = rb##i.z;                                                   \
  b_[3 * kStepPitchB + 8 * i] = rb##i.w;
#define STEP_STORE(buf)                                                                    \
  {                                                                                        \
    float* a_ = la + (buf) * 32 * kStepBK + lane * 4;                                      \
    float* b_ = lb + (buf) * kStepBK * kStepPitchB + bk * kStepPitchB + bc;                \
    STEP_STORE1(0) STEP_STORE1(1) STEP_STORE1(2) STEP_STORE1(3)                            \
  }

  // The kernel runs at the rate the L2 delivers the operands (every 32x32 output tile pulls
  // its full-depth strips of both), so one stage of lookahead is enough.
  stepx16 acc = {0};
  const float *ga = nullptr, *gb0 = nullptr, *gb1 = nullptr, *gb2 = nullptr, *gb3 = nullptr;
  for (int which = 0; which < 2; ++which) {
    const StepOperand op = which == 0 ? op0 : op1;
    if (op.Wp == nullptr) continue;  // uniform over the grid
    const unsigned kq = op.K / 4, k0 = wave * kq, nst = kq / kStepBK;
    ga = op.Wp + (size_t(rt) * op.K + k0) * 32 + lane * 4;
    // columns past the batch are computed on a clamped address and dropped
    auto column = [&](unsigned i) {
      const unsigned col = ct * 32 + bc + 8 * i;
      return op.v + size_t(col < B ? col : B - 1) * op.K + k0 + bk;
    };
    gb0 = column(0);
    gb1 = column(1);
    gb2 = column(2);
    gb3 = column(3);
    STEP_LOAD(0)
    STEP_STORE(0)
    if (nst > 1) { STEP_LOAD(1) }
    step_wave_sync();
    for (unsigned st = 0; st < nst; ++st) {
      const unsigned cur = st & 1;
      const float* a = la + cur * 32 * kStepBK + lhi * 32 + l32;
      const float* b = lb + cur * kStepBK * kStepPitchB + lhi * kStepPitchB + l32;
#pragma unroll
      for (int s = 0; s < kStepBK / 2; ++s)
        acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a[2 * s * 32], b[2 * s * kStepPitchB], acc, 0, 0, 0);
      if (st + 1 < nst) {
        STEP_STORE(cur ^ 1)
        if (st + 2 < nst) { STEP_LOAD(st + 2) }
      }
      step_wave_sync();  // the stages are private to the wave: no block barrier in the loop
    }
  }
  __syncthreads();
#undef STEP_LOAD1
#undef STEP_LOAD
#undef STEP_STORE1
#undef STEP_STORE

  // the four quarter sums meet in LDS (the stages are dead after the last barrier)
  float* red = lds;
#pragma unroll
  for (int r = 0; r < 16; ++r) {
    const unsigned row = 8 * (r / 4) + 4 * lhi + (r % 4);
    red[(wave * 32 + row) * kStepPitchR + l32] = acc[r];
  }
  __syncthreads();

  if (ecol >= B) return;
  const size_t g0 = size_t(ecol) * 4 * H + ej, s0 = size_t(ecol) * H + ej;
#pragma unroll
  for (int q = 0; q < 4; ++q) {
#pragma unroll
    for (int w = 0; w < 4; ++w) pre[q] += red[(w * 32 + q * 8 + eu) * kStepPitchR + ecc];
  }
  const float gi = logistic(mode, pre[0]), gf = logistic(mode, pre[1]), go = logistic(mode, pre[2]);
  const float gg = tanh_accurate(pre[3]);
  const float cv = c_prev != nullptr ? gi * gg + gf * cp : gi * gg;
  gates[g0] = gi;
  gates[g0 + H] = gf;
  gates[g0 + 2 * size_t(H)] = go;
  gates[g0 + 3 * size_t(H)] = gg;
  c[s0] = cv;
  h[s0] = go * tanh_accurate(cv);
}

static bool all_aligned16(std::initializer_list<const void*> ps) {
  for (const void* p : ps)
    if (p != nullptr && !aligned16(p)) return false;
  return true;
}

struct GatesInputs {
  unsigned I;
  bool dropout;
};

static int check_gates(unsigned num_inputs, const float* const* xs, const unsigned* x_dims, unsigned H, unsigned B,
                       const float* mask_x, unsigned mask_x_bd, const float* mask_h, unsigned mask_h_bd,
                       GatesInputs* out) {
  DYHIP_REQUIRE(num_inputs >= 1 && xs != nullptr && x_dims != nullptr, "Failed input count check in VanillaLSTMGates");
  DYHIP_REQUIRE(H >= 1 && B >= 1, "VanillaLSTMGates: bad hidden (%u) or batch (%u) size", H, B);
  unsigned I = 0;
  for (unsigned k = 0; k < num_inputs; ++k) {
    DYHIP_REQUIRE(xs[k] != nullptr && x_dims[k] >= 1, "VanillaLSTMGates: x_t[%u] expected to be a vector", k);
    I += x_dims[k];
  }
  DYHIP_REQUIRE((mask_x == nullptr) == (mask_h == nullptr), "VanillaLSTMGates: both dropout masks or none");
  out->dropout = mask_x != nullptr;
  if (out->dropout) {
    DYHIP_REQUIRE(mask_x_bd == B || mask_x_bd == 1,
                  "VanillaLSTMGates: dropout_mask_x expected to have batch size 1 or %u, was %u", B, mask_x_bd);
    DYHIP_REQUIRE(mask_h_bd == B || mask_h_bd == 1,
                  "VanillaLSTMGates: dropout_mask_h expected to have batch size 1 or %u, was %u", B, mask_h_bd);
  }
  out->I = I;
  return DYHIP_OK;
}

// Builds the effective x_t (concatenated and/or masked) in `buf` when needed;
// returns the pointer the GEMM should read.
static int prepare_x(dyhip_device* dev, unsigned num_inputs, const float* const* xs, const unsigned* x_dims,
                     unsigned I, unsigned B, const float* mask_x, unsigned mask_x_bd, float* buf,
                     const float** x_eff) {
  if (num_inputs == 1 && mask_x == nullptr) {
    *x_eff = xs[0];
    return DYHIP_OK;
  }
  unsigned off = 0;
  for (unsigned k = 0; k < num_inputs; ++k) {
    hipLaunchKernelGGL(rows_copy_mask_kernel, dim3(cdiv<unsigned>(x_dims[k], 256), grid_y(B)), dim3(256), 0, dev->stream,
                       x_dims[k], I, off, xs[k], mask_x, mask_x_bd > 1 ? 1 : 0, buf, B);
    off += x_dims[k];
  }
  DYHIP_CHECK_LAUNCH();
  *x_eff = buf;
  return DYHIP_OK;
}

static int prepare_h(dyhip_device* dev, unsigned H, unsigned B, const float* h, const float* mask_h,
                     unsigned mask_h_bd, float* buf, const float** h_eff) {
  if (mask_h == nullptr) {
    *h_eff = h;
    return DYHIP_OK;
  }
  hipLaunchKernelGGL(rows_copy_mask_kernel, dim3(cdiv<unsigned>(H, 256), grid_y(B)), dim3(256), 0, dev->stream, H, H, 0u,
                     h, mask_h, mask_h_bd > 1 ? 1 : 0, buf, B);
  DYHIP_CHECK_LAUNCH();
  *h_eff = buf;
  return DYHIP_OK;
}

}  // namespace dyhip

using namespace dyhip;

extern "C" {

int dyhip_lstm_gates_workspace(unsigned num_inputs, unsigned I, unsigned H, unsigned B, int dropout,
                               size_t* ws_bytes) {
  DYHIP_REQUIRE(ws_bytes != nullptr, "null output pointer");
  size_t n = 0;
  if (num_inputs > 1 || dropout) n += align256(sizeof(float) * size_t(I) * B);
  if (dropout) n += align256(sizeof(float) * size_t(H) * B);
  *ws_bytes = n;
  return DYHIP_OK;
}

int dyhip_lstm_gates_forward(dyhip_device* dev, unsigned num_inputs, const float* const* xs_host,
                             const unsigned* x_dims_host, unsigned H, unsigned B, const float* h_tm1,
                             const float* Wx, const float* Wh, const float* b, const float* mask_x,
                             unsigned mask_x_bd, const float* mask_h, unsigned mask_h_bd, int logistic_mode,
                             float* fx, void* ws, size_t ws_bytes) {
  DYHIP_CHECK_DEV(dev);
  GatesInputs gi;
  DYHIP_CHECK_STATUS(check_gates(num_inputs, xs_host, x_dims_host, H, B, mask_x, mask_x_bd, mask_h, mask_h_bd, &gi));
  DYHIP_REQUIRE(h_tm1 && Wx && Wh && b && fx, "VanillaLSTMGates: null tensor pointer");
  DYHIP_REQUIRE(logistic_mode == DYHIP_LOGISTIC_PACKET || logistic_mode == DYHIP_LOGISTIC_SCALAR,
                "unknown logistic mode %d", logistic_mode);
  size_t need = 0;
  DYHIP_CHECK_STATUS(dyhip_lstm_gates_workspace(num_inputs, gi.I, H, B, gi.dropout, &need));
  DYHIP_REQUIRE(need == 0 || (ws != nullptr && ws_bytes >= need), "VanillaLSTMGates needs %zu workspace bytes, got %zu",
                need, ws_bytes);
  char* wsp = static_cast<char*>(ws);
  float* xbuf = reinterpret_cast<float*>(wsp);
  float* hbuf = reinterpret_cast<float*>(wsp + ((num_inputs > 1 || gi.dropout) ? align256(sizeof(float) * size_t(gi.I) * B) : 0));
  const float *x_eff = nullptr, *h_eff = nullptr;
  DYHIP_CHECK_STATUS(prepare_x(dev, num_inputs, xs_host, x_dims_host, gi.I, B, mask_x, mask_x_bd, xbuf, &x_eff));
  DYHIP_CHECK_STATUS(prepare_h(dev, H, B, h_tm1, mask_h, mask_h_bd, hbuf, &h_eff));
  const size_t G = size_t(4) * H;
  GemmSeg segs[2] = {{Wx, G, x_eff, gi.I, gi.I}, {Wh, G, h_eff, H, H}};
  GemmEpiParams ep{kEpiLstmGates, 0.f, b, H, logistic_mode};
  return gemm_run(dev, false, true, G, B, 2, segs, fx, ep);
}

int dyhip_lstm_gates_dpre(dyhip_device* dev, unsigned H, unsigned B, const float* fx, const float* dEdf,
                          float* dpre) {
  DYHIP_CHECK_DEV(dev);
  DYHIP_REQUIRE(fx && dEdf && dpre, "null tensor pointer");
  if (H == 0 || B == 0) return DYHIP_OK;
  hipLaunchKernelGGL(lstm_dpre_kernel, dim3(cdiv<unsigned>(4 * H, 256), grid_y(B)), dim3(256), 0, dev->stream, H, fx, dEdf,
                     dpre, B);
  DYHIP_CHECK_LAUNCH();
  return DYHIP_OK;
}

int dyhip_lstm_gates_backward_workspace(unsigned num_inputs, unsigned I, unsigned H, unsigned B, int dropout,
                                        size_t* ws_bytes) {
  DYHIP_REQUIRE(ws_bytes != nullptr, "null output pointer");
  (void)num_inputs;
  (void)dropout;
  const unsigned big = I > H ? I : H;
  size_t red = 0;
  DYHIP_CHECK_STATUS(dyhip_batch_reduce_workspace(size_t(4) * H, B, &red));
  *ws_bytes = align256(sizeof(float) * size_t(4) * H * B) + align256(sizeof(float) * size_t(big) * B) + align256(red);
  return DYHIP_OK;
}

int dyhip_lstm_gates_backward(dyhip_device* dev, unsigned num_inputs, const float* const* xs_host,
                              const unsigned* x_dims_host, unsigned H, unsigned B, const float* h_tm1,
                              const float* Wx, const float* Wh, const float* mask_x, unsigned mask_x_bd,
                              const float* mask_h, unsigned mask_h_bd, const float* fx, const float* dEdf,
                              const float* dpre, unsigned i, float* dEdxi, void* ws, size_t ws_bytes) {
  DYHIP_CHECK_DEV(dev);
  GatesInputs gi;
  DYHIP_CHECK_STATUS(check_gates(num_inputs, xs_host, x_dims_host, H, B, mask_x, mask_x_bd, mask_h, mask_h_bd, &gi));
  DYHIP_REQUIRE(i <= num_inputs + 3, "VanillaLSTMGates has %u differentiable arguments (i = %u)", num_inputs + 4, i);
  DYHIP_REQUIRE(h_tm1 && Wx && Wh && fx && dEdf && dEdxi, "VanillaLSTMGates: null tensor pointer");
  size_t need = 0;
  DYHIP_CHECK_STATUS(dyhip_lstm_gates_backward_workspace(num_inputs, gi.I, H, B, gi.dropout, &need));
  DYHIP_REQUIRE(ws != nullptr && ws_bytes >= need, "VanillaLSTMGates backward needs %zu workspace bytes, got %zu", need,
                ws_bytes);
  const size_t G = size_t(4) * H;
  const unsigned big = gi.I > H ? gi.I : H;
  char* wsp = static_cast<char*>(ws);
  float* dpre_buf = reinterpret_cast<float*>(wsp);
  float* tmp = reinterpret_cast<float*>(wsp + align256(sizeof(float) * G * B));
  char* red_ws = wsp + align256(sizeof(float) * G * B) + align256(sizeof(float) * size_t(big) * B);
  const size_t red_bytes = ws_bytes - (red_ws - wsp);
  if (dpre == nullptr) {
    DYHIP_CHECK_STATUS(dyhip_lstm_gates_dpre(dev, H, B, fx, dEdf, dpre_buf));
    dpre = dpre_buf;
  }
  const GemmEpiParams acc{kEpiAxpby, 1.0f, nullptr, 0, 0}, ovw{kEpiAxpby, 0.0f, nullptr, 0, 0};
  if (i <= num_inputs) {
    // dx_i += Wx[:, slice]^T dpre   or   dh += Wh^T dpre
    unsigned off = 0, rows = H;
    const float* W = Wh;
    const float* mask = mask_h;
    unsigned mask_ld = H, mask_bd = mask_h_bd;
    if (i < num_inputs) {
      for (unsigned j = 0; j < i; ++j) off += x_dims_host[j];
      rows = x_dims_host[i];
      W = Wx + size_t(off) * G;
      mask = mask_x;
      mask_ld = gi.I;
      mask_bd = mask_x_bd;
    } else {
      off = 0;
    }
    GemmSeg s{W, G, dpre, G, G};
    if (!gi.dropout) return gemm_run(dev, true, true, rows, B, 1, &s, dEdxi, acc);
    DYHIP_CHECK_STATUS(gemm_run(dev, true, true, rows, B, 1, &s, tmp, ovw));
    hipLaunchKernelGGL(acc_mul_mask_kernel, dim3(cdiv<unsigned>(rows, 256), grid_y(B)), dim3(256), 0, dev->stream, rows,
                       mask_ld, off, tmp, mask, mask_bd > 1 ? 1 : 0, dEdxi, B);
    DYHIP_CHECK_LAUNCH();
    return DYHIP_OK;
  }
  if (i == num_inputs + 1) {  // dWx += dpre * x_t^T
    const float* x_eff = nullptr;
    DYHIP_CHECK_STATUS(prepare_x(dev, num_inputs, xs_host, x_dims_host, gi.I, B, mask_x, mask_x_bd, tmp, &x_eff));
    GemmSeg s{dpre, G, x_eff, gi.I, B};
    return gemm_run(dev, false, false, G, gi.I, 1, &s, dEdxi, acc);
  }
  if (i == num_inputs + 2) {  // dWh += dpre * h^T
    const float* h_eff = nullptr;
    DYHIP_CHECK_STATUS(prepare_h(dev, H, B, h_tm1, mask_h, mask_h_bd, tmp, &h_eff));
    GemmSeg s{dpre, G, h_eff, H, B};
    return gemm_run(dev, false, false, G, H, 1, &s, dEdxi, acc);
  }
  // db += sum_b dpre
  return batch_reduce(dev, G, B, dpre, nullptr, dEdxi, true, red_ws, red_bytes);
}

int dyhip_lstm_c_forward(dyhip_device* dev, unsigned H, unsigned B, const float* c_tm1, const float* gates, float* c) {
  DYHIP_CHECK_DEV(dev);
  DYHIP_REQUIRE(c_tm1 && gates && c, "VanillaLSTMC: null tensor pointer");
  return launch_pointwise<0>(dev, H, B, c_tm1, gates, nullptr, c);
}

int dyhip_lstm_c_backward(dyhip_device* dev, unsigned H, unsigned B, const float* c_tm1, const float* gates,
                          const float* dEdf, unsigned i, float* dEdxi) {
  DYHIP_CHECK_DEV(dev);
  DYHIP_REQUIRE(c_tm1 && gates && dEdf && dEdxi, "VanillaLSTMC: null tensor pointer");
  DYHIP_REQUIRE(i < 2, "VanillaLSTMC has two arguments (i = %u)", i);
  return i == 0 ? launch_pointwise<1>(dev, H, B, c_tm1, gates, dEdf, dEdxi)
                : launch_pointwise<2>(dev, H, B, c_tm1, gates, dEdf, dEdxi);
}

int dyhip_lstm_h_forward(dyhip_device* dev, unsigned H, unsigned B, const float* c, const float* gates, float* h) {
  DYHIP_CHECK_DEV(dev);
  DYHIP_REQUIRE(c && gates && h, "VanillaLSTMH: null tensor pointer");
  return launch_pointwise<3>(dev, H, B, c, gates, nullptr, h);
}

int dyhip_lstm_h_backward(dyhip_device* dev, unsigned H, unsigned B, const float* c, const float* gates,
                          const float* dEdf, unsigned i, float* dEdxi) {
  DYHIP_CHECK_DEV(dev);
  DYHIP_REQUIRE(c && gates && dEdf && dEdxi, "VanillaLSTMH: null tensor pointer");
  DYHIP_REQUIRE(i < 2, "VanillaLSTMH has two arguments (i = %u)", i);
  return i == 0 ? launch_pointwise<4>(dev, H, B, c, gates, dEdf, dEdxi)
                : launch_pointwise<5>(dev, H, B, c, gates, dEdf, dEdxi);
}

// ---- fused cell path ------------------------------------------------------------------
static int recurrent_partials(dyhip_device* dev, bool transposed, unsigned H, unsigned B, const float* Wh,
                              const float* v, void* ws, size_t ws_bytes, unsigned* splits) {
  DYHIP_REQUIRE(H >= 1 && B >= 1, "LSTM cell: bad hidden (%u) or batch (%u) size", H, B);
  DYHIP_REQUIRE(Wh && v && ws && splits, "LSTM cell: null pointer");
  const size_t G = size_t(4) * H;
  GemmEpiParams ep{};
  ep.kind = kEpiPartials;
  ep.partials = static_cast<float*>(ws);
  ep.partials_bytes = ws_bytes;
  ep.splits_out = splits;
  if (!transposed) {  // Wh[4H x H] * h[H x B]
    GemmSeg s{Wh, G, v, H, H};
    return gemm_run(dev, false, true, G, B, 1, &s, nullptr, ep);
  }
  GemmSeg s{Wh, G, v, G, G};  // Wh^T * dpre[4H x B]
  return gemm_run(dev, true, true, H, B, 1, &s, nullptr, ep);
}

int dyhip_lstm_cell_workspace(dyhip_device* dev, unsigned H, unsigned B, size_t* fwd_bytes, size_t* bwd_bytes) {
  DYHIP_CHECK_DEV(dev);
  DYHIP_REQUIRE(fwd_bytes && bwd_bytes, "null output pointer");
  // room for the largest split count the GEMM planner considers
  *fwd_bytes = align256(sizeof(float) * size_t(4) * H * B) * 32;
  *bwd_bytes = align256(sizeof(float) * size_t(H) * B) * 32;
  return DYHIP_OK;
}

int dyhip_lstm_recurrent_forward(dyhip_device* dev, unsigned H, unsigned B, const float* Wh, const float* h_tm1,
                                 void* ws, size_t ws_bytes, unsigned* splits) {
  DYHIP_CHECK_DEV(dev);
  return recurrent_partials(dev, false, H, B, Wh, h_tm1, ws, ws_bytes, splits);
}

int dyhip_lstm_recurrent_backward(dyhip_device* dev, unsigned H, unsigned B, const float* Wh, const float* dpre,
                                  void* ws, size_t ws_bytes, unsigned* splits) {
  DYHIP_CHECK_DEV(dev);
  return recurrent_partials(dev, true, H, B, Wh, dpre, ws, ws_bytes, splits);
}

int dyhip_lstm_cell_forward(dyhip_device* dev, unsigned H, unsigned B, const float* xproj, const float* b,
                            const float* rec, unsigned splits, const float* c_tm1, int logistic_mode, float* gates,
                            float* c, float* h) {
  DYHIP_CHECK_DEV(dev);
  DYHIP_REQUIRE(H >= 1 && B >= 1, "LSTM cell: bad hidden (%u) or batch (%u) size", H, B);
  DYHIP_REQUIRE(xproj && b && gates && c && h, "LSTM cell: null tensor pointer");
  DYHIP_REQUIRE(splits == 0 || rec != nullptr, "LSTM cell: %u recurrent slices but no buffer", splits);
  DYHIP_REQUIRE(logistic_mode == DYHIP_LOGISTIC_PACKET || logistic_mode == DYHIP_LOGISTIC_SCALAR,
                "unknown logistic mode %d", logistic_mode);
  const size_t slice = size_t(4) * H * B;
  const bool vec = H % 4 == 0 && all_aligned16({xproj, b, rec, c_tm1, gates, c, h});
  for (unsigned b0 = 0; b0 < B; b0 += 65535u) {  // the grid's second dimension holds at most 65535 blocks
    const unsigned nb = B - b0 < 65535u ? B - b0 : 65535u;
    if (vec)
      hipLaunchKernelGGL(lstm_cell_fwd_kernel<4>, dim3(cdiv<unsigned>(H, kCellThreads * 4), nb), dim3(kCellThreads), 0,
                         dev->stream, H, splits, slice, xproj, rec, b, c_tm1, logistic_mode, gates, c, h, b0);
    else
      hipLaunchKernelGGL(lstm_cell_fwd_kernel<1>, dim3(cdiv<unsigned>(H, kCellThreads), nb), dim3(kCellThreads), 0,
                         dev->stream, H, splits, slice, xproj, rec, b, c_tm1, logistic_mode, gates, c, h, b0);
  }
  DYHIP_CHECK_LAUNCH();
  return DYHIP_OK;
}

int dyhip_lstm_cell_backward(dyhip_device* dev, unsigned H, unsigned B, const float* gates, const float* c,
                             const float* c_tm1, const float* dh, const float* rec, unsigned splits, const float* dc,
                             float* dpre, float* dc_tm1) {
  DYHIP_CHECK_DEV(dev);
  DYHIP_REQUIRE(H >= 1 && B >= 1, "LSTM cell: bad hidden (%u) or batch (%u) size", H, B);
  DYHIP_REQUIRE(gates && c && dh && dpre, "LSTM cell: null tensor pointer");
  DYHIP_REQUIRE(splits == 0 || rec != nullptr, "LSTM cell: %u recurrent slices but no buffer", splits);
  const size_t slice = size_t(H) * B;
  const bool vec = H % 4 == 0 && all_aligned16({gates, c, c_tm1, dh, rec, dc, dpre, dc_tm1});
  for (unsigned b0 = 0; b0 < B; b0 += 65535u) {
    const unsigned nb = B - b0 < 65535u ? B - b0 : 65535u;
    if (vec)
      hipLaunchKernelGGL(lstm_cell_bwd_kernel<4>, dim3(cdiv<unsigned>(H, kCellThreads * 4), nb), dim3(kCellThreads), 0,
                         dev->stream, H, splits, slice, gates, c, c_tm1, dh, rec, dc, dpre, dc_tm1, b0);
    else
      hipLaunchKernelGGL(lstm_cell_bwd_kernel<1>, dim3(cdiv<unsigned>(H, kCellThreads), nb), dim3(kCellThreads), 0,
                         dev->stream, H, splits, slice, gates, c, c_tm1, dh, rec, dc, dpre, dc_tm1, b0);
  }
  DYHIP_CHECK_LAUNCH();
  return DYHIP_OK;
}

static bool step_depth_ok(unsigned K) { return K >= 128 && K % 128 == 0; }  // quarters in whole 32-deep stages

int dyhip_lstm_step_supported(dyhip_device* dev, unsigned H, unsigned B, int* supported) {
  DYHIP_CHECK_DEV(dev);
  DYHIP_REQUIRE(supported, "null output pointer");
  // grid and index ranges in 32 bits
  *supported = (step_depth_ok(H) && B >= 1 && B <= 65535 && size_t(4) * H * H < (size_t(1) << 32)) ? 1 : 0;
  return DYHIP_OK;
}

static int pack_weights(dyhip_device* dev, unsigned H, unsigned K, const float* W, float* packed) {
  DYHIP_REQUIRE(step_depth_ok(H) && step_depth_ok(K) && size_t(4) * H * K < (size_t(1) << 32),
                "LSTM step: hidden size %u and product depth %u must be multiples of 128", H, K);
  DYHIP_REQUIRE(W && packed, "LSTM step: null tensor pointer");
  const size_t n = size_t(4) * H * K;
  hipLaunchKernelGGL(lstm_pack_recurrent_kernel, dim3(unsigned(cdiv<size_t>(n, 256))), dim3(256), 0, dev->stream, H, K, W,
                     packed);
  DYHIP_CHECK_LAUNCH();
  return DYHIP_OK;
}

int dyhip_lstm_pack_recurrent(dyhip_device* dev, unsigned H, const float* Wh, float* packed) {
  DYHIP_CHECK_DEV(dev);
  return pack_weights(dev, H, H, Wh, packed);
}

int dyhip_lstm_pack_input(dyhip_device* dev, unsigned I, unsigned H, const float* Wx, float* packed) {
  DYHIP_CHECK_DEV(dev);
  return pack_weights(dev, H, I, Wx, packed);
}

static int step_forward(dyhip_device* dev, unsigned I, unsigned H, unsigned B, const float* packed_Wx, const float* x,
                        const float* packed_Wh, const float* h_tm1, const float* xproj, const float* b,
                        const float* c_tm1, int logistic_mode, float* gates, float* c, float* h) {
  int ok = 0;
  dyhip_lstm_step_supported(dev, H, B, &ok);
  DYHIP_REQUIRE(ok, "LSTM step: unsupported hidden (%u) or batch (%u) size", H, B);
  DYHIP_REQUIRE(b && gates && c && h, "LSTM step: null tensor pointer");
  DYHIP_REQUIRE((packed_Wx == nullptr) == (x == nullptr) && (packed_Wh == nullptr) == (h_tm1 == nullptr),
                "LSTM step: packed weights and their operand come together");
  DYHIP_REQUIRE(packed_Wx == nullptr || step_depth_ok(I), "LSTM step: input size %u is not a multiple of 128", I);
  DYHIP_REQUIRE(all_aligned16({packed_Wx, x, packed_Wh, h_tm1}), "LSTM step: weights and operands must be 16-byte aligned");
  DYHIP_REQUIRE(logistic_mode == DYHIP_LOGISTIC_PACKET || logistic_mode == DYHIP_LOGISTIC_SCALAR,
                "unknown logistic mode %d", logistic_mode);
  const StepOperand op0{packed_Wx, x, I}, op1{packed_Wh, h_tm1, H};
  const unsigned blocks = (H / 8) * cdiv<unsigned>(B, 32);
  hipLaunchKernelGGL(lstm_step_fwd_kernel, dim3(blocks), dim3(256), 0, dev->stream, H, B, op0, op1, xproj, b, c_tm1,
                     logistic_mode, gates, c, h);
  DYHIP_CHECK_LAUNCH();
  return DYHIP_OK;
}

int dyhip_lstm_step_forward(dyhip_device* dev, unsigned H, unsigned B, const float* packed_Wh, const float* h_tm1,
                            const float* xproj, const float* b, const float* c_tm1, int logistic_mode, float* gates,
                            float* c, float* h) {
  DYHIP_CHECK_DEV(dev);
  DYHIP_REQUIRE(packed_Wh && h_tm1 && xproj && c_tm1, "LSTM step: null tensor pointer");
  return step_forward(dev, 0, H, B, nullptr, nullptr, packed_Wh, h_tm1, xproj, b, c_tm1, logistic_mode, gates, c, h);
}

int dyhip_lstm_step_forward_x(dyhip_device* dev, unsigned I, unsigned H, unsigned B, const float* packed_Wx,
                              const float* x, const float* packed_Wh, const float* h_tm1, const float* b,
                              const float* c_tm1, int logistic_mode, float* gates, float* c, float* h) {
  DYHIP_CHECK_DEV(dev);
  DYHIP_REQUIRE(packed_Wx && x, "LSTM step: null tensor pointer");
  return step_forward(dev, I, H, B, packed_Wx, x, packed_Wh, h_tm1, nullptr, b, c_tm1, logistic_mode, gates, c, h);
}

}  // extern "C"
