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
  // four slices at a time, all their loads in flight (a slice past the end repeats the last one and is not added)
  for (unsigned k0 = 0; k0 < splits; k0 += 4) {
    Pack<V> r[4][4];
#pragma unroll
    for (int u = 0; u < 4; ++u)
#pragma unroll
      for (int q = 0; q < 4; ++q) r[u][q].load(rec + size_t(min(k0 + u, splits - 1)) * slice + g0 + size_t(q) * H);
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      if (k0 + u < splits) {
#pragma unroll
        for (int q = 0; q < 4; ++q)
#pragma unroll
          for (int e = 0; e < V; ++e) pre[q].v[e] += r[u][q].v[e];
      }
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
                                                                     float* dc_prev, unsigned b_first,
                                                                     float* __restrict__ dpre_packed) {
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
  for (unsigned k0 = 0; k0 < splits; k0 += 4) {  // four slices in flight, added in ascending order
    Pack<V> r[4];
#pragma unroll
    for (int u = 0; u < 4; ++u) r[u].load(rec + size_t(min(k0 + u, splits - 1)) * slice + s0);
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      if (k0 + u < splits) {
#pragma unroll
        for (int e = 0; e < V; ++e) dh.v[e] += r[u].v[e];
      }
    }
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
  // dpre again in the fragment order of the next recurrent product (depth 4H): see lstm_pack_state_kernel
  if (dpre_packed != nullptr) {
    const size_t tile = size_t(b / 32) * (H / 2) * 256 + (b % 32) * 4;  // column tile of 4H/8 groups of 256 floats
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      const unsigned k = q * H + j;  // k .. k+V-1 are the slots of one lane: k = 8*kg + 4*lhi + s
      out[q].store(dpre_packed + tile + size_t(k / 8) * 256 + ((k % 8) / 4) * 128 + k % 4);
    }
  }
}

// ---- single-launch forward step: recurrent product and cell update in one kernel -------
// A block owns 16 hidden units x 32 batch columns.  Its 64 weight rows are the four gate rows
// (i, f, o, g) of those units, so after the product all four pre-activations of a hidden unit
// sit in the same block and the cell update runs in the epilogue: the 4H x B product never goes
// to memory.  The four waves split the depth of the sum in quarters and meet in LDS; each wave
// multiplies two 32-row tiles by one 32-column tile, so a fragment of the state feeds two MFMAs.
//
// The kernel is bound by the MFMA issue of its one wavefront per SIMD (256 MFMAs per wave at H = 1024);
// the tile is the one with the fewest operand bytes per block that still gives every CU a block at
// H = 1024, B = 128, (64 + 32) rows and columns of depth H.  Blocks b and b + 8k run on the same XCD,
// so the column tiles of one row pair share its L2 and the weights arrive from beyond it once per
// launch, not once per block.  Both operands are read in MFMA fragment order straight into
// registers (no LDS stage, no barrier in the loop): for a 32-wide tile and a group of 8 consecutive
// k, lane l = 32*lhi + l32 holds k = 8*kg + 4*lhi + s, s = 0..3, of row (or column) l32 as one
// float4 (MFMA step s of the group multiplies k = 8*kg + s and 8*kg + 4 + s; the order inside a
// group is free as long as both operands agree), and a group of a tile is 1 KiB contiguous.
//   weights  Wp[rows/32][K/8][64][4]   forward: row g*H + rt*8 + u of W at l32 = g*8 + u of tile rt;
//                                      backward: row rt*32 + l32 of W^T (dyhip_lstm_pack_*)
//   state    vp[ceil(B/32)][K/8][64][4]   column ct*32 + l32 (dyhip_lstm_pack_state, or the packed h /
//            dpre the step kernels write for the next timestep); columns past B hold zeros or stale
//            values and only feed output columns that are dropped
// Blocks that share weight rows are a multiple of 8 apart in launch order, so they land on the same
// XCD and share that L2's copy of the rows.
constexpr int kStepPitchR = 33;  // partial-sum exchange: [row][col]
typedef float stepx16 __attribute__((ext_vector_type(16)));

// W is 4H x K column-major (Wh: K = H, Wx: K = the input size): gate-interleaved row tiles.  A block packs the
// tiles rt0 .. rt0 + 7 of one group of 8 k: for a gate and a k their 64 units are one 256-byte run of W, which goes
// through LDS ([gate][k][unit]) into the eight 1 KiB fragment groups (H is a multiple of 64).
__global__ __launch_bounds__(256) void lstm_pack_weights_kernel(unsigned H, unsigned K, const float* __restrict__ W,
                                                                float* __restrict__ Wp) {
  __shared__ float tile[4 * 8 * 65];
  const unsigned kg = blockIdx.x % (K / 8), rt0 = (blockIdx.x / (K / 8)) * 8;
  const unsigned t = threadIdx.x;
#pragma unroll
  for (int pass = 0; pass < 8; ++pass) {
    const unsigned pair = pass * 4 + t / 64, g = pair / 8, k = pair % 8, unit = t % 64;
    tile[(g * 8 + k) * 65 + unit] = W[size_t(g) * H + rt0 * 8 + unit + size_t(8 * kg + k) * 4 * H];
  }
  __syncthreads();
#pragma unroll
  for (int j = 0; j < 2; ++j) {
    const unsigned q = j * 256 + t, r = q / 64, lane = q % 64, l32 = lane % 32, lhi = lane / 32;
    const unsigned g = l32 / 8, unit = r * 8 + l32 % 8;
    float4 v;
    v.x = tile[(g * 8 + 4 * lhi + 0) * 65 + unit];
    v.y = tile[(g * 8 + 4 * lhi + 1) * 65 + unit];
    v.z = tile[(g * 8 + 4 * lhi + 2) * 65 + unit];
    v.w = tile[(g * 8 + 4 * lhi + 3) * 65 + unit];
    float* dst = Wp + ((size_t(rt0 + r) * (K / 8) + kg) * 64 + lane) * 4;  // packed buffers are 16-byte aligned or not:
    dst[0] = v.x; dst[1] = v.y; dst[2] = v.z; dst[3] = v.w;              // four stores the compiler may merge
  }
}

// Wh is 4H x H column-major; the packed matrix is Wh^T (H rows, depth 4H) in plain 32-row tiles
__global__ __launch_bounds__(256) void lstm_pack_transposed_kernel(unsigned H, const float* __restrict__ W,
                                                                   float* __restrict__ Wp) {
  const size_t o = size_t(blockIdx.x) * 256 + threadIdx.x;  // ((rt*(4H/8) + kg)*64 + lane)*4 + s
  if (o >= size_t(4) * H * H) return;
  const unsigned s = o % 4, lane = (o / 4) % 64, l32 = lane % 32, lhi = lane / 32;
  const size_t tg = o / 256;
  const unsigned kg = tg % (H / 2), rt = tg / (H / 2);
  Wp[o] = W[size_t(rt * 32 + l32) * 4 * H + 8 * kg + 4 * lhi + s];
}

// v is K x B column-major
__global__ __launch_bounds__(256) void lstm_pack_state_kernel(unsigned K, unsigned B, const float* __restrict__ v,
                                                              float* __restrict__ vp) {
  const size_t o = size_t(blockIdx.x) * 256 + threadIdx.x;  // ((ct*(K/8) + kg)*64 + lane)*4 + s
  if (o >= size_t(K) * cdiv<unsigned>(B, 32) * 32) return;
  const unsigned s = o % 4, lane = (o / 4) % 64, l32 = lane % 32, lhi = lane / 32;
  const size_t tg = o / 256;
  const unsigned kg = tg % (K / 8), ct = tg / (K / 8);
  const unsigned col = ct * 32 + l32, k = 8 * kg + 4 * lhi + s;
  vp[o] = col < B ? v[size_t(col) * K + k] : 0.f;
}

// acc0 / acc1 += (two 32-row tiles of packed weights) x (one 32-column tile of packed state) over `groups`
// groups of 8 k (a multiple of 4), starting at the group the pointers name.  Eight groups at a time run as a
// branch-free double buffer: four groups are multiplied while the next four are in flight (the last round
// re-reads its own groups instead of branching around the loads, so the compiler counts the outstanding
// loads exactly; the scheduling barriers keep it from sinking the loads down to their uses).
// Every pointer names this lane's fragment of the first group; the next group is 256 floats on for a packed
// operand and 8 floats on for a plain one (PLAIN_A / PLAIN_B): a matrix stored with k contiguous per row (or
// column) needs no packing, its fragment is the 128-bit load of four consecutive k at row l32, offset 4 * lhi
// (32 segments of 32 bytes per wave and load where the packed form has 1 KiB contiguous).
// A_MODE 2 is a matrix stored with the ROW index contiguous (leading dimension lda between consecutive k, e.g.
// DyNet's 4H x K weights as they lie): the four k of a fragment are four 32-bit loads, each one 128-byte run
// over the 32 rows of the tile; pa then points at row l32 of k = first k + 4 * lhi.
// TILES = 1 leaves the second row tile out (pa1 and acc1 unused): small problems get twice the blocks.
enum { kFragPacked = 0, kFragAlongK = 1, kFragAlongRows = 2 };
// B_BYTES = 8: a plain B whose columns start on 8-byte boundaries only (an odd multiple of two floats apart): its
// fragment is two 64-bit loads.
template <int B_BYTES>
__device__ __forceinline__ float4 step_load_b(const float* p) {
  if (B_BYTES == 16) return *reinterpret_cast<const float4*>(p);
  const float2 lo = *reinterpret_cast<const float2*>(p), hi = *reinterpret_cast<const float2*>(p + 2);
  return make_float4(lo.x, lo.y, hi.x, hi.y);
}

template <int A_MODE, bool PLAIN_B, int TILES = 2, int B_BYTES = 16>
__device__ __forceinline__ void step_product(stepx16& acc0, stepx16& acc1, const float* __restrict__ pa0,
                                             const float* __restrict__ pa1, const float* __restrict__ pb,
                                             unsigned groups, size_t lda = 0) {
  constexpr size_t SA = A_MODE == kFragAlongK ? 8 : 256, SB = PLAIN_B ? 8 : 256;
  float4 a0[4], a1[4], b0[4], c0[4], c1[4], d0[4];
#define STEP_LOAD_A(dst, p, g_)                                                                      \
  if (A_MODE == kFragAlongRows) {                                                                    \
    const float* q_ = p + size_t(g_) * 8 * lda;                                                      \
    dst = make_float4(q_[0], q_[lda], q_[2 * lda], q_[3 * lda]);                                     \
  } else {                                                                                           \
    dst = *reinterpret_cast<const float4*>(p + size_t(g_) * SA);                                     \
  }
#define STEP_LOAD(A0, A1, BB, grp)                                                                   \
  _Pragma("unroll") for (int u = 0; u < 4; ++u) {                                                    \
    STEP_LOAD_A(A0[u], pa0, (grp) + u)                                                               \
    if (TILES == 2) { STEP_LOAD_A(A1[u], pa1, (grp) + u) }                                           \
    BB[u] = step_load_b<B_BYTES>(pb + size_t((grp) + u) * SB);                                       \
  }                                                                                                  \
  __builtin_amdgcn_sched_barrier(0);
#define STEP_MMA1(x, y, acc) acc = __builtin_amdgcn_mfma_f32_32x32x2f32(x, y, acc, 0, 0, 0);
#define STEP_MMA(A0, A1, BB)                       \
  _Pragma("unroll") for (int u = 0; u < 4; ++u) {  \
    STEP_MMA1(A0[u].x, BB[u].x, acc0)              \
    if (TILES == 2) STEP_MMA1(A1[u].x, BB[u].x, acc1) \
    STEP_MMA1(A0[u].y, BB[u].y, acc0)              \
    if (TILES == 2) STEP_MMA1(A1[u].y, BB[u].y, acc1) \
    STEP_MMA1(A0[u].z, BB[u].z, acc0)              \
    if (TILES == 2) STEP_MMA1(A1[u].z, BB[u].z, acc1) \
    STEP_MMA1(A0[u].w, BB[u].w, acc0)              \
    if (TILES == 2) STEP_MMA1(A1[u].w, BB[u].w, acc1) \
  }                                                \
  __builtin_amdgcn_sched_barrier(0);
  const unsigned full = groups / 8 * 8;
  if (full > 0) {
    STEP_LOAD(a0, a1, b0, 0u)
    for (unsigned g = 0; g < full; g += 8) {
      const unsigned nx = g + 8 < full ? g + 8 : g;  // the last round's prefetch lands on its own groups
      STEP_LOAD(c0, c1, d0, g + 4)
      STEP_MMA(a0, a1, b0)
      STEP_LOAD(a0, a1, b0, nx)
      STEP_MMA(c0, c1, d0)
    }
  }
  if (full < groups) {
    STEP_LOAD(a0, a1, b0, full)
    STEP_MMA(a0, a1, b0)
  }
#undef STEP_LOAD_A
#undef STEP_LOAD
#undef STEP_MMA1
#undef STEP_MMA
}

// Up to two products feed the pre-activations: Wx * x (depth I) and Wh * h_tm1 (depth H), both operands
// packed; either product may be absent (null), and Wx * x may instead arrive precomputed in xproj.
struct StepOperand {
  const float* Wp;
  const float* vp;
  unsigned K;
};

// Waves 0..3 form the product.  The cell update has one thread per (hidden unit, column) of the block, 32 * UB of
// them: with 64-row tiles that is eight waves, and the four that take no part in the product wait at the barrier
// (one wavefront per SIMD issues dependent VALU work at a fraction of the rate two can).
template <bool PLAIN, int TILES>
__global__ __launch_bounds__(256 * TILES) void lstm_step_fwd_kernel(unsigned H, unsigned B, StepOperand op0,
                                                                    StepOperand op1, const float* xproj,
                                                                    const float* __restrict__ bias,
                                                                    const float* __restrict__ c_prev, int mode,
                                                                    float* gates, float* __restrict__ c,
                                                                    float* __restrict__ h, float* __restrict__ hp,
                                                                    const float* __restrict__ mask_h) {
  constexpr int UB = 8 * TILES;       // hidden units of a block (its 32*TILES weight rows are their four gate rows)
  constexpr int ROWS = 32 * TILES;
  __shared__ float red[4 * ROWS * kStepPitchR];
  const unsigned RP = H / UB;
  const unsigned rp = blockIdx.x % RP, ct = blockIdx.x / RP;
  const unsigned wave = threadIdx.x / 64, lane = threadIdx.x % 64;
  const unsigned l32 = lane % 32, lhi = lane / 32;

  // The epilogue's thread owns hidden unit eu (of UB) of batch column col; its operands are fetched now so that
  // their latency hides behind the product, and kept as loaded: any arithmetic on them here would make the wave
  // wait for them before its first MFMA (1.3 us at H = 1024, B = 128).
  const unsigned eu = threadIdx.x % UB, col = threadIdx.x / UB, ej = rp * UB + eu;
  const unsigned ecol = ct * 32 + col, lcol = ecol < B ? ecol : B - 1;  // past the batch: clamped, dropped
  float bq[4], xq[4];
#pragma unroll
  for (int q = 0; q < 4; ++q) {
    bq[q] = bias[q * H + ej];
    xq[q] = xproj != nullptr ? xproj[size_t(lcol) * 4 * H + ej + size_t(q) * H] : 0.f;
  }
  const float cp = c_prev != nullptr ? c_prev[size_t(lcol) * H + ej] : 0.f;
  // the recurrent dropout mask of the sequence (H x B): the next timestep multiplies Wh by h (.) mask_h, so the packed
  // copy of h that it reads is written masked; the plain h (the layer's output) is not
  const float mh = mask_h != nullptr ? mask_h[size_t(lcol) * H + ej] : 1.f;

  if (wave < 4) {
    stepx16 acc0 = {0}, acc1 = {0};
    for (int which = 0; which < 2; ++which) {
      const StepOperand op = which == 0 ? op0 : op1;
      if (op.Wp == nullptr) continue;  // uniform over the grid
      const unsigned G = op.K / 8, gq = G / 4, g0 = wave * gq;
      const float* pa = op.Wp + ((size_t(TILES * rp) * G + g0) * 64 + lane) * 4;
      // plain state: columns past the batch are computed on a clamped address and dropped
      const unsigned pcol = ct * 32 + l32 < B ? ct * 32 + l32 : B - 1;
      const float* pb = PLAIN ? op.vp + size_t(pcol) * op.K + size_t(g0) * 8 + 4 * lhi : op.vp + ((size_t(ct) * G + g0) * 64 + lane) * 4;
      step_product<kFragPacked, PLAIN, TILES>(acc0, acc1, pa, pa + size_t(G) * 256, pb, gq);
    }
    // the four quarter sums meet in LDS: rows 0..31 = first tile, 32..63 = second
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      const unsigned row = 8 * (r / 4) + 4 * lhi + (r % 4);
      red[(wave * ROWS + row) * kStepPitchR + l32] = acc0[r];
      if (TILES == 2) red[(wave * ROWS + 32 + row) * kStepPitchR + l32] = acc1[r];
    }
  }
  __syncthreads();
  if (ecol >= B) return;

  const unsigned tile = eu / 8, u = eu % 8;
  float pre[4];
#pragma unroll
  for (int q = 0; q < 4; ++q) {
    pre[q] = (q == 1 ? bq[q] + 1.0f : bq[q]) + xq[q];
#pragma unroll
    for (int w = 0; w < 4; ++w) pre[q] += red[(w * ROWS + tile * 32 + q * 8 + u) * kStepPitchR + col];
  }
  const float gi = logistic(mode, pre[0]), gf = logistic(mode, pre[1]), go = logistic(mode, pre[2]);
  const float gg = tanh_accurate(pre[3]);
  const float cv = c_prev != nullptr ? gi * gg + gf * cp : gi * gg;
  const float hv = go * tanh_accurate(cv);
  const size_t g0 = size_t(ecol) * 4 * H + ej, s0 = size_t(ecol) * H + ej;
  gates[g0] = gi;
  gates[g0 + H] = gf;
  gates[g0 + 2 * size_t(H)] = go;
  gates[g0 + 3 * size_t(H)] = gg;
  c[s0] = cv;
  h[s0] = hv;
  // h again, as the next timestep's packed operand: unit ej is k = 8*(TILES*rp + tile) + u
  if (hp != nullptr) hp[((size_t(ct) * (H / 8) + TILES * rp + tile) * 64 + (u / 4) * 32 + col) * 4 + u % 4] = hv * mh;
}

// ---- single-launch backward step: recurrent product Wh^T * dpre_{t+1} and the cell backward of step t -----------
// The mirror of lstm_step_fwd_kernel.  The output of the product is H x B with a 4H-deep sum, so a block that is to
// run the cell backward in its epilogue must keep the whole depth: it owns 16 hidden units x 32 batch columns (256
// blocks at H = 1024, B = 128) and uses v_mfma_f32_16x16x4_f32, one 16-row tile times two 16-column tiles per wave,
// the four waves splitting the depth in quarters.  Operands in the fragment order of that MFMA: for a 16-wide tile and
// a group of 16 consecutive k, lane 16*lq + l16 holds k = 16*kg + 4*lq + s, s = 0..3, of row (or column) l16 as one
// float4 (step s of the group multiplies k = 16*kg + 4*lq + s over lq = 0..3; the order inside a group is free as long
// as both operands agree); a group of a tile is 1 KiB contiguous.
//   weights  Wp[H/16][4H/16][64][4]          row rt*16 + l16 of Wh^T (dyhip_lstm_pack_recurrent_transposed16)
//   dpre     vp[2*ceil(B/32)][4H/16][64][4]  column ct*16 + l16 (written by the previous launch of this kernel)
// The epilogue has one thread per (unit, column): it adds the four quarter sums to dh, applies the formulas of
// lstm_cell_bwd_kernel and writes dpre of this step plain (for the weight-gradient products over all timesteps) and in
// fragment order (for the next launch), and dc_tm1.  Per block the product reads (16 + 32) x 4H floats, twice the
// forward kernel's bytes per flop: 12.5 us for the bare product against 11.4 us forward, but one launch instead of
// two and no slices through memory.
// One 128-bit group per thread: the four k of a lane's fragment are consecutive in Wh's column as well.  When the
// operands are not 16-byte aligned the group is moved float by float.
__global__ void lstm_pack_transposed16_kernel(unsigned H, const float* __restrict__ W, float* __restrict__ Wp, int vec) {
  const size_t o4 = size_t(blockIdx.x) * 256 + threadIdx.x;  // (rt*(4H/16) + kg)*64 + lane
  if (o4 >= size_t(H) * H) return;
  const unsigned lane = o4 % 64, l16 = lane % 16, lq = lane / 16;
  const size_t tg = o4 / 64;
  const unsigned G = H / 4, kg = tg % G, rt = tg / G;
  const unsigned unit = rt * 16 + l16, k = 16 * kg + 4 * lq;
  const float* src = W + k + size_t(unit) * 4 * H;  // Wh is 4H x H, column-major: Wh^T(unit, k) = Wh(k, unit)
  if (vec) {
    reinterpret_cast<float4*>(Wp)[o4] = *reinterpret_cast<const float4*>(src);
  } else {
#pragma unroll
    for (int q = 0; q < 4; ++q) Wp[o4 * 4 + q] = src[q];
  }
}

__global__ void lstm_pack_state16_kernel(unsigned K, unsigned B, const float* __restrict__ v, float* __restrict__ vp) {
  const size_t o = size_t(blockIdx.x) * 256 + threadIdx.x;  // ((ct*(K/16) + kg)*64 + lane)*4 + s
  const size_t total = size_t(2) * cdiv<unsigned>(B, 32) * K * 16;
  if (o >= total) return;
  const unsigned s = o % 4, lane = (o / 4) % 64, l16 = lane % 16, lq = lane / 16;
  const size_t tg = o / 256;
  const unsigned kg = tg % (K / 16), ct = tg / (K / 16);
  const unsigned col = ct * 16 + l16, k = 16 * kg + 4 * lq + s;
  vp[o] = col < B ? v[size_t(col) * K + k] : 0.f;
}

typedef float stepx4 __attribute__((ext_vector_type(4)));

__global__ __launch_bounds__(512) void lstm_step_bwd_kernel(unsigned H, unsigned B, const float* __restrict__ WTp,
                                                            const float* __restrict__ dpre_next_p,
                                                            const float* __restrict__ gates,
                                                            const float* __restrict__ c,
                                                            const float* __restrict__ c_prev,
                                                            const float* __restrict__ dh_in, const float* dc_in,
                                                            float* __restrict__ dpre, float* dc_prev,
                                                            float* __restrict__ dpre_p,
                                                            const float* __restrict__ mask_h) {
  __shared__ float red[4 * 16 * kStepPitchR];
  const unsigned RT = H / 16;
  const unsigned rt = blockIdx.x % RT, ct = blockIdx.x / RT;  // ct: pair of 16-column tiles
  const unsigned wave = threadIdx.x / 64, lane = threadIdx.x % 64;

  // the epilogue's thread owns hidden unit eu of batch column col; its operands are fetched now and kept as loaded
  const unsigned eu = threadIdx.x % 16, col = threadIdx.x / 16, ej = rt * 16 + eu;
  const unsigned ecol = ct * 32 + col, lcol = ecol < B ? ecol : B - 1;  // past the batch: clamped, dropped
  const size_t g0 = size_t(lcol) * 4 * H + ej, s0 = size_t(lcol) * H + ej;
  float gt[4];
#pragma unroll
  for (int q = 0; q < 4; ++q) gt[q] = gates[g0 + size_t(q) * H];
  const float cv = c[s0], dhv = dh_in[s0];
  const float cpv = c_prev != nullptr ? c_prev[s0] : 0.f;
  const float dcv_in = dc_in != nullptr ? dc_in[s0] : 0.f;
  // recurrent dropout: timestep t+1 multiplied Wh by h_t (.) mask_h, so its gradient reaches h_t through the mask
  const float mh = mask_h != nullptr ? mask_h[s0] : 1.f;

  if (wave < 4 && dpre_next_p != nullptr) {
    const unsigned G = H / 4, gq = G / 4, g_first = wave * gq;  // groups of 16 k; a quarter of the depth per wave
    const float4* pa = reinterpret_cast<const float4*>(WTp) + (size_t(rt) * G + g_first) * 64 + lane;
    const float4* pb0 = reinterpret_cast<const float4*>(dpre_next_p) + (size_t(2 * ct) * G + g_first) * 64 + lane;
    const float4* pb1 = pb0 + size_t(G) * 64;
    stepx4 acc0 = {0.f, 0.f, 0.f, 0.f}, acc1 = {0.f, 0.f, 0.f, 0.f};
    float4 a[3][4], b0[3][4], b1[3][4];
#define BWD_LOAD(buf, grp)                                   \
  _Pragma("unroll") for (int u = 0; u < 4; ++u) {            \
    a[buf][u] = pa[size_t((grp) + u) * 64];                  \
    b0[buf][u] = pb0[size_t((grp) + u) * 64];                \
    b1[buf][u] = pb1[size_t((grp) + u) * 64];                \
  }                                                          \
  __builtin_amdgcn_sched_barrier(0);
#define BWD_MMA1(x, y, acc) acc = __builtin_amdgcn_mfma_f32_16x16x4f32(x, y, acc, 0, 0, 0);
#define BWD_MMA(buf)                                                                            \
  _Pragma("unroll") for (int u = 0; u < 4; ++u) {                                               \
    BWD_MMA1(a[buf][u].x, b0[buf][u].x, acc0) BWD_MMA1(a[buf][u].x, b1[buf][u].x, acc1)         \
    BWD_MMA1(a[buf][u].y, b0[buf][u].y, acc0) BWD_MMA1(a[buf][u].y, b1[buf][u].y, acc1)         \
    BWD_MMA1(a[buf][u].z, b0[buf][u].z, acc0) BWD_MMA1(a[buf][u].z, b1[buf][u].z, acc1)         \
    BWD_MMA1(a[buf][u].w, b0[buf][u].w, acc0) BWD_MMA1(a[buf][u].w, b1[buf][u].w, acc1)         \
  }                                                                                             \
  __builtin_amdgcn_sched_barrier(0);
    // Rounds of four groups through three register buffers: one is multiplied while the next two are in flight.  A
    // wave's 3 KiB per group against 8 MFMAs is twice the forward kernel's bytes per MFMA cycle, about what a CU gets
    // from its L2, so the bytes in flight, not the MFMAs, set the pace.  Loads past the quarter's end re-read its last
    // round (unconditional: the compiler counts what is in flight only in straight-line code).
    const unsigned last_round = gq - 4;
    BWD_LOAD(0, 0u)
    BWD_LOAD(1, min(4u, last_round))
    for (unsigned g = 0; g < gq; g += 12) {
      BWD_LOAD(2, min(g + 8, last_round))
      BWD_MMA(0)
      BWD_LOAD(0, min(g + 12, last_round))
      if (g + 4 < gq) { BWD_MMA(1) }
      BWD_LOAD(1, min(g + 16, last_round))
      if (g + 8 < gq) { BWD_MMA(2) }
    }
#undef BWD_LOAD
#undef BWD_MMA1
#undef BWD_MMA
    // D of the 16x16 MFMA: lane holds column lane%16, rows 4*(lane/16) + r
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const unsigned row = 4 * (lane / 16) + r;
      red[(wave * 16 + row) * kStepPitchR + lane % 16] = acc0[r];
      red[(wave * 16 + row) * kStepPitchR + 16 + lane % 16] = acc1[r];
    }
  }
  __syncthreads();
  if (ecol >= B) return;

  float dh = dhv;
  if (dpre_next_p != nullptr) {
    float rec = red[eu * kStepPitchR + col];
#pragma unroll
    for (int w = 1; w < 4; ++w) rec += red[(w * 16 + eu) * kStepPitchR + col];
    dh += mask_h != nullptr ? rec * mh : rec;
  }
  const float gi = gt[0], gf = gt[1], go = gt[2], gg = gt[3];
  const float t = tanh_accurate(cv);
  const float dcv = dcv_in + dh * go * (1.f - t * t);
  const float d_o = dh * t;
  const float d_i = dcv * gg, d_f = c_prev != nullptr ? dcv * cpv : 0.f, d_g = dcv * gi;
  float out[4];
  out[0] = d_i * gi * (1.f - gi);
  out[1] = d_f * gf * (1.f - gf);
  out[2] = d_o * go * (1.f - go);
  out[3] = d_g * (1.f - gg * gg);
#pragma unroll
  for (int q = 0; q < 4; ++q) dpre[g0 + size_t(q) * H] = out[q];
  if (dc_prev != nullptr) dc_prev[s0] = dcv * gf;
  if (dpre_p != nullptr) {
    // depth index of gate row q of this unit: k = q*H + ej; its slot: group k/16, lane 16*((k%16)/4) + column%16, s = k%4
    const unsigned G = H / 4;
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      const unsigned k = q * H + ej;
      dpre_p[((size_t(ecol / 16) * G + k / 16) * 64 + ((k % 16) / 4) * 16 + ecol % 16) * 4 + k % 4] = out[q];
    }
  }
}

// Skinny transposed product: slice[split] = A^T[M rows, depth range] x B[depth range, N columns] for M x N small
// and the depth K large (the backward timestep's Wh^T * dpre, and dx = Wx^T * dpre of the gates node): the same
// 64x32 tile and operand order as the forward kernel; K is cut into gridDim.y ranges so that every CU has a block,
// and whoever consumes the slices adds them in ascending order.  A is K x M and B is K x N, both with k contiguous
// (leading dimensions lda, ldb), read plain, or packed in fragment order.  Rows and columns past M and N are
// computed on clamped addresses and dropped.
template <bool PLAIN_A, bool PLAIN_B>
__global__ __launch_bounds__(256) void skinny_tn_kernel(unsigned M, unsigned N, unsigned K, const float* __restrict__ A,
                                                        size_t lda, const float* __restrict__ Bm, size_t ldb,
                                                        float* __restrict__ slices) {
  __shared__ float red[4 * 64 * kStepPitchR];
  const unsigned RP = cdiv<unsigned>(M, 64);
  const unsigned rp = blockIdx.x % RP, ct = blockIdx.x / RP, split = blockIdx.y;
  const unsigned wave = threadIdx.x / 64, lane = threadIdx.x % 64;
  const unsigned l32 = lane % 32, lhi = lane / 32;
  const unsigned G = K / 8, gq = G / (4 * gridDim.y), g0 = (split * 4 + wave) * gq;
  stepx16 acc0 = {0}, acc1 = {0};
  const float *pa0, *pa1, *pb;
  if (PLAIN_A) {
    const unsigned r0 = rp * 64 + l32, r1 = r0 + 32;
    pa0 = A + size_t(r0 < M ? r0 : M - 1) * lda + size_t(g0) * 8 + 4 * lhi;
    pa1 = A + size_t(r1 < M ? r1 : M - 1) * lda + size_t(g0) * 8 + 4 * lhi;
  } else {
    pa0 = A + ((size_t(2 * rp) * G + g0) * 64 + lane) * 4;
    pa1 = pa0 + size_t(G) * 256;
  }
  if (PLAIN_B) {
    const unsigned c0 = ct * 32 + l32;
    pb = Bm + size_t(c0 < N ? c0 : N - 1) * ldb + size_t(g0) * 8 + 4 * lhi;
  } else {
    pb = Bm + ((size_t(ct) * G + g0) * 64 + lane) * 4;
  }
  step_product<PLAIN_A ? kFragAlongK : kFragPacked, PLAIN_B, 2>(acc0, acc1, pa0, pa1, pb, gq);
#pragma unroll
  for (int r = 0; r < 16; ++r) {
    const unsigned row = 8 * (r / 4) + 4 * lhi + (r % 4);
    red[(wave * 64 + row) * kStepPitchR + l32] = acc0[r];
    red[(wave * 64 + 32 + row) * kStepPitchR + l32] = acc1[r];
  }
  __syncthreads();
  float* out = slices + size_t(split) * M * N;
  for (unsigned o = threadIdx.x; o < 64 * 32; o += 256) {
    const unsigned row = o % 64, col = o / 64, erow = rp * 64 + row, ecol = ct * 32 + col;
    if (erow >= M || ecol >= N) continue;
    float s = red[row * kStepPitchR + col];
#pragma unroll
    for (int w = 1; w < 4; ++w) s += red[(w * 64 + row) * kStepPitchR + col];
    out[size_t(ecol) * M + erow] = s;
  }
}

// C = epilogue(W0 v0 [+ W1 v1]) for a right operand that is a few 32-column tiles wide, one launch: the gates node's
// forward, fx = act(b + [f: +1] + Wx x + Wh h), and l * r / the affine layer of a small batch.  The weights as DyNet
// stores them (M x K, rows contiguous) and v plain (k contiguous per column).  A block owns 32 or 64 consecutive rows
// x 32 columns over the full depth of both products, its four waves split the depth in quarters and meet in LDS;
// nothing goes through a workspace.
struct NnOperand {
  const float* W;  // M x K, rows contiguous, leading dimension ldw
  const float* v;  // K x N, k contiguous, leading dimension ldv
  unsigned K;
  size_t ldw, ldv;
};
enum { kNnGates = 0, kNnBias = 1, kNnAxpby = 2 };

// TILES = 1: a block owns 32 rows (twice the blocks and half the matrix-core steps a wavefront: the smallest
// baseline cell, 16 blocks of 64 rows, 8.0 us; 5.6 us with 32 of 32)
template <int TILES, int EPI, int B_BYTES>
__global__ __launch_bounds__(256) void skinny_nn_kernel(unsigned M, unsigned H, unsigned B, NnOperand op0, NnOperand op1,
                                                        const float* __restrict__ bias, float beta, int mode,
                                                        float* __restrict__ fx) {
  constexpr unsigned ROWS = 32 * TILES;
  __shared__ float red[4 * ROWS * kStepPitchR];
  const unsigned RP = (M + ROWS - 1) / ROWS;  // rows past the end are computed on the last row and dropped
  const unsigned rp = blockIdx.x % RP, ct = blockIdx.x / RP;
  const unsigned wave = threadIdx.x / 64, lane = threadIdx.x % 64;
  const unsigned l32 = lane % 32, lhi = lane / 32;
  stepx16 acc0 = {0}, acc1 = {0};
  const unsigned pcol = ct * 32 + l32 < B ? ct * 32 + l32 : B - 1;
  // every output of this thread lies in row rp*ROWS + threadIdx.x % ROWS: its bias is fetched under the product
  const float bias_row = EPI == kNnAxpby ? 0.f : bias[min(rp * ROWS + threadIdx.x % ROWS, M - 1)];
  const unsigned r0 = min(rp * ROWS + l32, M - 1), r1 = min(rp * ROWS + 32 + l32, M - 1);
  // The four waves split the depth of BOTH products taken together into quarters (with I = H two waves multiply by
  // Wx and two by Wh): one run of the load pipeline per wave instead of one per product (its start costs ~1.5 us).
  if (op0.K % 32 == 0 && op1.K % 32 == 0 && (op0.K + op1.K) % 128 == 0) {
    const unsigned G0 = op0.K / 8, Gt = G0 + op1.K / 8, lo = wave * (Gt / 4), hi = lo + Gt / 4;
    for (int which = 0; which < 2; ++which) {
      const NnOperand op = which == 0 ? op0 : op1;
      const unsigned base = which == 0 ? 0 : G0, G = op.K / 8;
      const unsigned glo = lo > base ? lo : base, ghi = hi < base + G ? hi : base + G;
      if (glo >= ghi) continue;
      const unsigned g0 = glo - base;
      const float* pk = op.W + (size_t(g0) * 8 + 4 * lhi) * op.ldw;
      const float* pb = op.v + size_t(pcol) * op.ldv + size_t(g0) * 8 + 4 * lhi;
      step_product<kFragAlongRows, true, TILES, B_BYTES>(acc0, acc1, pk + r0, pk + r1, pb, ghi - glo, op.ldw);
    }
  } else {
    // Depths off that grid (even all the same): the waves are dealt to the two products in proportion to their depths
    // (all four to a single product), so that a wave still runs one pass of the load pipeline.  The waves of a product
    // split its leading whole rounds of four groups each; what is left of it, fewer than four groups a wave and a
    // group cut short after 2, 4 or 6 k, is dealt to them one group at a time and multiplied in one round of loads
    // (a pair of k past the end is fetched from k = 0 and its v entries zeroed).
    const unsigned Kt = op0.K + op1.K;
    unsigned w0 = 4;
    if (op1.K != 0) {
      w0 = (4 * op0.K + Kt / 2) / Kt;
      w0 = w0 < 1 ? 1 : w0 > 3 ? 3 : w0;
    }
    const bool first = wave < w0;
    const NnOperand op = first ? op0 : op1;
    const unsigned wq = first ? w0 : 4 - w0, wl = first ? wave : wave - w0;
    const unsigned G = op.K / 8, per = G / (4 * wq) * 4, main = per * wq;
    if (per > 0) {
      const unsigned g0 = wl * per;
      const float* pk = op.W + (size_t(g0) * 8 + 4 * lhi) * op.ldw;
      const float* pb = op.v + size_t(pcol) * op.ldv + size_t(g0) * 8 + 4 * lhi;
      step_product<kFragAlongRows, true, TILES, B_BYTES>(acc0, acc1, pk + r0, pk + r1, pb, per, op.ldw);
    }
    const unsigned rem = op.K - 8 * G, items = G - main + (rem != 0 ? 1u : 0u);  // rem: 0, 2, 4 or 6 k past the groups
    if (wl < items) {
      float a0[4][4], a1[4][4], bf[4][4];
#pragma unroll
      for (int it = 0; it < 4; ++it) {
        const unsigned idx = wl + wq * it, g = main + idx, k = 8 * g + 4 * lhi;
#pragma unroll
        for (int pr = 0; pr < 2; ++pr) {  // the fragment's two pairs of k: inside the depth together or not at all
          const bool valid = idx < items && k + 2 * pr + 1 < op.K;
          const unsigned kp = valid ? k + 2 * pr : 0u;
          const float2 t = *reinterpret_cast<const float2*>(op.v + size_t(pcol) * op.ldv + kp);
          bf[it][2 * pr] = valid ? t.x : 0.f;
          bf[it][2 * pr + 1] = valid ? t.y : 0.f;
#pragma unroll
          for (int j = 0; j < 2; ++j) {
            a0[it][2 * pr + j] = op.W[r0 + size_t(kp + j) * op.ldw];
            if (TILES == 2) a1[it][2 * pr + j] = op.W[r1 + size_t(kp + j) * op.ldw];
          }
        }
      }
#pragma unroll
      for (int it = 0; it < 4; ++it) {
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          acc0 = __builtin_amdgcn_mfma_f32_32x32x2f32(a0[it][j], bf[it][j], acc0, 0, 0, 0);
          if (TILES == 2) acc1 = __builtin_amdgcn_mfma_f32_32x32x2f32(a1[it][j], bf[it][j], acc1, 0, 0, 0);
        }
      }
    }
  }
#pragma unroll
  for (int r = 0; r < 16; ++r) {
    const unsigned row = 8 * (r / 4) + 4 * lhi + (r % 4);
    red[(wave * ROWS + row) * kStepPitchR + l32] = acc0[r];
    if (TILES == 2) red[(wave * ROWS + 32 + row) * kStepPitchR + l32] = acc1[r];
  }
  __syncthreads();
  for (unsigned o = threadIdx.x; o < ROWS * 32; o += 256) {
    const unsigned row = o % ROWS, col = o / ROWS, erow = rp * ROWS + row, ecol = ct * 32 + col;
    if (ecol >= B || erow >= M) continue;
    float* out = fx + size_t(ecol) * M + erow;
    if (EPI == kNnGates) {
      float pre = bias_row;
      if (erow >= H && erow < 2 * H) pre += 1.0f;  // forget-gate bias
#pragma unroll
      for (int w = 0; w < 4; ++w) pre += red[(w * ROWS + row) * kStepPitchR + col];
      *out = erow < 3 * H ? logistic(mode, pre) : tanh_accurate(pre);
    } else {
      float t = red[row * kStepPitchR + col];
#pragma unroll
      for (int w = 1; w < 4; ++w) t += red[(w * ROWS + row) * kStepPitchR + col];
      if (EPI == kNnBias) t += bias_row;
      else if (beta != 0.f) t += beta * *out;
      *out = t;
    }
  }
}

// 32-row blocks as long as they do not outnumber the CUs (gates forward, I = H = 1024: B = 20 13.9 us against 25 us
// with 64-row blocks and 17.0 us for the two-launch small-batch product; B = 64 15.4 against 23.7 us; I = H = 2048,
// B = 20 32.4 against 42.3 and 36.6 us; more blocks than CUs lose: B = 96 39.3 against 24.4 us, B = 128 39.8 against
// 25.7 us).  Not for a block that would walk more than 2 MB of weights alone (a few rows over a very long depth), nor
// for odd depths (v's fragments are 128-bit loads along k, or two 64-bit ones).
int skinny_nn_gemm(dyhip_device* dev, size_t M, size_t N, int nseg, const GemmSeg* segs, float* C, const GemmEpiParams& epi,
                   bool* taken) {
  *taken = false;
  if (nseg < 1 || nseg > 2 || C == nullptr || N == 0 || N > 256 || M < 1 || M >= (size_t(1) << 31)) return DYHIP_OK;
  const int kind = epi.kind == kEpiLstmGates ? kNnGates : epi.kind == kEpiBias ? kNnBias : epi.kind == kEpiAxpby ? kNnAxpby : -1;
  if (kind < 0 || (kind != kNnAxpby && epi.bias == nullptr) || (nseg == 2 && kind != kNnGates)) return DYHIP_OK;
  size_t Kt = 0;
  bool b16 = true;
  for (int q = 0; q < nseg; ++q) {
    const GemmSeg& g = segs[q];
    if (g.A == nullptr || g.B == nullptr || g.K == 0 || g.K % 2 != 0 || g.K >= (size_t(1) << 31) || g.ldb % 2 != 0 ||
        (reinterpret_cast<uintptr_t>(g.B) & 7u) != 0)
      return DYHIP_OK;
    b16 = b16 && g.ldb % 4 == 0 && aligned16(g.B);  // 128-bit fragments of v; 64-bit halves otherwise
    Kt += g.K;
  }
  // fewer than 32 rows (one ragged row tile: an output layer with a handful of classes) up to a depth of 1024, where
  // its few blocks still beat the depth-split forms (20 x 128 x 1024: 15.9 -> 8.6 us; at 4096 deep 14.0 against 22.7 us)
  if (M < 32 && Kt > 1024) return DYHIP_OK;
  const unsigned cus = unsigned(dev->num_cus > 0 ? dev->num_cus : 256);
  const unsigned ct = cdiv<unsigned>(unsigned(N), 32);
  const unsigned blocks64 = cdiv<unsigned>(unsigned(M), 64) * ct;
  const unsigned tiles = blocks64 <= cus / 2 ? 1 : 2;
  if (size_t(32) * tiles * Kt * sizeof(float) > (size_t(2) << 20)) return DYHIP_OK;
  const NnOperand op0{segs[0].A, segs[0].B, unsigned(segs[0].K), segs[0].lda, segs[0].ldb};
  const NnOperand op1 = nseg > 1 ? NnOperand{segs[1].A, segs[1].B, unsigned(segs[1].K), segs[1].lda, segs[1].ldb}
                                 : NnOperand{segs[0].A, segs[0].B, 0u, segs[0].lda, segs[0].ldb};
  const dim3 grid(cdiv<unsigned>(unsigned(M), 32 * tiles) * ct), block(256);
  const float beta = kind == kNnAxpby ? epi.beta : 0.f;
#define DYHIP_SKINNY_NN_B(T, E, BB)                                                                                 \
  hipLaunchKernelGGL((skinny_nn_kernel<T, E, BB>), grid, block, 0, dev->stream, unsigned(M), epi.H, unsigned(N), op0, op1, \
                     epi.bias, beta, epi.logistic_mode, C)
#define DYHIP_SKINNY_NN(T, E)        \
  do {                               \
    if (b16) DYHIP_SKINNY_NN_B(T, E, 16); \
    else DYHIP_SKINNY_NN_B(T, E, 8);      \
  } while (0)
  if (tiles == 1) {
    if (kind == kNnGates) DYHIP_SKINNY_NN(1, kNnGates);
    else if (kind == kNnBias) DYHIP_SKINNY_NN(1, kNnBias);
    else DYHIP_SKINNY_NN(1, kNnAxpby);
  } else {
    if (kind == kNnGates) DYHIP_SKINNY_NN(2, kNnGates);
    else if (kind == kNnBias) DYHIP_SKINNY_NN(2, kNnBias);
    else DYHIP_SKINNY_NN(2, kNnAxpby);
  }
#undef DYHIP_SKINNY_NN_B
#undef DYHIP_SKINNY_NN
  DYHIP_CHECK_LAUNCH();
  *taken = true;
  return DYHIP_OK;
}

// out[e] = beta * out[e] + (slices[0][e] + slices[1][e] + ...), slices added in ascending order
__global__ __launch_bounds__(256) void slices_accumulate_kernel(size_t total, unsigned splits,
                                                                const float* __restrict__ slices, float beta,
                                                                float* __restrict__ out) {
  const size_t e = size_t(blockIdx.x) * 256 + threadIdx.x;
  if (e >= total) return;
  const float old = beta != 0.f ? out[e] : 0.f;  // fetched beside the slices
  float s = 0.f;
  for (unsigned k0 = 0; k0 < splits; k0 += 8) {  // eight slices in flight, added in ascending order
    float v[8];
#pragma unroll
    for (int u = 0; u < 8; ++u) v[u] = slices[size_t(min(k0 + u, splits - 1)) * total + e];
#pragma unroll
    for (int u = 0; u < 8; ++u)
      if (k0 + u < splits) s += v[u];
  }
  out[e] = beta != 0.f ? beta * old + s : s;
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

// Depth ranges of a skinny transposed product: enough blocks for every CU, whole sets of four groups of 8 k per
// wave.  0 when the depth does not divide that way (the caller then takes the general GEMM).
static unsigned skinny_tn_splits(unsigned M, unsigned N, unsigned K) {
  if (K < 128 || K % 128 != 0) return 0;
  const unsigned tiles = cdiv<unsigned>(M, 64) * cdiv<unsigned>(N, 32);
  unsigned s = 1;
  while (s < 16 && tiles * s < 256 && (K / 8) % (s * 2 * 16) == 0) s *= 2;
  return s;
}

// slices[s] = A^T B over depth range s (s < *splits); see skinny_tn_kernel for the operand forms
static int skinny_tn(dyhip_device* dev, unsigned M, unsigned N, unsigned K, const float* A, size_t lda, bool plain_a,
                     const float* B, size_t ldb, bool plain_b, float* slices, size_t slices_bytes, unsigned* splits) {
  const unsigned s = skinny_tn_splits(M, N, K);
  DYHIP_REQUIRE(s >= 1, "skinny product: depth %u is not a multiple of 128", K);
  DYHIP_REQUIRE(aligned16(A) && aligned16(B) && lda % 4 == 0 && ldb % 4 == 0, "skinny product: operands must be 16-byte aligned");
  DYHIP_REQUIRE(slices != nullptr && slices_bytes >= sizeof(float) * size_t(M) * N * s,
                "skinny product: %u slices of %u x %u floats do not fit %zu bytes", s, M, N, slices_bytes);
  const dim3 grid(cdiv<unsigned>(M, 64) * cdiv<unsigned>(N, 32), s), block(256);
#define DYHIP_SKINNY(PA, PB) \
  hipLaunchKernelGGL((skinny_tn_kernel<PA, PB>), grid, block, 0, dev->stream, M, N, K, A, lda, B, ldb, slices)
  if (plain_a && plain_b) DYHIP_SKINNY(true, true);
  else if (plain_a) DYHIP_SKINNY(true, false);
  else if (plain_b) DYHIP_SKINNY(false, true);
  else DYHIP_SKINNY(false, false);
#undef DYHIP_SKINNY
  DYHIP_CHECK_LAUNCH();
  *splits = s;
  return DYHIP_OK;
}

// ---- C[M x N] = beta * C + A^T B for at most 32 columns of B (dx and dh of the gates node at a small batch) --------
// A (K x M, a weight matrix) is read once from memory and is the whole cost; B (K x N) is small and stays in the L2.
// A block owns four columns of A and all columns of B: its 256 threads split the depth in 128-bit groups, every thread
// multiplies its group of each of the four A columns with its group of every B column, and the 4 x N partial sums
// cross the block once at the end (wavefront sums, then LDS in ascending wavefront order).  No matrix cores: at 20
// columns the product is 80 multiply-adds per 16 bytes of A, and a 32-column matrix-core tile would read A in
// 128-byte pieces (the fragment-order kernel above takes 13.6 us for 16.8 MB of A at N = 20).
// kThinTnCols: columns of A a block owns: four for more than 4096 output rows, two down to 513, one below (more,
// smaller blocks: 1024 x 1 x 4096 6.3 -> 5.4 us, 256 x 1 x 1024 3.7 -> 2.7 us; 10 000 x 1 x 1024 9.2 against 9.5 us)
template <int NP, int kThinTnCols>  // NP: N rounded up to a multiple of four
__global__ __launch_bounds__(256) void gemm_tn_thin_kernel(unsigned M, unsigned N, unsigned K4, const float* __restrict__ A,
                                                           size_t lda, const float* __restrict__ B, size_t ldb, float beta,
                                                           float* __restrict__ C, size_t stride_a, size_t stride_b,
                                                           size_t stride_c) {
  __shared__ float red[4][kThinTnCols][NP];
  // item blockIdx.y of a strided batch (strides 0 otherwise)
  A += size_t(blockIdx.y) * stride_a;
  B += size_t(blockIdx.y) * stride_b;
  C += size_t(blockIdx.y) * stride_c;
  const unsigned i0 = blockIdx.x * kThinTnCols;
  const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
  float acc[kThinTnCols][NP];
#pragma unroll
  for (int c = 0; c < kThinTnCols; ++c)
#pragma unroll
    for (int n = 0; n < NP; ++n) acc[c][n] = 0.f;
  const float4* a4[kThinTnCols];
#pragma unroll
  for (int c = 0; c < kThinTnCols; ++c)
    a4[c] = reinterpret_cast<const float4*>(A + size_t(min(i0 + c, M - 1)) * lda);  // columns past the end: not stored
  for (unsigned k4 = threadIdx.x; k4 < K4; k4 += 256) {
    float4 a[kThinTnCols], b[NP];
#pragma unroll
    for (int c = 0; c < kThinTnCols; ++c) a[c] = ldg4<true>(a4[c] + k4);  // read once: streaming
#pragma unroll
    for (int n = 0; n < NP; ++n)
      b[n] = reinterpret_cast<const float4*>(B + size_t(min(unsigned(n), N - 1)) * ldb)[k4];
#pragma unroll
    for (int c = 0; c < kThinTnCols; ++c)
#pragma unroll
      for (int n = 0; n < NP; ++n) {
        float t = acc[c][n];
        t = fmaf(a[c].x, b[n].x, t);
        t = fmaf(a[c].y, b[n].y, t);
        t = fmaf(a[c].z, b[n].z, t);
        t = fmaf(a[c].w, b[n].w, t);
        acc[c][n] = t;
      }
  }
#pragma unroll
  for (int c = 0; c < kThinTnCols; ++c)
#pragma unroll
    for (int n = 0; n < NP; ++n) {
      const float t = wave_sum(acc[c][n]);
      if (lane == 0) red[w][c][n] = t;
    }
  __syncthreads();
  if (threadIdx.x < kThinTnCols * NP) {
    const unsigned c = threadIdx.x / NP, n = threadIdx.x % NP;
    if (i0 + c < M && n < N) {
      const float t = ((red[0][c][n] + red[1][c][n]) + red[2][c][n]) + red[3][c][n];
      float* out = C + size_t(n) * M + i0 + c;
      *out = beta != 0.f ? beta * *out + t : t;
    }
  }
}

// ---- C[M x N] = beta * C + A^T B for 5..256 columns of B (in tiles of 32) on the matrix cores, the operands as they lie --
// A's columns (the depth contiguous) are fetched by coalesced 128-bit loads, 32 depth indices of 32 columns a
// wavefront at a time (128-byte runs), and turned into matrix-core fragments through a wavefront's own LDS tile:
// lane l reads column l % 32 at four depth indices of the lower or upper half of an 8-index group.  B's columns the
// same way.  A block's four wavefronts take a quarter of its depth range each (tiles added through LDS), blocks split
// the depth further and slices_accumulate_kernel adds their slices.  The fragment-order kernel reads A in 32-byte
// pieces and wants depths that are multiples of 128 (1024 x 20 x 4096: 10.7 us, here 9.1; 384 x 32 x 1536: 10.6 us,
// here 6.2); the streaming kernel above fetches all of B once per four columns of A (1024 x 20 x 10 000: 25 us, here
// 15.8).
// 32 depth indices a round: 128-byte runs and 37 KB of LDS a block (64: 10.1 against 9.2 us for 1024 x 20 x 4096;
// 128: 10.9 us); one block a CU's worth of slices (two: 9.2 against 9.1 us, 7.5 against 6.8 us at a depth of 2048)
constexpr unsigned kTnMidDepth = 32;
constexpr unsigned kTnMidPitch = kTnMidDepth + 4;
template <int NB4>  // B's columns in loads of four: ceil(N / 4)
__global__ __launch_bounds__(256) void gemm_tn_mid_kernel(unsigned M, unsigned N, unsigned K, unsigned chunk,
                                                          unsigned per_wave, const float* __restrict__ A, size_t lda,
                                                          const float* __restrict__ B, size_t ldb, float beta,
                                                          float* __restrict__ C, float* __restrict__ partial) {
  __shared__ __attribute__((aligned(16))) float tiles[4][2][32 * kTnMidPitch];
  const unsigned lane = threadIdx.x & 63, w = threadIdx.x >> 6, l32 = lane & 31, hi = lane >> 5;
  const unsigned i0 = blockIdx.x * 32;
  const unsigned n0 = blockIdx.z * 32, Nt = min(32u, N - n0);  // this block's tile of B's columns
  const unsigned k0 = blockIdx.y * chunk, k1 = min(K, k0 + chunk);
  const unsigned kw0 = k0 + w * per_wave, kw1 = min(k1, kw0 + per_wave);
  float* la = tiles[w][0];
  float* lb = tiles[w][1];
  constexpr unsigned kLanesDeep = kTnMidDepth / 4, kColsPerLoad = 64 / kLanesDeep;
  const unsigned q = lane % kLanesDeep, cq = lane / kLanesDeep;  // a load: kLanesDeep lanes along the depth of one of kColsPerLoad columns
  stepx16 acc;
#pragma unroll
  for (int r = 0; r < 16; ++r) acc[r] = 0.f;
  // The next round's loads leave before this round's fragments are multiplied.
  constexpr int kLoadsA = 32 / kColsPerLoad, kLoadsB = (4 * NB4 + kColsPerLoad - 1) / kColsPerLoad;
  float4 ta[kLoadsA], tb[kLoadsB];
  bool in = false;
  auto fetch = [&](unsigned t) __attribute__((always_inline)) {
    const unsigned kq = kw0 + t + 4 * q;       // this lane's four depth indices
    in = kq < kw1;                             // K, the ranges and kq are multiples of four
    const size_t kc = in ? kq : (K - 4);
#pragma unroll
    for (int u = 0; u < kLoadsA; ++u) ta[u] = ldg4<true>(reinterpret_cast<const float4*>(A + size_t(min(i0 + kColsPerLoad * u + cq, M - 1)) * lda + kc));
#pragma unroll
    for (int u = 0; u < kLoadsB; ++u) tb[u] = *reinterpret_cast<const float4*>(B + size_t(n0 + min(kColsPerLoad * u + cq, Nt - 1)) * ldb + kc);
  };
  fetch(0);
  for (unsigned t = 0; kw0 + t < kw1; t += kTnMidDepth) {
    // the tiles are this wavefront's own: its LDS accesses execute in order, so the compiler only has to keep the
    // writes behind the last round's reads and ahead of this round's (no block barrier: the wavefronts drift apart
    // and one multiplies while another waits for its loads)
    __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
    __builtin_amdgcn_wave_barrier();
#pragma unroll
    for (int u = 0; u < kLoadsA; ++u) {
      const float4 v = ta[u];
      *reinterpret_cast<float4*>(la + (kColsPerLoad * u + cq) * kTnMidPitch + 4 * q) =
          make_float4(in ? v.x : 0.f, in ? v.y : 0.f, in ? v.z : 0.f, in ? v.w : 0.f);
    }
#pragma unroll
    for (int u = 0; u < kLoadsB; ++u) {
      const float4 v = tb[u];
      if (kColsPerLoad * u + cq < 32)
      *reinterpret_cast<float4*>(lb + (kColsPerLoad * u + cq) * kTnMidPitch + 4 * q) =
          make_float4(in ? v.x : 0.f, in ? v.y : 0.f, in ? v.z : 0.f, in ? v.w : 0.f);
    }
    __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
    __builtin_amdgcn_wave_barrier();
    if (kw0 + t + kTnMidDepth < kw1) fetch(t + kTnMidDepth);
#pragma unroll
    for (int s8 = 0; s8 < int(kTnMidDepth) / 8; ++s8) {
      const float4 a4 = *reinterpret_cast<const float4*>(la + l32 * kTnMidPitch + 8 * s8 + 4 * hi);
      const float4 b4 = *reinterpret_cast<const float4*>(lb + min(l32, 4u * NB4 - 1) * kTnMidPitch + 8 * s8 + 4 * hi);
      const bool col = l32 < Nt;
      acc = __builtin_amdgcn_mfma_f32_32x32x2f32(col ? b4.x : 0.f, a4.x, acc, 0, 0, 0);
      acc = __builtin_amdgcn_mfma_f32_32x32x2f32(col ? b4.y : 0.f, a4.y, acc, 0, 0, 0);
      acc = __builtin_amdgcn_mfma_f32_32x32x2f32(col ? b4.z : 0.f, a4.z, acc, 0, 0, 0);
      acc = __builtin_amdgcn_mfma_f32_32x32x2f32(col ? b4.w : 0.f, a4.w, acc, 0, 0, 0);
    }
  }
  // acc[r] of lane l: output row i0 + l % 32, column 8 * (r / 4) + 4 * (l / 32) + r % 4
  __syncthreads();
  float* red = &tiles[0][0][0];  // [wave][16][64]
#pragma unroll
  for (int r = 0; r < 16; ++r) red[(w * 16 + r) * 64 + lane] = acc[r];
  __syncthreads();
  float* out = partial != nullptr ? partial + size_t(blockIdx.y) * M * N : C;
  const unsigned row = i0 + l32;
#pragma unroll
  for (int rr = 0; rr < 4; ++rr) {  // wavefront w finishes registers 4 w .. 4 w + 3
    const unsigned r = 4 * w + rr, n = n0 + 8 * (r / 4) + 4 * hi + (r % 4);
    float v = red[r * 64 + lane];
#pragma unroll
    for (int x = 1; x < 4; ++x) v += red[(x * 16 + r) * 64 + lane];
    if (row < M && n < N) {
      float* p = out + size_t(n) * M + row;
      *p = (partial == nullptr && beta != 0.f) ? beta * *p + v : v;
    }
  }
}

static bool mid_tn_eligible(const dyhip_device* dev, size_t M, size_t N, size_t K, const float* A, size_t lda, const float* B,
                            size_t ldb) {
  return N >= 5 && N <= 256 && M >= 32 && M <= (size_t(1) << 30) && K >= 256 && K % 4 == 0 && K <= 0x7FFFFFF0ull &&
         lda % 4 == 0 && ldb % 4 == 0 && aligned16(A) && aligned16(B) && dev->gemm_ws != nullptr;
}

static int mid_tn_run(dyhip_device* dev, size_t M, size_t N, size_t K, const float* A, size_t lda, const float* B, size_t ldb,
                      float beta, float* C) {
  const unsigned tiles = static_cast<unsigned>(cdiv<size_t>(M, 32)), Ku = static_cast<unsigned>(K);
  // depth slices: a block a CU, each with at least one round per wavefront
  const unsigned ct = cdiv<unsigned>(unsigned(N), 32);
  unsigned slabs = cdiv<unsigned>(unsigned(dev->num_cus > 0 ? dev->num_cus : 256), tiles * ct);
  const unsigned max_by_depth = cdiv<unsigned>(Ku, 4 * kTnMidDepth);
  if (slabs > max_by_depth) slabs = max_by_depth;
  if (slabs < 1) slabs = 1;
  unsigned chunk = cdiv<unsigned>(Ku, slabs);
  chunk = (chunk + 4 * kTnMidDepth - 1) / (4 * kTnMidDepth) * (4 * kTnMidDepth);
  slabs = cdiv<unsigned>(Ku, chunk);
  const unsigned per_wave = chunk / 4;
  float* partial = nullptr;
  if (slabs > 1) {
    DYHIP_REQUIRE(dev->gemm_ws_bytes >= sizeof(float) * M * N * slabs, "transposed small-batch product: workspace too small");
    partial = static_cast<float*>(dev->gemm_ws);
  }
  const dim3 grid(tiles, slabs, ct), block(256);
#define DYHIP_TN_MID(NB4)                                                                                          \
  hipLaunchKernelGGL(gemm_tn_mid_kernel<NB4>, grid, block, 0, dev->stream, static_cast<unsigned>(M), static_cast<unsigned>(N), \
                     Ku, chunk, per_wave, A, lda, B, ldb, beta, C, partial)
  switch (N >= 32 ? 8u : unsigned(N + 3) / 4) {
    case 2: DYHIP_TN_MID(2); break;
    case 3: DYHIP_TN_MID(3); break;
    case 4: DYHIP_TN_MID(4); break;
    case 5: DYHIP_TN_MID(5); break;
    case 6: DYHIP_TN_MID(6); break;
    case 7: DYHIP_TN_MID(7); break;
    default: DYHIP_TN_MID(8); break;
  }
#undef DYHIP_TN_MID
  DYHIP_CHECK_LAUNCH();
  if (partial != nullptr) {
    const size_t total = M * N;
    hipLaunchKernelGGL(slices_accumulate_kernel, dim3(unsigned(cdiv<size_t>(total, 256))), dim3(256), 0, dev->stream, total,
                       slabs, partial, beta, C);
    DYHIP_CHECK_LAUNCH();
  }
  return DYHIP_OK;
}

static bool thin_tn_eligible(size_t M, size_t N, size_t K, const float* A, size_t lda, const float* B, size_t ldb) {
  return N >= 1 && N <= 32 && M >= 1 && M <= (size_t(1) << 30) && K >= 256 && K % 4 == 0 && K / 4 <= 0xFFFFFFFFull &&
         lda % 4 == 0 && ldb % 4 == 0 && aligned16(A) && aligned16(B);
}

static int thin_tn_run(dyhip_device* dev, size_t M, size_t N, size_t K, const float* A, size_t lda, const float* B,
                       size_t ldb, float beta, float* C, const GemmBatch* batch = nullptr) {
  const unsigned items = batch != nullptr && batch->count > 1 ? batch->count : 1;
  const size_t sa = items > 1 ? batch->stride_a : 0, sb = items > 1 ? batch->stride_b : 0, sc = items > 1 ? batch->stride_c : 0;
  const int cols = M * items > 4096 ? 4 : M * items > 512 ? 2 : 1;
  const dim3 grid(static_cast<unsigned>(cdiv<size_t>(M, cols)), items), block(256);
#define DYHIP_THIN_TN_C(NP, CC)                                                                                 \
  hipLaunchKernelGGL((gemm_tn_thin_kernel<NP, CC>), grid, block, 0, dev->stream, static_cast<unsigned>(M),     \
                     static_cast<unsigned>(N), static_cast<unsigned>(K / 4), A, lda, B, ldb, beta, C, sa, sb, sc)
#define DYHIP_THIN_TN(NP)                      \
  do {                                         \
    if (cols == 4) DYHIP_THIN_TN_C(NP, 4);     \
    else if (cols == 2) DYHIP_THIN_TN_C(NP, 2); \
    else DYHIP_THIN_TN_C(NP, 1);               \
  } while (0)
  switch ((N + 3) / 4) {
    case 1: DYHIP_THIN_TN(4); break;
    case 2: DYHIP_THIN_TN(8); break;
    case 3: DYHIP_THIN_TN(12); break;
    case 4: DYHIP_THIN_TN(16); break;
    case 5: DYHIP_THIN_TN(20); break;
    case 6: DYHIP_THIN_TN(24); break;
    case 7: DYHIP_THIN_TN(28); break;
    default: DYHIP_THIN_TN(32); break;
  }
#undef DYHIP_THIN_TN_C
#undef DYHIP_THIN_TN
  DYHIP_CHECK_LAUNCH();
  return DYHIP_OK;
}

// The streaming kernel over the items of a strided batch (da += H^T * dctx of an attention over a batch: 35 x 1 x 1024
// times 128 items 12.7 us with a matrix-core tile per wavefront).  *taken = false when the shape is not its own.
int thin_tn_batched(dyhip_device* dev, size_t M, size_t N, size_t K, const float* A, size_t lda, const float* B, size_t ldb,
                    float beta, float* C, const GemmBatch* batch, bool* taken) {
  *taken = false;
  if (batch == nullptr || batch->count <= 1 || batch->count > 65535u || N > 4 || C == nullptr ||
      !thin_tn_eligible(M, N, K, A, lda, B, ldb) || batch->stride_a % 4 != 0 || batch->stride_b % 4 != 0 ||
      batch->stride_c < M * N)
    return DYHIP_OK;
  DYHIP_CHECK_STATUS(thin_tn_run(dev, M, N, K, A, lda, B, ldb, beta, C, batch));
  *taken = true;
  return DYHIP_OK;
}

// C[M x N] = beta * C + A^T B for a small output with a deep sum, A (K x M) and B (K x N) plain with k contiguous:
// the fragment-order product leaves a few slices in the queue's GEMM workspace and a second launch folds them into
// C.  *taken = false (nothing launched) when the shape is not one this form is faster on.
int skinny_tn_gemm(dyhip_device* dev, size_t M, size_t N, size_t K, const float* A, size_t lda, const float* B,
                   size_t ldb, float beta, float* C, bool* taken) {
  *taken = false;
  // At most 32 columns of B: up to four the streaming kernel (1024 x 1 x 4096: 7.1 against 11.4 us for the
  // fragment-order product below), from five on the matrix-core kernel on LDS tiles (faster than the fragment-order
  // product on every shape measured up to 64 MB of A, and without its conditions on the depth); the streaming kernel
  // still takes what neither does.  More than 32 columns: the fragment-order product.
  const bool thin_ok = C != nullptr && thin_tn_eligible(M, N, K, A, lda, B, ldb);
  bool frag_ok = !(M == 0 || N == 0 || M > 4096 || N > 256 || K < 1024 || K > (size_t(1) << 24)) &&
                 !(M * N > (size_t(1) << 19) || lda % 4 != 0 || ldb % 4 != 0 || !aligned16(A) || !aligned16(B));
  frag_ok = frag_ok && skinny_tn_splits(unsigned(M), unsigned(N), unsigned(K)) != 0 && dev->gemm_ws != nullptr &&
            dev->gemm_ws_bytes >= sizeof(float) * M * N * 16;
  // beyond 64 columns (tiles of 32, each re-reading A) only for a small A or where the fragment-order product does
  // not apply: 256 x 128 x 4096 9.8 against 11.1 us, 1024 x 40 x 10 000 24.1 against 31.6 us, but 1024 x 128 x 4096
  // 20.4 against 18.4 us
  if (C != nullptr && mid_tn_eligible(dev, M, N, K, A, lda, B, ldb) &&
      (N <= 64 || !frag_ok || M * K * sizeof(float) <= (size_t(8) << 20))) {
    DYHIP_CHECK_STATUS(mid_tn_run(dev, M, N, K, A, lda, B, ldb, beta, C));
    *taken = true;
    return DYHIP_OK;
  }
  if (thin_ok && (N <= 4 || !frag_ok)) {
    DYHIP_CHECK_STATUS(thin_tn_run(dev, M, N, K, A, lda, B, ldb, beta, C));
    *taken = true;
    return DYHIP_OK;
  }
  if (!frag_ok) return DYHIP_OK;
  const unsigned m = unsigned(M), n = unsigned(N), k = unsigned(K);
  unsigned splits = 0;
  DYHIP_CHECK_STATUS(skinny_tn(dev, m, n, k, A, lda, true, B, ldb, true, static_cast<float*>(dev->gemm_ws),
                               dev->gemm_ws_bytes, &splits));
  const size_t total = M * N;
  hipLaunchKernelGGL(slices_accumulate_kernel, dim3(unsigned(cdiv<size_t>(total, 256))), dim3(256), 0, dev->stream, total,
                     splits, static_cast<const float*>(dev->gemm_ws), beta, C);
  DYHIP_CHECK_LAUNCH();
  *taken = true;
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
  // gemm_run picks the form: up to four columns (the un-batched graph, decoding) the matrix-times-vector kernels,
  // whose second kernel adds the depth slabs with the gates' epilogue (I = H = 1024, one column: 22 -> 9.4 us); from
  // five columns the one-launch fragment-order kernel on the operands as they lie (see skinny_nn_gemm)
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
    if (!gi.dropout) {  // a small output with a 4H-deep sum: the fragment-order product when the shape suits it
      bool taken = false;
      DYHIP_CHECK_STATUS(skinny_tn_gemm(dev, rows, B, G, W, G, dpre, G, 1.0f, dEdxi, &taken));
      if (taken) return DYHIP_OK;
    }
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
  // Wh^T * dpre[4H x B]: a small output with a deep sum, both operands with k contiguous as they lie
  if (B <= 512 && skinny_tn_splits(H, B, unsigned(G)) >= 1 && aligned16(Wh) && aligned16(v) &&
      ws_bytes >= sizeof(float) * size_t(H) * B * skinny_tn_splits(H, B, unsigned(G)))
    return skinny_tn(dev, H, B, unsigned(G), Wh, G, true, v, G, true, static_cast<float*>(ws), ws_bytes, splits);
  GemmSeg s{Wh, G, v, G, G};
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

static int cell_backward(dyhip_device* dev, unsigned H, unsigned B, const float* gates, const float* c,
                         const float* c_tm1, const float* dh, const float* rec, unsigned splits, const float* dc,
                         float* dpre, float* dc_tm1, float* dpre_packed) {
  DYHIP_REQUIRE(H >= 1 && B >= 1, "LSTM cell: bad hidden (%u) or batch (%u) size", H, B);
  DYHIP_REQUIRE(gates && c && dh && dpre, "LSTM cell: null tensor pointer");
  DYHIP_REQUIRE(splits == 0 || rec != nullptr, "LSTM cell: %u recurrent slices but no buffer", splits);
  const size_t slice = size_t(H) * B;
  const bool vec = H % 4 == 0 && all_aligned16({gates, c, c_tm1, dh, rec, dc, dpre, dc_tm1});
  for (unsigned b0 = 0; b0 < B; b0 += 65535u) {
    const unsigned nb = B - b0 < 65535u ? B - b0 : 65535u;
    if (vec)
      hipLaunchKernelGGL(lstm_cell_bwd_kernel<4>, dim3(cdiv<unsigned>(H, kCellThreads * 4), nb), dim3(kCellThreads), 0,
                         dev->stream, H, splits, slice, gates, c, c_tm1, dh, rec, dc, dpre, dc_tm1, b0, dpre_packed);
    else
      hipLaunchKernelGGL(lstm_cell_bwd_kernel<1>, dim3(cdiv<unsigned>(H, kCellThreads), nb), dim3(kCellThreads), 0,
                         dev->stream, H, splits, slice, gates, c, c_tm1, dh, rec, dc, dpre, dc_tm1, b0, dpre_packed);
  }
  DYHIP_CHECK_LAUNCH();
  return DYHIP_OK;
}

int dyhip_lstm_cell_backward(dyhip_device* dev, unsigned H, unsigned B, const float* gates, const float* c,
                             const float* c_tm1, const float* dh, const float* rec, unsigned splits, const float* dc,
                             float* dpre, float* dc_tm1) {
  DYHIP_CHECK_DEV(dev);
  return cell_backward(dev, H, B, gates, c, c_tm1, dh, rec, splits, dc, dpre, dc_tm1, nullptr);
}

static bool step_depth_ok(unsigned K) { return K >= 128 && K % 128 == 0; }  // quarters in whole sets of 4 groups of 8

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
  hipLaunchKernelGGL(lstm_pack_weights_kernel, dim3(unsigned(n / 2048)), dim3(256), 0, dev->stream, H, K, W, packed);
  DYHIP_CHECK_LAUNCH();
  return DYHIP_OK;
}

static size_t packed_state_floats(unsigned K, unsigned B) { return size_t(K) * cdiv<unsigned>(B, 32) * 32; }

static int pack_state(dyhip_device* dev, unsigned K, unsigned B, const float* v, float* packed) {
  DYHIP_REQUIRE(step_depth_ok(K) && B >= 1 && B <= 65535, "LSTM step: state of %u rows x %u columns cannot be packed", K, B);
  DYHIP_REQUIRE(v && packed, "LSTM step: null tensor pointer");
  const size_t n = packed_state_floats(K, B);
  hipLaunchKernelGGL(lstm_pack_state_kernel, dim3(unsigned(cdiv<size_t>(n, 256))), dim3(256), 0, dev->stream, K, B, v,
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

int dyhip_lstm_pack_recurrent_transposed(dyhip_device* dev, unsigned H, const float* Wh, float* packed) {
  DYHIP_CHECK_DEV(dev);
  DYHIP_REQUIRE(step_depth_ok(H) && size_t(4) * H * H < (size_t(1) << 32), "LSTM step: hidden size %u must be a multiple of 128", H);
  DYHIP_REQUIRE(Wh && packed, "LSTM step: null tensor pointer");
  const size_t n = size_t(4) * H * H;
  hipLaunchKernelGGL(lstm_pack_transposed_kernel, dim3(unsigned(cdiv<size_t>(n, 256))), dim3(256), 0, dev->stream, H, Wh,
                     packed);
  DYHIP_CHECK_LAUNCH();
  return DYHIP_OK;
}

int dyhip_lstm_pack_recurrent_transposed16(dyhip_device* dev, unsigned H, const float* Wh, float* packed) {
  DYHIP_CHECK_DEV(dev);
  DYHIP_REQUIRE(step_depth_ok(H) && size_t(4) * H * H < (size_t(1) << 32), "LSTM step: hidden size %u must be a multiple of 128", H);
  DYHIP_REQUIRE(Wh && packed, "LSTM step: null tensor pointer");
  const size_t n = size_t(4) * H * H;
  hipLaunchKernelGGL(lstm_pack_transposed16_kernel, dim3(unsigned(cdiv<size_t>(n / 4, 256))), dim3(256), 0, dev->stream, H,
                     Wh, packed, aligned16(Wh) && aligned16(packed) ? 1 : 0);
  DYHIP_CHECK_LAUNCH();
  return DYHIP_OK;
}

int dyhip_lstm_packed_state16_floats(unsigned rows, unsigned B, size_t* floats) {
  DYHIP_REQUIRE(floats != nullptr, "null output pointer");
  *floats = size_t(2) * cdiv<unsigned>(B, 32) * 16 * rows;  // pairs of 16-column tiles
  return DYHIP_OK;
}

int dyhip_lstm_pack_state16(dyhip_device* dev, unsigned rows, unsigned B, const float* v, float* packed) {
  DYHIP_CHECK_DEV(dev);
  DYHIP_REQUIRE(v && packed, "LSTM step: null tensor pointer");
  DYHIP_REQUIRE(rows % 16 == 0 && rows > 0 && B > 0, "LSTM step: %u rows are not a multiple of 16", rows);
  const size_t n = size_t(2) * cdiv<unsigned>(B, 32) * 16 * rows;
  DYHIP_REQUIRE(n < (size_t(1) << 32), "LSTM step: state too large to pack");
  hipLaunchKernelGGL(lstm_pack_state16_kernel, dim3(unsigned(cdiv<size_t>(n, 256))), dim3(256), 0, dev->stream, rows, B, v,
                     packed);
  DYHIP_CHECK_LAUNCH();
  return DYHIP_OK;
}

int dyhip_lstm_step_backward_packed(dyhip_device* dev, unsigned H, unsigned B, const float* packed_WhT16,
                                    const float* dpre_next_packed16, const float* gates, const float* c,
                                    const float* c_tm1, const float* dh, const float* dc, float* dpre, float* dc_tm1,
                                    float* dpre_packed16) {
  return dyhip_lstm_step_backward_packed_dropout(dev, H, B, packed_WhT16, dpre_next_packed16, gates, c, c_tm1, dh, dc,
                                                 nullptr, dpre, dc_tm1, dpre_packed16);
}

int dyhip_lstm_step_backward_packed_dropout(dyhip_device* dev, unsigned H, unsigned B, const float* packed_WhT16,
                                            const float* dpre_next_packed16, const float* gates, const float* c,
                                            const float* c_tm1, const float* dh, const float* dc, const float* mask_h,
                                            float* dpre, float* dc_tm1, float* dpre_packed16) {
  DYHIP_CHECK_DEV(dev);
  int ok = 0;
  dyhip_lstm_step_supported(dev, H, B, &ok);
  DYHIP_REQUIRE(ok, "LSTM step: unsupported hidden (%u) or batch (%u) size", H, B);
  DYHIP_REQUIRE(gates && c && dh && dpre, "LSTM step: null tensor pointer");
  DYHIP_REQUIRE(dpre_next_packed16 == nullptr || packed_WhT16 != nullptr, "LSTM step: packed weights and their operand come together");
  DYHIP_REQUIRE(all_aligned16({packed_WhT16, dpre_next_packed16}), "LSTM step: weights and operands must be 16-byte aligned");
  hipLaunchKernelGGL(lstm_step_bwd_kernel, dim3((H / 16) * cdiv<unsigned>(B, 32)), dim3(512), 0, dev->stream, H, B,
                     packed_WhT16, dpre_next_packed16, gates, c, c_tm1, dh, dc, dpre, dc_tm1, dpre_packed16, mask_h);
  DYHIP_CHECK_LAUNCH();
  return DYHIP_OK;
}

int dyhip_lstm_packed_state_floats(unsigned rows, unsigned B, size_t* floats) {
  DYHIP_REQUIRE(floats != nullptr, "null output pointer");
  *floats = packed_state_floats(rows, B);
  return DYHIP_OK;
}

int dyhip_lstm_pack_state(dyhip_device* dev, unsigned rows, unsigned B, const float* v, float* packed) {
  DYHIP_CHECK_DEV(dev);
  return pack_state(dev, rows, B, v, packed);
}

// x and h_tm1 are both packed or both plain (the plain form reads them with strided loads, no extra launch).
static int step_forward(dyhip_device* dev, unsigned I, unsigned H, unsigned B, const float* packed_Wx, const float* x,
                        const float* packed_Wh, const float* h_tm1, bool states_packed, const float* xproj,
                        const float* b, const float* c_tm1, int logistic_mode, float* gates, float* c, float* h,
                        float* hp_out, const float* mask_h = nullptr) {
  int ok = 0;
  dyhip_lstm_step_supported(dev, H, B, &ok);
  DYHIP_REQUIRE(ok, "LSTM step: unsupported hidden (%u) or batch (%u) size", H, B);
  DYHIP_REQUIRE(b && gates && c && h, "LSTM step: null tensor pointer");
  DYHIP_REQUIRE((packed_Wx == nullptr) == (x == nullptr) && (packed_Wh == nullptr) == (h_tm1 == nullptr),
                "LSTM step: packed weights and their operand come together");
  DYHIP_REQUIRE(packed_Wx == nullptr || step_depth_ok(I), "LSTM step: input size %u is not a multiple of 128", I);
  DYHIP_REQUIRE(all_aligned16({packed_Wx, x, packed_Wh, h_tm1, hp_out}),
                "LSTM step: weights and operands must be 16-byte aligned");
  DYHIP_REQUIRE(logistic_mode == DYHIP_LOGISTIC_PACKET || logistic_mode == DYHIP_LOGISTIC_SCALAR,
                "unknown logistic mode %d", logistic_mode);
  const StepOperand op0{packed_Wx, x, I}, op1{packed_Wh, h_tm1, H};
  // 64-row tiles (fewest operand bytes per CU) once they give half the CUs a block, 32-row tiles below that
  const unsigned blocks2 = (H / 16) * cdiv<unsigned>(B, 32);
  const bool two = blocks2 * 2 >= unsigned(dev->num_cus > 0 ? dev->num_cus : 256);
  const dim3 grid(two ? blocks2 : blocks2 * 2), block(two ? 512 : 256);
#define DYHIP_STEP(PLAIN, TILES)                                                                                     \
  hipLaunchKernelGGL((lstm_step_fwd_kernel<PLAIN, TILES>), grid, block, 0, dev->stream, H, B, op0, op1, xproj, b, c_tm1, \
                     logistic_mode, gates, c, h, hp_out, mask_h)
  if (states_packed) {
    if (two) DYHIP_STEP(false, 2);
    else DYHIP_STEP(false, 1);
  } else {
    if (two) DYHIP_STEP(true, 2);
    else DYHIP_STEP(true, 1);
  }
#undef DYHIP_STEP
  DYHIP_CHECK_LAUNCH();
  return DYHIP_OK;
}

int dyhip_lstm_step_forward(dyhip_device* dev, unsigned H, unsigned B, const float* packed_Wh, const float* h_tm1,
                            const float* xproj, const float* b, const float* c_tm1, int logistic_mode, float* gates,
                            float* c, float* h) {
  DYHIP_CHECK_DEV(dev);
  DYHIP_REQUIRE(packed_Wh && h_tm1 && xproj && c_tm1, "LSTM step: null tensor pointer");
  return step_forward(dev, 0, H, B, nullptr, nullptr, packed_Wh, h_tm1, false, xproj, b, c_tm1, logistic_mode, gates, c,
                      h, nullptr);
}

int dyhip_lstm_step_forward_packed(dyhip_device* dev, unsigned H, unsigned B, const float* packed_Wh,
                                   const float* h_tm1_packed, const float* xproj, const float* b, const float* c_tm1,
                                   int logistic_mode, float* gates, float* c, float* h, float* h_packed) {
  DYHIP_CHECK_DEV(dev);
  DYHIP_REQUIRE(xproj != nullptr, "LSTM step: null tensor pointer");
  DYHIP_REQUIRE((packed_Wh == nullptr) == (h_tm1_packed == nullptr) && (packed_Wh == nullptr) == (c_tm1 == nullptr),
                "LSTM step: the recurrent weights, the packed state and c_tm1 come together (all null = zero state)");
  return step_forward(dev, 0, H, B, nullptr, nullptr, packed_Wh, h_tm1_packed, true, xproj, b, c_tm1, logistic_mode,
                      gates, c, h, h_packed);
}

int dyhip_lstm_step_forward_packed_dropout(dyhip_device* dev, unsigned H, unsigned B, const float* packed_Wh,
                                           const float* h_tm1_packed, const float* xproj, const float* b,
                                           const float* c_tm1, const float* mask_h, int logistic_mode, float* gates,
                                           float* c, float* h, float* h_packed) {
  DYHIP_CHECK_DEV(dev);
  DYHIP_REQUIRE(xproj != nullptr, "LSTM step: null tensor pointer");
  DYHIP_REQUIRE((packed_Wh == nullptr) == (h_tm1_packed == nullptr) && (packed_Wh == nullptr) == (c_tm1 == nullptr),
                "LSTM step: the recurrent weights, the packed state and c_tm1 come together (all null = zero state)");
  return step_forward(dev, 0, H, B, nullptr, nullptr, packed_Wh, h_tm1_packed, true, xproj, b, c_tm1, logistic_mode,
                      gates, c, h, h_packed, mask_h);
}

int dyhip_lstm_step_forward_x(dyhip_device* dev, unsigned I, unsigned H, unsigned B, const float* packed_Wx,
                              const float* x, const float* packed_Wh, const float* h_tm1, const float* b,
                              const float* c_tm1, int logistic_mode, float* gates, float* c, float* h) {
  DYHIP_CHECK_DEV(dev);
  DYHIP_REQUIRE(packed_Wx && x, "LSTM step: null tensor pointer");
  return step_forward(dev, I, H, B, packed_Wx, x, packed_Wh, h_tm1, false, nullptr, b, c_tm1, logistic_mode, gates, c, h,
                      nullptr);
}

int dyhip_lstm_recurrent_backward_packed(dyhip_device* dev, unsigned H, unsigned B, const float* packed_WhT,
                                         const float* dpre_packed, void* ws, size_t ws_bytes, unsigned* splits) {
  DYHIP_CHECK_DEV(dev);
  int ok = 0;
  dyhip_lstm_step_supported(dev, H, B, &ok);
  DYHIP_REQUIRE(ok, "LSTM step: unsupported hidden (%u) or batch (%u) size", H, B);
  DYHIP_REQUIRE(packed_WhT && dpre_packed && ws && splits, "LSTM step: null pointer");
  return skinny_tn(dev, H, B, 4 * H, packed_WhT, 0, false, dpre_packed, 0, false, static_cast<float*>(ws), ws_bytes, splits);
}

int dyhip_lstm_cell_backward_packed(dyhip_device* dev, unsigned H, unsigned B, const float* gates, const float* c,
                                    const float* c_tm1, const float* dh, const float* rec, unsigned splits,
                                    const float* dc, float* dpre, float* dc_tm1, float* dpre_packed) {
  DYHIP_CHECK_DEV(dev);
  DYHIP_REQUIRE(dpre_packed == nullptr || (H % 8 == 0 && aligned16(dpre_packed)), "LSTM cell: packed dpre needs H %% 8 == 0");
  return cell_backward(dev, H, B, gates, c, c_tm1, dh, rec, splits, dc, dpre, dc_tm1, dpre_packed);
}

}  // extern "C"
