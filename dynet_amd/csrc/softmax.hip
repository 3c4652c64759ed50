// Row-wise log-sum-exp, PickNegLogSoftmax, the LogSumExp node and argmax.
//
// Replaces TensorTools::logsumexp_dev (dynet/tensor.cc:468-507: three Eigen
// launches that read x twice), PickNegLogSoftmax (dynet/nodes-pickneglogsoftmax.cc
// :79-145, which adds a pick kernel, an Eigen subtract, a full-size exp pass and
// an atomic subtract), LogSumExp (dynet/nodes-logsumexp.cc:38-97) and
// TensorTools::argmax_dev (dynet/tensor.cc:527-538).
//
// Layout: x is rows x bd, one softmax per batch element (column), contiguous.
// Forward reads every element exactly once: each thread keeps a running
// (max, sum of exp(x - max)) pair over its 128-bit slices, pairs are merged by
// wave butterfly and then across waves through LDS.  Backward is one
// elementwise read-modify-write pass with the one-hot subtraction folded in.
#include <cmath>
#include <vector>

#include "common.h"

namespace dyhip {

constexpr int kLseThreads = 1024;
constexpr int kLseWaves = kLseThreads / 64;

struct MaxSum {
  float m, s;
};

// The running maximum starts at the most negative finite float, never at -inf: a thread whose first
// values are all -inf (masked logits) then adds exp(-inf - finite) = 0 instead of exp(-inf + inf) = NaN.
// Any finite input is >= this start value, so the final maximum is exact; a column that holds nothing
// but -inf ends with s == 0 and is given the reference's result (m = -inf, z = NaN: its
// exp(x - m) is exp(NaN), dynet/tensor.cc:468-507) when the block writes its outputs.
constexpr float kLseStartMax = -3.402823466e+38f;

__device__ __forceinline__ void ms_push4(MaxSum& a, const float4 v) {
  const float cm = fmaxf(fmaxf(v.x, v.y), fmaxf(v.z, v.w));
  if (cm > a.m) {
    a.s *= __expf(a.m - cm);
    a.m = cm;
  }
  a.s += (__expf(v.x - a.m) + __expf(v.y - a.m)) + (__expf(v.z - a.m) + __expf(v.w - a.m));
}

__device__ __forceinline__ void ms_push1(MaxSum& a, const float v) {
  if (v > a.m) {
    a.s *= __expf(a.m - v);
    a.m = v;
  }
  a.s += __expf(v - a.m);
}

__device__ __forceinline__ MaxSum ms_merge(const MaxSum a, const MaxSum b) {
  MaxSum r;
  r.m = fmaxf(a.m, b.m);
  // both maxima are finite (see kLseStartMax), so neither exponent can be inf - inf
  r.s = a.s * __expf(a.m - r.m) + b.s * __expf(b.m - r.m);
  return r;
}

// One block per batch element.  Writes m[b], z[b]; if ids != nullptr also
// fx[b] = z[b] - x[ids[b]] (the pick of PickNegLogSoftmax).
template <bool VEC, bool NT>
__global__ __launch_bounds__(kLseThreads) void lse_cols_kernel(size_t rows, const float* __restrict__ x,
                                                               float* __restrict__ m_out, float* __restrict__ z_out,
                                                               const unsigned* __restrict__ ids,
                                                               float* __restrict__ fx) {
  __shared__ float lm[kLseWaves], ls[kLseWaves];
  const unsigned b = blockIdx.x;
  const float* px = x + size_t(b) * rows;
  MaxSum a;
  a.m = kLseStartMax;
  a.s = 0.f;
  // the picked logit is fetched up front so that its two dependent loads overlap the streaming pass
  float picked = 0.f;
  if (ids != nullptr && threadIdx.x == 0) picked = x[ids[b]];
  if (VEC) {
    // A column starts wherever b * rows falls: up to three leading elements bring it to a 16-byte boundary, the body
    // runs in 128-bit groups, up to three elements trail (taken by the last threads of the block).  With rows a
    // multiple of four and an aligned x there is only the body.
    const size_t head = min(size_t((4u - unsigned((reinterpret_cast<uintptr_t>(px) >> 2) & 3u)) & 3u), rows);
    const size_t n4 = (rows - head) >> 2;
    if (threadIdx.x < head) ms_push1(a, px[threadIdx.x]);
    {
      const size_t e = head + (n4 << 2) + (kLseThreads - 1 - threadIdx.x);
      if (e < rows) ms_push1(a, px[e]);
    }
    const float4* p4 = reinterpret_cast<const float4*>(px + head);
    size_t i = threadIdx.x;
    // eight independent 128-bit loads in flight per thread before the first exp
    for (; i + 7 * kLseThreads < n4; i += 8 * kLseThreads) {
      float4 v[8];
#pragma unroll
      for (int u = 0; u < 8; ++u) v[u] = ldg4<NT>(p4 + i + u * kLseThreads);
#pragma unroll
      for (int u = 0; u < 8; ++u) ms_push4(a, v[u]);
    }
    for (; i + 3 * kLseThreads < n4; i += 4 * kLseThreads) {
      const float4 v0 = ldg4<NT>(p4 + i), v1 = ldg4<NT>(p4 + i + kLseThreads),
                   v2 = ldg4<NT>(p4 + i + 2 * kLseThreads), v3 = ldg4<NT>(p4 + i + 3 * kLseThreads);
      ms_push4(a, v0);
      ms_push4(a, v1);
      ms_push4(a, v2);
      ms_push4(a, v3);
    }
    for (; i < n4; i += kLseThreads) ms_push4(a, ldg4<NT>(p4 + i));
  } else {
    for (size_t i = threadIdx.x; i < rows; i += kLseThreads) ms_push1(a, px[i]);
  }
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) {
    MaxSum o;
    o.m = __shfl_xor(a.m, off, kWave);
    o.s = __shfl_xor(a.s, off, kWave);
    a = ms_merge(a, o);
  }
  const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
  if (lane == 0) {
    lm[w] = a.m;
    ls[w] = a.s;
  }
  __syncthreads();
  if (w == 0) {
    // wave 0 merges the per-wave pairs with a butterfly over the first kLseWaves lanes
    MaxSum t;
    t.m = lane < kLseWaves ? lm[lane] : kLseStartMax;
    t.s = lane < kLseWaves ? ls[lane] : 0.f;
#pragma unroll
    for (int off = kLseWaves / 2; off > 0; off >>= 1) {
      MaxSum o;
      o.m = __shfl_xor(t.m, off, kWave);
      o.s = __shfl_xor(t.s, off, kWave);
      t = ms_merge(t, o);
    }
    if (lane == 0) {
      const bool empty = t.s == 0.f;  // every input was -inf
      const float z = empty ? NAN : logf(t.s) + t.m;
      if (empty) t.m = -INFINITY;
      m_out[b] = t.m;
      z_out[b] = z;
      if (ids != nullptr) fx[b] = z - picked;
    }
  }
}

// Short columns (rows <= 64 * U): one wavefront per column, four columns per block, every load of a column in flight
// at once.  A 1024-thread block per column of 33 rows (a tagger's label set over a large batch) is 1023 idle threads
// and a barrier per column: 337 us for 100 000 columns against 8 us here.
template <int U>
__global__ __launch_bounds__(256) void lse_cols_wave_kernel(unsigned rows, unsigned bd, const float* __restrict__ x,
                                                            float* __restrict__ m_out, float* __restrict__ z_out,
                                                            const unsigned* __restrict__ ids, float* __restrict__ fx) {
  const unsigned b = blockIdx.x * 4 + (threadIdx.x >> 6);
  if (b >= bd) return;  // whole wavefronts leave; the kernel has no barrier
  const int lane = threadIdx.x & 63;
  const float* px = x + size_t(b) * rows;
  float picked = 0.f;
  if (ids != nullptr && lane == 0) picked = x[ids[b]];
  float v[U];
#pragma unroll
  for (int u = 0; u < U; ++u) {
    const unsigned i = lane + 64 * u;
    v[u] = px[i < rows ? i : rows - 1];  // unconditional loads; a lane past the end does not push its value
  }
  MaxSum a;
  a.m = kLseStartMax;
  a.s = 0.f;
#pragma unroll
  for (int u = 0; u < U; ++u)
    if (lane + 64 * u < rows) ms_push1(a, v[u]);
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) {
    MaxSum o;
    o.m = __shfl_xor(a.m, off, kWave);
    o.s = __shfl_xor(a.s, off, kWave);
    a = ms_merge(a, o);
  }
  if (lane == 0) {
    const bool empty = a.s == 0.f;  // every input was -inf
    const float z = empty ? NAN : logf(a.s) + a.m;
    m_out[b] = empty ? -INFINITY : a.m;
    z_out[b] = z;
    if (ids != nullptr) fx[b] = z - picked;
  }
}

// Columns of at most 64 rows: one thread per column, eight loads in flight, no cross-lane step at all (with a
// wavefront per column the six merge steps of the butterfly, two exp each, cost more than the column's own terms:
// 23 us for 100 000 columns of 33 rows, vector-instruction bound).  A wavefront reads 64 neighbouring columns, i.e.
// one contiguous span, line by line through its L1.
__global__ __launch_bounds__(256) void lse_cols_thread_kernel(unsigned rows, unsigned bd, const float* __restrict__ x,
                                                              float* __restrict__ m_out, float* __restrict__ z_out,
                                                              const unsigned* __restrict__ ids, float* __restrict__ fx) {
  const unsigned b = blockIdx.x * 256 + threadIdx.x;
  if (b >= bd) return;
  const float* px = x + size_t(b) * rows;
  float picked = 0.f;
  if (ids != nullptr) picked = x[ids[b]];
  MaxSum a;
  a.m = kLseStartMax;
  a.s = 0.f;
  unsigned i = 0;
  for (; i + 8 <= rows; i += 8) {
    float v[8];
#pragma unroll
    for (int u = 0; u < 8; ++u) v[u] = px[i + u];
#pragma unroll
    for (int u = 0; u < 8; ++u) ms_push1(a, v[u]);
  }
  for (; i < rows; ++i) ms_push1(a, px[i]);
  const bool empty = a.s == 0.f;  // every input was -inf
  const float z = empty ? NAN : logf(a.s) + a.m;
  m_out[b] = empty ? -INFINITY : a.m;
  z_out[b] = z;
  if (ids != nullptr) fx[b] = z - picked;
}

// The backward pass over short columns, one wavefront per column as above.
template <int U, bool ACC>
__global__ __launch_bounds__(256) void pnls_bwd_wave_kernel(unsigned rows, unsigned bd, const float* __restrict__ x,
                                                            const float* __restrict__ z,
                                                            const unsigned* __restrict__ ids,
                                                            const float* __restrict__ dEdf, float* __restrict__ dEdx) {
  const unsigned b = blockIdx.x * 4 + (threadIdx.x >> 6);
  if (b >= bd) return;
  const int lane = threadIdx.x & 63;
  const size_t col0 = size_t(b) * rows;
  const float zb = z[b], dy = dEdf[b];
  const unsigned hot = unsigned(size_t(ids[b]) - col0);
  float xv[U], dv[U];
#pragma unroll
  for (int u = 0; u < U; ++u) {
    const unsigned i = lane + 64 * u, ic = i < rows ? i : rows - 1;
    xv[u] = x[col0 + ic];
    dv[u] = ACC ? dEdx[col0 + ic] : 0.f;
  }
#pragma unroll
  for (int u = 0; u < U; ++u) {
    const unsigned i = lane + 64 * u;
    if (i < rows) {
      float r = dv[u] + __expf(xv[u] - zb) * dy;
      if (i == hot) r -= dy;
      dEdx[col0 + i] = r;
    }
  }
}

constexpr unsigned kLseWaveMaxRows = 512;
constexpr int kPbThreads = 256;
constexpr int kPbUnroll = 4;

// dx[:, b] += exp(x[:, b] - z[b]) * dy[b]; dx[ids[b]] -= dy[b]   (ACC == false: = instead of +=)
template <bool VEC, bool NT, bool ACC>
__global__ __launch_bounds__(kPbThreads) void pnls_bwd_kernel(size_t rows, unsigned tiles_per_col,
                                                              const float* __restrict__ x,
                                                              const float* __restrict__ z,
                                                              const unsigned* __restrict__ ids,
                                                              const float* __restrict__ dEdf,
                                                              float* __restrict__ dEdx) {
  const unsigned b = blockIdx.x / tiles_per_col;
  const unsigned tile = blockIdx.x - b * tiles_per_col;
  const float zb = z[b], dy = dEdf[b];
  const size_t col0 = size_t(b) * rows;
  const size_t hot = size_t(ids[b]) - col0;  // row of the picked element
  if (VEC) {
    // x and dEdx start at the same offset from a 16-byte boundary (checked by the host): up to three leading elements,
    // a body of 128-bit groups, up to three trailing elements; the first tile's first and last threads take the ends
    const size_t head = min(size_t((4u - unsigned((reinterpret_cast<uintptr_t>(x + col0) >> 2) & 3u)) & 3u), rows);
    const size_t n4 = (rows - head) >> 2;
    if (tile == 0) {
      size_t e = rows;  // none
      if (threadIdx.x < head) e = threadIdx.x;
      else if (head + (n4 << 2) + (kPbThreads - 1 - threadIdx.x) < rows) e = head + (n4 << 2) + (kPbThreads - 1 - threadIdx.x);
      if (e < rows) {
        float r = (ACC ? dEdx[col0 + e] : 0.f) + __expf(x[col0 + e] - zb) * dy;
        if (e == hot) r -= dy;
        dEdx[col0 + e] = r;
      }
    }
    const bool hot_in_body = hot >= head && hot < head + (n4 << 2);
    const size_t hot_b = hot - head;  // index inside the body (only used when hot_in_body)
    const float4* x4 = reinterpret_cast<const float4*>(x + col0 + head);
    float4* d4 = reinterpret_cast<float4*>(dEdx + col0 + head);
    const size_t j0 = size_t(tile) * (kPbThreads * kPbUnroll) + threadIdx.x;
    float4 xv[kPbUnroll], dv[kPbUnroll];
#pragma unroll
    for (int u = 0; u < kPbUnroll; ++u) {
      const size_t j = j0 + size_t(u) * kPbThreads;
      if (j < n4) {
        xv[u] = ldg4<NT>(x4 + j);
        dv[u] = ACC ? d4[j] : make_float4(0.f, 0.f, 0.f, 0.f);
      }
    }
#pragma unroll
    for (int u = 0; u < kPbUnroll; ++u) {
      const size_t j = j0 + size_t(u) * kPbThreads;
      if (j < n4) {
        float4 r;
        r.x = dv[u].x + __expf(xv[u].x - zb) * dy;
        r.y = dv[u].y + __expf(xv[u].y - zb) * dy;
        r.z = dv[u].z + __expf(xv[u].z - zb) * dy;
        r.w = dv[u].w + __expf(xv[u].w - zb) * dy;
        if (hot_in_body && (hot_b >> 2) == j) {
          const unsigned c = hot_b & 3;
          if (c == 0) r.x -= dy;
          else if (c == 1) r.y -= dy;
          else if (c == 2) r.z -= dy;
          else r.w -= dy;
        }
        stg4<NT>(d4 + j, r);
      }
    }
  } else {
    const size_t j0 = size_t(tile) * (kPbThreads * kPbUnroll) + threadIdx.x;
#pragma unroll
    for (int u = 0; u < kPbUnroll; ++u) {
      const size_t j = j0 + size_t(u) * kPbThreads;
      if (j < rows) {
        float r = (ACC ? dEdx[col0 + j] : 0.f) + __expf(x[col0 + j] - zb) * dy;
        if (j == hot) r -= dy;
        dEdx[col0 + j] = r;
      }
    }
  }
}

// ---- LogSumExp node over k <= 8 arguments -----------------------------------
constexpr unsigned kLseNodeMaxArgs = 32;  // arguments a launch takes; more are chained (below)
struct LseNodeArgs {
  const float* x[kLseNodeMaxArgs];
  unsigned bcast;  // bit i: argument i has batch 1 and is indexed by e % n
  unsigned k;
  unsigned last;   // the launch that leaves the node's value (not a link of a chain)
};

__global__ __launch_bounds__(256) void lse_node_fwd_kernel(LseNodeArgs a, size_t n, size_t total,
                                                           float* __restrict__ fx) {
  const size_t e = size_t(blockIdx.x) * 256 + threadIdx.x;
  if (e >= total) return;
  const size_t j = e % n;
  // the arguments' values are fetched once, four at a time in flight, into a running (max, sum of exp) pair
  float m = -INFINITY, s = 0.f;
  for (unsigned i0 = 0; i0 < a.k; i0 += 4) {
    float v[4];
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const unsigned i = min(i0 + u, a.k - 1);
      v[u] = a.x[i][(a.bcast >> i) & 1u ? j : e];
    }
    float mg = v[0];
#pragma unroll
    for (int u = 1; u < 4; ++u)
      if (i0 + u < a.k) mg = fmaxf(mg, v[u]);
    const float mn = fmaxf(m, mg);
    // exp(-inf - -inf) would be NaN: a running maximum of -inf has no terms yet (or only -inf ones)
    float t = mn == -INFINITY ? 0.f : s * expf(m - mn);
#pragma unroll
    for (int u = 0; u < 4; ++u)
      if (i0 + u < a.k) t += mn == -INFINITY ? 1.f : expf(v[u] - mn);
    m = mn;
    s = t;
  }
  // arguments that are all -inf: the reference's exp(x - max) is exp(-inf + inf) = NaN there; a link of a chain keeps
  // -inf, which later finite arguments absorb
  fx[e] = (a.last != 0 && m == -INFINITY) ? __builtin_nanf("") : logf(s) + m;
}

// dxi[e] += exp(xi[e] - fx[e]) * dEdf[e]
__global__ __launch_bounds__(256) void lse_node_bwd_kernel(size_t total, const float* __restrict__ xi,
                                                           const float* __restrict__ fx,
                                                           const float* __restrict__ dEdf,
                                                           float* __restrict__ dEdxi) {
  const size_t e = size_t(blockIdx.x) * 256 + threadIdx.x;
  if (e < total) dEdxi[e] += expf(xi[e] - fx[e]) * dEdf[e];
}

// broadcast argument: tmp[b*n + j] = exp(xi[j] - fx[b*n+j]) * dEdf[b*n+j]
__global__ __launch_bounds__(256) void lse_node_bwd_bcast_kernel(size_t n, size_t total,
                                                                 const float* __restrict__ xi,
                                                                 const float* __restrict__ fx,
                                                                 const float* __restrict__ dEdf,
                                                                 float* __restrict__ tmp) {
  const size_t e = size_t(blockIdx.x) * 256 + threadIdx.x;
  if (e < total) tmp[e] = expf(xi[e % n] - fx[e]) * dEdf[e];
}

// The Argmax node's output (dynet/nodes-argmax.cc:44-55): 1 at each batch element's argmax, 0 elsewhere.  The
// reference copies the indices to the host and sets the ones one element at a time; here they never leave the device.
__global__ __launch_bounds__(256) void onehot_kernel(size_t rows, size_t total, const long long* __restrict__ idx,
                                                     float* __restrict__ fx) {
  const size_t e = size_t(blockIdx.x) * 256 + threadIdx.x;
  if (e < total) fx[e] = (long long)(e % rows) == idx[e / rows] ? 1.0f : 0.0f;
}

// ---- argmax along dim 0, first maximum ---------------------------------------
// (value, index) of the better of two candidates: the greater value, the lower index among equal values; an index of
// ~0 marks "none yet"
__device__ __forceinline__ void argmax_take(float& bv, unsigned long long& bi, float ov, unsigned long long oi) {
  if (oi != ~0ull && (bi == ~0ull || ov > bv || (ov == bv && oi < bi))) {
    bv = ov;
    bi = oi;
  }
}

// A thread's scan of elements first, first + step, ... of a column: eight loads in flight (one load and one compare
// a step is one memory round trip a step: 50 000 rows x 512 columns took 93 us, 1.1 TB/s); ascending order, so a
// strict > keeps the first maximum.  Entries past the end are fetched from the column's last row and skipped.
__device__ __forceinline__ void argmax_scan(const float* __restrict__ px, size_t rows, size_t first, size_t step, float& bv,
                                            unsigned long long& bi) {
  for (size_t i0 = first; i0 < rows; i0 += 8 * step) {
    float v[8];
#pragma unroll
    for (int u = 0; u < 8; ++u) {
      const size_t i = i0 + u * step;
      v[u] = px[i < rows ? i : rows - 1];
    }
#pragma unroll
    for (int u = 0; u < 8; ++u) {
      const size_t i = i0 + u * step;
      if (i < rows && (bi == ~0ull || v[u] > bv)) {
        bv = v[u];
        bi = i;
      }
    }
  }
}

__device__ __forceinline__ void argmax_wave(float& bv, unsigned long long& bi) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) {
    const float ov = __shfl_xor(bv, off, kWave);
    const unsigned long long oi = __shfl_xor(bi, off, kWave);
    argmax_take(bv, bi, ov, oi);
  }
}

// one block per column (columns of more than 2048 rows)
template <int T>
__global__ __launch_bounds__(T) void argmax_cols_kernel(size_t rows, const float* __restrict__ x,
                                                        long long* __restrict__ idx) {
  __shared__ float lv[T / 64];
  __shared__ unsigned long long li[T / 64];
  const float* px = x + size_t(blockIdx.x) * rows;
  float bv = -INFINITY;
  unsigned long long bi = ~0ull;
  argmax_scan(px, rows, threadIdx.x, T, bv, bi);
  argmax_wave(bv, bi);
  const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
  if (lane == 0) {
    lv[w] = bv;
    li[w] = bi;
  }
  __syncthreads();
  if (threadIdx.x == 0) {
    for (int k = 1; k < T / 64; ++k) argmax_take(bv, bi, lv[k], li[k]);
    idx[blockIdx.x] = static_cast<long long>(bi);
  }
}

// one wavefront per column (33..2048 rows), four columns a block
__global__ __launch_bounds__(256) void argmax_cols_wave_kernel(size_t rows, unsigned cols, const float* __restrict__ x,
                                                               long long* __restrict__ idx) {
  const unsigned c = blockIdx.x * 4 + (threadIdx.x >> 6);
  if (c >= cols) return;
  float bv = -INFINITY;
  unsigned long long bi = ~0ull;
  argmax_scan(x + size_t(c) * rows, rows, threadIdx.x & 63, 64, bv, bi);
  argmax_wave(bv, bi);
  if ((threadIdx.x & 63) == 0) idx[c] = static_cast<long long>(bi);
}

// one thread per column (at most 32 rows: a block per column left 252 of 256 threads idle on 4-row columns)
__global__ __launch_bounds__(256) void argmax_cols_thread_kernel(size_t rows, unsigned cols, const float* __restrict__ x,
                                                                 long long* __restrict__ idx) {
  const unsigned c = blockIdx.x * 256 + threadIdx.x;
  if (c >= cols) return;
  float bv = -INFINITY;
  unsigned long long bi = ~0ull;
  argmax_scan(x + size_t(c) * rows, rows, 0, 1, bv, bi);
  idx[c] = static_cast<long long>(bi);
}

static void launch_argmax_cols(dyhip_device* dev, size_t rows, unsigned bd, const float* x, long long* idx);

static void launch_argmax_cols_blocks(dyhip_device* dev, size_t rows, unsigned bd, const float* x, long long* idx) {
  if (rows <= 32)
    hipLaunchKernelGGL(argmax_cols_thread_kernel, dim3(cdiv<unsigned>(bd, 256)), dim3(256), 0, dev->stream, rows, bd, x, idx);
  else if (rows <= 2048)
    hipLaunchKernelGGL(argmax_cols_wave_kernel, dim3(cdiv<unsigned>(bd, 4)), dim3(256), 0, dev->stream, rows, bd, x, idx);
  else if (rows <= 8192)
    hipLaunchKernelGGL(argmax_cols_kernel<256>, dim3(bd), dim3(256), 0, dev->stream, rows, x, idx);
  else
    hipLaunchKernelGGL(argmax_cols_kernel<1024>, dim3(bd), dim3(1024), 0, dev->stream, rows, x, idx);
}

// ---- columns of a vocabulary's length in a batch of a few (decoding, a batch of one): a block per column is a handful
// of blocks (100 000 x 1: 8.4 us for the log-sum-exp, 12.7 us for the softmax backward's dot, 300 000 x 2: 20 / 34 us,
// a million rows: 57 / 114 us and 76 us for the argmax).  The column is cut into chunks of kColChunk rows over
// (chunks, columns) blocks of 256 threads; a chunk leaves its (max, sum of exp), its sum of a * b or its first maximum
// in the device's scratch, and a wavefront per column merges the chunks in ascending order. -------------------------
constexpr unsigned kColChunk = 8192;
constexpr size_t kColChunkMinRows = 65536;

static bool col_chunked(const dyhip_device* dev, size_t rows, unsigned cols, unsigned* chunks) {
  const size_t cus = dev->num_cus > 0 ? size_t(dev->num_cus) : 256, c = cdiv<size_t>(rows, kColChunk);
  *chunks = static_cast<unsigned>(c);
  return rows >= kColChunkMinRows && size_t(cols) * 4 <= cus && c <= 0xFFFFFFu && dev->gemm_ws != nullptr &&
         dev->gemm_ws_bytes >= 2 * sizeof(float) * c * cols + 256;
}

// MODE 0: (max, sum exp(x - max))   1: sum a * (b ? b : 1)   2: first maximum (value, row as two 32-bit halves)
template <int MODE>
__global__ __launch_bounds__(256) void col_chunk_kernel(size_t rows, const float* __restrict__ a,
                                                        const float* __restrict__ b, float* __restrict__ part) {
  __shared__ float l0[4], l1[4];
  __shared__ unsigned long long li[4];
  const size_t r0 = size_t(blockIdx.x) * kColChunk, r1 = min(rows, r0 + kColChunk);
  const float* pa = a + size_t(blockIdx.y) * rows;
  const float* pb = MODE == 1 && b != nullptr ? b + size_t(blockIdx.y) * rows : nullptr;
  constexpr int U = 8;
  MaxSum ms;
  ms.m = kLseStartMax;
  ms.s = 0.f;
  float dot = 0.f, bv = -INFINITY;
  unsigned long long bi = ~0ull;
  for (size_t i0 = r0 + threadIdx.x; i0 < r1; i0 += size_t(U) * 256) {
    float x[U], y[U];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const size_t i = min(i0 + size_t(u) * 256, r1 - 1);  // clamped, masked below
      x[u] = pa[i];
      y[u] = pb != nullptr ? pb[i] : 1.f;
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const size_t i = i0 + size_t(u) * 256;
      if (i >= r1) continue;
      if (MODE == 0) ms_push1(ms, x[u]);
      else if (MODE == 1) dot += pb != nullptr ? x[u] * y[u] : x[u];
      else if (bi == ~0ull || x[u] > bv) {
        bv = x[u];
        bi = i;
      }
    }
  }
  const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
  const size_t at = size_t(blockIdx.y) * gridDim.x + blockIdx.x;
  if (MODE == 0) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
      MaxSum o;
      o.m = __shfl_xor(ms.m, off, kWave);
      o.s = __shfl_xor(ms.s, off, kWave);
      ms = ms_merge(ms, o);
    }
    if (lane == 0) {
      l0[w] = ms.m;
      l1[w] = ms.s;
    }
    __syncthreads();
    if (threadIdx.x == 0) {
      for (int k = 1; k < 4; ++k) {
        MaxSum o;
        o.m = l0[k];
        o.s = l1[k];
        ms = ms_merge(ms, o);
      }
      part[2 * at] = ms.m;
      part[2 * at + 1] = ms.s;
    }
  } else if (MODE == 1) {
    const float t = block_sum<4>(dot, l0);
    if (threadIdx.x == 0) part[at] = t;
  } else {
    argmax_wave(bv, bi);
    if (lane == 0) {
      l0[w] = bv;
      li[w] = bi;
    }
    __syncthreads();
    if (threadIdx.x == 0) {
      for (int k = 1; k < 4; ++k) argmax_take(bv, bi, l0[k], li[k]);
      part[2 * at] = bv;
      reinterpret_cast<unsigned*>(part)[2 * at + 1] = static_cast<unsigned>(bi - r0);  // row inside the chunk
    }
  }
}

// one wavefront per column: lane l merges chunks l, l + 64, ... in ascending order, then the lanes merge
template <int MODE>
__global__ __launch_bounds__(64) void col_finish_kernel(size_t rows, unsigned chunks, const float* __restrict__ part,
                                                        const float* __restrict__ x, const unsigned* __restrict__ ids,
                                                        float* __restrict__ out0, float* __restrict__ out1,
                                                        float* __restrict__ fx, long long* __restrict__ idx) {
  const unsigned b = blockIdx.x, lane = threadIdx.x;
  const float* p = part + size_t(b) * chunks * (MODE == 1 ? 1 : 2);
  if (MODE == 0) {
    float picked = 0.f;
    if (ids != nullptr && lane == 0) picked = x[ids[b]];
    MaxSum t;
    t.m = kLseStartMax;
    t.s = 0.f;
    for (unsigned c = lane; c < chunks; c += 64) {
      MaxSum o;
      o.m = p[2 * c];
      o.s = p[2 * c + 1];
      t = ms_merge(t, o);
    }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
      MaxSum o;
      o.m = __shfl_xor(t.m, off, kWave);
      o.s = __shfl_xor(t.s, off, kWave);
      t = ms_merge(t, o);
    }
    if (lane == 0) {
      const bool empty = t.s == 0.f;  // every input was -inf
      const float z = empty ? NAN : logf(t.s) + t.m;
      out0[b] = empty ? -INFINITY : t.m;
      out1[b] = z;
      if (ids != nullptr) fx[b] = z - picked;
    }
  } else if (MODE == 1) {
    float s = 0.f;
    for (unsigned c = lane; c < chunks; c += 64) s += p[c];
    s = wave_sum(s);
    if (lane == 0) out0[b] = s;
  } else {
    float bv = -INFINITY;
    unsigned long long bi = ~0ull;
    for (unsigned c = lane; c < chunks; c += 64) {
      const float v = p[2 * c];
      const unsigned long long i = size_t(c) * kColChunk + reinterpret_cast<const unsigned*>(p)[2 * c + 1];
      argmax_take(bv, bi, v, i);
    }
    argmax_wave(bv, bi);
    if (lane == 0) idx[b] = static_cast<long long>(bi);
  }
  (void)rows;
}

static void launch_argmax_cols(dyhip_device* dev, size_t rows, unsigned bd, const float* x, long long* idx) {
  unsigned chunks = 0;
  if (col_chunked(dev, rows, bd, &chunks)) {
    float* part = static_cast<float*>(dev->gemm_ws);
    hipLaunchKernelGGL(col_chunk_kernel<2>, dim3(chunks, bd), dim3(256), 0, dev->stream, rows, x, nullptr, part);
    hipLaunchKernelGGL(col_finish_kernel<2>, dim3(bd), dim3(64), 0, dev->stream, rows, chunks, part, nullptr, nullptr,
                       nullptr, nullptr, nullptr, idx);
    return;
  }
  launch_argmax_cols_blocks(dev, rows, bd, x, idx);
}

int batch_reduce(dyhip_device* dev, size_t n, unsigned bd, const float* in0, const float* in1, float* out,
                 bool accumulate, void* ws, size_t ws_bytes);

static int launch_lse(dyhip_device* dev, size_t rows, unsigned bd, const float* x, float* m, float* z,
                      const unsigned* ids, float* fx) {
  if (rows <= kLseWaveMaxRows) {
    const dim3 grid(cdiv<unsigned>(bd, 4)), block(256);
    const unsigned r = static_cast<unsigned>(rows);
#define DYHIP_LSE_WAVE(U) hipLaunchKernelGGL(lse_cols_wave_kernel<U>, grid, block, 0, dev->stream, r, bd, x, m, z, ids, fx)
    if (r <= 64)
      hipLaunchKernelGGL(lse_cols_thread_kernel, dim3(cdiv<unsigned>(bd, 256)), block, 0, dev->stream, r, bd, x, m, z, ids, fx);
    else if (r <= 128) DYHIP_LSE_WAVE(2);
    else if (r <= 256) DYHIP_LSE_WAVE(4);
    else DYHIP_LSE_WAVE(8);
#undef DYHIP_LSE_WAVE
    DYHIP_CHECK_LAUNCH();
    return DYHIP_OK;
  }
  unsigned chunks = 0;
  if (col_chunked(dev, rows, bd, &chunks)) {
    float* part = static_cast<float*>(dev->gemm_ws);
    hipLaunchKernelGGL(col_chunk_kernel<0>, dim3(chunks, bd), dim3(256), 0, dev->stream, rows, x, nullptr, part);
    hipLaunchKernelGGL(col_finish_kernel<0>, dim3(bd), dim3(64), 0, dev->stream, rows, chunks, part, x, ids, m, z, fx,
                       nullptr);
    DYHIP_CHECK_LAUNCH();
    return DYHIP_OK;
  }
  const bool vec = true;  // any column: its ends are peeled off around a body of 128-bit groups
  const bool stream = rows * size_t(bd) * sizeof(float) >= dev->stream_threshold;
  if (vec && stream)
    hipLaunchKernelGGL((lse_cols_kernel<true, true>), dim3(bd), dim3(kLseThreads), 0, dev->stream, rows, x, m, z, ids, fx);
  else if (vec)
    hipLaunchKernelGGL((lse_cols_kernel<true, false>), dim3(bd), dim3(kLseThreads), 0, dev->stream, rows, x, m, z, ids, fx);
  else
    hipLaunchKernelGGL((lse_cols_kernel<false, false>), dim3(bd), dim3(kLseThreads), 0, dev->stream, rows, x, m, z, ids, fx);
  DYHIP_CHECK_LAUNCH();
  return DYHIP_OK;
}

// ---- Softmax / LogSoftmax over dim 0 ---------------------------------------------------
// Column statistics come from lse_cols_kernel (forward) or col_dot_kernel (backward); the
// element pass is one kernel over (column, tile) with the column's scalars read once per block.
constexpr int kSmThreads = 256;
constexpr int kSmUnroll = 4;

// red[c] = sum_i a[i,c] * (b ? b[i,c] : 1), one block per column, fixed summation tree
constexpr int kColDotThreads = 1024;  // columns of more than 16 384 rows: 256 threads walked 50 000 rows x 20 columns in 20 us
__global__ __launch_bounds__(kColDotThreads) void col_dot_kernel(size_t rows, const float* __restrict__ a,
                                                               const float* __restrict__ b, float* __restrict__ red) {
  __shared__ float sh[kColDotThreads / 64];
  const size_t c0 = size_t(blockIdx.x) * rows;
  // eight loads in flight a thread (a loop of one load and one add runs one memory round trip per step: 50 000 rows
  // x 20 columns took 59 us); entries past the end are fetched from the column's last row and not added
  float s = 0.f;
  for (size_t i0 = threadIdx.x; i0 < rows; i0 += size_t(kColDotThreads) * 4) {
    float x[4], y[4];
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const size_t i = i0 + size_t(u) * kColDotThreads, ic = i < rows ? i : rows - 1;
      x[u] = a[c0 + ic];
      y[u] = b ? b[c0 + ic] : 1.f;
    }
#pragma unroll
    for (int u = 0; u < 4; ++u)
      if (i0 + size_t(u) * kColDotThreads < rows) s += b ? x[u] * y[u] : x[u];
  }
  const float t = block_sum<kColDotThreads / 64>(s, sh);
  if (threadIdx.x == 0) red[blockIdx.x] = t;
}

static void launch_col_dot(dyhip_device* dev, size_t rows, unsigned cols, const float* a, const float* b, float* red) {
  unsigned chunks = 0;
  if (col_chunked(dev, rows, cols, &chunks)) {
    float* part = static_cast<float*>(dev->gemm_ws);
    hipLaunchKernelGGL(col_chunk_kernel<1>, dim3(chunks, cols), dim3(256), 0, dev->stream, rows, a, b, part);
    hipLaunchKernelGGL(col_finish_kernel<1>, dim3(cols), dim3(64), 0, dev->stream, rows, chunks, part, nullptr, nullptr, red,
                       nullptr, nullptr, nullptr);
    return;
  }
  hipLaunchKernelGGL(col_dot_kernel, dim3(cols), dim3(kColDotThreads), 0, dev->stream, rows, a, b, red);
}

template <int MODE>
__global__ __launch_bounds__(kSmThreads) void col_apply_kernel(size_t rows, unsigned tiles_per_col,
                                                              const float* __restrict__ a,
                                                              const float* __restrict__ b,
                                                              const float* __restrict__ s0,
                                                              const float* __restrict__ s1, float* __restrict__ out) {
  const unsigned c = blockIdx.x / tiles_per_col, tile = blockIdx.x - c * tiles_per_col;
  const size_t c0 = size_t(c) * rows;
  const float p0 = s0[c];
  const float p1 = MODE == 0 ? expf(p0 - s1[c]) : 0.f;
  const size_t i0 = size_t(tile) * kSmThreads * kSmUnroll + threadIdx.x;
  // every load of the tile first, on indices clamped into the column (loads inside the per-element branch wait for
  // one another: 50 000 rows x 20 columns backward 25 us)
  float va[kSmUnroll], vb[kSmUnroll], vo[kSmUnroll];
#pragma unroll
  for (int u = 0; u < kSmUnroll; ++u) {
    const size_t i = i0 + size_t(u) * kSmThreads, e = c0 + (i < rows ? i : rows - 1);
    va[u] = a[e];
    vb[u] = MODE >= 2 ? b[e] : 0.f;
    vo[u] = MODE >= 2 ? out[e] : 0.f;
  }
#pragma unroll
  for (int u = 0; u < kSmUnroll; ++u) {
    const size_t i = i0 + size_t(u) * kSmThreads;
    if (i >= rows) break;
    const size_t e = c0 + i;
    if (MODE == 0) out[e] = expf(va[u] - p0) * p1;
    else if (MODE == 1) out[e] = va[u] - p0;
    else if (MODE == 2) out[e] = vo[u] + (vb[u] - p0) * va[u];
    else out[e] = vo[u] + ((expf(va[u]) * -p0) + vb[u]);
  }
}

template <int MODE>
static int launch_col_apply(dyhip_device* dev, size_t rows, unsigned cols, const float* a, const float* b,
                            const float* s0, const float* s1, float* out) {
  const size_t tiles = cdiv<size_t>(rows, size_t(kSmThreads) * kSmUnroll);
  DYHIP_REQUIRE(tiles * cols < (size_t(1) << 31), "softmax launch too large");
  hipLaunchKernelGGL(col_apply_kernel<MODE>, dim3(static_cast<unsigned>(tiles * cols)), dim3(kSmThreads), 0, dev->stream,
                     rows, static_cast<unsigned>(tiles), a, b, s0, s1, out);
  DYHIP_CHECK_LAUNCH();
  return DYHIP_OK;
}

// ---- Softmax / LogSoftmax over dim 0 with the column held in registers: ONE kernel, the column read once -----------
// T threads own a column (a wavefront for columns of up to 512 rows, four columns to a block; a block of 256 threads up
// to 4096 rows, of 1024 threads up to 16384), thread t holding rows t, t + T, ... (U of them), so that every access of
// the group is one contiguous run.  The statistics-then-apply pair of kernels below reads the column twice (forward)
// or three times (backward) and launches twice; it remains for longer columns.  Same formulas as that pair, MODE as
// in col_apply_kernel; MODE 0 / 1 also leave z (and m) where the pair leaves them.
template <int T>
__device__ __forceinline__ float sm_group_sum(float v, float* red) {
  if (T == 64) return wave_sum(v);
  return block_sum<(T >= 64 ? T / 64 : 1)>(v, red);
}
template <int T>
__device__ __forceinline__ float sm_group_max(float v, float* red) {
  if (T == 64) return wave_max(v);
  return block_max<(T >= 64 ? T / 64 : 1)>(v, red);
}

template <int MODE, int T, int U>
__global__ __launch_bounds__(T == 64 ? 256 : T) void softmax_resident_kernel(unsigned rows, unsigned cols,
                                                                            const float* __restrict__ a,
                                                                            const float* __restrict__ b,
                                                                            float* __restrict__ s0, float* __restrict__ s1,
                                                                            float* __restrict__ out) {
  __shared__ float red[16];
  const unsigned c = T == 64 ? blockIdx.x * 4 + (threadIdx.x >> 6) : blockIdx.x;
  if (c >= cols) return;  // T == 64: whole wavefronts leave and that form has no barrier; else c == blockIdx.x < cols
  const unsigned t = T == 64 ? (threadIdx.x & 63) : threadIdx.x;
  const size_t c0 = size_t(c) * rows;
  float av[U], bv[U], ov[U];
#pragma unroll
  for (int u = 0; u < U; ++u) {
    const unsigned i = t + T * u, ic = i < rows ? i : rows - 1;  // unconditional loads; rows past the end are masked
    av[u] = a[c0 + ic];
    if (MODE >= 2) {
      bv[u] = b[c0 + ic];
      ov[u] = out[c0 + ic];
    }
  }
  if (MODE == 0 || MODE == 1) {
    float mx = -INFINITY;
#pragma unroll
    for (int u = 0; u < U; ++u)
      if (t + T * u < rows) mx = av[u] > mx ? av[u] : mx;
    const float m = sm_group_max<T>(mx, red);
    float e[U], sum = 0.f;
#pragma unroll
    for (int u = 0; u < U; ++u) {
      e[u] = expf(av[u] - m);
      if (t + T * u < rows) sum += e[u];
    }
    const float z = logf(sm_group_sum<T>(sum, red)) + m;
    if (t == 0) {
      s0[c] = z;
      if (s1 != nullptr) s1[c] = m;
    }
    const float p1 = expf(m - z);
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const unsigned i = t + T * u;
      if (i < rows) out[c0 + i] = MODE == 0 ? e[u] * p1 : av[u] - z;
    }
  } else {
    float part = 0.f;
#pragma unroll
    for (int u = 0; u < U; ++u)
      if (t + T * u < rows) part += MODE == 2 ? av[u] * bv[u] : bv[u];
    const float r = sm_group_sum<T>(part, red);
    if (t == 0 && s0 != nullptr) s0[c] = r;
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const unsigned i = t + T * u;
      if (i < rows) out[c0 + i] = MODE == 2 ? ov[u] + (bv[u] - r) * av[u] : ov[u] + ((expf(av[u]) * -r) + bv[u]);
    }
  }
}

constexpr size_t kSmResidentMaxRows = 16384;

// true: the column-resident kernel was launched
template <int MODE>
static bool launch_softmax_resident(dyhip_device* dev, size_t rows, unsigned cols, const float* a, const float* b,
                                    float* s0, float* s1, float* out) {
  if (rows > kSmResidentMaxRows) return false;
  const unsigned r = static_cast<unsigned>(rows);
#define DYHIP_SM(T, U, GRID)                                                                                           \
  hipLaunchKernelGGL((softmax_resident_kernel<MODE, T, U>), dim3(GRID), dim3(T == 64 ? 256 : T), 0, dev->stream, r, cols, \
                     a, b, s0, s1, out)
  const unsigned g4 = cdiv<unsigned>(cols, 4);
  if (r <= 64) DYHIP_SM(64, 1, g4);
  else if (r <= 128) DYHIP_SM(64, 2, g4);
  else if (r <= 256) DYHIP_SM(64, 4, g4);
  else if (r <= 512) DYHIP_SM(64, 8, g4);
  else if (r <= 1024) DYHIP_SM(256, 4, cols);
  else if (r <= 2048) DYHIP_SM(256, 8, cols);
  else if (r <= 4096) DYHIP_SM(256, 16, cols);
  else if (r <= 8192) DYHIP_SM(1024, 8, cols);
  else DYHIP_SM(1024, 16, cols);
#undef DYHIP_SM
  return true;
}

// ---- reductions along dim 1 (Softmax with dimension 1, LogSumExpDimension) --------------------------------
// x is rows x cols column-major per batch element.  A block is 64 lanes (consecutive rows: coalesced) x
// kRowWaves waves (wave w takes columns w, w + kRowWaves, ...); the per-row maximum, then the per-row sum of
// exp(x - max), cross the waves through LDS, the sum in ascending wave order.  The second read of x comes
// from cache for all but very large matrices.
constexpr int kRowWaves = 8;

// MODE 0: m_out = max, z_out = log(sum) + max     (TensorTools::logsumexp_dev along axis 1)
// MODE 1: out = exp(x - max) / sum                (Softmax forward, dimension 1)
// MODE 2: out += (b - sum_j a*b) * a              (Softmax backward, dimension 1; a = fx, b = dEdf)
template <int MODE, int U>  // U: loads in flight a thread and pass (2 for few columns a thread, 8 otherwise)
__global__ __launch_bounds__(64 * kRowWaves) void rowwise_kernel(unsigned rows, unsigned cols, unsigned bd, unsigned rw_shift,
                                                                 const float* __restrict__ a,
                                                                 const float* __restrict__ b,
                                                                 float* __restrict__ m_out, float* __restrict__ out) {
  __shared__ float red[kRowWaves][64];
  // A wavefront's lanes: RW = 2^rw_shift consecutive rows x 64 / RW columns (matrices of fewer than 64 rows would
  // leave lanes idle: 3 rows x 50 000 columns took 1.8 ms).  U loads in flight a thread in every pass, on column
  // indices clamped into the matrix (one load and one compare a step is one memory round trip a step).
  const unsigned lane = threadIdx.x & 63, w = threadIdx.x >> 6;
  const unsigned RW = 1u << rw_shift, nsub = 64u >> rw_shift, rl = lane & (RW - 1), sub = lane >> rw_shift;
  const unsigned stride = kRowWaves * nsub, j0 = w * nsub + sub;
  const unsigned row = blockIdx.x * RW + rl;
  const bool live = row < rows;
  const unsigned rowc = live ? row : rows - 1;
  for (unsigned bi = blockIdx.y; bi < bd; bi += gridDim.y) {
    const size_t base = size_t(bi) * rows * cols + rowc;
    float mx = -INFINITY;
    if (MODE != 2) {
      for (unsigned j = j0; j < cols; j += U * stride) {
        float v[U];
#pragma unroll
        for (int u = 0; u < U; ++u) v[u] = a[base + size_t(min(j + u * stride, cols - 1)) * rows];
#pragma unroll
        for (int u = 0; u < U; ++u)
          if (j + u * stride < cols) mx = v[u] > mx ? v[u] : mx;  // a NaN entry is skipped here and turns the row's sum into NaN below
      }
      red[w][lane] = mx;
      __syncthreads();
      mx = -INFINITY;
      for (unsigned k = 0; k < kRowWaves; ++k)
        for (unsigned s2 = 0; s2 < nsub; ++s2) {
          const float o = red[k][(s2 << rw_shift) + rl];
          mx = o > mx ? o : mx;
        }
      __syncthreads();
    }
    float s = 0.f;
    for (unsigned j = j0; j < cols; j += U * stride) {
      float v[U], y[U];
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const size_t e = base + size_t(min(j + u * stride, cols - 1)) * rows;
        v[u] = a[e];
        y[u] = MODE == 2 ? b[e] : 0.f;
      }
#pragma unroll
      for (int u = 0; u < U; ++u)
        if (j + u * stride < cols) s += MODE == 2 ? v[u] * y[u] : expf(v[u] - mx);
    }
    red[w][lane] = s;
    __syncthreads();
    s = 0.f;
    for (unsigned k = 0; k < kRowWaves; ++k)
      for (unsigned s2 = 0; s2 < nsub; ++s2) s += red[k][(s2 << rw_shift) + rl];
    __syncthreads();
    if (MODE == 0) {
      if (live && w == 0 && sub == 0) {
        m_out[size_t(bi) * rows + row] = mx;
        out[size_t(bi) * rows + row] = logf(s) + mx;
      }
    } else {
      for (unsigned j = j0; j < cols; j += U * stride) {
        float v[U], y[U], o[U];
#pragma unroll
        for (int u = 0; u < U; ++u) {
          const size_t e = base + size_t(min(j + u * stride, cols - 1)) * rows;
          v[u] = a[e];
          y[u] = MODE == 2 ? b[e] : 0.f;
          o[u] = MODE == 2 ? out[e] : 0.f;
        }
#pragma unroll
        for (int u = 0; u < U; ++u) {
          if (!live || j + u * stride >= cols) continue;
          const size_t e = base + size_t(j + u * stride) * rows;
          if (MODE == 1) out[e] = expf(v[u] - mx) / s;
          else out[e] = o[u] + (y[u] - s) * v[u];
        }
      }
    }
  }
}

// ---- the same three when rows x bd gives that kernel fewer blocks than the device has CUs (512 x 512 x 8: 64 blocks,
// 0.8 TB/s; 2048 x 2048: 32 blocks) --------------------------------------------------------------------------------
// The columns are cut into slabs over gridDim.y as well.  rows_slab_kernel leaves, per row and slab, the running
// (maximum, sum of exp(x - maximum)) of one pass over the slab (DOT: the slab's sum of a * b); rows_finish_kernel
// merges a row's slabs (the block's threads share them out and meet in LDS) and writes its own slab of the output,
// or the row's (max, log-sum-exp) from a grid with gridDim.y == 1.  Lane layout as in rowwise_kernel with four waves.
constexpr int kSlabWaves = 4;

// (m, s) of every thread of the block merged per row; every thread leaves with its row's pair.  A thread that saw
// nothing brings (-inf, 0); a NaN sum stays NaN whatever its maximum.
__device__ __forceinline__ void rows_merge(float& m, float& s, float (*red_m)[64], float (*red_s)[64], unsigned w,
                                           unsigned lane, unsigned rw_shift, unsigned rl, bool dot) {
  red_m[w][lane] = m;
  red_s[w][lane] = s;
  __syncthreads();
  const unsigned nsub = 64u >> rw_shift;
  float mm = -INFINITY;
  if (!dot)
    for (unsigned k = 0; k < kSlabWaves; ++k)
      for (unsigned s2 = 0; s2 < nsub; ++s2) {
        const float o = red_m[k][(s2 << rw_shift) + rl];
        mm = o > mm ? o : mm;
      }
  const float ref = mm > -INFINITY ? mm : 0.f;
  float ss = 0.f;
  for (unsigned k = 0; k < kSlabWaves; ++k)
    for (unsigned s2 = 0; s2 < nsub; ++s2) {
      const unsigned at = (s2 << rw_shift) + rl;
      ss += dot ? red_s[k][at] : red_s[k][at] * expf(red_m[k][at] - ref);
    }
  __syncthreads();
  m = mm;
  s = ss;
}

template <bool DOT>
__global__ __launch_bounds__(64 * kSlabWaves) void rows_slab_kernel(unsigned rows, unsigned cols, unsigned rw_shift,
                                                                   unsigned slab, const float* __restrict__ a,
                                                                   const float* __restrict__ b,
                                                                   float* __restrict__ part_m, float* __restrict__ part_s) {
  __shared__ float red_m[kSlabWaves][64], red_s[kSlabWaves][64];
  constexpr int U = 8;
  const unsigned lane = threadIdx.x & 63, w = threadIdx.x >> 6;
  const unsigned RW = 1u << rw_shift, nsub = 64u >> rw_shift, rl = lane & (RW - 1), sub = lane >> rw_shift;
  const unsigned stride = kSlabWaves * nsub;
  const unsigned row = blockIdx.x * RW + rl;
  const bool live = row < rows;
  const unsigned c0 = blockIdx.y * slab, c1 = min(cols, c0 + slab);
  const size_t base = size_t(blockIdx.z) * rows * cols + (live ? row : rows - 1);
  float m = -INFINITY, s = 0.f;
  for (unsigned j = c0 + w * nsub + sub; j < c1; j += U * stride) {
    float v[U], y[U];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const size_t e = base + size_t(min(j + u * stride, c1 - 1)) * rows;
      v[u] = a[e];
      y[u] = DOT ? b[e] : 0.f;
    }
    if (DOT) {
#pragma unroll
      for (int u = 0; u < U; ++u)
        if (j + u * stride < c1) s += v[u] * y[u];
    } else {
      float lm = m;
#pragma unroll
      for (int u = 0; u < U; ++u)
        if (j + u * stride < c1) lm = v[u] > lm ? v[u] : lm;  // a NaN entry is skipped here and makes the sum NaN below
      const float ref = lm > -INFINITY ? lm : 0.f;
      s *= expf(m - ref);
#pragma unroll
      for (int u = 0; u < U; ++u)
        if (j + u * stride < c1) s += expf(v[u] - ref);
      m = lm;
    }
  }
  rows_merge(m, s, red_m, red_s, w, lane, rw_shift, rl, DOT);
  if (live && w == 0 && sub == 0) {
    const size_t at = (size_t(blockIdx.z) * gridDim.y + blockIdx.y) * rows + row;
    if (!DOT) part_m[at] = m;
    part_s[at] = s;
  }
}

// MODE as in rowwise_kernel; nslabs: slabs the partial results hold per row (gridDim.y of the slab kernel)
template <int MODE>
__global__ __launch_bounds__(64 * kSlabWaves) void rows_finish_kernel(unsigned rows, unsigned cols, unsigned rw_shift,
                                                                     unsigned slab, unsigned nslabs,
                                                                     const float* __restrict__ part_m,
                                                                     const float* __restrict__ part_s,
                                                                     const float* __restrict__ a,
                                                                     const float* __restrict__ b,
                                                                     float* __restrict__ m_out, float* __restrict__ out) {
  __shared__ float red_m[kSlabWaves][64], red_s[kSlabWaves][64];
  constexpr int U = 8;
  const unsigned lane = threadIdx.x & 63, w = threadIdx.x >> 6;
  const unsigned RW = 1u << rw_shift, nsub = 64u >> rw_shift, rl = lane & (RW - 1), sub = lane >> rw_shift;
  const unsigned stride = kSlabWaves * nsub;
  const unsigned row = blockIdx.x * RW + rl;
  const bool live = row < rows;
  const unsigned rowc = live ? row : rows - 1;
  float m = -INFINITY, s = 0.f;
  for (unsigned k = w * nsub + sub; k < nslabs; k += U * stride) {
    float pm[U], ps[U];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const size_t at = (size_t(blockIdx.z) * nslabs + min(k + u * stride, nslabs - 1)) * rows + rowc;
      pm[u] = MODE == 2 ? 0.f : part_m[at];
      ps[u] = part_s[at];
    }
    if (MODE == 2) {
#pragma unroll
      for (int u = 0; u < U; ++u)
        if (k + u * stride < nslabs) s += ps[u];
    } else {
      float lm = m;
#pragma unroll
      for (int u = 0; u < U; ++u)
        if (k + u * stride < nslabs) lm = pm[u] > lm ? pm[u] : lm;
      const float ref = lm > -INFINITY ? lm : 0.f;
      s *= expf(m - ref);
#pragma unroll
      for (int u = 0; u < U; ++u)
        if (k + u * stride < nslabs) s += ps[u] * expf(pm[u] - ref);
      m = lm;
    }
  }
  rows_merge(m, s, red_m, red_s, w, lane, rw_shift, rl, MODE == 2);
  if (MODE != 2 && m == -INFINITY) s = NAN;  // a row of -inf: exp(-inf - -inf), as in the one-kernel form
  if (MODE == 0) {
    if (live && w == 0 && sub == 0) {
      m_out[size_t(blockIdx.z) * rows + row] = m;
      out[size_t(blockIdx.z) * rows + row] = logf(s) + m;
    }
    return;
  }
  const unsigned c0 = blockIdx.y * slab, c1 = min(cols, c0 + slab);
  const size_t base = size_t(blockIdx.z) * rows * cols + rowc;
  for (unsigned j = c0 + w * nsub + sub; j < c1; j += U * stride) {
    float v[U], y[U], o[U];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const size_t e = base + size_t(min(j + u * stride, c1 - 1)) * rows;
      v[u] = a[e];
      y[u] = MODE == 2 ? b[e] : 0.f;
      o[u] = MODE == 2 ? out[e] : 0.f;
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
      if (!live || j + u * stride >= c1) continue;
      const size_t e = base + size_t(j + u * stride) * rows;
      if (MODE == 1) out[e] = expf(v[u] - m) / s;
      else out[e] = o[u] + (y[u] - s) * v[u];
    }
  }
}

template <int MODE>
static int launch_rowwise(dyhip_device* dev, size_t rows, size_t cols, unsigned bd, const float* a, const float* b,
                          float* m_out, float* out) {
  DYHIP_REQUIRE(rows < (size_t(1) << 31) && cols < (size_t(1) << 31), "matrix dimension too large");
  unsigned rw_shift = 6;  // row lanes a wavefront: the power of two that reaches the row count, at most 64
  while (rw_shift > 0 && (size_t(1) << (rw_shift - 1)) >= rows) --rw_shift;
  const size_t tiles = cdiv<size_t>(rows, size_t(1) << rw_shift), cus = dev->num_cus > 0 ? size_t(dev->num_cus) : 256;
  if (tiles * bd < cus && cols >= 256) {
    const size_t sstride = size_t(kSlabWaves) * (64u >> rw_shift);
    size_t nslabs = std::min(cdiv<size_t>(2 * cus, tiles * bd), cols / 64);
    const size_t slab = cdiv<size_t>(cdiv<size_t>(cols, nslabs), sstride) * sstride;  // whole passes of the block
    nslabs = cdiv<size_t>(cols, slab);
    const size_t part = size_t(bd) * nslabs * rows;
    if (nslabs >= 2 && dev->gemm_ws != nullptr && dev->gemm_ws_bytes >= 2 * part * sizeof(float)) {
      float* part_m = static_cast<float*>(dev->gemm_ws);
      float* part_s = part_m + part;
      const unsigned r = static_cast<unsigned>(rows), c = static_cast<unsigned>(cols), sl = static_cast<unsigned>(slab),
                     ns = static_cast<unsigned>(nslabs), t = static_cast<unsigned>(tiles);
      hipLaunchKernelGGL((rows_slab_kernel<MODE == 2>), dim3(t, ns, bd), dim3(64 * kSlabWaves), 0, dev->stream, r, c,
                         rw_shift, sl, a, b, part_m, part_s);
      hipLaunchKernelGGL((rows_finish_kernel<MODE>), dim3(t, MODE == 0 ? 1 : ns, bd), dim3(64 * kSlabWaves), 0, dev->stream,
                         r, c, rw_shift, sl, ns, part_m, part_s, a, b, m_out, out);
      DYHIP_CHECK_LAUNCH();
      return DYHIP_OK;
    }
  }
  const dim3 grid(static_cast<unsigned>(tiles), bd < 65535u ? bd : 65535u);
  const size_t stride = size_t(kRowWaves) * (64u >> rw_shift);  // columns between a thread's consecutive elements
  if (cols >= 4 * stride)
    hipLaunchKernelGGL((rowwise_kernel<MODE, 8>), grid, dim3(64 * kRowWaves), 0, dev->stream, static_cast<unsigned>(rows),
                       static_cast<unsigned>(cols), bd, rw_shift, a, b, m_out, out);
  else
    hipLaunchKernelGGL((rowwise_kernel<MODE, 2>), grid, dim3(64 * kRowWaves), 0, dev->stream, static_cast<unsigned>(rows),
                       static_cast<unsigned>(cols), bd, rw_shift, a, b, m_out, out);
  DYHIP_CHECK_LAUNCH();
  return DYHIP_OK;
}

// LogSumExpDimension backward: dx[i,j,b] += exp(x[i,j,b] - fx[o,b]) * dEdf[o,b], o = j (dim 0) or i (dim 1)
__global__ __launch_bounds__(256) void lse_dim_bwd_kernel(unsigned rows, unsigned cols, size_t total, unsigned dim,
                                                          const float* __restrict__ x, const float* __restrict__ fx,
                                                          const float* __restrict__ dEdf, float* __restrict__ dEdx) {
  for (size_t e = size_t(blockIdx.x) * 256 + threadIdx.x; e < total; e += size_t(gridDim.x) * 256) {
    const size_t col = e / rows;  // column index over (cols x batch)
    const size_t o = dim == 0 ? col : (col / cols) * rows + (e - col * rows);
    dEdx[e] += expf(x[e] - fx[o]) * dEdf[o];
  }
}

template <bool ACC>
static int pnls_backward(dyhip_device* dev, size_t rows, unsigned bd, const float* x, const void* aux, const float* dEdf,
                         float* dEdx) {
  DYHIP_REQUIRE(rows >= 1 && x && aux && dEdf && dEdx, "PickNegLogSoftmax needs non-empty tensors");
  if (bd == 0) return DYHIP_OK;
  const float* z = static_cast<const float*>(aux);
  const unsigned* ids = reinterpret_cast<const unsigned*>(z + 2 * size_t(bd));
  if (rows <= kLseWaveMaxRows) {
    const dim3 grid(cdiv<unsigned>(bd, 4)), block(256);
    const unsigned r = static_cast<unsigned>(rows);
#define DYHIP_PB_WAVE(U) \
  hipLaunchKernelGGL((pnls_bwd_wave_kernel<U, ACC>), grid, block, 0, dev->stream, r, bd, x, z, ids, dEdf, dEdx)
    if (r <= 64) DYHIP_PB_WAVE(1);
    else if (r <= 128) DYHIP_PB_WAVE(2);
    else if (r <= 256) DYHIP_PB_WAVE(4);
    else DYHIP_PB_WAVE(8);
#undef DYHIP_PB_WAVE
    DYHIP_CHECK_LAUNCH();
    return DYHIP_OK;
  }
  // 128-bit accesses when x and dEdx sit at the same offset from a 16-byte boundary (every column then does too);
  // a column's ends are peeled off inside the kernel
  const bool vec = ((reinterpret_cast<uintptr_t>(x) ^ reinterpret_cast<uintptr_t>(dEdx)) & 15u) == 0 && rows >= 8;
  const size_t per_tile = size_t(kPbThreads) * kPbUnroll * (vec ? 4 : 1);
  const size_t tiles = cdiv(rows, per_tile);
  DYHIP_REQUIRE(tiles * bd < (size_t(1) << 31), "PickNegLogSoftmax backward launch too large");
  const dim3 grid(static_cast<unsigned>(tiles * bd));
  const bool stream = rows * size_t(bd) * sizeof(float) >= dev->stream_threshold;
  if (vec && stream)
    hipLaunchKernelGGL((pnls_bwd_kernel<true, true, ACC>), grid, dim3(kPbThreads), 0, dev->stream, rows, (unsigned)tiles, x, z, ids, dEdf, dEdx);
  else if (vec)
    hipLaunchKernelGGL((pnls_bwd_kernel<true, false, ACC>), grid, dim3(kPbThreads), 0, dev->stream, rows, (unsigned)tiles, x, z, ids, dEdf, dEdx);
  else
    hipLaunchKernelGGL((pnls_bwd_kernel<false, false, ACC>), grid, dim3(kPbThreads), 0, dev->stream, rows, (unsigned)tiles, x, z, ids, dEdf, dEdx);
  DYHIP_CHECK_LAUNCH();
  return DYHIP_OK;
}

}  // namespace dyhip

using namespace dyhip;

extern "C" {

int dyhip_logsumexp_cols(dyhip_device* dev, size_t rows, unsigned bd, const float* x, float* m, float* z) {
  DYHIP_CHECK_DEV(dev);
  DYHIP_REQUIRE(rows >= 1 && x && m && z, "logsumexp needs a non-empty tensor");
  if (bd == 0) return DYHIP_OK;
  return launch_lse(dev, rows, bd, x, m, z, nullptr, nullptr);
}

int dyhip_pnls_forward(dyhip_device* dev, size_t rows, unsigned bd, const float* x, const unsigned* labels_host,
                       void* aux, float* fx) {
  DYHIP_CHECK_DEV(dev);
  DYHIP_REQUIRE(rows >= 1 && x && labels_host && aux && fx, "PickNegLogSoftmax needs non-empty tensors");
  if (bd == 0) return DYHIP_OK;
  DYHIP_REQUIRE(rows * size_t(bd) <= (size_t(1) << 32), "PickNegLogSoftmax: %zu x %u elements overflow 32-bit ids",
                rows, bd);
  std::vector<unsigned> ids(bd);
  for (unsigned b = 0; b < bd; ++b) {
    DYHIP_REQUIRE(labels_host[b] < rows, "Index error in PickNegLogSoftmax: Index %u out of bounds for input tensor of %zu rows",
                  labels_host[b], rows);
    ids[b] = static_cast<unsigned>(rows * b + labels_host[b]);
  }
  float* z = static_cast<float*>(aux);
  float* m = z + bd;
  unsigned* ids_dev = reinterpret_cast<unsigned*>(m + bd);
  // pageable source: the copy has been staged by the time the call returns
  DYHIP_CHECK_HIP(hipMemcpyAsync(ids_dev, ids.data(), sizeof(unsigned) * bd, hipMemcpyHostToDevice, dev->stream));
  DYHIP_CHECK_HIP(hipStreamSynchronize(dev->stream));
  return launch_lse(dev, rows, bd, x, m, z, ids_dev, fx);
}

int dyhip_pnls_forward_staged(dyhip_device* dev, size_t rows, unsigned bd, const float* x, void* aux, float* fx) {
  DYHIP_CHECK_DEV(dev);
  DYHIP_REQUIRE(rows >= 1 && x && aux && fx, "PickNegLogSoftmax needs non-empty tensors");
  if (bd == 0) return DYHIP_OK;
  float* z = static_cast<float*>(aux);
  float* m = z + bd;
  return launch_lse(dev, rows, bd, x, m, z, reinterpret_cast<const unsigned*>(m + bd), fx);
}

int dyhip_pnls_backward(dyhip_device* dev, size_t rows, unsigned bd, const float* x, const void* aux,
                        const float* dEdf, float* dEdx) {
  DYHIP_CHECK_DEV(dev);
  return pnls_backward<true>(dev, rows, bd, x, aux, dEdf, dEdx);
}

int dyhip_pnls_backward_assign(dyhip_device* dev, size_t rows, unsigned bd, const float* x, const void* aux,
                               const float* dEdf, float* dEdx) {
  DYHIP_CHECK_DEV(dev);
  return pnls_backward<false>(dev, rows, bd, x, aux, dEdf, dEdx);
}

int dyhip_logsumexp_node_forward(dyhip_device* dev, unsigned k, size_t n, unsigned bd, const float* const* xs_host,
                                 const unsigned* bds_host, float* fx) {
  DYHIP_CHECK_DEV(dev);
  DYHIP_REQUIRE(k >= 1, "LogSumExp needs at least one argument");
  DYHIP_REQUIRE(xs_host && bds_host && fx, "null pointer");
  const size_t total = n * size_t(bd);
  if (total == 0) return DYHIP_OK;
  for (unsigned i = 0; i < k; ++i)
    DYHIP_REQUIRE(bds_host[i] == bd || bds_host[i] == 1, "Mismatched input dimensions in LogSumExp");
  // up to 32 arguments a launch; more are chained through the output, which joins the next launch as one more
  // argument: logsumexp(a, b) with a = logsumexp of the earlier arguments is the logsumexp of all of them
  unsigned at = 0;
  while (at < k) {
    LseNodeArgs a;
    unsigned cnt = 0;
    a.bcast = 0;
    if (at > 0) a.x[cnt++] = fx;
    while (cnt < kLseNodeMaxArgs && at < k) {
      if (bds_host[at] != bd) a.bcast |= 1u << cnt;
      a.x[cnt++] = xs_host[at++];
    }
    for (unsigned i = cnt; i < kLseNodeMaxArgs; ++i) a.x[i] = a.x[0];
    a.k = cnt;
    a.last = at == k ? 1u : 0u;
    hipLaunchKernelGGL(lse_node_fwd_kernel, dim3((unsigned)cdiv<size_t>(total, 256)), dim3(256), 0, dev->stream, a, n,
                       total, fx);
    DYHIP_CHECK_LAUNCH();
  }
  return DYHIP_OK;
}

int dyhip_logsumexp_node_backward(dyhip_device* dev, unsigned k, size_t n, unsigned bd, const float* const* xs_host,
                                  const unsigned* bds_host, const float* fx, const float* dEdf, unsigned i,
                                  float* dEdxi, void* ws, size_t ws_bytes) {
  DYHIP_CHECK_DEV(dev);
  DYHIP_REQUIRE(k >= 1 && i < k, "bad argument index %u of %u", i, k);
  DYHIP_REQUIRE(xs_host && bds_host && fx && dEdf && dEdxi, "null pointer");
  const size_t total = n * size_t(bd);
  if (total == 0) return DYHIP_OK;
  const dim3 grid((unsigned)cdiv<size_t>(total, 256));
  if (k == 1) return dyhip_accumulate(dev, total, dEdf, dEdxi);
  if (bds_host[i] == bd) {
    hipLaunchKernelGGL(lse_node_bwd_kernel, grid, dim3(256), 0, dev->stream, total, xs_host[i], fx, dEdf, dEdxi);
    DYHIP_CHECK_LAUNCH();
    return DYHIP_OK;
  }
  // broadcast argument: materialise the products, then reduce over the batch
  size_t red = 0;
  DYHIP_CHECK_STATUS(dyhip_batch_reduce_workspace(n, bd, &red));
  const size_t tmp_bytes = cdiv<size_t>(total * sizeof(float), 256) * 256;
  DYHIP_REQUIRE(ws != nullptr && ws_bytes >= tmp_bytes + red, "LogSumExp backward needs %zu workspace bytes, got %zu",
                tmp_bytes + red, ws_bytes);
  float* tmp = static_cast<float*>(ws);
  hipLaunchKernelGGL(lse_node_bwd_bcast_kernel, grid, dim3(256), 0, dev->stream, n, total, xs_host[i], fx, dEdf, tmp);
  DYHIP_CHECK_LAUNCH();
  return batch_reduce(dev, n, bd, tmp, nullptr, dEdxi, true, static_cast<char*>(ws) + tmp_bytes, ws_bytes - tmp_bytes);
}

int dyhip_argmax_cols(dyhip_device* dev, size_t rows, unsigned bd, const float* x, long long* idx) {
  DYHIP_CHECK_DEV(dev);
  DYHIP_REQUIRE(rows >= 1 && x && idx, "argmax needs a non-empty tensor");
  if (bd == 0) return DYHIP_OK;
  launch_argmax_cols(dev, rows, bd, x, idx);
  DYHIP_CHECK_LAUNCH();
  return DYHIP_OK;
}

int dyhip_argmax_onehot_forward(dyhip_device* dev, size_t rows, unsigned bd, const float* x, long long* idx, float* fx) {
  DYHIP_CHECK_DEV(dev);
  DYHIP_REQUIRE(rows >= 1 && x && idx && fx, "argmax needs a non-empty tensor");
  if (bd == 0) return DYHIP_OK;
  launch_argmax_cols(dev, rows, bd, x, idx);
  DYHIP_CHECK_LAUNCH();
  const size_t total = rows * size_t(bd);
  hipLaunchKernelGGL(onehot_kernel, dim3((unsigned)cdiv<size_t>(total, 256)), dim3(256), 0, dev->stream, rows, total, idx, fx);
  DYHIP_CHECK_LAUNCH();
  return DYHIP_OK;
}

int dyhip_softmax_forward(dyhip_device* dev, size_t rows, unsigned cols, const float* x, float* fx, void* ws,
                          size_t ws_bytes) {
  DYHIP_CHECK_DEV(dev);
  DYHIP_REQUIRE(rows >= 1 && x && fx, "Softmax needs non-empty tensors");
  if (cols == 0) return DYHIP_OK;
  DYHIP_REQUIRE(ws != nullptr && ws_bytes >= 2 * sizeof(float) * cols, "Softmax needs %zu workspace bytes, got %zu",
                2 * sizeof(float) * cols, ws_bytes);
  float* z = static_cast<float*>(ws);
  float* m = z + cols;
  if (launch_softmax_resident<0>(dev, rows, cols, x, nullptr, z, m, fx)) {
    DYHIP_CHECK_LAUNCH();
    return DYHIP_OK;
  }
  DYHIP_CHECK_STATUS(launch_lse(dev, rows, cols, x, m, z, nullptr, nullptr));
  return launch_col_apply<0>(dev, rows, cols, x, nullptr, m, z, fx);
}

int dyhip_softmax_backward(dyhip_device* dev, size_t rows, unsigned cols, const float* fx, const float* dEdf,
                           float* dEdx, void* ws, size_t ws_bytes) {
  DYHIP_CHECK_DEV(dev);
  DYHIP_REQUIRE(rows >= 1 && fx && dEdf && dEdx, "Softmax needs non-empty tensors");
  if (cols == 0) return DYHIP_OK;
  DYHIP_REQUIRE(ws != nullptr && ws_bytes >= sizeof(float) * cols, "Softmax backward needs %zu workspace bytes, got %zu",
                sizeof(float) * cols, ws_bytes);
  float* r = static_cast<float*>(ws);
  if (launch_softmax_resident<2>(dev, rows, cols, fx, dEdf, r, nullptr, dEdx)) {
    DYHIP_CHECK_LAUNCH();
    return DYHIP_OK;
  }
  launch_col_dot(dev, rows, cols, fx, dEdf, r);
  DYHIP_CHECK_LAUNCH();
  return launch_col_apply<2>(dev, rows, cols, fx, dEdf, r, nullptr, dEdx);
}

int dyhip_softmax_rows_forward(dyhip_device* dev, size_t rows, size_t cols, unsigned bd, const float* x, float* fx) {
  DYHIP_CHECK_DEV(dev);
  DYHIP_REQUIRE(rows >= 1 && cols >= 1 && x && fx, "Softmax needs non-empty tensors");
  if (bd == 0) return DYHIP_OK;
  return launch_rowwise<1>(dev, rows, cols, bd, x, nullptr, nullptr, fx);
}

int dyhip_softmax_rows_backward(dyhip_device* dev, size_t rows, size_t cols, unsigned bd, const float* fx,
                                const float* dEdf, float* dEdx) {
  DYHIP_CHECK_DEV(dev);
  DYHIP_REQUIRE(rows >= 1 && cols >= 1 && fx && dEdf && dEdx, "Softmax needs non-empty tensors");
  if (bd == 0) return DYHIP_OK;
  return launch_rowwise<2>(dev, rows, cols, bd, fx, dEdf, nullptr, dEdx);
}

int dyhip_logsumexp_dim_forward(dyhip_device* dev, size_t rows, size_t cols, unsigned bd, const float* x, unsigned dim,
                                float* m, float* fx) {
  DYHIP_CHECK_DEV(dev);
  DYHIP_REQUIRE(dim <= 1, "LogSumExpDimension reduces dimension 0 or 1, got %u", dim);
  DYHIP_REQUIRE(rows >= 1 && cols >= 1 && x && m && fx, "LogSumExpDimension needs non-empty tensors");
  if (bd == 0) return DYHIP_OK;
  if (dim == 0) {
    DYHIP_REQUIRE(cols * size_t(bd) <= 0xffffffffu, "too many columns");
    return launch_lse(dev, rows, static_cast<unsigned>(cols * bd), x, m, fx, nullptr, nullptr);
  }
  return launch_rowwise<0>(dev, rows, cols, bd, x, nullptr, m, fx);
}

int dyhip_logsumexp_dim_backward(dyhip_device* dev, size_t rows, size_t cols, unsigned bd, const float* x,
                                 const float* fx, const float* dEdf, unsigned dim, float* dEdx) {
  DYHIP_CHECK_DEV(dev);
  DYHIP_REQUIRE(dim <= 1, "LogSumExpDimension reduces dimension 0 or 1, got %u", dim);
  DYHIP_REQUIRE(rows >= 1 && cols >= 1 && rows < (size_t(1) << 31) && cols < (size_t(1) << 31) && x && fx && dEdf && dEdx,
                "LogSumExpDimension needs non-empty tensors");
  const size_t total = rows * cols * bd;
  if (total == 0) return DYHIP_OK;
  const size_t blocks = cdiv<size_t>(total, 256);
  hipLaunchKernelGGL(lse_dim_bwd_kernel, dim3(static_cast<unsigned>(blocks < 65536 * 16 ? blocks : 65536 * 16)), dim3(256), 0,
                     dev->stream, static_cast<unsigned>(rows), static_cast<unsigned>(cols), total, dim, x, fx, dEdf, dEdx);
  DYHIP_CHECK_LAUNCH();
  return DYHIP_OK;
}

int dyhip_log_softmax_forward(dyhip_device* dev, size_t rows, unsigned cols, const float* x, void* aux, float* fx) {
  DYHIP_CHECK_DEV(dev);
  DYHIP_REQUIRE(rows >= 1 && x && aux && fx, "LogSoftmax needs non-empty tensors");
  if (cols == 0) return DYHIP_OK;
  float* z = static_cast<float*>(aux);
  float* m = z + cols;
  if (launch_softmax_resident<1>(dev, rows, cols, x, nullptr, z, m, fx)) {
    DYHIP_CHECK_LAUNCH();
    return DYHIP_OK;
  }
  DYHIP_CHECK_STATUS(launch_lse(dev, rows, cols, x, m, z, nullptr, nullptr));
  return launch_col_apply<1>(dev, rows, cols, x, nullptr, z, nullptr, fx);
}

int dyhip_log_softmax_backward(dyhip_device* dev, size_t rows, unsigned cols, const float* fx, const float* dEdf,
                               void* aux, float* dEdx) {
  DYHIP_CHECK_DEV(dev);
  DYHIP_REQUIRE(rows >= 1 && fx && dEdf && aux && dEdx, "LogSoftmax needs non-empty tensors");
  if (cols == 0) return DYHIP_OK;
  float* r = static_cast<float*>(aux);  // the reference overwrites z in aux_mem with the column sums of dEdf
  if (launch_softmax_resident<3>(dev, rows, cols, fx, dEdf, r, nullptr, dEdx)) {
    DYHIP_CHECK_LAUNCH();
    return DYHIP_OK;
  }
  launch_col_dot(dev, rows, cols, dEdf, nullptr, r);
  DYHIP_CHECK_LAUNCH();
  return launch_col_apply<3>(dev, rows, cols, fx, dEdf, r, nullptr, dEdx);
}

}  // extern "C"
