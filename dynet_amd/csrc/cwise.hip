// CwiseSum / CwiseMultiply / CwiseQuotient with broadcast over any dimension (and the batch), and the
// scalar-constant nodes ConstantPlusX / ConstantMinusX.
//
// Replaces the Eigen broadcast / reduce statements of dynet/nodes-arith-cwise.cc (forward :50-97, :196-243,
// :338-351; backward and backward_helper :99-156, :245-307, :353-421) and dynet/nodes-arith-const.cc:33-75.
// The batch-only cases keep their streaming kernels (elementwise.hip); this file adds the general case, which
// the unfused layer_norm composite needs (x - mean, (x - mean) / (sigma + eps): Dim({n}, bd) against Dim({1}, bd)).
//
// Layout: a tensor is dims[5] = {d0, d1, d2, d3, bd}, column-major with the batch outermost; on every axis
// the two arguments agree or one of them is 1.
//   forward / backward without reduction: one thread per 4 consecutive elements along d0 (128-bit accesses
//     when d0 % 4 == 0), operands that are 1 along an axis are indexed with stride 0;
//   backward of an argument that was broadcast: dEdxi[o] += sum of the terms over the broadcast axes.
//     kept axes = a prefix and the other operand is full size: the batch reduction of reduce.hip (coalesced);
//     otherwise one wavefront per output element (>= 64 terms, lanes walk the broadcast axes fastest-first,
//     fixed summation order) or one thread per output element (fewer terms).
#include <algorithm>

#include "common.h"

namespace dyhip {

int batch_reduce(dyhip_device* dev, size_t n, unsigned bd, const float* in0, const float* in1, float* out,
                 bool accumulate, void* ws, size_t ws_bytes);

struct CwShape {
  unsigned d[5];      // dimensions of the full (output-sized) index space
  size_t s[3][5];     // element strides of the three operands; 0 on an axis the operand is broadcast over
};

// FN: 0: p0 + p1   1: p0 * p1   2: p0 / p1                                   (forward, overwrite)
//     3: out + p0  4: out + p0 * p1   5: out + p0 / p1   6: out - p0 / (p1 * p1) * p2   (backward, accumulate)
template <int FN>
__device__ __forceinline__ float cw_apply(float p0, float p1, float p2, float old) {
  if (FN == 0) return p0 + p1;
  if (FN == 1) return p0 * p1;
  if (FN == 2) return p0 / p1;
  if (FN == 3) return old + p0;
  if (FN == 4) return old + p0 * p1;
  if (FN == 5) return old + p0 / p1;
  return old - p0 / (p1 * p1) * p2;
}
template <int FN>
__device__ __forceinline__ float cw_term(float p0, float p1, float p2) {  // what a reduction sums (added to the output)
  if (FN == 3) return p0;
  if (FN == 4) return p0 * p1;
  return -(p0 / (p1 * p1) * p2);
}
constexpr int cw_inputs(int fn) { return fn == 3 ? 1 : fn == 6 ? 3 : 2; }

// ---- no reduction: out[e] = f(operands at the broadcast index of e) ------------------------------
template <int FN, int W>  // W = 4: d0 % 4 == 0 and every pointer 16-byte aligned; W = 1 otherwise
__global__ __launch_bounds__(256) void cwise_bcast_kernel(CwShape sh, const float* __restrict__ p0,
                                                          const float* __restrict__ p1, const float* __restrict__ p2,
                                                          float* __restrict__ out, size_t groups) {
  constexpr int NIN = cw_inputs(FN);
  constexpr bool ACC = FN >= 3;
  const unsigned d0g = sh.d[0] / W;
  for (size_t g = size_t(blockIdx.x) * 256 + threadIdx.x; g < groups; g += size_t(gridDim.x) * 256) {
    size_t r = g / d0g;
    unsigned idx[5];
    idx[0] = unsigned(g - r * d0g) * W;
#pragma unroll
    for (int j = 1; j < 4; ++j) {
      const size_t q = r / sh.d[j];
      idx[j] = unsigned(r - q * sh.d[j]);
      r = q;
    }
    idx[4] = unsigned(r);
    const float* ps[3] = {p0, p1, p2};
    float v[3][W];
#pragma unroll
    for (int k = 0; k < 3; ++k) {
      if (k < NIN) {
        size_t off = 0;
#pragma unroll
        for (int j = 0; j < 5; ++j) off += size_t(idx[j]) * sh.s[k][j];
        if (W == 4 && sh.s[k][0] == 1) {
          const float4 t = *reinterpret_cast<const float4*>(ps[k] + off);
          v[k][0] = t.x; v[k][1 % W] = t.y; v[k][2 % W] = t.z; v[k][3 % W] = t.w;
        } else {
#pragma unroll
          for (int e = 0; e < W; ++e) v[k][e] = ps[k][off + size_t(e) * sh.s[k][0]];
        }
      } else {
#pragma unroll
        for (int e = 0; e < W; ++e) v[k][e] = 0.f;
      }
    }
    float* po = out + g * W;
    float o[W];
    if (W == 4) {
      float4 t = make_float4(0.f, 0.f, 0.f, 0.f);
      if (ACC) t = *reinterpret_cast<const float4*>(po);
      o[0] = t.x; o[1 % W] = t.y; o[2 % W] = t.z; o[3 % W] = t.w;
    } else {
      o[0] = ACC ? po[0] : 0.f;
    }
#pragma unroll
    for (int e = 0; e < W; ++e) o[e] = cw_apply<FN>(v[0][e], v[1][e], v[2][e], o[e]);
    if (W == 4) *reinterpret_cast<float4*>(po) = make_float4(o[0], o[1 % W], o[2 % W], o[3 % W]);
    else po[0] = o[0];
  }
}

// The same when the index space collapses to two axes (the usual case: a matrix against a row or a column of it, e.g.
// x - mean and x / sigma of the layer_norm composite): no index arithmetic beyond the block's own coordinates, kRows
// rows of the outer axis per block with all their loads issued first, streaming accesses for large tensors.
struct CwShape2 {
  unsigned d0g, d1, d2;  // groups of W elements along the inner axis; extents of the middle and the outer axis
  unsigned tx_shift;     // a block is 2^tx_shift threads along the inner axis x 256 / 2^tx_shift rows of the middle one
  size_t s0[3], s1[3], s2[3];  // element strides of the three operands along the three axes (0 = broadcast)
};
constexpr int kCwRows = 4;

template <int FN, int W, bool NT>
__global__ __launch_bounds__(256) void cwise_bcast2_kernel(CwShape2 sh, const float* __restrict__ p0,
                                                           const float* __restrict__ p1, const float* __restrict__ p2,
                                                           float* __restrict__ out) {
  constexpr int NIN = cw_inputs(FN);
  constexpr bool ACC = FN >= 3;
  constexpr int kRows = kCwRows;  // rows in flight per thread (sixteen for the one-float form measured slower than four)
  // a short inner axis does not idle most of the block: the block's threads fold over rows of the middle axis
  const unsigned tx = threadIdx.x & ((1u << sh.tx_shift) - 1u), ty = threadIdx.x >> sh.tx_shift;
  const unsigned rows_per_block = (256u >> sh.tx_shift) * kRows;
  const unsigned gx = (blockIdx.x << sh.tx_shift) + tx;
  if (gx >= sh.d0g) return;
  for (unsigned z = blockIdx.z; z < sh.d2; z += gridDim.z) {
  const float* ps[3] = {p0 + size_t(z) * sh.s2[0], p1 + (NIN > 1 ? size_t(z) * sh.s2[1] : 0),
                        p2 + (NIN > 2 ? size_t(z) * sh.s2[2] : 0)};
  float* const outz = out + size_t(z) * sh.d1 * sh.d0g * W;
  for (unsigned y0 = blockIdx.y * rows_per_block + ty * kRows; y0 < sh.d1; y0 += gridDim.y * rows_per_block) {
    float v[kRows][3][W], o[kRows][W];
#pragma unroll
    for (int r = 0; r < kRows; ++r) {
      const unsigned y = min(y0 + r, sh.d1 - 1);  // rows past the end repeat the last one and are not stored
#pragma unroll
      for (int k = 0; k < 3; ++k) {
        if (k < NIN) {
          const float* q = ps[k] + size_t(y) * sh.s1[k] + size_t(gx) * W * sh.s0[k];
          if (W == 4 && sh.s0[k] == 1) {
            const float4 t = ldg4<NT>(reinterpret_cast<const float4*>(q));
            v[r][k][0] = t.x; v[r][k][1 % W] = t.y; v[r][k][2 % W] = t.z; v[r][k][3 % W] = t.w;
          } else {
#pragma unroll
            for (int e = 0; e < W; ++e) v[r][k][e] = q[size_t(e) * sh.s0[k]];
          }
        } else {
#pragma unroll
          for (int e = 0; e < W; ++e) v[r][k][e] = 0.f;
        }
      }
      const float* po = outz + (size_t(y) * sh.d0g + gx) * W;
      if (ACC && W == 4) {
        const float4 t = *reinterpret_cast<const float4*>(po);  // read-modify-write: a plain load
        o[r][0] = t.x; o[r][1 % W] = t.y; o[r][2 % W] = t.z; o[r][3 % W] = t.w;
      } else {
#pragma unroll
        for (int e = 0; e < W; ++e) o[r][e] = ACC ? po[e] : 0.f;
      }
    }
#pragma unroll
    for (int r = 0; r < kRows; ++r) {
      if (y0 + r >= sh.d1) break;
      float* po = outz + (size_t(y0 + r) * sh.d0g + gx) * W;
#pragma unroll
      for (int e = 0; e < W; ++e) o[r][e] = cw_apply<FN>(v[r][0][e], v[r][1][e], v[r][2][e], o[r][e]);
      if (W == 4) stg4<NT>(reinterpret_cast<float4*>(po), make_float4(o[r][0], o[r][1 % W], o[r][2 % W], o[r][3 % W]));
      else po[0] = o[r][0];
    }
  }
  }
}

// ---- reduction over the broadcast axes ------------------------------------------------------------
struct CwReduce {
  unsigned kd[5], rd[5];   // sizes of the kept / reduced axes, in axis order, padded with 1
  size_t ks[3][5];         // strides of the three operands along the kept axes (same order)
  size_t rs[3][5];         // ... along the reduced axes
  size_t n_out, n_red;
  // cwise_reduce_row_kernel only: the reduced axis in `chunks` pieces of chunk_len (a multiple of 1024) indices, piece
  // ch of output o summed into out[o * chunks + ch]
  unsigned chunks, chunk_len;
  int overwrite;  // out = sum instead of out += sum (a stage that writes scratch)
};

template <int FN>
__device__ __forceinline__ float cw_reduce_one(const CwReduce& c, size_t o, size_t q0, size_t qstep, const float* p0,
                                               const float* p1, const float* p2) {
  constexpr int NIN = cw_inputs(FN);
  size_t base[3] = {0, 0, 0};
  {
    size_t r = o;
#pragma unroll
    for (int j = 0; j < 5; ++j) {
      const size_t q = r / c.kd[j];
      const size_t i = r - q * c.kd[j];
      r = q;
#pragma unroll
      for (int k = 0; k < NIN; ++k) base[k] += i * c.ks[k][j];
    }
  }
  float acc = 0.f;
  for (size_t q = q0; q < c.n_red; q += qstep) {
    size_t off[3] = {base[0], base[1], base[2]};
    size_t r = q;
#pragma unroll
    for (int j = 0; j < 5; ++j) {
      const size_t t = r / c.rd[j];
      const size_t i = r - t * c.rd[j];
      r = t;
#pragma unroll
      for (int k = 0; k < NIN; ++k) off[k] += i * c.rs[k][j];
    }
    acc += cw_term<FN>(p0[off[0]], NIN > 1 ? p1[off[1]] : 0.f, NIN > 2 ? p2[off[2]] : 0.f);
  }
  return acc;
}

template <int FN>
__global__ __launch_bounds__(256) void cwise_reduce_wave_kernel(CwReduce c, const float* __restrict__ p0,
                                                                const float* __restrict__ p1,
                                                                const float* __restrict__ p2, float* __restrict__ out) {
  const int lane = threadIdx.x & 63;
  for (size_t o = size_t(blockIdx.x) * 4 + (threadIdx.x >> 6); o < c.n_out; o += size_t(gridDim.x) * 4) {
    const float t = wave_sum(cw_reduce_one<FN>(c, o, size_t(lane), 64, p0, p1, p2));
    if (lane == 0) out[o] = c.overwrite ? t : out[o] + t;
  }
}

// The reduced axes collapse to one (the usual case: the sum over the row of a matrix): the kept index is decomposed
// once per output, the walk along the reduced axis needs no division, and four terms per lane are in flight.
// VEC: every operand runs along the reduced axis with stride 1 (128-bit loads) or stride 0.
template <int FN, bool VEC, bool NT>
__global__ __launch_bounds__(256) void cwise_reduce_row_kernel(CwReduce c, const float* __restrict__ p0,
                                                               const float* __restrict__ p1,
                                                               const float* __restrict__ p2, float* __restrict__ out) {
  constexpr int NIN = cw_inputs(FN);
  const unsigned lane = threadIdx.x & 63;
  const float* ps[3] = {p0, p1, p2};
  for (size_t item = size_t(blockIdx.x) * 4 + (threadIdx.x >> 6); item < c.n_out * c.chunks; item += size_t(gridDim.x) * 4) {
    const size_t o = c.chunks == 1 ? item : item / c.chunks;
    const unsigned ch = c.chunks == 1 ? 0 : unsigned(item - o * c.chunks);
    size_t base[3] = {0, 0, 0};
    size_t r = o;  // the same in every lane of the wave: the branches below are uniform
#pragma unroll
    for (int j = 0; j < 5; ++j) {
      const unsigned kd = c.kd[j];
      if (kd == 1) continue;
      // no division once the rest fits the axis (always so with one kept axis: the kernel's loads used to start
      // behind five 64-bit divisions), a 32-bit one while it fits 32 bits
      size_t q, i;
      if (r < kd) {
        q = 0;
        i = r;
      } else if (r <= 0xFFFFFFFFull) {
        const unsigned r32 = unsigned(r), q32 = r32 / kd;
        q = q32;
        i = r32 - q32 * kd;
      } else {
        q = r / kd;
        i = r - q * kd;
      }
      r = q;
#pragma unroll
      for (int k = 0; k < NIN; ++k) base[k] += i * c.ks[k][j];
    }
    const unsigned qb = ch * c.chunk_len;
    const unsigned nr = c.chunks == 1 ? unsigned(c.n_red) : unsigned(min(c.n_red, size_t(qb) + c.chunk_len));
    const float old = lane == 0 && !c.overwrite ? out[item] : 0.f;  // fetched beside the terms, not after the sum
    float acc = 0.f;
    if (VEC) {
      for (unsigned q0 = qb; q0 < nr; q0 += 4 * 64 * 4) {
        float4 v[4][3];
#pragma unroll
        for (int u = 0; u < 4; ++u) {
          const unsigned q = min(q0 + 4 * (lane + 64 * u), nr - 4);  // clamped, masked below
#pragma unroll
          for (int k = 0; k < 3; ++k) {
            if (k >= NIN) v[u][k] = make_float4(0.f, 0.f, 0.f, 0.f);
            else if (c.rs[k][0] == 1) v[u][k] = ldg4<NT>(reinterpret_cast<const float4*>(ps[k] + base[k] + q));
            else {
              const float b = ps[k][base[k]];
              v[u][k] = make_float4(b, b, b, b);
            }
          }
        }
#pragma unroll
        for (int u = 0; u < 4; ++u) {
          if (q0 + 4 * (lane + 64 * u) < nr) {
            acc += cw_term<FN>(v[u][0].x, v[u][1].x, v[u][2].x);
            acc += cw_term<FN>(v[u][0].y, v[u][1].y, v[u][2].y);
            acc += cw_term<FN>(v[u][0].z, v[u][1].z, v[u][2].z);
            acc += cw_term<FN>(v[u][0].w, v[u][1].w, v[u][2].w);
          }
        }
      }
    } else {
      for (unsigned q0 = qb; q0 < nr; q0 += 64 * 4) {
        float v[4][3];
#pragma unroll
        for (int u = 0; u < 4; ++u) {
          const unsigned q = min(q0 + lane + 64 * u, nr - 1);
#pragma unroll
          for (int k = 0; k < 3; ++k) v[u][k] = k < NIN ? ps[k][base[k] + size_t(q) * c.rs[k][0]] : 0.f;
        }
#pragma unroll
        for (int u = 0; u < 4; ++u)
          if (q0 + lane + 64 * u < nr) acc += cw_term<FN>(v[u][0], v[u][1], v[u][2]);
      }
    }
    const float t = wave_sum(acc);
    if (lane == 0) out[item] = old + t;
  }
}

template <int FN>
__global__ __launch_bounds__(256) void cwise_reduce_thread_kernel(CwReduce c, const float* __restrict__ p0,
                                                                  const float* __restrict__ p1,
                                                                  const float* __restrict__ p2,
                                                                  float* __restrict__ out) {
  for (size_t o = size_t(blockIdx.x) * 256 + threadIdx.x; o < c.n_out; o += size_t(gridDim.x) * 256)
    out[o] = c.overwrite ? cw_reduce_one<FN>(c, o, 0, 1, p0, p1, p2) : out[o] + cw_reduce_one<FN>(c, o, 0, 1, p0, p1, p2);
}

// ---- host side ---------------------------------------------------------------------------------------
static int cw_check(int op, const unsigned* da, const unsigned* db, const char* what) {
  DYHIP_REQUIRE(op >= DYHIP_CWISE_SUM && op <= DYHIP_CWISE_QUOTIENT, "%s: unknown operator %d", what, op);
  DYHIP_REQUIRE(da != nullptr && db != nullptr, "%s: null dimension array", what);
  for (int j = 0; j < 5; ++j) {
    DYHIP_REQUIRE(da[j] >= 1 && db[j] >= 1, "%s: empty dimension %d", what, j);
    if (op == DYHIP_CWISE_QUOTIENT)
      DYHIP_REQUIRE(da[j] == db[j] || db[j] == 1,
                    "CwiseQuotient: For each dimension, the dim size needs to match or the right side needs to equal 1 "
                    "(axis %d: %u and %u)", j, da[j], db[j]);
    else
      DYHIP_REQUIRE(da[j] == db[j] || da[j] == 1 || db[j] == 1,
                    "%s: For each dimension, the dim size needs to match or equal 1 (axis %d: %u and %u)", what, j, da[j],
                    db[j]);
  }
  return DYHIP_OK;
}

static void cw_strides(const unsigned* dims, const unsigned* full, size_t* s) {
  size_t stride = 1;
  for (int j = 0; j < 5; ++j) {
    s[j] = (dims[j] == 1 && full[j] > 1) ? 0 : stride;
    stride *= dims[j];
  }
}

static size_t cw_size(const unsigned* d) { return size_t(d[0]) * d[1] * d[2] * d[3] * d[4]; }

static unsigned cw_grid(size_t work_items, unsigned per_block, const dyhip_device* dev) {
  const size_t want = cdiv<size_t>(work_items, per_block);
  const size_t cap = size_t(dev->num_cus) * 16;
  return static_cast<unsigned>(want < cap ? (want ? want : 1) : cap);
}

// The reduced axes collapse to one that is NOT the contiguous one (the gradient of a column vector added to every
// column of a matrix: kept rows, reduced columns, kept batch): lanes run along the contiguous kept axis, so every load
// of a wavefront is one contiguous run, the block's 8 wavefronts split the reduced axis (four terms in flight each) and
// meet in LDS in ascending order.  With a wavefront per output walking the reduced axis each lane touched a line of
// its own (46.7 us for 256 x 64 x 256 summed over the 64; 8 us here).
constexpr int kCwMidWaves = 8;
template <int FN>
__global__ __launch_bounds__(64 * kCwMidWaves) void cwise_reduce_mid_kernel(CwReduce c, const float* __restrict__ p0,
                                                                           const float* __restrict__ p1,
                                                                           const float* __restrict__ p2,
                                                                           float* __restrict__ out) {
  constexpr int NIN = cw_inputs(FN);
  __shared__ float red[kCwMidWaves][64];
  const unsigned lane = threadIdx.x & 63, w = threadIdx.x >> 6;
  const unsigned i = blockIdx.x * 64 + lane;  // along the contiguous kept axis
  const bool live = i < c.kd[0];
  const unsigned ic = live ? i : c.kd[0] - 1;
  const float* ps[3] = {p0, p1, p2};
  const size_t n_rest = c.n_out / c.kd[0];  // the other kept axes, flattened
  const unsigned nr = unsigned(c.n_red);
  for (size_t z = blockIdx.y; z < n_rest; z += gridDim.y) {
    size_t base[3] = {0, 0, 0};
    size_t r = z;  // the same in every thread of the block
#pragma unroll
    for (int j = 1; j < 5; ++j) {
      const unsigned kd = c.kd[j];
      if (kd == 1) continue;
      const size_t q = r / kd, e = r - q * kd;
      r = q;
#pragma unroll
      for (int k = 0; k < NIN; ++k) base[k] += e * c.ks[k][j];
    }
#pragma unroll
    for (int k = 0; k < NIN; ++k) base[k] += size_t(ic) * c.ks[k][0];
    float acc = 0.f;
    for (unsigned q0 = w; q0 < nr; q0 += 4 * kCwMidWaves) {
      float v[4][3];
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const unsigned q = min(q0 + u * kCwMidWaves, nr - 1);  // clamped, masked below
#pragma unroll
        for (int k = 0; k < 3; ++k) v[u][k] = k < NIN ? ps[k][base[k] + size_t(q) * c.rs[k][0]] : 0.f;
      }
#pragma unroll
      for (int u = 0; u < 4; ++u)
        if (q0 + u * kCwMidWaves < nr) acc += cw_term<FN>(v[u][0], v[u][1], v[u][2]);
    }
    __syncthreads();  // the previous round's sums have been read
    red[w][lane] = acc;
    __syncthreads();
    if (w == 0 && live) {
      float t = red[0][lane];
#pragma unroll
      for (int k = 1; k < kCwMidWaves; ++k) t += red[k][lane];
      out[z * c.kd[0] + i] = c.overwrite ? t : out[z * c.kd[0] + i] + t;
    }
  }
}

// Axes of extent 1 dropped, neighbouring axes merged when every operand treats them alike (broadcast over both, or
// laid out contiguously across both).  Returns the number of axes left; d / s are padded with 1 / 0.
static int cw_collapse(const unsigned* d_in, const size_t s_in[3][5], int nin, unsigned* d, size_t s[3][5]) {
  int r = 0;
  for (int j = 0; j < 5; ++j) {
    if (d_in[j] == 1) continue;
    if (r > 0 && size_t(d[r - 1]) * d_in[j] <= 0xFFFFFFFFull) {
      bool ok = true;
      for (int k = 0; k < nin; ++k)
        ok = ok && ((s[k][r - 1] == 0 && s_in[k][j] == 0) || (s[k][r - 1] != 0 && s_in[k][j] == s[k][r - 1] * d[r - 1]));
      if (ok) {
        d[r - 1] *= d_in[j];
        continue;
      }
    }
    d[r] = d_in[j];
    for (int k = 0; k < 3; ++k) s[k][r] = k < nin ? s_in[k][j] : 0;
    ++r;
  }
  for (int j = r; j < 5; ++j) {
    d[j] = 1;
    for (int k = 0; k < 3; ++k) s[k][j] = 0;
  }
  return r;
}

template <int FN>
static int cw_launch_bcast(dyhip_device* dev, const CwShape& sh_in, const float* p0, const float* p1, const float* p2,
                           float* out) {
  const size_t total = cw_size(sh_in.d);
  if (total == 0) return DYHIP_OK;
  CwShape sh;
  const int rank = cw_collapse(sh_in.d, sh_in.s, cw_inputs(FN), sh.d, sh.s);
  bool vec = sh.d[0] % 4 == 0 && aligned16(out);
  const float* ps[3] = {p0, p1, p2};
  for (int k = 0; k < cw_inputs(FN); ++k) {
    if (sh.s[k][0] == 1) {  // 128-bit loads of an operand that follows d0
      vec = vec && aligned16(ps[k]);
      for (int j = 1; j < 5; ++j) vec = vec && sh.s[k][j] % 4 == 0;
    }
  }
  if (rank <= 3) {  // up to three axes: no index arithmetic, several rows in flight per block
    CwShape2 s2;
    s2.d0g = sh.d[0] / (vec ? 4 : 1);
    s2.d1 = sh.d[1];
    s2.d2 = sh.d[2];
    for (int k = 0; k < 3; ++k) {
      s2.s0[k] = sh.s[k][0];
      s2.s1[k] = sh.s[k][1];
      s2.s2[k] = sh.s[k][2];
    }
    s2.tx_shift = 8;
    while (s2.tx_shift > 4 && (128u >> (8 - s2.tx_shift)) >= s2.d0g) --s2.tx_shift;  // 16..256 threads along the inner axis
    const unsigned tx = 1u << s2.tx_shift, gy = cdiv<unsigned>(s2.d1, (256u / tx) * kCwRows);
    const dim3 grid(cdiv<unsigned>(s2.d0g, tx), gy < 65535u ? gy : 65535u, s2.d2 < 65535u ? s2.d2 : 65535u), block(256);
    const bool nt = total * sizeof(float) >= dev->stream_threshold;
    if (vec && nt) hipLaunchKernelGGL((cwise_bcast2_kernel<FN, 4, true>), grid, block, 0, dev->stream, s2, p0, p1, p2, out);
    else if (vec) hipLaunchKernelGGL((cwise_bcast2_kernel<FN, 4, false>), grid, block, 0, dev->stream, s2, p0, p1, p2, out);
    else hipLaunchKernelGGL((cwise_bcast2_kernel<FN, 1, false>), grid, block, 0, dev->stream, s2, p0, p1, p2, out);
  } else if (vec) {
    const size_t groups = total / 4;
    hipLaunchKernelGGL((cwise_bcast_kernel<FN, 4>), dim3(cw_grid(groups, 256, dev)), dim3(256), 0, dev->stream, sh, p0, p1,
                       p2, out, groups);
  } else {
    hipLaunchKernelGGL((cwise_bcast_kernel<FN, 1>), dim3(cw_grid(total, 256, dev)), dim3(256), 0, dev->stream, sh, p0, p1,
                       p2, out, total);
  }
  DYHIP_CHECK_LAUNCH();
  return DYHIP_OK;
}

// scratch / scratch_floats: device memory a stage may leave intermediate sums in (none: single-stage forms only)
template <int FN>
static int cw_launch_reduce(dyhip_device* dev, const unsigned* full, const unsigned* dself, const size_t s[3][5],
                            const float* p0, const float* p1, const float* p2, float* out, bool overwrite, float* scratch,
                            size_t scratch_floats) {
  CwReduce c;
  int nk = 0, nr = 0, runs = 0, first_run_end = 5;
  bool in_run = false;
  for (int j = 0; j < 5; ++j) {
    c.kd[j] = c.rd[j] = 1;
    for (int k = 0; k < 3; ++k) c.ks[k][j] = c.rs[k][j] = 0;
  }
  for (int j = 0; j < 5; ++j) {
    const bool reduced = dself[j] == 1 && full[j] > 1;
    if (reduced) {
      c.rd[nr] = full[j];
      for (int k = 0; k < 3; ++k) c.rs[k][nr] = s[k][j];
      ++nr;
      if (!in_run) ++runs;
      in_run = true;
    } else {
      c.kd[nk] = full[j];
      for (int k = 0; k < 3; ++k) c.ks[k][nk] = s[k][j];
      ++nk;
      if (full[j] > 1) {
        if (in_run && runs == 1 && first_run_end == 5) first_run_end = j;
        in_run = false;
      }
    }
  }
  c.n_out = cw_size(c.kd);
  c.n_red = cw_size(c.rd);
  c.chunks = 1;
  c.chunk_len = 0;
  c.overwrite = overwrite ? 1 : 0;
  const size_t cus = dev->num_cus > 0 ? size_t(dev->num_cus) : 256;
  {
    // the reduced axes as one axis, if every operand walks them alike
    unsigned rd2[5];
    size_t rs2[3][5], rs_in[3][5];
    for (int k = 0; k < 3; ++k)
      for (int j = 0; j < 5; ++j) rs_in[k][j] = c.rs[k][j];
    if (c.n_red >= 2 && c.n_red <= 0xFFFFFFFFull && cw_collapse(c.rd, rs_in, cw_inputs(FN), rd2, rs2) == 1) {
      const float* ps[3] = {p0, p1, p2};
      bool vec = c.n_red % 4 == 0;
      for (int k = 0; k < cw_inputs(FN); ++k) {
        vec = vec && (rs2[k][0] == 0 || rs2[k][0] == 1);
        if (rs2[k][0] == 1) {
          vec = vec && aligned16(ps[k]);
          for (int j = 0; j < 5; ++j) vec = vec && c.ks[k][j] % 4 == 0;
        }
      }
      // the first kept axis is the contiguous one (and not a short one) and the reduced axis is not: lanes along it
      bool mid = c.kd[0] >= 16;
      for (int k = 0; k < cw_inputs(FN); ++k) mid = mid && (c.ks[k][0] == 1 || c.ks[k][0] == 0) && rs2[k][0] != 1;
      // ... and there are enough (kept row tile, other kept index) pairs to fill the GPU: a block owns one
      mid = mid && cdiv<size_t>(c.kd[0], 64) * (c.n_out / c.kd[0]) >= 128;
      // a short reduced axis (a thread per output walked its 35 terms one round trip at a time: 26 us for
      // 1024 x 35 x 16 summed over the 35) takes these kernels too; the shortest stay with a thread per output
      if (mid || c.n_red >= 8) {
        for (int j = 0; j < 5; ++j) {
          c.rd[j] = rd2[j];
          for (int k = 0; k < 3; ++k) c.rs[k][j] = rs2[k][j];
        }
      }
      if (mid) {
        const size_t n_rest = c.n_out / c.kd[0];
        const dim3 grid(cdiv<unsigned>(c.kd[0], 64), unsigned(n_rest < 65535 ? n_rest : 65535)), block(64 * kCwMidWaves);
        hipLaunchKernelGGL(cwise_reduce_mid_kernel<FN>, grid, block, 0, dev->stream, c, p0, p1, p2, out);
        DYHIP_CHECK_LAUNCH();
        return DYHIP_OK;
      }
      if (c.n_red >= 8) {
        // Few outputs with a long reduced axis (3 outputs of 100 000 terms: 12..190 us with a wavefront per output):
        // the axis in pieces over more wavefronts, the pieces' sums in scratch, then summed per output in a fixed order.
        float* target = out;
        if (c.n_out < 8 * cus && c.n_red >= 8192) {
          // a wavefront takes 256 terms a round trip with scalar loads, 1024 with 128-bit loads: about four round trips
          unsigned chunks = unsigned(std::min(cdiv<size_t>(c.n_red, vec ? 4096 : 1024), cdiv<size_t>(16 * cus, c.n_out)));
          const unsigned len = unsigned(cdiv<size_t>(cdiv<size_t>(c.n_red, chunks), 1024) * 1024);
          chunks = unsigned(cdiv<size_t>(c.n_red, len));
          if (chunks >= 2 && scratch != nullptr && scratch_floats >= c.n_out * chunks) {
            c.chunks = chunks;
            c.chunk_len = len;
            c.overwrite = 1;
            target = scratch;
          }
        }
        const dim3 grid(cw_grid(c.n_out * c.chunks, 4, dev)), block(256);
        // operands far larger than the caches are read once: streaming loads
        const bool nt = vec && c.n_out * c.n_red * sizeof(float) >= dev->stream_threshold;
        if (nt) hipLaunchKernelGGL((cwise_reduce_row_kernel<FN, true, true>), grid, block, 0, dev->stream, c, p0, p1, p2, target);
        else if (vec) hipLaunchKernelGGL((cwise_reduce_row_kernel<FN, true, false>), grid, block, 0, dev->stream, c, p0, p1, p2, target);
        else hipLaunchKernelGGL((cwise_reduce_row_kernel<FN, false, false>), grid, block, 0, dev->stream, c, p0, p1, p2, target);
        DYHIP_CHECK_LAUNCH();
        if (target != out) {
          CwReduce f;
          for (int j = 0; j < 5; ++j) {
            f.kd[j] = f.rd[j] = 1;
            for (int k = 0; k < 3; ++k) f.ks[k][j] = f.rs[k][j] = 0;
          }
          f.kd[0] = unsigned(c.n_out);
          f.ks[0][0] = c.chunks;
          f.rd[0] = c.chunks;
          f.rs[0][0] = 1;
          f.n_out = c.n_out;
          f.n_red = c.chunks;
          f.chunks = 1;
          f.chunk_len = 0;
          f.overwrite = overwrite ? 1 : 0;
          hipLaunchKernelGGL((cwise_reduce_row_kernel<3, false, false>), dim3(cw_grid(f.n_out, 4, dev)), dim3(256), 0,
                             dev->stream, f, scratch, nullptr, nullptr, out);
          DYHIP_CHECK_LAUNCH();
        }
        return DYHIP_OK;
      }
    }
  }
  // Reduced axes with kept axes between them (a 512 x 512 x batch-8 tensor summed over its rows and the batch: 47 us
  // with a wavefront per output decomposing every index): the first run of adjacent reduced axes into scratch by the
  // kernels above, the rest from there.
  if (runs >= 2 && c.n_red >= 64 && scratch != nullptr) {
    unsigned dstage[5], full2[5];
    size_t left = 1;
    for (int j = 0; j < 5; ++j) {
      const bool reduced = dself[j] == 1 && full[j] > 1;
      dstage[j] = reduced && j < first_run_end ? 1 : full[j];
      full2[j] = dstage[j];
      left *= full2[j];
    }
    if (left <= scratch_floats / 2) {
      DYHIP_CHECK_STATUS(cw_launch_reduce<FN>(dev, full, dstage, s, p0, p1, p2, scratch, true, scratch + left,
                                              scratch_floats - left));
      size_t s2[3][5];
      cw_strides(full2, full2, s2[0]);
      for (int j = 0; j < 5; ++j) s2[1][j] = s2[2][j] = 0;
      return cw_launch_reduce<3>(dev, full2, dself, s2, scratch, nullptr, nullptr, out, overwrite, scratch + left,
                                 scratch_floats - left);
    }
  }
  if (c.n_red >= 64)
    hipLaunchKernelGGL(cwise_reduce_wave_kernel<FN>, dim3(cw_grid(c.n_out, 4, dev)), dim3(256), 0, dev->stream, c, p0, p1, p2,
                       out);
  else
    hipLaunchKernelGGL(cwise_reduce_thread_kernel<FN>, dim3(cw_grid(c.n_out, 256, dev)), dim3(256), 0, dev->stream, c, p0,
                       p1, p2, out);
  DYHIP_CHECK_LAUNCH();
  return DYHIP_OK;
}

// kept axes form a prefix of the axes and every later axis is reduced (or has size 1)?  Then the reduction is
// out[j] += sum_b in[b * n + j] with n = the prefix's size: the coalesced batch reduction.
static bool cw_prefix_split(const unsigned* full, const unsigned* dself, size_t* n, size_t* bd) {
  int first_red = 5;
  for (int j = 0; j < 5; ++j)
    if (dself[j] == 1 && full[j] > 1) {
      first_red = j;
      break;
    }
  *n = 1;
  *bd = 1;
  for (int j = 0; j < 5; ++j) {
    if (j < first_red) *n *= full[j];
    else {
      if (dself[j] != 1) return false;
      *bd *= full[j];
    }
  }
  return first_red < 5;
}

struct AddConst {
  float c;
  __device__ float operator()(float x) const { return c + x; }
};
struct SubFromConst {
  float c;
  __device__ float operator()(float x) const { return c - x; }
};

template <class F>
__global__ __launch_bounds__(256) void const_op_kernel(size_t n, const float* __restrict__ x, float* __restrict__ y, F f) {
  for (size_t j = size_t(blockIdx.x) * 256 + threadIdx.x; j < n; j += size_t(gridDim.x) * 256) y[j] = f(x[j]);
}

}  // namespace dyhip

using namespace dyhip;

extern "C" {

int dyhip_cwise_forward(dyhip_device* dev, int op, const unsigned* dims_a, const unsigned* dims_b, const float* a,
                        const float* b, float* fx) {
  DYHIP_CHECK_DEV(dev);
  DYHIP_CHECK_STATUS(cw_check(op, dims_a, dims_b, "cwise forward"));
  DYHIP_REQUIRE(a && b && fx, "null tensor pointer");
  bool dims_equal = true;
  for (int j = 0; j < 4; ++j) dims_equal = dims_equal && dims_a[j] == dims_b[j];
  const size_t n = size_t(dims_a[0]) * dims_a[1] * dims_a[2] * dims_a[3];
  if (dims_equal && op == DYHIP_CWISE_SUM) return dyhip_csum_forward(dev, n, dims_a[4], dims_b[4], a, b, fx);
  if (dims_equal && op == DYHIP_CWISE_MULT) return dyhip_cmult_forward(dev, n, dims_a[4], dims_b[4], a, b, fx);
  CwShape sh;
  for (int j = 0; j < 5; ++j) sh.d[j] = dims_a[j] > dims_b[j] ? dims_a[j] : dims_b[j];
  cw_strides(dims_a, sh.d, sh.s[0]);
  cw_strides(dims_b, sh.d, sh.s[1]);
  for (int j = 0; j < 5; ++j) sh.s[2][j] = 0;
  if (op == DYHIP_CWISE_SUM) return cw_launch_bcast<0>(dev, sh, a, b, nullptr, fx);
  if (op == DYHIP_CWISE_MULT) return cw_launch_bcast<1>(dev, sh, a, b, nullptr, fx);
  return cw_launch_bcast<2>(dev, sh, a, b, nullptr, fx);
}

int dyhip_cwise_backward_workspace(const unsigned* dims_a, const unsigned* dims_b, unsigned i, size_t* ws_bytes) {
  DYHIP_REQUIRE(ws_bytes != nullptr && dims_a != nullptr && dims_b != nullptr && i < 2, "bad argument");
  unsigned full[5];
  for (int j = 0; j < 5; ++j) full[j] = dims_a[j] > dims_b[j] ? dims_a[j] : dims_b[j];
  size_t n = 0, bd = 0;
  *ws_bytes = 0;
  if (cw_prefix_split(full, i == 0 ? dims_a : dims_b, &n, &bd) && bd <= 0xFFFFFFFFull)
    return dyhip_batch_reduce_workspace(n, static_cast<unsigned>(bd), ws_bytes);
  return DYHIP_OK;
}

int dyhip_cwise_backward(dyhip_device* dev, int op, const unsigned* dims_a, const unsigned* dims_b, const float* a,
                         const float* b, const float* dEdf, unsigned i, float* dEdxi, void* ws, size_t ws_bytes) {
  DYHIP_CHECK_DEV(dev);
  DYHIP_CHECK_STATUS(cw_check(op, dims_a, dims_b, "cwise backward"));
  DYHIP_REQUIRE(i < 2, "the operator has two arguments (i = %u)", i);
  DYHIP_REQUIRE(a && b && dEdf && dEdxi, "null tensor pointer");
  unsigned full[5];
  for (int j = 0; j < 5; ++j) full[j] = dims_a[j] > dims_b[j] ? dims_a[j] : dims_b[j];
  const unsigned* dself = i == 0 ? dims_a : dims_b;
  const unsigned* dother = i == 0 ? dims_b : dims_a;
  const float* other = i == 0 ? b : a;
  bool reduces = false, other_full = true;
  for (int j = 0; j < 5; ++j) {
    reduces = reduces || (dself[j] == 1 && full[j] > 1);
    other_full = other_full && dother[j] == full[j];
  }
  // operands of the term: p0 = dEdf (full size); sum: -, multiply: p1 = other, quotient: p1 = b, p2 = a
  size_t s[3][5];
  cw_strides(full, full, s[0]);
  const float *p1 = nullptr, *p2 = nullptr;
  for (int j = 0; j < 5; ++j) s[1][j] = s[2][j] = 0;
  if (op == DYHIP_CWISE_MULT) {
    p1 = other;
    cw_strides(dother, full, s[1]);
  } else if (op == DYHIP_CWISE_QUOTIENT) {
    p1 = b;
    cw_strides(dims_b, full, s[1]);
    p2 = a;
    cw_strides(dims_a, full, s[2]);
  }
  if (!reduces) {
    CwShape sh;
    for (int j = 0; j < 5; ++j) {
      sh.d[j] = full[j];
      for (int k = 0; k < 3; ++k) sh.s[k][j] = s[k][j];
    }
    if (op == DYHIP_CWISE_SUM) return cw_launch_bcast<3>(dev, sh, dEdf, nullptr, nullptr, dEdxi);
    if (op == DYHIP_CWISE_MULT) return cw_launch_bcast<4>(dev, sh, dEdf, p1, nullptr, dEdxi);
    if (i == 0) return cw_launch_bcast<5>(dev, sh, dEdf, p1, nullptr, dEdxi);
    return cw_launch_bcast<6>(dev, sh, dEdf, p1, p2, dEdxi);
  }
  DYHIP_REQUIRE(!(op == DYHIP_CWISE_QUOTIENT && i == 0), "CwiseQuotient: the left argument is never broadcast");
  size_t n = 0, bd = 0;
  if (op != DYHIP_CWISE_QUOTIENT && cw_prefix_split(full, dself, &n, &bd) && bd <= 0xFFFFFFFFull &&
      (op == DYHIP_CWISE_SUM || other_full))
    return batch_reduce(dev, n, static_cast<unsigned>(bd), dEdf, op == DYHIP_CWISE_MULT ? other : nullptr, dEdxi, true, ws,
                        ws_bytes);
  // intermediate sums of the multi-stage reductions: the device's own scratch (stream-ordered like every other use)
  float* scratch = static_cast<float*>(dev->gemm_ws);
  const size_t scratch_floats = scratch != nullptr ? dev->gemm_ws_bytes / sizeof(float) : 0;
  if (op == DYHIP_CWISE_SUM)
    return cw_launch_reduce<3>(dev, full, dself, s, dEdf, nullptr, nullptr, dEdxi, false, scratch, scratch_floats);
  if (op == DYHIP_CWISE_MULT)
    return cw_launch_reduce<4>(dev, full, dself, s, dEdf, p1, nullptr, dEdxi, false, scratch, scratch_floats);
  return cw_launch_reduce<6>(dev, full, dself, s, dEdf, p1, p2, dEdxi, false, scratch, scratch_floats);
}

int dyhip_const_plus_x_forward(dyhip_device* dev, size_t n, float c, const float* x, float* fx) {
  DYHIP_CHECK_DEV(dev);
  if (n == 0) return DYHIP_OK;
  DYHIP_REQUIRE(x && fx, "null tensor pointer");
  hipLaunchKernelGGL(const_op_kernel<AddConst>, dim3(cw_grid(n, 256, dev)), dim3(256), 0, dev->stream, n, x, fx, AddConst{c});
  DYHIP_CHECK_LAUNCH();
  return DYHIP_OK;
}

int dyhip_const_minus_x_forward(dyhip_device* dev, size_t n, float c, const float* x, float* fx) {
  DYHIP_CHECK_DEV(dev);
  if (n == 0) return DYHIP_OK;
  DYHIP_REQUIRE(x && fx, "null tensor pointer");
  hipLaunchKernelGGL(const_op_kernel<SubFromConst>, dim3(cw_grid(n, 256, dev)), dim3(256), 0, dev->stream, n, x, fx,
                     SubFromConst{c});
  DYHIP_CHECK_LAUNCH();
  return DYHIP_OK;
}

}  // extern "C"
