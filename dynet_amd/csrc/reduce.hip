// Reductions: sum over the batch dimension (sum_batches and the broadcast-side
// backward of cmult / csum), mean_elems / std_elems, and the fused LayerNorm.
//
// Replaces the Eigen reductions of SumDimension (dynet/nodes-arith-sum.cc:197-248),
// MomentDimension (dynet/nodes-moments.cc:181-309), StdDimension (:434-555) and the
// eight-node layer_norm composite of dynet/expr.cc:248-253.
//
// All reductions are deterministic: partial sums are combined in a fixed order
// (lanes by xor-butterfly, waves and grid partials by ascending index), never
// with floating-point atomics.
#include "common.h"

namespace dyhip {

// ============================================================================
// batch reduction: out[j] (+)= sum_b in0[b*n + j] * (in1 ? in1[b*n + j] : 1)
// ============================================================================
//
// Block = 64 column lanes x NW waves.  Lane l owns VEC consecutive columns
// (VEC = 4: one 128-bit access); wave w of split s sums batch elements
// s*per_split + w, + NW, ...; the NW wave partials are combined through LDS in
// ascending w.  With more than one split the block writes its partial row to
// the workspace and a second kernel adds the splits in ascending s.
constexpr int kBrWaves = 16;
constexpr unsigned kBrMaxSplits = 64;

struct BrPlan {
  unsigned tiles;      // column tiles of 64*VEC columns
  unsigned splits;     // batch splits
  unsigned per_split;  // batch elements per split
  int vec;
};

static BrPlan br_plan(size_t n, unsigned bd, bool vec_ok) {
  BrPlan p;
  // A reduction of at most 4 MB is bound by launches, not bytes: one launch of scalar tiles (four times as
  // many blocks as vector tiles) beats split partial sums plus a combining launch when there are enough of them.
  if (n * size_t(bd) <= (size_t(1) << 20) && n >= 32 * 64) {
    p.vec = 1;
    p.tiles = static_cast<unsigned>(cdiv<size_t>(n, 64));
    p.splits = 1;
    p.per_split = bd;
    return p;
  }
  p.vec = vec_ok ? 4 : 1;
  p.tiles = static_cast<unsigned>(cdiv<size_t>(n, size_t(64) * p.vec));
  unsigned want = p.tiles >= 192 ? 1u : cdiv<unsigned>(512u, p.tiles);
  unsigned max_by_work = cdiv<unsigned>(bd, kBrWaves * 2);
  if (want > max_by_work) want = max_by_work;
  if (want > kBrMaxSplits) want = kBrMaxSplits;
  if (want < 1) want = 1;
  p.per_split = cdiv<unsigned>(bd, want);
  p.splits = cdiv<unsigned>(bd, p.per_split);
  return p;
}

template <int VEC, bool MUL, bool NT>
__global__ __launch_bounds__(64 * kBrWaves) void batch_reduce_kernel(size_t n, unsigned bd, unsigned per_split,
                                                                    const float* __restrict__ in0,
                                                                    const float* __restrict__ in1,
                                                                    float* __restrict__ out, int accumulate,
                                                                    float* __restrict__ partial) {
  __shared__ float lds[kBrWaves][64 * VEC];
  const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
  const size_t col = (size_t(blockIdx.x) * 64 + lane) * VEC;
  const unsigned b0 = blockIdx.y * per_split;
  const unsigned b1 = min(bd, b0 + per_split);
  float acc[VEC];
#pragma unroll
  for (int v = 0; v < VEC; ++v) acc[v] = 0.f;
  if (col < n) {
    constexpr int U = 4;
    unsigned b = b0 + w;
    for (; b + (U - 1) * kBrWaves < b1; b += U * kBrWaves) {
      float x[U][VEC], y[U][VEC];
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const size_t off = size_t(b + u * kBrWaves) * n + col;
        if (VEC == 4) {
          const float4 t = ldg4<NT>(reinterpret_cast<const float4*>(in0 + off));
          x[u][0] = t.x; x[u][1 % VEC] = t.y; x[u][2 % VEC] = t.z; x[u][3 % VEC] = t.w;
          if (MUL) {
            const float4 s = ldg4<NT>(reinterpret_cast<const float4*>(in1 + off));
            y[u][0] = s.x; y[u][1 % VEC] = s.y; y[u][2 % VEC] = s.z; y[u][3 % VEC] = s.w;
          }
        } else {
          x[u][0] = in0[off];
          if (MUL) y[u][0] = in1[off];
        }
      }
#pragma unroll
      for (int u = 0; u < U; ++u)
#pragma unroll
        for (int v = 0; v < VEC; ++v) acc[v] += MUL ? x[u][v] * y[u][v] : x[u][v];
    }
    for (; b < b1; b += kBrWaves) {
      const size_t off = size_t(b) * n + col;
#pragma unroll
      for (int v = 0; v < VEC; ++v) acc[v] += MUL ? in0[off + v] * in1[off + v] : in0[off + v];
    }
  }
#pragma unroll
  for (int v = 0; v < VEC; ++v) lds[w][lane * VEC + v] = acc[v];
  __syncthreads();
  if (w == 0 && col < n) {
#pragma unroll
    for (int v = 0; v < VEC; ++v) {
      float t = lds[0][lane * VEC + v];
#pragma unroll
      for (int k = 1; k < kBrWaves; ++k) t += lds[k][lane * VEC + v];
      if (partial)
        partial[size_t(blockIdx.y) * n + col + v] = t;
      else
        out[col + v] = accumulate ? out[col + v] + t : t;
    }
  }
}

// out[j] (+)= sum_s partial[s*n + j].  Block = 64 columns x kCombSlices slices:
// slice q adds splits q, q+16, ... in ascending order with up to sixteen loads in flight,
// then the slices are added in ascending q.  blockIdx.y selects one of two
// (partial, out) pairs so that two outputs share a launch.
constexpr int kCombSlices = 16;
__global__ __launch_bounds__(64 * kCombSlices) void combine_partials_kernel(size_t n, unsigned splits,
                                                                           const float* __restrict__ partial0,
                                                                           float* __restrict__ out0,
                                                                           const float* __restrict__ partial1,
                                                                           float* __restrict__ out1,
                                                                           int accumulate) {
  __shared__ float lds[kCombSlices][64];
  const float* partial = blockIdx.y == 0 ? partial0 : partial1;
  float* out = blockIdx.y == 0 ? out0 : out1;
  const int lane = threadIdx.x & 63, q = threadIdx.x >> 6;
  const size_t j = size_t(blockIdx.x) * 64 + lane;
  float acc = 0.f;
  if (j < n) {
    unsigned sp = q;
    constexpr int U = 16;  // loads in flight per thread
    for (; sp + (U - 1) * kCombSlices < splits; sp += U * kCombSlices) {
      float a[U];
#pragma unroll
      for (int u = 0; u < U; ++u) a[u] = partial[size_t(sp + u * kCombSlices) * n + j];
#pragma unroll
      for (int u = 0; u < U; ++u) acc += a[u];
    }
    for (; sp + 3 * kCombSlices < splits; sp += 4 * kCombSlices) {
      const float a0 = partial[size_t(sp) * n + j], a1 = partial[size_t(sp + kCombSlices) * n + j],
                  a2 = partial[size_t(sp + 2 * kCombSlices) * n + j],
                  a3 = partial[size_t(sp + 3 * kCombSlices) * n + j];
      acc += a0;
      acc += a1;
      acc += a2;
      acc += a3;
    }
    for (; sp < splits; sp += kCombSlices) acc += partial[size_t(sp) * n + j];
  }
  lds[q][lane] = acc;
  __syncthreads();
  if (q == 0 && j < n) {
    float t = lds[0][lane];
#pragma unroll
    for (int k = 1; k < kCombSlices; ++k) t += lds[k][lane];
    out[j] = accumulate ? out[j] + t : t;
  }
}

// The same for rows of float4 with many more blocks: a block owns 8 float4 columns (one 128-byte line of every
// partial row) and kCombVecSlots row slots (32, or 64 for more than 128 partial rows, so that 256 rows are one batch of
// four loads per thread, all in flight at once, instead of two dependent batches); slot q adds rows q, q+slots, ...
// in ascending order, then eight threads per column add every eighth slot and one adds those eight: a fixed order
// again for a given number of partial rows.
constexpr int kCombVecCols = 8;
template <int kCombVecSlots>
__global__ __launch_bounds__(kCombVecCols * kCombVecSlots) void combine_partials_vec_kernel(unsigned n4, unsigned splits,
                                                                               const float4* __restrict__ partial0,
                                                                               float4* __restrict__ out0,
                                                                               const float4* __restrict__ partial1,
                                                                               float4* __restrict__ out1,
                                                                               int accumulate, int nt) {
  __shared__ float4 lds[kCombVecSlots][kCombVecCols];
  const float4* partial = blockIdx.y == 0 ? partial0 : partial1;
  float4* out = blockIdx.y == 0 ? out0 : out1;
  const unsigned c = threadIdx.x % kCombVecCols, q = threadIdx.x / kCombVecCols;
  const unsigned col = blockIdx.x * kCombVecCols + c;
  const bool in = col < n4;
  float4 acc = make_float4(0.f, 0.f, 0.f, 0.f);
  float4 old = acc;
  if (in && q == 0 && accumulate) old = out[col];
  if (in) {
    unsigned sp = q;
    for (; sp + 3 * kCombVecSlots < splits; sp += 4 * kCombVecSlots) {
      // nt (the same for every thread): the partial rows are larger than the L2s and read once
      float4 a0, a1, a2, a3;
      if (nt) {
        a0 = ldg4<true>(partial + size_t(sp) * n4 + col);
        a1 = ldg4<true>(partial + size_t(sp + kCombVecSlots) * n4 + col);
        a2 = ldg4<true>(partial + size_t(sp + 2 * kCombVecSlots) * n4 + col);
        a3 = ldg4<true>(partial + size_t(sp + 3 * kCombVecSlots) * n4 + col);
      } else {
        a0 = partial[size_t(sp) * n4 + col];
        a1 = partial[size_t(sp + kCombVecSlots) * n4 + col];
        a2 = partial[size_t(sp + 2 * kCombVecSlots) * n4 + col];
        a3 = partial[size_t(sp + 3 * kCombVecSlots) * n4 + col];
      }
      acc.x += a0.x; acc.y += a0.y; acc.z += a0.z; acc.w += a0.w;
      acc.x += a1.x; acc.y += a1.y; acc.z += a1.z; acc.w += a1.w;
      acc.x += a2.x; acc.y += a2.y; acc.z += a2.z; acc.w += a2.w;
      acc.x += a3.x; acc.y += a3.y; acc.z += a3.z; acc.w += a3.w;
    }
    for (; sp < splits; sp += kCombVecSlots) {
      const float4 a = partial[size_t(sp) * n4 + col];
      acc.x += a.x; acc.y += a.y; acc.z += a.z; acc.w += a.w;
    }
  }
  lds[q][c] = acc;
  __syncthreads();
  if (q < 8) {
    float4 t = lds[q][c];
    for (int k = q + 8; k < kCombVecSlots; k += 8) {
      const float4 a = lds[k][c];
      t.x += a.x; t.y += a.y; t.z += a.z; t.w += a.w;
    }
    acc = t;
  }
  __syncthreads();
  if (q < 8) lds[q][c] = acc;
  __syncthreads();
  if (q == 0 && in) {
    float4 t = lds[0][c];
    for (int k = 1; k < 8; ++k) {
      const float4 a = lds[k][c];
      t.x += a.x; t.y += a.y; t.z += a.z; t.w += a.w;
    }
    out[col] = make_float4(old.x + t.x, old.y + t.y, old.z + t.z, old.w + t.w);
  }
}

static void launch_combine(dyhip_device* dev, size_t n, unsigned splits, const float* p0, float* o0, const float* p1,
                           float* o1, int accumulate, int nt = 0) {
  if (n % 4 == 0 && splits >= 32 && aligned16(p0) && aligned16(o0) && (p1 == nullptr || (aligned16(p1) && aligned16(o1)))) {
    const unsigned n4 = static_cast<unsigned>(n / 4);
    const dim3 grid(cdiv<unsigned>(n4, kCombVecCols), p1 != nullptr ? 2 : 1);
    if (splits > 128)
      hipLaunchKernelGGL(combine_partials_vec_kernel<64>, grid, dim3(kCombVecCols * 64), 0, dev->stream, n4, splits,
                         reinterpret_cast<const float4*>(p0), reinterpret_cast<float4*>(o0),
                         reinterpret_cast<const float4*>(p1), reinterpret_cast<float4*>(o1), accumulate, nt);
    else
      hipLaunchKernelGGL(combine_partials_vec_kernel<32>, grid, dim3(kCombVecCols * 32), 0, dev->stream, n4, splits,
                         reinterpret_cast<const float4*>(p0), reinterpret_cast<float4*>(o0),
                         reinterpret_cast<const float4*>(p1), reinterpret_cast<float4*>(o1), accumulate, nt);
    return;
  }
  const dim3 grid((unsigned)cdiv<size_t>(n, 64), p1 != nullptr ? 2 : 1);
  hipLaunchKernelGGL(combine_partials_kernel, grid, dim3(64 * kCombSlices), 0, dev->stream, n, splits, p0, o0, p1, o1,
                     accumulate);
}

// out[j] (+)= sum_s partial[s * n + j] for other files' split sums (ascending s; the float4 form from 32 slices on)
int combine_partial_rows(dyhip_device* dev, size_t n, unsigned splits, const float* partial, float* out, bool accumulate) {
  launch_combine(dev, n, splits, partial, out, nullptr, nullptr, accumulate ? 1 : 0);
  DYHIP_CHECK_LAUNCH();
  return DYHIP_OK;
}

// ---- batch elements of at most 32 floats, many of them (a scalar or a handful of values per batch element: the
// tile kernel above has n of a wavefront's 64 lanes at work, 68 us for a million scalars) -----------------------
// The tensor is walked flat: a block owns a contiguous piece that starts at a multiple of S = (256 / n) * n entries
// and thread t < S steps through it by S, so all its entries belong to column t % n; eight loads in flight.  The
// threads of a column meet in LDS in ascending order, the blocks' partial rows in the combine kernel.
constexpr unsigned kBrFlatMaxN = 32;
constexpr unsigned kBrFlatMaxBlocks = 512;
constexpr size_t kBrFlatMinTotal = 32768;

static bool br_flat(size_t n, unsigned bd) { return n <= kBrFlatMaxN && n * size_t(bd) >= kBrFlatMinTotal; }

template <bool MUL>
__global__ __launch_bounds__(256) void batch_reduce_flat_kernel(unsigned n, size_t total, size_t per_block,
                                                                const float* __restrict__ in0,
                                                                const float* __restrict__ in1,
                                                                float* __restrict__ partial) {
  __shared__ float lds[256];
  const unsigned t = threadIdx.x, S = 256 / n * n;
  const size_t b0 = size_t(blockIdx.x) * per_block, b1 = min(total, b0 + per_block);
  float acc = 0.f;
  if (t < S && b0 < b1) {
    constexpr int U = 8;
    for (size_t e = b0 + t; e < b1; e += size_t(U) * S) {
      float x[U], y[U];
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const size_t at = min(e + size_t(u) * S, b1 - 1);  // clamped, masked below
        x[u] = in0[at];
        y[u] = MUL ? in1[at] : 1.f;
      }
#pragma unroll
      for (int u = 0; u < U; ++u)
        if (e + size_t(u) * S < b1) acc += MUL ? x[u] * y[u] : x[u];
    }
  }
  __shared__ float lds2[256];
  lds[t] = acc;
  __syncthreads();
  // column c is held by threads c, c + n, ...: eight threads a column add every eighth of them, then one adds the eight
  // (one thread walking all 256 entries of a scalar's column was 7 us of dependent LDS reads)
  if (t < 8 * n) {
    const unsigned c = t % n, j = t / n;
    float s = 0.f;
    for (unsigned k = c + j * n; k < S; k += 8 * n) s += lds[k];
    lds2[t] = s;
  }
  __syncthreads();
  if (t < n) {
    float s = 0.f;
#pragma unroll
    for (unsigned j = 0; j < 8; ++j) s += lds2[t + j * n];
    partial[size_t(blockIdx.x) * n + t] = s;
  }
}

int batch_reduce(dyhip_device* dev, size_t n, unsigned bd, const float* in0, const float* in1, float* out,
                 bool accumulate, void* ws, size_t ws_bytes) {
  if (n == 0) return DYHIP_OK;
  DYHIP_REQUIRE(bd >= 1, "batch reduction over an empty batch");
  if (br_flat(n, bd)) {
    const unsigned nn = static_cast<unsigned>(n), S = 256 / nn * nn;
    const size_t total = n * size_t(bd);
    // about four passes of eight loads a thread, at most kBrFlatMaxBlocks blocks
    const size_t want = std::min<size_t>(kBrFlatMaxBlocks, cdiv<size_t>(total, size_t(S) * 32));
    const size_t per_block = cdiv<size_t>(cdiv<size_t>(total, want), S) * S;
    const unsigned blocks = static_cast<unsigned>(cdiv<size_t>(total, per_block));
    const size_t need = size_t(blocks) * n * sizeof(float);
    DYHIP_REQUIRE(ws != nullptr && ws_bytes >= need, "batch reduction needs %zu workspace bytes, got %zu", need, ws_bytes);
    float* partial = static_cast<float*>(ws);
    if (in1)
      hipLaunchKernelGGL(batch_reduce_flat_kernel<true>, dim3(blocks), dim3(256), 0, dev->stream, nn, total, per_block, in0,
                         in1, partial);
    else
      hipLaunchKernelGGL(batch_reduce_flat_kernel<false>, dim3(blocks), dim3(256), 0, dev->stream, nn, total, per_block, in0,
                         in1, partial);
    DYHIP_CHECK_LAUNCH();
    launch_combine(dev, n, blocks, partial, out, nullptr, nullptr, accumulate ? 1 : 0);
    DYHIP_CHECK_LAUNCH();
    return DYHIP_OK;
  }
  const bool vec_ok = (n % 4 == 0) && aligned16(in0) && (in1 == nullptr || aligned16(in1));
  const BrPlan p = br_plan(n, bd, vec_ok);
  float* partial = nullptr;
  if (p.splits > 1) {
    const size_t need = size_t(p.splits) * n * sizeof(float);
    DYHIP_REQUIRE(ws != nullptr && ws_bytes >= need, "batch reduction needs %zu workspace bytes, got %zu", need,
                  ws_bytes);
    partial = static_cast<float*>(ws);
  }
  const dim3 grid(p.tiles, p.splits), block(64 * kBrWaves);
  const int acc = accumulate ? 1 : 0;
  const bool stream = n * size_t(bd) * sizeof(float) >= dev->stream_threshold;
#define DYHIP_BR_LAUNCH(VEC, MUL, NT)                                                                           \
  hipLaunchKernelGGL((batch_reduce_kernel<VEC, MUL, NT>), grid, block, 0, dev->stream, n, bd, p.per_split, in0, \
                     in1, out, acc, partial)
  if (p.vec == 4) {
    if (stream) {
      if (in1) DYHIP_BR_LAUNCH(4, true, true); else DYHIP_BR_LAUNCH(4, false, true);
    } else {
      if (in1) DYHIP_BR_LAUNCH(4, true, false); else DYHIP_BR_LAUNCH(4, false, false);
    }
  } else {
    if (in1) DYHIP_BR_LAUNCH(1, true, false); else DYHIP_BR_LAUNCH(1, false, false);
  }
#undef DYHIP_BR_LAUNCH
  DYHIP_CHECK_LAUNCH();
  if (partial) {
    launch_combine(dev, n, p.splits, partial, out, nullptr, nullptr, acc);
    DYHIP_CHECK_LAUNCH();
  }
  return DYHIP_OK;
}

// ============================================================================
// mean_elems / std_elems: one value per batch element (block per batch element)
// ============================================================================
// Block-per-element forms for elements longer than the register-resident kernels below take: 1024 threads, four
// independent loads in flight per thread and pass (the second pass finds the element in the caches).
constexpr int kMomThreads = 1024;
template <bool STD>
__global__ __launch_bounds__(kMomThreads) void moment_fwd_kernel(size_t n, const float* __restrict__ x,
                                                                 float* __restrict__ y) {
  __shared__ float red[kMomThreads / 64];
  const float* px = x + size_t(blockIdx.x) * n;
  float s = 0.f;
  for (size_t j0 = threadIdx.x; j0 < n; j0 += 4 * kMomThreads) {
    float a[4];
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const size_t j = j0 + size_t(u) * kMomThreads;
      a[u] = px[j < n ? j : n - 1];
    }
#pragma unroll
    for (int u = 0; u < 4; ++u)
      if (j0 + size_t(u) * kMomThreads < n) s += a[u];
  }
  const float mean = block_sum<kMomThreads / 64>(s, red) / float(n);
  if (!STD) {
    if (threadIdx.x == 0) y[blockIdx.x] = mean;
    return;
  }
  float v = 0.f;
  for (size_t j0 = threadIdx.x; j0 < n; j0 += 4 * kMomThreads) {
    float a[4];
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const size_t j = j0 + size_t(u) * kMomThreads;
      a[u] = px[j < n ? j : n - 1];
    }
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      if (j0 + size_t(u) * kMomThreads < n) {
        const float d = a[u] - mean;
        v += d * d;
      }
    }
  }
  const float var = block_sum<kMomThreads / 64>(v, red) / float(n);
  if (threadIdx.x == 0) y[blockIdx.x] = sqrtf(var);
}

// dx[b, j] += dEdf[b] / n
__global__ __launch_bounds__(256) void mean_bwd_kernel(size_t n, unsigned bd, const float* __restrict__ dEdf,
                                                       float* __restrict__ dEdx) {
  const size_t j = size_t(blockIdx.x) * 256 + threadIdx.x;
  if (j >= n) return;
  for (unsigned b = blockIdx.y; b < bd; b += gridDim.y)  // the grid's second dimension holds at most 65535 blocks
    dEdx[size_t(b) * n + j] += dEdf[b] / float(n);
}

// dx[b, j] += (2/n) * (x - mean_b) * (dEdf[b] / (2 * fx[b]))
__global__ __launch_bounds__(kMomThreads) void std_bwd_kernel(size_t n, const float* __restrict__ x,
                                                              const float* __restrict__ fx,
                                                              const float* __restrict__ dEdf, float* __restrict__ dEdx) {
  __shared__ float red[kMomThreads / 64];
  const float* px = x + size_t(blockIdx.x) * n;
  float s = 0.f;
  for (size_t j0 = threadIdx.x; j0 < n; j0 += 4 * kMomThreads) {
    float a[4];
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const size_t j = j0 + size_t(u) * kMomThreads;
      a[u] = px[j < n ? j : n - 1];
    }
#pragma unroll
    for (int u = 0; u < 4; ++u)
      if (j0 + size_t(u) * kMomThreads < n) s += a[u];
  }
  const float mean = block_sum<kMomThreads / 64>(s, red) / float(n);
  const float sb = dEdf[blockIdx.x] / (2.f * fx[blockIdx.x]);
  const float c = 2.f / float(n);
  float* pd = dEdx + size_t(blockIdx.x) * n;
  for (size_t j0 = threadIdx.x; j0 < n; j0 += 4 * kMomThreads) {
    float a[4], o[4];
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const size_t j = j0 + size_t(u) * kMomThreads, jc = j < n ? j : n - 1;
      a[u] = px[jc];
      o[u] = pd[jc];
    }
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const size_t j = j0 + size_t(u) * kMomThreads;
      if (j < n) pd[j] = o[u] + c * (a[u] - mean) * sb;
    }
  }
}

// ---- long elements of a small batch (a block per element is then a handful of blocks: 4 elements of 1M floats took
// 60 / 117 / 326 us for mean / std / std backward): an element is cut into chunks of kMomChunk floats, a 256-thread
// block holds its chunk in registers and leaves the chunk's sum (MODE 0) or its mean and centered sum of squares
// (MODE 1); a wavefront per element then merges the chunks in a fixed order (for the variance by the pairwise
// update of means and centered sums, which is at least as accurate as the two passes it replaces).
constexpr unsigned kMomChunk = 8192;
template <int MODE>
__global__ __launch_bounds__(256) void moment_chunk_kernel(size_t n, const float* __restrict__ x, float* __restrict__ stats) {
  __shared__ float red[4];
  const size_t c0 = size_t(blockIdx.x) * kMomChunk, c1 = min(n, c0 + kMomChunk);
  const float* px = x + size_t(blockIdx.y) * n;
  constexpr int U = kMomChunk / 256;
  float v[U];
#pragma unroll
  for (int u = 0; u < U; ++u) {
    const size_t j = c0 + threadIdx.x + size_t(u) * 256;
    v[u] = px[j < c1 ? j : c1 - 1];
  }
  float s = 0.f;
#pragma unroll
  for (int u = 0; u < U; ++u)
    if (c0 + threadIdx.x + size_t(u) * 256 < c1) s += v[u];
  const float sum = block_sum<4>(s, red);
  const size_t at = size_t(blockIdx.y) * gridDim.x + blockIdx.x;
  if (MODE == 0) {
    if (threadIdx.x == 0) stats[at] = sum;
    return;
  }
  const float mean = sum / float(c1 - c0);
  float q = 0.f;
#pragma unroll
  for (int u = 0; u < U; ++u) {
    if (c0 + threadIdx.x + size_t(u) * 256 < c1) {
      const float d = v[u] - mean;
      q += d * d;
    }
  }
  const float m2 = block_sum<4>(q, red);
  if (threadIdx.x == 0) {
    stats[2 * at] = mean;
    stats[2 * at + 1] = m2;
  }
}

// the mean of an element from its chunk sums, by one wavefront (every lane returns it)
__device__ __forceinline__ float moment_mean_of_chunks(const float* __restrict__ sums, unsigned chunks, size_t n, int lane) {
  float s = 0.f;
  for (unsigned c = lane; c < chunks; c += 64) s += sums[c];
  return wave_sum(s) / float(n);
}

template <int MODE>
__global__ __launch_bounds__(64) void moment_finish_kernel(size_t n, unsigned chunks, const float* __restrict__ stats,
                                                          float* __restrict__ y) {
  const int lane = threadIdx.x;
  const unsigned b = blockIdx.x;
  if (MODE == 0) {
    const float mean = moment_mean_of_chunks(stats + size_t(b) * chunks, chunks, n, lane);
    if (lane == 0) y[b] = mean;
    return;
  }
  const float* st = stats + size_t(b) * chunks * 2;
  auto count = [&](unsigned c) { return float(min(n, size_t(c + 1) * kMomChunk) - size_t(c) * kMomChunk); };
  float s = 0.f;
  for (unsigned c = lane; c < chunks; c += 64) s += count(c) * st[2 * c];
  const float mean = wave_sum(s) / float(n);
  float q = 0.f;
  for (unsigned c = lane; c < chunks; c += 64) {
    const float d = st[2 * c] - mean;
    q += st[2 * c + 1] + count(c) * d * d;
  }
  const float m2 = wave_sum(q);
  if (lane == 0) y[b] = sqrtf(m2 / float(n));
}

// dx[b, j] += (2/n) * (x - mean_b) * (dEdf[b] / (2 * fx[b])) with the mean from the chunk sums; a block per 1024 entries
__global__ __launch_bounds__(256) void std_bwd_chunked_kernel(size_t n, unsigned chunks, const float* __restrict__ x,
                                                              const float* __restrict__ sums, const float* __restrict__ fx,
                                                              const float* __restrict__ dEdf, float* __restrict__ dEdx) {
  const unsigned b = blockIdx.y;
  const float mean = moment_mean_of_chunks(sums + size_t(b) * chunks, chunks, n, threadIdx.x & 63);
  const float sb = dEdf[b] / (2.f * fx[b]);
  const float c = 2.f / float(n);
  const float* px = x + size_t(b) * n;
  float* pd = dEdx + size_t(b) * n;
  const size_t j0 = size_t(blockIdx.x) * 1024 + threadIdx.x;
  float a[4], o[4];
#pragma unroll
  for (int u = 0; u < 4; ++u) {
    const size_t j = j0 + size_t(u) * 256, jc = j < n ? j : n - 1;
    a[u] = px[jc];
    o[u] = pd[jc];
  }
#pragma unroll
  for (int u = 0; u < 4; ++u) {
    const size_t j = j0 + size_t(u) * 256;
    if (j < n) pd[j] = o[u] + c * (a[u] - mean) * sb;
  }
}

// true: the element is long and the batch small enough for the chunked kernels, and the device's scratch holds the
// chunk statistics
static bool moment_chunked_fits(const dyhip_device* dev, size_t n, unsigned bd, unsigned* chunks) {
  const size_t c = cdiv<size_t>(n, kMomChunk), cus = dev->num_cus > 0 ? size_t(dev->num_cus) : 256;
  *chunks = static_cast<unsigned>(c);
  return n > 16384 && bd < 2 * cus && c <= 0x7FFFFFFFull && bd <= 65535u && dev->gemm_ws != nullptr &&
         dev->gemm_ws_bytes >= sizeof(float) * 2 * c * bd && cdiv<size_t>(n, 1024) <= 0x7FFFFFFFull;
}

// ---- the same three with the batch element held in registers: T threads own a batch element (a wavefront up to 512
// floats, four elements to a block; a block of 256 threads up to 4096 floats, of 1024 threads up to 16384), thread t
// holding entries t, t + T, ... (U of them): x is read once, every access of the group is one contiguous run, and a
// short element does not occupy a 256-thread block (80 000 elements of 50 floats: 42 -> a few us for std_elems).
// MODE 0: mean   1: std   2: std backward.  Longer elements take the chunked kernels above when the batch is small and
// the block-per-element kernels otherwise; elements of at most 32 floats take moment_group_kernel below.
// the sum over a group of G adjacent lanes (G a power of two, 4..64), left in every lane of the group
template <int G>
__device__ __forceinline__ float group_sum(float v) {
  v += dpp_move<0xB1, 0xF>(v, 0.f);                // quad_perm [1,0,3,2]
  v += dpp_move<0x4E, 0xF>(v, 0.f);                // quad_perm [2,3,0,1]
  if (G >= 8) v += dpp_move<0x141, 0xF>(v, 0.f);   // row_half_mirror
  if (G >= 16) v += dpp_move<0x140, 0xF>(v, 0.f);  // row_mirror
  if (G >= 32) v += __shfl_xor(v, 16);             // the other DPP row of the half
  if (G >= 64) v += __shfl_xor(v, 32);
  return v;
}

template <int T>
__device__ __forceinline__ float mom_group_sum(float v, float* red) {
  if (T == 64) return wave_sum(v);
  return block_sum<(T >= 64 ? T / 64 : 1)>(v, red);
}

template <int MODE, int T, int U>
__global__ __launch_bounds__(T == 64 ? 256 : T) void moment_resident_kernel(unsigned n, unsigned bd,
                                                                           const float* __restrict__ x,
                                                                           const float* __restrict__ fx,
                                                                           const float* __restrict__ dEdf,
                                                                           float* __restrict__ out) {
  __shared__ float red[16];
  const unsigned b = T == 64 ? blockIdx.x * 4 + (threadIdx.x >> 6) : blockIdx.x;
  if (b >= bd) return;  // T == 64: whole wavefronts leave and that form has no barrier
  const unsigned t = T == 64 ? (threadIdx.x & 63) : threadIdx.x;
  const size_t b0 = size_t(b) * n;
  float v[U], o[U];
#pragma unroll
  for (int u = 0; u < U; ++u) {
    const unsigned i = t + T * u, ic = i < n ? i : n - 1;  // unconditional loads; entries past the end are masked
    v[u] = x[b0 + ic];
    if (MODE == 2) o[u] = out[b0 + ic];
  }
  float s = 0.f;
#pragma unroll
  for (int u = 0; u < U; ++u)
    if (t + T * u < n) s += v[u];
  const float mean = mom_group_sum<T>(s, red) / float(n);
  if (MODE == 0) {
    if (t == 0) out[b] = mean;
  } else if (MODE == 1) {
    float q = 0.f;
#pragma unroll
    for (int u = 0; u < U; ++u) {
      if (t + T * u < n) {
        const float d = v[u] - mean;
        q += d * d;
      }
    }
    const float var = mom_group_sum<T>(q, red) / float(n);
    if (t == 0) out[b] = sqrtf(var);
  } else {
    const float sb = dEdf[b] / (2.f * fx[b]);
    const float c = 2.f / float(n);
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const unsigned i = t + T * u;
      if (i < n) out[b0 + i] = o[u] + c * (v[u] - mean) * sb;
    }
  }
}

// Elements of at most 32 floats: G lanes (4..32) hold one, a block of 256 threads takes RPG * 256 / G of them with all
// loads issued before the first sum (a wavefront per 7-float element used 7 of its 64 lanes: 100 000 of them took
// 7.9 / 12.8 / 15.3 us).
template <int MODE, int G, int RPG>
__global__ __launch_bounds__(256) void moment_group_kernel(unsigned n, unsigned bd, const float* __restrict__ x,
                                                           const float* __restrict__ fx, const float* __restrict__ dEdf,
                                                           float* __restrict__ out) {
  constexpr unsigned PER = 256 / G;
  const unsigned gl = threadIdx.x % G;
  const unsigned e0 = blockIdx.x * (PER * RPG) + threadIdx.x / G;
  const bool in = gl < n;
  float v[RPG], o[RPG];
#pragma unroll
  for (int k = 0; k < RPG; ++k) {
    const unsigned e = e0 + k * PER;
    const size_t at = size_t(e < bd ? e : bd - 1) * n + (in ? gl : n - 1);
    v[k] = x[at];
    if (MODE == 2) o[k] = out[at];
  }
  const float fn = float(n);
#pragma unroll
  for (int k = 0; k < RPG; ++k) {
    const unsigned e = e0 + k * PER;
    const float mean = group_sum<G>(in ? v[k] : 0.f) / fn;
    if (MODE == 0) {
      if (gl == 0 && e < bd) out[e] = mean;
    } else if (MODE == 1) {
      const float d = in ? v[k] - mean : 0.f;
      const float var = group_sum<G>(d * d) / fn;
      if (gl == 0 && e < bd) out[e] = sqrtf(var);
    } else if (e < bd) {
      const float sb = dEdf[e] / (2.f * fx[e]);
      if (in) out[size_t(e) * n + gl] = o[k] + (2.f / fn) * (v[k] - mean) * sb;
    }
  }
}

// true: the register-resident kernel was launched
template <int MODE>
static bool launch_moment_resident(dyhip_device* dev, size_t n, unsigned bd, const float* x, const float* fx,
                                   const float* dEdf, float* out) {
  if (n > 16384) return false;
  const unsigned r = static_cast<unsigned>(n);
#define DYHIP_MOM(T, U, GRID)                                                                                          \
  hipLaunchKernelGGL((moment_resident_kernel<MODE, T, U>), dim3(GRID), dim3(T == 64 ? 256 : T), 0, dev->stream, r, bd, x, \
                     fx, dEdf, out)
  const unsigned g4 = cdiv<unsigned>(bd, 4);
#define DYHIP_MOMG(G)                                                                                              \
  hipLaunchKernelGGL((moment_group_kernel<MODE, G, 4>), dim3(cdiv<unsigned>(bd, 4 * 256 / G)), dim3(256), 0, dev->stream, \
                     r, bd, x, fx, dEdf, out)
  if (r <= 4) DYHIP_MOMG(4);
  else if (r <= 8) DYHIP_MOMG(8);
  else if (r <= 16) DYHIP_MOMG(16);
  else if (r <= 32) DYHIP_MOMG(32);
  else if (r <= 64) DYHIP_MOM(64, 1, g4);
  else if (r <= 128) DYHIP_MOM(64, 2, g4);
  else if (r <= 256) DYHIP_MOM(64, 4, g4);
  else if (r <= 512) DYHIP_MOM(64, 8, g4);
  else if (r <= 1024) DYHIP_MOM(256, 4, bd);
  else if (r <= 2048) DYHIP_MOM(256, 8, bd);
  else if (r <= 4096) DYHIP_MOM(256, 16, bd);
  else if (r <= 8192) DYHIP_MOM(1024, 8, bd);
  else DYHIP_MOM(1024, 16, bd);
#undef DYHIP_MOM
#undef DYHIP_MOMG
  return true;
}

// dx[b, j] += dEdf[b] / n over the flat tensor: four entries a thread, the batch index by one 32-bit division
__global__ __launch_bounds__(256) void mean_bwd_flat_kernel(unsigned n, size_t total, const float* __restrict__ dEdf,
                                                            float* __restrict__ dEdx) {
  const size_t e0 = size_t(blockIdx.x) * 1024 + threadIdx.x;
  float o[4];
#pragma unroll
  for (int k = 0; k < 4; ++k) o[k] = dEdx[e0 + 256 * k < total ? e0 + 256 * k : total - 1];
#pragma unroll
  for (int k = 0; k < 4; ++k) {
    const size_t e = e0 + 256 * k;
    if (e < total) dEdx[e] = o[k] + dEdf[e / n] / float(n);
  }
}

// ============================================================================
// fused LayerNorm
// ============================================================================
//
// Fast path (n % 4 == 0, n <= 2048, 16-byte aligned): one wavefront per batch
// element, the whole row held in registers as VPL float4 per lane (lane l owns
// float4 slots l, l+64, ...), so x (and dy) are read from HBM exactly once.
// mean and the two-pass population variance are wave-butterfly reductions.
//
// Backward keeps per-lane partial sums of dg / db across the rows a wave owns,
// combines the waves of a block through LDS in ascending wave order, writes one
// partial row per block to the workspace, and a second kernel adds the block
// partials in ascending block order into dg / db.
constexpr int kLnWavesFwd = 4;
constexpr int kLnWavesBwd = 8;
constexpr unsigned kLnBwdMaxBlocks = 256;
constexpr float kLnEps = 1e-8f;

template <int VPL, bool NT>
__global__ __launch_bounds__(64 * kLnWavesFwd) void ln_fwd_wave_kernel(unsigned n4, unsigned bd,
                                                                      const float4* __restrict__ x,
                                                                      const float4* __restrict__ g,
                                                                      const float4* __restrict__ b,
                                                                      float4* __restrict__ y) {
  const int lane = threadIdx.x & 63;
  const unsigned row = blockIdx.x * kLnWavesFwd + (threadIdx.x >> 6);
  if (row >= bd) return;
  const float fn = float(n4 * 4);
  const float4* px = x + size_t(row) * n4;
  float4 v[VPL];
#pragma unroll
  for (int u = 0; u < VPL; ++u) {
    const unsigned idx = lane + 64 * u;
    v[u] = idx < n4 ? ldg4<NT>(px + idx) : make_float4(0.f, 0.f, 0.f, 0.f);
  }
  float s = 0.f;
#pragma unroll
  for (int u = 0; u < VPL; ++u) s += (v[u].x + v[u].y) + (v[u].z + v[u].w);
  const float mean = wave_sum(s) / fn;
  float ss = 0.f;
#pragma unroll
  for (int u = 0; u < VPL; ++u) {
    if (lane + 64 * u < n4) {
      const float dx = v[u].x - mean, dy = v[u].y - mean, dz = v[u].z - mean, dw = v[u].w - mean;
      ss += (dx * dx + dy * dy) + (dz * dz + dw * dw);
    }
  }
  const float sigma = sqrtf(wave_sum(ss) / fn);
  // one exact division per row; per element a multiply (within 1.5 ulp of x / (sigma + eps))
  const float sden = 1.0f / (kLnEps + sigma);
  const float neg = -mean;
  float4* py = y + size_t(row) * n4;
#pragma unroll
  for (int u = 0; u < VPL; ++u) {
    const unsigned idx = lane + 64 * u;
    if (idx < n4) {
      const float4 gg = g[idx], bb = b[idx];
      float4 r;
      r.x = gg.x * ((v[u].x + neg) * sden) + bb.x;
      r.y = gg.y * ((v[u].y + neg) * sden) + bb.y;
      r.z = gg.z * ((v[u].z + neg) * sden) + bb.z;
      r.w = gg.w * ((v[u].w + neg) * sden) + bb.w;
      stg4<NT>(py + idx, r);
    }
  }
}

// ---- rows of at most 256 floats: G lanes (4, 8 or 16) hold a row, a wavefront 64 / G rows at a time ---------------------
// With a wavefront per row, rows of 64 floats use 16 of its lanes and one 128-bit load per lane (0.27 of the HBM peak
// forward and backward; 0.08 at 16 floats).  The sums over a row stay inside a 16-lane DPP row: quad permutes, then
// the half-row and row mirrors (group_sum above), after which every lane of the group holds the group's sum.
// RPG: rows a group takes, all fetched before the first is reduced (one 128-bit load a lane is too little in flight:
// 64-float rows 7.6 us for 16 MB with one, against 6.0 us for 128-float rows with two)
template <int G, int VPL, int RPG, bool NT>
__global__ __launch_bounds__(64 * kLnWavesFwd) void ln_fwd_group_kernel(unsigned n4, unsigned bd,
                                                                       const float4* __restrict__ x,
                                                                       const float4* __restrict__ g,
                                                                       const float4* __restrict__ b,
                                                                       float4* __restrict__ y) {
  constexpr unsigned R = 64 / G;
  const unsigned lane = threadIdx.x & 63, gl = lane % G;
  const unsigned row0 = (blockIdx.x * kLnWavesFwd + (threadIdx.x >> 6)) * (R * RPG) + lane / G;
  const float fn = float(n4 * 4);
  float4 v[RPG][VPL];
#pragma unroll
  for (int k = 0; k < RPG; ++k) {
    const unsigned row = row0 + k * R;  // a group past the end works on the last row and stores nothing
    const float4* px = x + size_t(row < bd ? row : bd - 1) * n4;
#pragma unroll
    for (int u = 0; u < VPL; ++u) {
      const unsigned idx = gl + G * u;
      v[k][u] = ldg4<NT>(px + (idx < n4 ? idx : n4 - 1));
    }
  }
#pragma unroll
  for (int k = 0; k < RPG; ++k) {
    const unsigned row = row0 + k * R;
#pragma unroll
    for (int u = 0; u < VPL; ++u)
      if (!(gl + G * u < n4)) v[k][u] = make_float4(0.f, 0.f, 0.f, 0.f);
    float s = 0.f;
#pragma unroll
    for (int u = 0; u < VPL; ++u) s += (v[k][u].x + v[k][u].y) + (v[k][u].z + v[k][u].w);
    const float mean = group_sum<G>(s) / fn;
    float ss = 0.f;
#pragma unroll
    for (int u = 0; u < VPL; ++u) {
      if (gl + G * u < n4) {
        const float dx = v[k][u].x - mean, dy = v[k][u].y - mean, dz = v[k][u].z - mean, dw = v[k][u].w - mean;
        ss += (dx * dx + dy * dy) + (dz * dz + dw * dw);
      }
    }
    const float sigma = sqrtf(group_sum<G>(ss) / fn);
    const float sden = 1.0f / (kLnEps + sigma);
    const float neg = -mean;
    float4* py = y + size_t(row) * n4;
#pragma unroll
    for (int u = 0; u < VPL; ++u) {
      const unsigned idx = gl + G * u;
      if (row < bd && idx < n4) {
        const float4 gg = g[idx], bb = b[idx];  // here, not ahead of the reductions: 6.0 against 7.3 us at 128-256 floats
        float4 r;
        r.x = gg.x * ((v[k][u].x + neg) * sden) + bb.x;
        r.y = gg.y * ((v[k][u].y + neg) * sden) + bb.y;
        r.z = gg.z * ((v[k][u].z + neg) * sden) + bb.z;
        r.w = gg.w * ((v[k][u].w + neg) * sden) + bb.w;
        stg4<NT>(py + idx, r);
      }
    }
  }
}

// Rows of 2052..16384 floats: a team of WPT waves holds one row in registers (four float4 per thread) and
// reduces through LDS, one barrier per reduction (each reduction has its own slots).
constexpr int kLnTeamVpt = 4;

template <int WPT>
__device__ __forceinline__ float team_sum(float v, float* slot, int w, int team) {
  v = wave_sum(v);
  if ((threadIdx.x & 63) == 0) slot[w] = v;
  __syncthreads();
  float t = slot[team * WPT];
#pragma unroll
  for (int k = 1; k < WPT; ++k) t += slot[team * WPT + k];
  return t;
}

template <int WPT, bool NT>
__global__ __launch_bounds__(64 * WPT) void ln_fwd_team_kernel(unsigned n4, const float4* __restrict__ x,
                                                               const float4* __restrict__ g,
                                                               const float4* __restrict__ b, float4* __restrict__ y) {
  __shared__ float red[2][16];
  constexpr int TEAM = 64 * WPT;
  const int w = threadIdx.x >> 6;
  const float fn = float(n4 * 4);
  const float4* px = x + size_t(blockIdx.x) * n4;
  float4 v[kLnTeamVpt];
#pragma unroll
  for (int u = 0; u < kLnTeamVpt; ++u) {
    const unsigned idx = threadIdx.x + TEAM * u;
    v[u] = idx < n4 ? ldg4<NT>(px + idx) : make_float4(0.f, 0.f, 0.f, 0.f);
  }
  float s = 0.f;
#pragma unroll
  for (int u = 0; u < kLnTeamVpt; ++u) s += (v[u].x + v[u].y) + (v[u].z + v[u].w);
  const float mean = team_sum<WPT>(s, red[0], w, 0) / fn;
  float ss = 0.f;
#pragma unroll
  for (int u = 0; u < kLnTeamVpt; ++u) {
    if (threadIdx.x + TEAM * u < n4) {
      const float dx = v[u].x - mean, dy = v[u].y - mean, dz = v[u].z - mean, dw = v[u].w - mean;
      ss += (dx * dx + dy * dy) + (dz * dz + dw * dw);
    }
  }
  const float sigma = sqrtf(team_sum<WPT>(ss, red[1], w, 0) / fn);
  const float sden = 1.0f / (kLnEps + sigma);
  const float neg = -mean;
  float4* py = y + size_t(blockIdx.x) * n4;
#pragma unroll
  for (int u = 0; u < kLnTeamVpt; ++u) {
    const unsigned idx = threadIdx.x + TEAM * u;
    if (idx < n4) {
      const float4 gg = g[idx], bb = b[idx];
      float4 r;
      r.x = gg.x * ((v[u].x + neg) * sden) + bb.x;
      r.y = gg.y * ((v[u].y + neg) * sden) + bb.y;
      r.z = gg.z * ((v[u].z + neg) * sden) + bb.z;
      r.w = gg.w * ((v[u].w + neg) * sden) + bb.w;
      stg4<NT>(py + idx, r);
    }
  }
}

// ---- rows of at most 2048 floats that cannot take 128-bit accesses (n % 4 != 0, or a pointer off a 16-byte
// boundary: every second row then starts off one too): the same one-wavefront-per-row scheme with VS floats per lane,
// lane l owning elements l, l + 64, ...  A wavefront's access is still one contiguous 256-byte run.  The arithmetic
// and its order per element are those of the 128-bit kernels; the block-per-row fallback these rows used to take ran
// at 0.2 of the HBM peak (n = 650: forward 19 us, backward 44 us for 16 MB).
template <int VS, bool NT>
__global__ __launch_bounds__(64 * kLnWavesFwd) void ln_fwd_lane_kernel(unsigned n, unsigned bd, const float* __restrict__ x,
                                                                      const float* __restrict__ g,
                                                                      const float* __restrict__ b, float* __restrict__ y) {
  const int lane = threadIdx.x & 63;
  const unsigned row = blockIdx.x * kLnWavesFwd + (threadIdx.x >> 6);
  if (row >= bd) return;
  const float fn = float(n);
  const float* px = x + size_t(row) * n;
  float v[VS];
#pragma unroll
  for (int u = 0; u < VS; ++u) {
    const unsigned idx = lane + 64 * u;
    v[u] = ldg1<NT>(px + (idx < n ? idx : n - 1));  // unconditional; a lane past the end drops what it fetched
  }
  float s = 0.f;
#pragma unroll
  for (int u = 0; u < VS; ++u)
    if (lane + 64 * u < n) s += v[u];
  const float mean = wave_sum(s) / fn;
  float ss = 0.f;
#pragma unroll
  for (int u = 0; u < VS; ++u) {
    if (lane + 64 * u < n) {
      const float d = v[u] - mean;
      ss += d * d;
    }
  }
  const float sigma = sqrtf(wave_sum(ss) / fn);
  const float sden = 1.0f / (kLnEps + sigma);
  const float neg = -mean;
  float* py = y + size_t(row) * n;
#pragma unroll
  for (int u = 0; u < VS; ++u) {
    const unsigned idx = lane + 64 * u;
    if (idx < n) stg1<NT>(py + idx, g[idx] * ((v[u] + neg) * sden) + b[idx]);
  }
}

template <int VS>
struct LnLaneRow {
  float v[VS], d[VS], o[VS];
};

// Up to 16 floats per lane (rows of at most 1024 floats): with 32 the row, the gain, both partial sums and the old dx
// do not fit the registers, and the spilling kernel (54-63 us for 16 MB) lost to the block-per-row fallback (41 us),
// which rows of 1025..2048 floats that cannot take 128-bit accesses therefore keep.
template <int VS, bool NT, bool PREFETCH>
__global__ __launch_bounds__(64 * kLnWavesBwd) void ln_bwd_lane_kernel(unsigned n, unsigned bd, const float* __restrict__ x,
                                                                      const float* __restrict__ g,
                                                                      const float* __restrict__ dEdf, float* __restrict__ dx,
                                                                      float* __restrict__ part_dg,
                                                                      float* __restrict__ part_db) {
  extern __shared__ float lds[];  // [dg | db][wave][n] when partial rows are requested
  constexpr int WAVES = kLnWavesBwd;
  const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
  const float fn = float(n);
  const bool want_g = part_dg != nullptr, want_b = part_db != nullptr;
  float gg[VS], pdg[VS], pdb[VS];
#pragma unroll
  for (int u = 0; u < VS; ++u) {
    const unsigned idx = lane + 64 * u;
    gg[u] = idx < n ? g[idx] : 0.f;
    pdg[u] = 0.f;
    pdb[u] = 0.f;
  }
  const unsigned wave_count = gridDim.x * WAVES;
  const float* dxr = dx != nullptr ? dx : x;  // without a dx the old values are fetched from x and not used
  LnLaneRow<VS> cur, nxt;
  // unconditional loads on addresses clamped into the row; lanes past the end hold zeros
  auto load = [&](LnLaneRow<VS>& r, unsigned row) __attribute__((always_inline)) {
    const float *px = x + size_t(row) * n, *pdy = dEdf + size_t(row) * n, *po = dxr + size_t(row) * n;
#pragma unroll
    for (int u = 0; u < VS; ++u) {
      const unsigned idx = lane + 64 * u, ic = idx < n ? idx : n - 1;
      r.v[u] = ldg1<NT>(px + ic);
      r.d[u] = ldg1<NT>(pdy + ic);
      r.o[u] = ldg1<NT>(po + ic);
    }
#pragma unroll
    for (int u = 0; u < VS; ++u) {
      if (!(lane + 64 * u < n)) {
        r.v[u] = 0.f;
        r.d[u] = 0.f;
      }
    }
  };
  // the block's partial rows: waves added in ascending order through LDS, then stored (every wave runs it once)
  auto stage = [&]() __attribute__((always_inline)) {
    __syncthreads();
#pragma unroll
    for (int u = 0; u < VS; ++u) {
      const unsigned idx = lane + 64 * u;
      if (idx < n) {
        if (want_g) lds[size_t(w) * n + idx] = pdg[u];
        if (want_b) lds[size_t(WAVES + w) * n + idx] = pdb[u];
      }
    }
    __syncthreads();
    for (unsigned j = threadIdx.x; j < 2 * n; j += 64 * WAVES) {
      const unsigned which = j >= n ? 1u : 0u;
      float* part = which == 0 ? part_dg : part_db;
      if (part == nullptr) continue;
      const unsigned c = j - which * n;
      const float* src = lds + size_t(which) * WAVES * n + c;
      float t = src[0];
#pragma unroll
      for (int k = 1; k < WAVES; ++k) t += src[size_t(k) * n];
      part[size_t(blockIdx.x) * n + c] = t;
    }
  };
  auto process = [&](const LnLaneRow<VS>& cur, unsigned row, bool last) __attribute__((always_inline)) {
    float s = 0.f;
#pragma unroll
    for (int u = 0; u < VS; ++u) s += cur.v[u];
    const float mean = wave_sum(s) / fn;
    float ss = 0.f;
#pragma unroll
    for (int u = 0; u < VS; ++u) {
      if (lane + 64 * u < n) {
        const float a = cur.v[u] - mean;
        ss += a * a;
      }
    }
    const float sigma = sqrtf(wave_sum(ss) / fn);
    const float rs = 1.0f / (kLnEps + sigma);
    const float neg = -mean;
    float sxq = 0.f, sq = 0.f;
#pragma unroll
    for (int u = 0; u < VS; ++u) {
      if (lane + 64 * u < n) {
        const float xc = cur.v[u] + neg;
        const float dq = cur.d[u] * gg[u];
        sxq = fmaf(dq, xc, sxq);
        sq += dq;
        if (want_g) pdg[u] = fmaf(cur.d[u], xc * rs, pdg[u]);
        if (want_b) pdb[u] += cur.d[u];
      }
    }
    if (last && (want_g || want_b)) stage();  // before this row's dx: the LDS pass and the stores run under it
    if (dx != nullptr) {
      const float ds = -(wave_sum(sxq) * rs) * rs;
      const float dmu = -(wave_sum(sq) * rs);
      const float sb = ds / (2.f * sigma);
      const float c = 2.f / fn;
      const float dmu_n = dmu / fn;
      float* pdx = dx + size_t(row) * n;
#pragma unroll
      for (int u = 0; u < VS; ++u) {
        const unsigned idx = lane + 64 * u;
        if (idx < n) {
          float acc = cur.o[u];
          acc += c * (cur.v[u] - mean) * sb;
          acc += (cur.d[u] * gg[u]) * rs;
          acc += dmu_n;
          stg1<NT>(pdx + idx, acc);
        }
      }
    }
  };
  unsigned r = __builtin_amdgcn_readfirstlane(blockIdx.x * WAVES + w);
  if (r < bd) {
    load(cur, r);
    for (unsigned next = r + wave_count; next < bd; next += wave_count) {
      if (PREFETCH) {
        load(nxt, next);
        process(cur, r, false);
        cur = nxt;
      } else {
        process(cur, r, false);
        load(cur, next);
      }
      r = next;
    }
    process(cur, r, true);
  } else if (want_g || want_b) {
    stage();  // a wave without rows still takes part in the block's barriers
  }
}

// generic fallback (rows wider than the register-resident kernels take, or wide rows that cannot take 128-bit
// accesses): one block per batch element, three passes over the row (the second and third find it in the caches), four
// independent loads in flight per thread and pass.  256 threads for rows of up to 4096 floats (more rows per CU at
// once), 1024 beyond (65536 floats x 64 rows: 190 -> 35 us forward against 256 threads and one load in flight).
template <int kLnBlockThreads>
__global__ __launch_bounds__(kLnBlockThreads) void ln_fwd_block_kernel(size_t n, const float* __restrict__ x,
                                                                       const float* __restrict__ g,
                                                                       const float* __restrict__ b,
                                                                       float* __restrict__ y) {
  __shared__ float red[kLnBlockThreads / 64];
  const float* px = x + size_t(blockIdx.x) * n;
  float s = 0.f;
  for (size_t j0 = threadIdx.x; j0 < n; j0 += 4 * kLnBlockThreads) {
    float a[4];
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const size_t j = j0 + size_t(u) * kLnBlockThreads;
      a[u] = px[j < n ? j : n - 1];
    }
#pragma unroll
    for (int u = 0; u < 4; ++u)
      if (j0 + size_t(u) * kLnBlockThreads < n) s += a[u];
  }
  const float mean = block_sum<kLnBlockThreads / 64>(s, red) / float(n);
  float v = 0.f;
  for (size_t j0 = threadIdx.x; j0 < n; j0 += 4 * kLnBlockThreads) {
    float a[4];
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const size_t j = j0 + size_t(u) * kLnBlockThreads;
      a[u] = px[j < n ? j : n - 1];
    }
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      if (j0 + size_t(u) * kLnBlockThreads < n) {
        const float d = a[u] - mean;
        v += d * d;
      }
    }
  }
  const float sigma = sqrtf(block_sum<kLnBlockThreads / 64>(v, red) / float(n));
  const float sden = kLnEps + sigma, neg = -mean;
  float* py = y + size_t(blockIdx.x) * n;
  for (size_t j0 = threadIdx.x; j0 < n; j0 += 4 * kLnBlockThreads) {
    float a[4], gg[4], bb[4];
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const size_t j = j0 + size_t(u) * kLnBlockThreads, jc = j < n ? j : n - 1;
      a[u] = px[jc];
      gg[u] = g[jc];
      bb[u] = b[jc];
    }
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const size_t j = j0 + size_t(u) * kLnBlockThreads;
      if (j < n) py[j] = gg[u] * ((a[u] + neg) / sden) + bb[u];
    }
  }
}

// accumulate helper for float4 with a per-component functor
#define DYHIP_F4_EACH(stmt) \
  { stmt(x) stmt(y) stmt(z) stmt(w) }

// Registers of one row: x, dy and (when dx is requested) the old dx.
template <int VPL>
struct LnRow {
  float4 v[VPL], d[VPL], o[VPL];
};

// FULL: the row fills every lane's groups and pdx is set, so the loads are unconditional.  Loads inside branches
// cannot be counted by the compiler, which then waits for everything in flight (the row fetched ahead included)
// before the first use of any of them.
template <int VPL, bool NT, bool FULL = false>
__device__ __forceinline__ void ln_row_load(LnRow<VPL>& r, unsigned n4, int lane, const float4* __restrict__ px,
                                            const float4* __restrict__ pdy, const float4* __restrict__ pdx) {
  if (FULL) {
#pragma unroll
    for (int u = 0; u < VPL; ++u) {
      r.v[u] = ldg4<NT>(px + lane + 64 * u);
      r.d[u] = ldg4<NT>(pdy + lane + 64 * u);
      r.o[u] = ldg4<NT>(pdx + lane + 64 * u);
    }
    return;
  }
#pragma unroll
  for (int u = 0; u < VPL; ++u) {
    const unsigned idx = lane + 64 * u;
    const bool in = idx < n4;
    r.v[u] = in ? ldg4<NT>(px + idx) : make_float4(0.f, 0.f, 0.f, 0.f);
    r.d[u] = in ? ldg4<NT>(pdy + idx) : make_float4(0.f, 0.f, 0.f, 0.f);
    if (pdx != nullptr) r.o[u] = in ? ldg4<NT>(pdx + idx) : make_float4(0.f, 0.f, 0.f, 0.f);
  }
}

// FULL: n4 == 64 * VPL and dx is wanted (the usual case): no per-lane bounds, and the row fetched ahead is always a
// valid one (the last iteration fetches its own row again), so the kernel's main loop has no branch around a load.
template <int VPL, bool NT, int WAVES, bool PREFETCH, bool FULL = false>
__global__ __launch_bounds__(64 * WAVES) void ln_bwd_wave_kernel(unsigned n4, unsigned bd,
                                                                      const float4* __restrict__ x,
                                                                      const float4* __restrict__ g,
                                                                      const float4* __restrict__ dEdf,
                                                                      float4* __restrict__ dx,
                                                                      float* __restrict__ part_dg,
                                                                      float* __restrict__ part_db) {
  extern __shared__ float lds[];  // [WAVES][n] when partials are requested
  const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
  const float fn = float(n4 * 4);
  const bool want_g = part_dg != nullptr, want_b = part_db != nullptr;
  float4 gg[VPL], pdg[VPL], pdb[VPL];
#pragma unroll
  for (int u = 0; u < VPL; ++u) {
    const unsigned idx = lane + 64 * u;
    gg[u] = idx < n4 ? g[idx] : make_float4(0.f, 0.f, 0.f, 0.f);
    pdg[u] = make_float4(0.f, 0.f, 0.f, 0.f);
    pdb[u] = make_float4(0.f, 0.f, 0.f, 0.f);
  }
  const unsigned wave_count = gridDim.x * WAVES;
  unsigned row = blockIdx.x * WAVES + w;
  LnRow<VPL> cur, nxt;
  // This block's dg / db partial rows: the waves are combined in ascending wave order, both outputs in one pass
  // through LDS (layout [which][wave][n]), and leave with 128-bit stores.  Two barriers; every wave of the block
  // runs it exactly once.
  auto stage = [&]() __attribute__((always_inline)) {
    const unsigned n = n4 * 4;
    __syncthreads();
#pragma unroll
    for (int u = 0; u < VPL; ++u) {
      const unsigned idx = lane + 64 * u;
      if (idx < n4) {
        if (want_g) reinterpret_cast<float4*>(lds + size_t(w) * n)[idx] = pdg[u];
        if (want_b) reinterpret_cast<float4*>(lds + size_t(WAVES + w) * n)[idx] = pdb[u];
      }
    }
    __syncthreads();
    for (unsigned j4 = threadIdx.x; j4 < 2 * n4; j4 += 64 * WAVES) {
      const unsigned which = j4 >= n4 ? 1u : 0u;
      float* part = which == 0 ? part_dg : part_db;
      if (part == nullptr) continue;
      const unsigned c4 = j4 - which * n4;
      const float4* src = reinterpret_cast<const float4*>(lds + size_t(which) * WAVES * n) + c4;
      float4 t = src[0];
#pragma unroll
      for (int k = 1; k < WAVES; ++k) {
        const float4 a = src[size_t(k) * n4];
        t.x += a.x; t.y += a.y; t.z += a.z; t.w += a.w;
      }
      reinterpret_cast<float4*>(part + size_t(blockIdx.x) * n)[c4] = t;
    }
  };
  // one row: the row sums, dx, and this wave's dg / db partial sums.  `last`: this is the wave's last row, whose
  // contribution completes the partial sums: the block's partial rows are combined and stored *before* the row's dx is
  // formed, so that the LDS pass and the partial rows' stores run under the dx arithmetic and stores instead of after
  // them, at the very end of the kernel, where nothing hides them (16.8 -> 15.x us for 4096 rows of 1024).
  auto process = [&](const LnRow<VPL>& cur, unsigned row, bool last) __attribute__((always_inline)) {
  float s = 0.f;
#pragma unroll
  for (int u = 0; u < VPL; ++u) s += (cur.v[u].x + cur.v[u].y) + (cur.v[u].z + cur.v[u].w);
  const float mean = wave_sum(s) / fn;
  float ss = 0.f;
#pragma unroll
  for (int u = 0; u < VPL; ++u) {
    if (FULL || lane + 64 * u < n4) {
      const float ax = cur.v[u].x - mean, ay = cur.v[u].y - mean, az = cur.v[u].z - mean, aw = cur.v[u].w - mean;
      ss += (ax * ax + ay * ay) + (az * az + aw * aw);
    }
  }
  const float sigma = sqrtf(wave_sum(ss) / fn);
  const float rs = 1.0f / (kLnEps + sigma);  // one exact division per row
  const float neg = -mean;
  // row sums: sum dq*xc and sum dq, with dq = dy*g
  float sxq = 0.f, sq = 0.f;
#pragma unroll
  for (int u = 0; u < VPL; ++u) {
    if (FULL || lane + 64 * u < n4) {
#define DYHIP_LN_ROW(c)                                  \
  {                                                      \
  const float xc = cur.v[u].c + neg;                   \
  const float dq = cur.d[u].c * gg[u].c;               \
  sxq = fmaf(dq, xc, sxq);                             \
  sq += dq;                                            \
  if (want_g) pdg[u].c = fmaf(cur.d[u].c, xc * rs, pdg[u].c); \
  if (want_b) pdb[u].c += cur.d[u].c;                  \
  }
      DYHIP_F4_EACH(DYHIP_LN_ROW)
#undef DYHIP_LN_ROW
    }
  }
  if (last && (want_g || want_b)) stage();
  if (FULL || dx != nullptr) {
    const float ds = -(wave_sum(sxq) * rs) * rs;   // CwiseQuotient: -sum dq/s^2 * xc
    const float dmu = -(wave_sum(sq) * rs);        // Negate(CwiseSum): -sum dq/s
    const float sb = ds / (2.f * sigma);           // StdDimension: d / (2*sigma)
    const float c = 2.f / fn;
    const float dmu_n = dmu / fn;
    float4* pdx = dx + size_t(row) * n4;
#pragma unroll
    for (int u = 0; u < VPL; ++u) {
      const unsigned idx = lane + 64 * u;
      if (FULL || idx < n4) {
        float4 o = cur.o[u];
#define DYHIP_LN_DX(c_)                                            \
  {                                                                \
  float acc = o.c_;                                              \
  acc += c * (cur.v[u].c_ - mean) * sb;                          \
  acc += (cur.d[u].c_ * gg[u].c_) * rs;                          \
  acc += dmu_n;                                                  \
  o.c_ = acc;                                                    \
  }
        DYHIP_F4_EACH(DYHIP_LN_DX)
#undef DYHIP_LN_DX
        stg4<NT>(pdx + idx, o);
      }
    }
  }
  };
  if (FULL) {
    // Straight-line loads only: the row after this one is fetched before this one is reduced, and the last row is
    // processed after the loop, so that no load sits inside a branch.  The row index is the same in every lane.
    unsigned r = __builtin_amdgcn_readfirstlane(row);
    if (r < bd) {
      ln_row_load<VPL, NT, true>(cur, n4, lane, x + size_t(r) * n4, dEdf + size_t(r) * n4, dx + size_t(r) * n4);
      for (unsigned next = r + wave_count; next < bd; next += wave_count) {
        ln_row_load<VPL, NT, true>(nxt, n4, lane, x + size_t(next) * n4, dEdf + size_t(next) * n4, dx + size_t(next) * n4);
        process(cur, r, false);
        cur = nxt;
        r = next;
      }
      process(cur, r, true);
    } else if (want_g || want_b) {
      stage();  // a wave without rows still takes part in the block's barriers
    }
    return;
  } else {
    if (PREFETCH && row < bd)
      ln_row_load<VPL, NT>(cur, n4, lane, x + size_t(row) * n4, dEdf + size_t(row) * n4,
                           dx ? dx + size_t(row) * n4 : nullptr);
    while (row < bd) {
      // the next row's loads are in flight while this row is reduced and written
      const unsigned next = row + wave_count;
      if (!PREFETCH)
        ln_row_load<VPL, NT>(cur, n4, lane, x + size_t(row) * n4, dEdf + size_t(row) * n4,
                             dx ? dx + size_t(row) * n4 : nullptr);
      if (PREFETCH && next < bd)
        ln_row_load<VPL, NT>(nxt, n4, lane, x + size_t(next) * n4, dEdf + size_t(next) * n4,
                             dx ? dx + size_t(next) * n4 : nullptr);
      process(cur, row, false);
      if (PREFETCH && next < bd) cur = nxt;
      row = next;
    }
  }
  if (want_g || want_b) stage();
}

// Backward for rows of at most 256 floats, G lanes a row (see ln_fwd_group_kernel).  A wavefront walks 64 / G rows at a
// time and fetches the next set before it reduces the current one; a group past the last row works on the last row
// again and neither stores nor accumulates.  Its dg / db partial sums are first added across the groups that share a
// 16-lane DPP row (row rotations), then across the block's 4 x WAVES DPP rows through LDS in ascending order.
template <int VPL>
struct LnGroupRow {
  float4 v[VPL], d[VPL], o[VPL];
};

template <int G, int VPL, bool NT>
__global__ __launch_bounds__(64 * kLnWavesBwd) void ln_bwd_group_kernel(unsigned n4, unsigned bd,
                                                                       const float4* __restrict__ x,
                                                                       const float4* __restrict__ g,
                                                                       const float4* __restrict__ dEdf,
                                                                       float4* __restrict__ dx,
                                                                       float* __restrict__ part_dg,
                                                                       float* __restrict__ part_db) {
  extern __shared__ float lds[];  // [dg | db][wave * 4 + DPP row][n]
  constexpr int WAVES = kLnWavesBwd;
  constexpr unsigned R = 64 / G;
  const unsigned lane = threadIdx.x & 63, w = threadIdx.x >> 6, gl = lane % G, q = lane / G;
  const float fn = float(n4 * 4);
  const bool want_g = part_dg != nullptr, want_b = part_db != nullptr;
  float4 gg[VPL], pdg[VPL], pdb[VPL];
#pragma unroll
  for (int u = 0; u < VPL; ++u) {
    const unsigned idx = gl + G * u;
    gg[u] = idx < n4 ? g[idx] : make_float4(0.f, 0.f, 0.f, 0.f);
    pdg[u] = make_float4(0.f, 0.f, 0.f, 0.f);
    pdb[u] = make_float4(0.f, 0.f, 0.f, 0.f);
  }
  const unsigned stride = gridDim.x * WAVES * R;
  const float4* dxr = dx != nullptr ? dx : x;  // without a dx the old values are fetched from x and not used
  LnGroupRow<VPL> cur, nxt;
  auto load = [&](LnGroupRow<VPL>& r, unsigned row) __attribute__((always_inline)) {
    const size_t at = size_t(row < bd ? row : bd - 1) * n4;
#pragma unroll
    for (int u = 0; u < VPL; ++u) {
      const unsigned idx = gl + G * u, ic = idx < n4 ? idx : n4 - 1;
      r.v[u] = ldg4<NT>(x + at + ic);
      r.d[u] = ldg4<NT>(dEdf + at + ic);
      r.o[u] = ldg4<NT>(dxr + at + ic);
    }
#pragma unroll
    for (int u = 0; u < VPL; ++u) {
      if (!(gl + G * u < n4)) {
        r.v[u] = make_float4(0.f, 0.f, 0.f, 0.f);
        r.d[u] = make_float4(0.f, 0.f, 0.f, 0.f);
      }
    }
  };
  auto process = [&](const LnGroupRow<VPL>& cur, unsigned row) __attribute__((always_inline)) {
    const bool valid = row < bd;
    float s = 0.f;
#pragma unroll
    for (int u = 0; u < VPL; ++u) s += (cur.v[u].x + cur.v[u].y) + (cur.v[u].z + cur.v[u].w);
    const float mean = group_sum<G>(s) / fn;
    float ss = 0.f;
#pragma unroll
    for (int u = 0; u < VPL; ++u) {
      if (gl + G * u < n4) {
        const float ax = cur.v[u].x - mean, ay = cur.v[u].y - mean, az = cur.v[u].z - mean, aw = cur.v[u].w - mean;
        ss += (ax * ax + ay * ay) + (az * az + aw * aw);
      }
    }
    const float sigma = sqrtf(group_sum<G>(ss) / fn);
    const float rs = 1.0f / (kLnEps + sigma);
    const float neg = -mean;
    float sxq = 0.f, sq = 0.f;
#pragma unroll
    for (int u = 0; u < VPL; ++u) {
      if (gl + G * u < n4) {
#define DYHIP_LN_ROW(c)                                                 \
  {                                                                     \
    const float xc = cur.v[u].c + neg;                                  \
    const float dq = cur.d[u].c * gg[u].c;                              \
    sxq = fmaf(dq, xc, sxq);                                            \
    sq += dq;                                                           \
    if (want_g && valid) pdg[u].c = fmaf(cur.d[u].c, xc * rs, pdg[u].c); \
    if (want_b && valid) pdb[u].c += cur.d[u].c;                        \
  }
        DYHIP_F4_EACH(DYHIP_LN_ROW)
#undef DYHIP_LN_ROW
      }
    }
    if (dx != nullptr) {
      const float ds = -(group_sum<G>(sxq) * rs) * rs;
      const float dmu = -(group_sum<G>(sq) * rs);
      const float sb = ds / (2.f * sigma);
      const float c = 2.f / fn;
      const float dmu_n = dmu / fn;
      float4* pdx = dx + size_t(row) * n4;
#pragma unroll
      for (int u = 0; u < VPL; ++u) {
        const unsigned idx = gl + G * u;
        if (valid && idx < n4) {
          float4 o = cur.o[u];
#define DYHIP_LN_DX(c_)                     \
  {                                         \
    float acc = o.c_;                       \
    acc += c * (cur.v[u].c_ - mean) * sb;   \
    acc += (cur.d[u].c_ * gg[u].c_) * rs;   \
    acc += dmu_n;                           \
    o.c_ = acc;                             \
  }
          DYHIP_F4_EACH(DYHIP_LN_DX)
#undef DYHIP_LN_DX
          stg4<NT>(pdx + idx, o);
        }
      }
    }
  };
  unsigned base = (blockIdx.x * WAVES + w) * R;  // the wavefront's first row: the same in every lane
  if (base < bd) {
    load(cur, base + q);
    for (unsigned next = base + stride; next < bd; next += stride) {
      load(nxt, next + q);
      process(cur, base + q);
      cur = nxt;
      base = next;
    }
    process(cur, base + q);
  }
  if (!want_g && !want_b) return;
  const unsigned n = n4 * 4;
#pragma unroll
  for (int u = 0; u < VPL; ++u) {
#define DYHIP_LN_ACROSS(c)                                              \
  {                                                                     \
    if (G <= 8) {                                                       \
      pdg[u].c += dpp_move<0x128, 0xF>(pdg[u].c, 0.f); /* row_ror:8 */  \
      pdb[u].c += dpp_move<0x128, 0xF>(pdb[u].c, 0.f);                  \
    }                                                                   \
    if (G <= 4) {                                                       \
      pdg[u].c += dpp_move<0x124, 0xF>(pdg[u].c, 0.f); /* row_ror:4 */  \
      pdb[u].c += dpp_move<0x124, 0xF>(pdb[u].c, 0.f);                  \
    }                                                                   \
  }
    DYHIP_F4_EACH(DYHIP_LN_ACROSS)
#undef DYHIP_LN_ACROSS
  }
  const unsigned slot = w * 4 + lane / 16;
#pragma unroll
  for (int u = 0; u < VPL; ++u) {
    const unsigned idx = gl + G * u;
    if (lane % 16 < G && idx < n4) {
      if (want_g) reinterpret_cast<float4*>(lds + size_t(slot) * n)[idx] = pdg[u];
      if (want_b) reinterpret_cast<float4*>(lds + size_t(4 * WAVES + slot) * n)[idx] = pdb[u];
    }
  }
  __syncthreads();
  for (unsigned j4 = threadIdx.x; j4 < 2 * n4; j4 += 64 * WAVES) {
    const unsigned which = j4 >= n4 ? 1u : 0u;
    float* part = which == 0 ? part_dg : part_db;
    if (part == nullptr) continue;
    const unsigned c4 = j4 - which * n4;
    const float4* src = reinterpret_cast<const float4*>(lds + size_t(which) * 4 * WAVES * n) + c4;
    float4 t = src[0];
#pragma unroll 8
    for (int k = 1; k < 4 * WAVES; ++k) {
      const float4 a = src[size_t(k) * n4];
      t.x += a.x; t.y += a.y; t.z += a.z; t.w += a.w;
    }
    reinterpret_cast<float4*>(part + size_t(blockIdx.x) * n)[c4] = t;
  }
}

// ---- the same for short rows that cannot take 128-bit accesses (n % 4 != 0 or a pointer off a 16-byte boundary):
// lane l of a group owns elements l, l + G, ...; a group's access is one contiguous run ------------------------------
template <int G, int VS, int RPG, bool NT>
__global__ __launch_bounds__(64 * kLnWavesFwd) void ln_fwd_group1_kernel(unsigned n, unsigned bd, const float* __restrict__ x,
                                                                        const float* __restrict__ g,
                                                                        const float* __restrict__ b, float* __restrict__ y) {
  constexpr unsigned R = 64 / G;
  const unsigned lane = threadIdx.x & 63, gl = lane % G;
  const unsigned row0 = (blockIdx.x * kLnWavesFwd + (threadIdx.x >> 6)) * (R * RPG) + lane / G;
  const float fn = float(n);
  float v[RPG][VS];
#pragma unroll
  for (int k = 0; k < RPG; ++k) {
    const unsigned row = row0 + k * R;
    const float* px = x + size_t(row < bd ? row : bd - 1) * n;
#pragma unroll
    for (int u = 0; u < VS; ++u) {
      const unsigned idx = gl + G * u;
      v[k][u] = ldg1<NT>(px + (idx < n ? idx : n - 1));
    }
  }
#pragma unroll
  for (int k = 0; k < RPG; ++k) {
    const unsigned row = row0 + k * R;
    float s = 0.f;
#pragma unroll
    for (int u = 0; u < VS; ++u)
      if (gl + G * u < n) s += v[k][u];
    const float mean = group_sum<G>(s) / fn;
    float ss = 0.f;
#pragma unroll
    for (int u = 0; u < VS; ++u) {
      if (gl + G * u < n) {
        const float d = v[k][u] - mean;
        ss += d * d;
      }
    }
    const float sigma = sqrtf(group_sum<G>(ss) / fn);
    const float sden = 1.0f / (kLnEps + sigma);
    const float neg = -mean;
    float* py = y + size_t(row) * n;
#pragma unroll
    for (int u = 0; u < VS; ++u) {
      const unsigned idx = gl + G * u;
      if (row < bd && idx < n) stg1<NT>(py + idx, g[idx] * ((v[k][u] + neg) * sden) + b[idx]);
    }
  }
}

template <int VS>
struct LnGroupRow1 {
  float v[VS], d[VS], o[VS];
};

template <int G, int VS, bool NT>
__global__ __launch_bounds__(64 * kLnWavesBwd) void ln_bwd_group1_kernel(unsigned n, unsigned bd, const float* __restrict__ x,
                                                                        const float* __restrict__ g,
                                                                        const float* __restrict__ dEdf, float* __restrict__ dx,
                                                                        float* __restrict__ part_dg,
                                                                        float* __restrict__ part_db) {
  extern __shared__ float lds[];  // [dg | db][wave * RL + group (G >= 16) or DPP row][n]
  constexpr int WAVES = kLnWavesBwd;
  constexpr unsigned R = 64 / G, RL = G >= 16 ? R : 4;  // partial rows a wavefront leaves in LDS
  const unsigned lane = threadIdx.x & 63, w = threadIdx.x >> 6, gl = lane % G, q = lane / G;
  const float fn = float(n);
  const bool want_g = part_dg != nullptr, want_b = part_db != nullptr;
  float gg[VS], pdg[VS], pdb[VS];
#pragma unroll
  for (int u = 0; u < VS; ++u) {
    const unsigned idx = gl + G * u;
    gg[u] = idx < n ? g[idx] : 0.f;
    pdg[u] = 0.f;
    pdb[u] = 0.f;
  }
  const unsigned stride = gridDim.x * WAVES * R;
  const float* dxr = dx != nullptr ? dx : x;
  LnGroupRow1<VS> cur, nxt;
  auto load = [&](LnGroupRow1<VS>& r, unsigned row) __attribute__((always_inline)) {
    const size_t at = size_t(row < bd ? row : bd - 1) * n;
#pragma unroll
    for (int u = 0; u < VS; ++u) {
      const unsigned idx = gl + G * u, ic = idx < n ? idx : n - 1;
      r.v[u] = ldg1<NT>(x + at + ic);
      r.d[u] = ldg1<NT>(dEdf + at + ic);
      r.o[u] = ldg1<NT>(dxr + at + ic);
    }
#pragma unroll
    for (int u = 0; u < VS; ++u) {
      if (!(gl + G * u < n)) {
        r.v[u] = 0.f;
        r.d[u] = 0.f;
      }
    }
  };
  auto process = [&](const LnGroupRow1<VS>& cur, unsigned row) __attribute__((always_inline)) {
    const bool valid = row < bd;
    float s = 0.f;
#pragma unroll
    for (int u = 0; u < VS; ++u) s += cur.v[u];
    const float mean = group_sum<G>(s) / fn;
    float ss = 0.f;
#pragma unroll
    for (int u = 0; u < VS; ++u) {
      if (gl + G * u < n) {
        const float a = cur.v[u] - mean;
        ss += a * a;
      }
    }
    const float sigma = sqrtf(group_sum<G>(ss) / fn);
    const float rs = 1.0f / (kLnEps + sigma);
    const float neg = -mean;
    float sxq = 0.f, sq = 0.f;
#pragma unroll
    for (int u = 0; u < VS; ++u) {
      if (gl + G * u < n) {
        const float xc = cur.v[u] + neg;
        const float dq = cur.d[u] * gg[u];
        sxq = fmaf(dq, xc, sxq);
        sq += dq;
        if (want_g && valid) pdg[u] = fmaf(cur.d[u], xc * rs, pdg[u]);
        if (want_b && valid) pdb[u] += cur.d[u];
      }
    }
    if (dx != nullptr) {
      const float ds = -(group_sum<G>(sxq) * rs) * rs;
      const float dmu = -(group_sum<G>(sq) * rs);
      const float sb = ds / (2.f * sigma);
      const float c = 2.f / fn;
      const float dmu_n = dmu / fn;
      float* pdx = dx + size_t(row) * n;
#pragma unroll
      for (int u = 0; u < VS; ++u) {
        const unsigned idx = gl + G * u;
        if (valid && idx < n) {
          float acc = cur.o[u];
          acc += c * (cur.v[u] - mean) * sb;
          acc += (cur.d[u] * gg[u]) * rs;
          acc += dmu_n;
          stg1<NT>(pdx + idx, acc);
        }
      }
    }
  };
  unsigned base = (blockIdx.x * WAVES + w) * R;
  if (base < bd) {
    load(cur, base + q);
    for (unsigned next = base + stride; next < bd; next += stride) {
      load(nxt, next + q);
      process(cur, base + q);
      cur = nxt;
      base = next;
    }
    process(cur, base + q);
  }
  if (!want_g && !want_b) return;
#pragma unroll
  for (int u = 0; u < VS; ++u) {
    if (G <= 8) {
      pdg[u] += dpp_move<0x128, 0xF>(pdg[u], 0.f);  // row_ror:8
      pdb[u] += dpp_move<0x128, 0xF>(pdb[u], 0.f);
    }
    if (G <= 4) {
      pdg[u] += dpp_move<0x124, 0xF>(pdg[u], 0.f);  // row_ror:4
      pdb[u] += dpp_move<0x124, 0xF>(pdb[u], 0.f);
    }
  }
  const unsigned slot = w * RL + (G >= 16 ? q : lane / 16);
#pragma unroll
  for (int u = 0; u < VS; ++u) {
    const unsigned idx = gl + G * u;
    if ((G >= 16 || lane % 16 < G) && idx < n) {
      if (want_g) lds[size_t(slot) * n + idx] = pdg[u];
      if (want_b) lds[size_t(RL * WAVES + slot) * n + idx] = pdb[u];
    }
  }
  __syncthreads();
  for (unsigned j = threadIdx.x; j < 2 * n; j += 64 * WAVES) {
    const unsigned which = j >= n ? 1u : 0u;
    float* part = which == 0 ? part_dg : part_db;
    if (part == nullptr) continue;
    const unsigned c = j - which * n;
    const float* src = lds + size_t(which) * RL * WAVES * n + c;
    float t = src[0];
#pragma unroll 8
    for (int k = 1; k < int(RL) * WAVES; ++k) t += src[size_t(k) * n];
    part[size_t(blockIdx.x) * n + c] = t;
  }
}

// A partial row on its way to the combine kernel: streamed past the caches when the partial rows together are larger
// than the L2s (they are written once and read once by other CUs); `nt` is the same for every thread.
__device__ __forceinline__ void st_part(float4* p, const float4 v, int nt) {
  if (nt) stg4<true>(p, v);
  else *p = v;
}

// Backward for rows of 2052..16384 floats: a 1024-thread block is 16/WPT teams of WPT waves; a team owns rows
// blockIdx.x*T + team, + gridDim.x*T, ... and keeps its dg / db partial sums in registers.  All teams of a block
// run the same number of iterations (rows past the end are all-zero rows that store nothing), so the barriers of
// the team reductions match.  At the end the teams are added in ascending order through LDS ([which][team][n]);
// the block's partial rows go to the workspace.
template <int WPT, bool NT>
__global__ __launch_bounds__(1024) void ln_bwd_team_kernel(unsigned n4, unsigned bd, const float4* __restrict__ x,
                                                           const float4* __restrict__ g,
                                                           const float4* __restrict__ dEdf, float4* __restrict__ dx,
                                                           float* __restrict__ part_dg, float* __restrict__ part_db,
                                                           int part_nt) {
  extern __shared__ float lds[];
  __shared__ float red[4][16];
  constexpr int T = 16 / WPT, TEAM = 64 * WPT, VPT = kLnTeamVpt;
  const int w = threadIdx.x >> 6, team = w / WPT, tl = threadIdx.x - team * TEAM;
  const float fn = float(n4 * 4);
  const bool want_g = part_dg != nullptr, want_b = part_db != nullptr;
  float4 gg[VPT], pdg[VPT], pdb[VPT];
#pragma unroll
  for (int u = 0; u < VPT; ++u) {
    const unsigned idx = tl + TEAM * u;
    gg[u] = idx < n4 ? g[idx] : make_float4(0.f, 0.f, 0.f, 0.f);
    pdg[u] = make_float4(0.f, 0.f, 0.f, 0.f);
    pdb[u] = make_float4(0.f, 0.f, 0.f, 0.f);
  }
  // The block's dg / db partial rows: its teams added in ascending order through LDS, then stored, after the last
  // row.  (Run before the last row's dx, as the one-wave-per-row kernel does, it was slower here: 22.4 against
  // 19.6 us for 1024 rows of 4096 - four teams meet at block-wide barriers and the 8 MiB of partial rows go out
  // ahead of the dx stores.)
  auto stage = [&]() __attribute__((always_inline)) {
    const unsigned n = n4 * 4;
    if (T == 1) {
#pragma unroll
      for (int u = 0; u < VPT; ++u) {
        const unsigned idx = tl + TEAM * u;
        if (idx < n4) {
          if (want_g) st_part(reinterpret_cast<float4*>(part_dg + size_t(blockIdx.x) * n) + idx, pdg[u], part_nt);
          if (want_b) st_part(reinterpret_cast<float4*>(part_db + size_t(blockIdx.x) * n) + idx, pdb[u], part_nt);
        }
      }
      return;
    }
    __syncthreads();
#pragma unroll
    for (int u = 0; u < VPT; ++u) {
      const unsigned idx = tl + TEAM * u;
      if (idx < n4) {
        if (want_g) reinterpret_cast<float4*>(lds + size_t(team) * n)[idx] = pdg[u];
        if (want_b) reinterpret_cast<float4*>(lds + size_t(T + team) * n)[idx] = pdb[u];
      }
    }
    __syncthreads();
    for (unsigned j4 = threadIdx.x; j4 < 2 * n4; j4 += 1024) {
      const unsigned which = j4 >= n4 ? 1u : 0u;
      float* part = which == 0 ? part_dg : part_db;
      if (part == nullptr) continue;
      const unsigned c4 = j4 - which * n4;
      const float4* src = reinterpret_cast<const float4*>(lds + size_t(which) * T * n) + c4;
      float4 t = src[0];
#pragma unroll
      for (int k = 1; k < T; ++k) {
        const float4 a = src[size_t(k) * n4];
        t.x += a.x; t.y += a.y; t.z += a.z; t.w += a.w;
      }
      st_part(reinterpret_cast<float4*>(part + size_t(blockIdx.x) * n) + c4, t, part_nt);
    }
  };
  for (unsigned base = blockIdx.x * T; base < bd; base += gridDim.x * T) {
    const unsigned row = base + team;
    const bool live = row < bd;
    const float4 zero = make_float4(0.f, 0.f, 0.f, 0.f);
    float4 v[VPT], d[VPT], o[VPT];
#pragma unroll
    for (int u = 0; u < VPT; ++u) {
      const unsigned idx = tl + TEAM * u;
      const bool in = live && idx < n4;
      v[u] = in ? ldg4<NT>(x + size_t(row) * n4 + idx) : zero;
      d[u] = in ? ldg4<NT>(dEdf + size_t(row) * n4 + idx) : zero;
      if (dx != nullptr) o[u] = in ? ldg4<NT>(dx + size_t(row) * n4 + idx) : zero;
    }
    float s = 0.f;
#pragma unroll
    for (int u = 0; u < VPT; ++u) s += (v[u].x + v[u].y) + (v[u].z + v[u].w);
    const float mean = team_sum<WPT>(s, red[0], w, team) / fn;
    float ss = 0.f;
#pragma unroll
    for (int u = 0; u < VPT; ++u) {
      if (tl + TEAM * u < n4) {
        const float ax = v[u].x - mean, ay = v[u].y - mean, az = v[u].z - mean, aw = v[u].w - mean;
        ss += (ax * ax + ay * ay) + (az * az + aw * aw);
      }
    }
    const float sigma = sqrtf(team_sum<WPT>(ss, red[1], w, team) / fn);
    const float rs = 1.0f / (kLnEps + sigma);
    const float neg = -mean;
    float sxq = 0.f, sq = 0.f;
#pragma unroll
    for (int u = 0; u < VPT; ++u) {
      if (live && tl + TEAM * u < n4) {
#define DYHIP_LN_ROW(c)                                        \
  {                                                            \
    const float xc = v[u].c + neg;                             \
    const float dq = d[u].c * gg[u].c;                         \
    sxq = fmaf(dq, xc, sxq);                                   \
    sq += dq;                                                  \
    if (want_g) pdg[u].c = fmaf(d[u].c, xc * rs, pdg[u].c);    \
    if (want_b) pdb[u].c += d[u].c;                            \
  }
        DYHIP_F4_EACH(DYHIP_LN_ROW)
#undef DYHIP_LN_ROW
      }
    }
    if (dx != nullptr) {
      // both row sums cross the team behind one barrier
      sxq = wave_sum(sxq);
      sq = wave_sum(sq);
      if ((threadIdx.x & 63) == 0) {
        red[2][w] = sxq;
        red[3][w] = sq;
      }
      __syncthreads();
      float txq = red[2][team * WPT], tq = red[3][team * WPT];
#pragma unroll
      for (int k = 1; k < WPT; ++k) {
        txq += red[2][team * WPT + k];
        tq += red[3][team * WPT + k];
      }
      const float ds = -(txq * rs) * rs;
      const float dmu = -(tq * rs);
      const float sb = ds / (2.f * sigma);
      const float c = 2.f / fn;
      const float dmu_n = dmu / fn;
#pragma unroll
      for (int u = 0; u < VPT; ++u) {
        const unsigned idx = tl + TEAM * u;
        if (live && idx < n4) {
          float4 r = o[u];
#define DYHIP_LN_DX(c_)                           \
  {                                               \
    float acc = r.c_;                             \
    acc += c * (v[u].c_ - mean) * sb;             \
    acc += (d[u].c_ * gg[u].c_) * rs;             \
    acc += dmu_n;                                 \
    r.c_ = acc;                                   \
  }
          DYHIP_F4_EACH(DYHIP_LN_DX)
#undef DYHIP_LN_DX
          stg4<NT>(dx + size_t(row) * n4 + idx, r);
        }
      }
    }
  }
  if (want_g || want_b) stage();
}

// generic fallback, pass 1: per-row statistics and the dx update.
// stats[row] = {mean, sden}
template <int kLnBlockThreads>
__global__ __launch_bounds__(kLnBlockThreads) void ln_bwd_block_kernel(size_t n, const float* __restrict__ x,
                                                                       const float* __restrict__ g,
                                                                       const float* __restrict__ dEdf,
                                                                       float* __restrict__ dx,
                                                                       float2* __restrict__ stats) {
  constexpr int T = kLnBlockThreads, W = kLnBlockThreads / 64;
  __shared__ float red[W];
  const float fn = float(n);
  const float* px = x + size_t(blockIdx.x) * n;
  const float* pdy = dEdf + size_t(blockIdx.x) * n;
  float s = 0.f;
  for (size_t j0 = threadIdx.x; j0 < n; j0 += 4 * T) {
    float a[4];
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const size_t j = j0 + size_t(u) * T;
      a[u] = px[j < n ? j : n - 1];
    }
#pragma unroll
    for (int u = 0; u < 4; ++u)
      if (j0 + size_t(u) * T < n) s += a[u];
  }
  const float mean = block_sum<W>(s, red) / fn;
  float v = 0.f;
  for (size_t j0 = threadIdx.x; j0 < n; j0 += 4 * T) {
    float a[4];
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const size_t j = j0 + size_t(u) * T;
      a[u] = px[j < n ? j : n - 1];
    }
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      if (j0 + size_t(u) * T < n) {
        const float d = a[u] - mean;
        v += d * d;
      }
    }
  }
  const float sigma = sqrtf(block_sum<W>(v, red) / fn);
  const float sden = kLnEps + sigma, neg = -mean, s2 = sden * sden;
  if (stats != nullptr && threadIdx.x == 0) stats[blockIdx.x] = make_float2(mean, sden);
  if (dx == nullptr) return;
  float ds_p = 0.f, dneg_p = 0.f;
  for (size_t j0 = threadIdx.x; j0 < n; j0 += 4 * T) {
    float a[4], d[4], gg[4];
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const size_t j = j0 + size_t(u) * T, jc = j < n ? j : n - 1;
      a[u] = px[jc];
      d[u] = pdy[jc];
      gg[u] = g[jc];
    }
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      if (j0 + size_t(u) * T < n) {
        const float dq = d[u] * gg[u];
        ds_p -= dq / s2 * (a[u] + neg);
        dneg_p += dq / sden;
      }
    }
  }
  const float ds = block_sum<W>(ds_p, red);
  const float dmu = -block_sum<W>(dneg_p, red);
  const float sb = ds / (2.f * sigma), c = 2.f / fn, dmu_n = dmu / fn;
  float* pdx = dx + size_t(blockIdx.x) * n;
  for (size_t j0 = threadIdx.x; j0 < n; j0 += 4 * T) {
    float a[4], d[4], gg[4], o[4];
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const size_t j = j0 + size_t(u) * T, jc = j < n ? j : n - 1;
      a[u] = px[jc];
      d[u] = pdy[jc];
      gg[u] = g[jc];
      o[u] = pdx[jc];
    }
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const size_t j = j0 + size_t(u) * T;
      if (j < n) {
        float acc = o[u];
        acc += c * (a[u] - mean) * sb;
        acc += (d[u] * gg[u]) / sden;
        acc += dmu_n;
        pdx[j] = acc;
      }
    }
  }
}

// generic fallback, pass 2: dg[j] += sum_b dy*(x-mean_b)/sden_b ; db[j] += sum_b dy.
// Row-parallel like batch_reduce_kernel: a block is 64 column lanes x 16 waves, wave w of split s walks rows
// s*per_split + w, + 16, ... with four rows in flight; waves are combined through LDS in ascending order and the
// block's partial rows go to the workspace, where combine_partials adds the splits in ascending order.
constexpr int kLnColsWaves = 16;
__global__ __launch_bounds__(64 * kLnColsWaves) void ln_bwd_cols_kernel(size_t n, unsigned bd, unsigned per_split,
                                                                       const float* __restrict__ x,
                                                                       const float* __restrict__ dEdf,
                                                                       const float2* __restrict__ stats,
                                                                       float* __restrict__ part_dg,
                                                                       float* __restrict__ part_db) {
  __shared__ float lds[2][kLnColsWaves][64];
  const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
  const size_t j = size_t(blockIdx.x) * 64 + lane;
  const unsigned b0 = blockIdx.y * per_split, b1 = min(bd, b0 + per_split);
  float sg = 0.f, sb = 0.f;
  if (j < n) {
    constexpr int U = 4;
    unsigned r = b0 + w;
    for (; r + (U - 1) * kLnColsWaves < b1; r += U * kLnColsWaves) {
      float xv[U], dv[U];
      float2 st[U];
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const unsigned rr = r + u * kLnColsWaves;
        xv[u] = x[size_t(rr) * n + j];
        dv[u] = dEdf[size_t(rr) * n + j];
        st[u] = stats[rr];
      }
#pragma unroll
      for (int u = 0; u < U; ++u) {
        sg += dv[u] * ((xv[u] - st[u].x) / st[u].y);
        sb += dv[u];
      }
    }
    for (; r < b1; r += kLnColsWaves) {
      const float2 st = stats[r];
      const float d = dEdf[size_t(r) * n + j];
      sg += d * ((x[size_t(r) * n + j] - st.x) / st.y);
      sb += d;
    }
  }
  lds[0][w][lane] = sg;
  lds[1][w][lane] = sb;
  __syncthreads();
  if (w < 2 && j < n) {
    float t = lds[w][0][lane];
#pragma unroll
    for (int k = 1; k < kLnColsWaves; ++k) t += lds[w][k][lane];
    float* part = w == 0 ? part_dg : part_db;
    if (part) part[size_t(blockIdx.y) * n + j] = t;
  }
}

static unsigned ln_cols_splits(size_t n, unsigned bd) {
  const unsigned tiles = static_cast<unsigned>(cdiv<size_t>(n, 64));
  unsigned want = tiles >= 512 ? 1u : cdiv<unsigned>(512u, tiles);
  const unsigned max_by_work = cdiv<unsigned>(bd, 2 * kLnColsWaves);
  if (want > max_by_work) want = max_by_work;
  if (want > 64) want = 64;
  if (want < 1) want = 1;
  return cdiv<unsigned>(bd, cdiv<unsigned>(bd, want));
}

static size_t ln_stats_bytes(unsigned bd) { return cdiv<size_t>(size_t(bd) * sizeof(float2), 256) * 256; }

static bool ln_fast_ok(size_t n, const void* a, const void* b, const void* c, const void* d) {
  return n % 4 == 0 && n <= 2048 && aligned16(a) && aligned16(b) && (c == nullptr || aligned16(c)) &&
         (d == nullptr || aligned16(d));
}

static bool ln_team_ok(size_t n, const void* a, const void* b, const void* c, const void* d) {
  return n % 4 == 0 && n > 2048 && n <= 16384 && aligned16(a) && aligned16(b) && (c == nullptr || aligned16(c)) &&
         (d == nullptr || aligned16(d));
}

// waves per team of the wide-row kernels: the team's 64*WPT threads hold 16 floats each
static int ln_team_waves(size_t n) { return n <= 4096 ? 4 : n <= 8192 ? 8 : 16; }

static unsigned ln_bwd_blocks(size_t n, unsigned bd) {
  const unsigned per_block = n <= 2048 ? unsigned(kLnWavesBwd) : unsigned(16 / ln_team_waves(n));
  unsigned blocks = cdiv<unsigned>(bd, per_block);
  // one block per CU keeps the partial rows few; once every wave of those blocks would own eight rows or more the
  // partial rows no longer matter and a second block per CU (its 64 KB of LDS fits beside the first up to n = 1024)
  // hides the row reductions (65536 rows of 1024: 192 -> 188 us)
  const unsigned cap =
      n <= 1024 && bd / (kLnBwdMaxBlocks * per_block) >= 8 ? 2 * kLnBwdMaxBlocks : kLnBwdMaxBlocks;
  return blocks > cap ? cap : blocks;
}

// Scratch of dyhip_layer_norm_backward_static: the per-block dg / db partial rows (or the per-row
// statistics of the generic path) live in this array instead of a caller-provided workspace, so that
// entry point allocates nothing.  Every GPU the library runs on holds its own copy at its own address
// until the process ends.  Host code never uses the array's name as an address (on the host it is only
// a stand-in for the device symbol): ln_static_scratch_setup asks the runtime for the address on the
// current device once, when the device handle is created, and every later use goes through that pointer.
static __device__ __align__(256) unsigned char scratch[DYHIP_LN_STATIC_SCRATCH_BYTES];

int ln_static_scratch_setup(dyhip_device* dev) {
  void* ptr = nullptr;
  DYHIP_CHECK_HIP(hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)));
  dev->ln_scratch = ptr;
  return DYHIP_OK;
}

}  // namespace dyhip

using namespace dyhip;

extern "C" {

int dyhip_batch_reduce_workspace(size_t n, unsigned bd, size_t* ws_bytes) {
  DYHIP_REQUIRE(ws_bytes != nullptr, "null output pointer");
  if (n == 0 || bd == 0) {
    *ws_bytes = 0;
    return DYHIP_OK;
  }
  // the scalar plan has at least as many tiles, hence at most as many splits
  const BrPlan p = br_plan(n, bd, n % 4 == 0);
  const BrPlan q = br_plan(n, bd, false);
  unsigned splits = p.splits > q.splits ? p.splits : q.splits;
  if (br_flat(n, bd) && splits < kBrFlatMaxBlocks) splits = kBrFlatMaxBlocks;  // the flat walk's partial rows
  *ws_bytes = splits > 1 ? size_t(splits) * n * sizeof(float) : 0;
  return DYHIP_OK;
}

int dyhip_sum_batches_forward(dyhip_device* dev, size_t n, unsigned bd, const float* x, float* y, void* ws,
                              size_t ws_bytes) {
  DYHIP_CHECK_DEV(dev);
  DYHIP_REQUIRE(n == 0 || (x && y), "null tensor pointer");
  return batch_reduce(dev, n, bd, x, nullptr, y, false, ws, ws_bytes);
}

int dyhip_mean_elems_forward(dyhip_device* dev, size_t n, unsigned bd, const float* x, float* y) {
  DYHIP_CHECK_DEV(dev);
  DYHIP_REQUIRE(n >= 1 && x && y, "mean_elems needs a non-empty tensor");
  if (bd == 0) return DYHIP_OK;
  if (launch_moment_resident<0>(dev, n, bd, x, nullptr, nullptr, y)) {
    DYHIP_CHECK_LAUNCH();
    return DYHIP_OK;
  }
  unsigned chunks = 0;
  if (moment_chunked_fits(dev, n, bd, &chunks)) {
    float* stats = static_cast<float*>(dev->gemm_ws);
    hipLaunchKernelGGL(moment_chunk_kernel<0>, dim3(chunks, bd), dim3(256), 0, dev->stream, n, x, stats);
    hipLaunchKernelGGL(moment_finish_kernel<0>, dim3(bd), dim3(64), 0, dev->stream, n, chunks, stats, y);
    DYHIP_CHECK_LAUNCH();
    return DYHIP_OK;
  }
  hipLaunchKernelGGL(moment_fwd_kernel<false>, dim3(bd), dim3(kMomThreads), 0, dev->stream, n, x, y);
  DYHIP_CHECK_LAUNCH();
  return DYHIP_OK;
}

int dyhip_std_elems_forward(dyhip_device* dev, size_t n, unsigned bd, const float* x, float* y) {
  DYHIP_CHECK_DEV(dev);
  DYHIP_REQUIRE(n >= 1 && x && y, "std_elems needs a non-empty tensor");
  if (bd == 0) return DYHIP_OK;
  if (launch_moment_resident<1>(dev, n, bd, x, nullptr, nullptr, y)) {
    DYHIP_CHECK_LAUNCH();
    return DYHIP_OK;
  }
  unsigned chunks = 0;
  if (moment_chunked_fits(dev, n, bd, &chunks)) {
    float* stats = static_cast<float*>(dev->gemm_ws);
    hipLaunchKernelGGL(moment_chunk_kernel<1>, dim3(chunks, bd), dim3(256), 0, dev->stream, n, x, stats);
    hipLaunchKernelGGL(moment_finish_kernel<1>, dim3(bd), dim3(64), 0, dev->stream, n, chunks, stats, y);
    DYHIP_CHECK_LAUNCH();
    return DYHIP_OK;
  }
  hipLaunchKernelGGL(moment_fwd_kernel<true>, dim3(bd), dim3(kMomThreads), 0, dev->stream, n, x, y);
  DYHIP_CHECK_LAUNCH();
  return DYHIP_OK;
}

int dyhip_mean_elems_backward(dyhip_device* dev, size_t n, unsigned bd, const float* dEdf, float* dEdx) {
  DYHIP_CHECK_DEV(dev);
  DYHIP_REQUIRE(n >= 1 && dEdf && dEdx, "mean_elems needs a non-empty tensor");
  if (bd == 0) return DYHIP_OK;
  const size_t total = n * size_t(bd);
  if (n <= 0xFFFFFFFFull && cdiv<size_t>(total, 1024) < (size_t(1) << 31)) {
    hipLaunchKernelGGL(mean_bwd_flat_kernel, dim3((unsigned)cdiv<size_t>(total, 1024)), dim3(256), 0, dev->stream,
                       static_cast<unsigned>(n), total, dEdf, dEdx);
    DYHIP_CHECK_LAUNCH();
    return DYHIP_OK;
  }
  hipLaunchKernelGGL(mean_bwd_kernel, dim3((unsigned)cdiv<size_t>(n, 256), bd < 65535u ? bd : 65535u), dim3(256), 0,
                     dev->stream, n, bd, dEdf, dEdx);
  DYHIP_CHECK_LAUNCH();
  return DYHIP_OK;
}

int dyhip_std_elems_backward(dyhip_device* dev, size_t n, unsigned bd, const float* x, const float* fx,
                             const float* dEdf, float* dEdx) {
  DYHIP_CHECK_DEV(dev);
  DYHIP_REQUIRE(n >= 1 && x && fx && dEdf && dEdx, "std_elems needs a non-empty tensor");
  if (bd == 0) return DYHIP_OK;
  if (launch_moment_resident<2>(dev, n, bd, x, fx, dEdf, dEdx)) {
    DYHIP_CHECK_LAUNCH();
    return DYHIP_OK;
  }
  unsigned chunks = 0;
  if (moment_chunked_fits(dev, n, bd, &chunks)) {
    float* sums = static_cast<float*>(dev->gemm_ws);
    hipLaunchKernelGGL(moment_chunk_kernel<0>, dim3(chunks, bd), dim3(256), 0, dev->stream, n, x, sums);
    hipLaunchKernelGGL(std_bwd_chunked_kernel, dim3(static_cast<unsigned>(cdiv<size_t>(n, 1024)), bd), dim3(256), 0,
                       dev->stream, n, chunks, x, sums, fx, dEdf, dEdx);
    DYHIP_CHECK_LAUNCH();
    return DYHIP_OK;
  }
  hipLaunchKernelGGL(std_bwd_kernel, dim3(bd), dim3(kMomThreads), 0, dev->stream, n, x, fx, dEdf, dEdx);
  DYHIP_CHECK_LAUNCH();
  return DYHIP_OK;
}

int dyhip_layer_norm_forward(dyhip_device* dev, size_t n, unsigned bd, const float* x, const float* g,
                             const float* b, float* y) {
  DYHIP_CHECK_DEV(dev);
  DYHIP_REQUIRE(n >= 1 && x && g && b && y, "layer_norm needs non-empty tensors");
  if (bd == 0) return DYHIP_OK;
  if (ln_fast_ok(n, x, g, b, y)) {
    const unsigned n4 = static_cast<unsigned>(n / 4);
    const dim3 grid(cdiv<unsigned>(bd, kLnWavesFwd)), block(64 * kLnWavesFwd);
    const float4 *x4 = reinterpret_cast<const float4*>(x), *g4 = reinterpret_cast<const float4*>(g),
                 *b4 = reinterpret_cast<const float4*>(b);
    float4* y4 = reinterpret_cast<float4*>(y);
    const bool stream = n * size_t(bd) * sizeof(float) >= dev->stream_threshold;
#define DYHIP_LN_FWD_GROUP(G, VPL, RPG)                                                                           \
  do {                                                                                                            \
    const dim3 gg(cdiv<unsigned>(bd, kLnWavesFwd * (64 / G) * RPG));                                              \
    if (stream) hipLaunchKernelGGL((ln_fwd_group_kernel<G, VPL, RPG, true>), gg, block, 0, dev->stream, n4, bd, x4, g4, b4, y4); \
    else hipLaunchKernelGGL((ln_fwd_group_kernel<G, VPL, RPG, false>), gg, block, 0, dev->stream, n4, bd, x4, g4, b4, y4);       \
  } while (0)
#define DYHIP_LN_FWD(VPL)                                                                                       \
  do {                                                                                                          \
    if (stream) hipLaunchKernelGGL((ln_fwd_wave_kernel<VPL, true>), grid, block, 0, dev->stream, n4, bd, x4, g4, b4, y4); \
    else hipLaunchKernelGGL((ln_fwd_wave_kernel<VPL, false>), grid, block, 0, dev->stream, n4, bd, x4, g4, b4, y4);       \
  } while (0)
    // short rows: several rows a wavefront
    if (n4 <= 4) DYHIP_LN_FWD_GROUP(4, 1, 2);
    else if (n4 <= 8) DYHIP_LN_FWD_GROUP(8, 1, 2);
    else if (n4 <= 16) DYHIP_LN_FWD_GROUP(16, 1, 2);
    else if (n4 <= 32) DYHIP_LN_FWD_GROUP(16, 2, 2);
    else if (n4 <= 48) DYHIP_LN_FWD_GROUP(16, 3, 1);
    else if (n4 <= 64) DYHIP_LN_FWD_GROUP(16, 4, 1);
    else if (n4 <= 128) DYHIP_LN_FWD(2);
    else if (n4 <= 256) DYHIP_LN_FWD(4);
    else DYHIP_LN_FWD(8);
#undef DYHIP_LN_FWD
#undef DYHIP_LN_FWD_GROUP
  } else if (ln_team_ok(n, x, g, b, y)) {
    const unsigned n4 = static_cast<unsigned>(n / 4);
    const float4 *x4 = reinterpret_cast<const float4*>(x), *g4 = reinterpret_cast<const float4*>(g),
                 *b4 = reinterpret_cast<const float4*>(b);
    float4* y4 = reinterpret_cast<float4*>(y);
    const bool stream = n * size_t(bd) * sizeof(float) >= dev->stream_threshold;
#define DYHIP_LN_FWD(WPT)                                                                                         \
  do {                                                                                                            \
    if (stream) hipLaunchKernelGGL((ln_fwd_team_kernel<WPT, true>), dim3(bd), dim3(64 * WPT), 0, dev->stream, n4, x4, g4, b4, y4); \
    else hipLaunchKernelGGL((ln_fwd_team_kernel<WPT, false>), dim3(bd), dim3(64 * WPT), 0, dev->stream, n4, x4, g4, b4, y4);       \
  } while (0)
    switch (ln_team_waves(n)) {
      case 4: DYHIP_LN_FWD(4); break;
      case 8: DYHIP_LN_FWD(8); break;
      default: DYHIP_LN_FWD(16); break;
    }
#undef DYHIP_LN_FWD
  } else if (n <= 2048) {
    // rows that cannot take 128-bit accesses: one wavefront per row all the same, one float per lane and step
    const unsigned nn = static_cast<unsigned>(n);
    const dim3 grid(cdiv<unsigned>(bd, kLnWavesFwd)), block(64 * kLnWavesFwd);
    const bool stream = n * size_t(bd) * sizeof(float) >= dev->stream_threshold;
#define DYHIP_LN_FWD_GROUP(G, VS, RPG)                                                                            \
  do {                                                                                                            \
    const dim3 gg(cdiv<unsigned>(bd, kLnWavesFwd * (64 / G) * RPG));                                              \
    if (stream) hipLaunchKernelGGL((ln_fwd_group1_kernel<G, VS, RPG, true>), gg, block, 0, dev->stream, nn, bd, x, g, b, y); \
    else hipLaunchKernelGGL((ln_fwd_group1_kernel<G, VS, RPG, false>), gg, block, 0, dev->stream, nn, bd, x, g, b, y);       \
  } while (0)
#define DYHIP_LN_FWD(VS)                                                                                          \
  do {                                                                                                            \
    if (stream) hipLaunchKernelGGL((ln_fwd_lane_kernel<VS, true>), grid, block, 0, dev->stream, nn, bd, x, g, b, y); \
    else hipLaunchKernelGGL((ln_fwd_lane_kernel<VS, false>), grid, block, 0, dev->stream, nn, bd, x, g, b, y);       \
  } while (0)
    // short rows: several rows a wavefront
    // short rows: as many lanes a row as reach its end (a group's access is then one run), several rows a wavefront
    if (nn <= 4) DYHIP_LN_FWD_GROUP(4, 1, 4);
    else if (nn <= 8) DYHIP_LN_FWD_GROUP(8, 1, 4);
    else if (nn <= 16) DYHIP_LN_FWD_GROUP(16, 1, 4);
    else if (nn <= 32) DYHIP_LN_FWD_GROUP(32, 1, 4);
    else if (nn <= 64) DYHIP_LN_FWD_GROUP(64, 1, 4);
    else if (nn <= 128) DYHIP_LN_FWD_GROUP(64, 2, 2);
    else if (nn <= 192) DYHIP_LN_FWD_GROUP(64, 3, 2);  // 150 floats: 11.9 -> 10.6 us; 250 floats gain nothing from a second row
    else if (nn <= 512) DYHIP_LN_FWD(8);
    else if (nn <= 1024) DYHIP_LN_FWD(16);
    else DYHIP_LN_FWD(32);
#undef DYHIP_LN_FWD
#undef DYHIP_LN_FWD_GROUP
  } else {
    if (n <= 4096) hipLaunchKernelGGL(ln_fwd_block_kernel<256>, dim3(bd), dim3(256), 0, dev->stream, n, x, g, b, y);
    else hipLaunchKernelGGL(ln_fwd_block_kernel<1024>, dim3(bd), dim3(1024), 0, dev->stream, n, x, g, b, y);
  }
  DYHIP_CHECK_LAUNCH();
  return DYHIP_OK;
}

// Scratch of the backward pass by the path it takes: the register-resident kernels need one partial row of dg and of
// db per block, the generic path per-row statistics and one partial row per output and batch split; nothing at all
// when neither dg nor db is asked for.
static size_t ln_bwd_ws_fast(size_t n, unsigned bd) { return size_t(2) * ln_bwd_blocks(n, bd) * n * sizeof(float); }
static size_t ln_bwd_ws_generic(size_t n, unsigned bd) {
  return ln_stats_bytes(bd) + size_t(2) * ln_cols_splits(n, bd ? bd : 1) * n * sizeof(float);
}
static size_t ln_bwd_ws_of_call(size_t n, unsigned bd, const float* x, const float* g, const float* dEdf, const float* dx,
                                bool cols) {
  if (!cols || bd == 0) return 0;
  // rows of at most 1024 floats always take a one-wavefront-per-row kernel (128-bit, or one float per lane and step)
  return n <= 1024 || ln_fast_ok(n, x, g, dEdf, dx) || ln_team_ok(n, x, g, dEdf, dx) ? ln_bwd_ws_fast(n, bd)
                                                                                      : ln_bwd_ws_generic(n, bd);
}

int dyhip_layer_norm_backward_workspace(size_t n, unsigned bd, size_t* ws_bytes) {
  DYHIP_REQUIRE(ws_bytes != nullptr, "null output pointer");
  // the pointers are not known here: enough for whichever path the call takes
  const size_t fast = n <= 16384 ? ln_bwd_ws_fast(n, bd) : 0, generic = ln_bwd_ws_generic(n, bd);
  *ws_bytes = fast > generic ? fast : generic;
  return DYHIP_OK;
}

int dyhip_layer_norm_backward_static(dyhip_device* dev, size_t n, unsigned bd, const float* x, const float* g,
                                     const float* dEdf, float* dx, float* dg, float* db) {
  DYHIP_CHECK_DEV(dev);
  // what the path this call takes needs (its pointers are known here), not the larger of the two paths
  const size_t need = ln_bwd_ws_of_call(n, bd, x, g, dEdf, dx, dg != nullptr || db != nullptr);
  DYHIP_REQUIRE(need <= size_t(DYHIP_LN_STATIC_SCRATCH_BYTES),
                "layer_norm backward without a workspace is limited to %zu scratch bytes; n = %zu, bd = %u needs %zu",
                size_t(DYHIP_LN_STATIC_SCRATCH_BYTES), n, bd, need);
  DYHIP_REQUIRE(dev->ln_scratch != nullptr, "the static scratch array of this device was not set up");
  return dyhip_layer_norm_backward(dev, n, bd, x, g, dEdf, dx, dg, db, dev->ln_scratch,
                                   size_t(DYHIP_LN_STATIC_SCRATCH_BYTES));
}

int dyhip_layer_norm_backward(dyhip_device* dev, size_t n, unsigned bd, const float* x, const float* g,
                              const float* dEdf, float* dx, float* dg, float* db, void* ws, size_t ws_bytes) {
  DYHIP_CHECK_DEV(dev);
  DYHIP_REQUIRE(n >= 1 && x && g && dEdf, "layer_norm needs non-empty tensors");
  if (bd == 0 || (!dx && !dg && !db)) return DYHIP_OK;
  const bool cols = dg != nullptr || db != nullptr;
  const size_t need = ln_bwd_ws_of_call(n, bd, x, g, dEdf, dx, cols);
  DYHIP_REQUIRE(!cols || (ws != nullptr && ws_bytes >= need), "layer_norm backward needs %zu workspace bytes, got %zu",
                need, ws_bytes);
  if (ln_fast_ok(n, x, g, dEdf, dx)) {
    const unsigned n4 = static_cast<unsigned>(n / 4);
    const unsigned waves = kLnWavesBwd;
    unsigned blocks = ln_bwd_blocks(n, bd);
    float* part_dg = dg ? static_cast<float*>(ws) : nullptr;
    float* part_db = db ? static_cast<float*>(ws) + size_t(blocks) * n : nullptr;  // placed for the upper bound of the block count
    const size_t lds = cols ? size_t(2) * waves * n * sizeof(float) : 0;  // [dg | db][wave][n]
    const dim3 grid(blocks), block(64 * waves);
    const float4 *x4 = reinterpret_cast<const float4*>(x), *g4 = reinterpret_cast<const float4*>(g),
                 *d4 = reinterpret_cast<const float4*>(dEdf);
    float4* dx4 = reinterpret_cast<float4*>(dx);
    const bool stream = n * size_t(bd) * sizeof(float) >= dev->stream_threshold;
// The row after the current one is fetched ahead, except for rows of 1028..2044 floats: two rows of eight groups a
// lane do not fit the registers beside the partial sums, and with the bounds-checked loads of a row that does not
// fill every lane the spills cost more than the prefetch gains (2048 rows of 1536: 32.1 -> 15.4 us without it; rows
// of exactly 2048 floats keep it: 18.1 against 23.9 us).
#define DYHIP_LN_BWD_LAUNCH(VPL, NT, WAVES, FULL)                                                           \
  hipLaunchKernelGGL((ln_bwd_wave_kernel<VPL, NT, WAVES, (VPL < 8 || FULL), FULL>), grid, block, lds, dev->stream, n4, bd, x4, \
                     g4, d4, dx4, part_dg, part_db)
#define DYHIP_LN_BWD_LDS(VPL, NT, WAVES, FULL)                                                              \
  DYHIP_CHECK_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(&ln_bwd_wave_kernel<VPL, NT, WAVES, (VPL < 8 || FULL), FULL>), \
                                      hipFuncAttributeMaxDynamicSharedMemorySize, 128 << 10))
#define DYHIP_LN_BWD(VPL)                                                                                  \
  do {                                                                                                     \
    static bool big_lds_ok = false;                                                                        \
    if (lds > (size_t(64) << 10) && !big_lds_ok) {                                                          \
      DYHIP_LN_BWD_LDS(VPL, true, kLnWavesBwd, true);                                                      \
      DYHIP_LN_BWD_LDS(VPL, false, kLnWavesBwd, true);                                                     \
      DYHIP_LN_BWD_LDS(VPL, true, kLnWavesBwd, false);                                                     \
      DYHIP_LN_BWD_LDS(VPL, false, kLnWavesBwd, false);                                                    \
      big_lds_ok = true;                                                                                   \
    }                                                                                                      \
    const bool full = dx4 != nullptr && n4 == 64u * VPL;                                                   \
    if (stream && full) DYHIP_LN_BWD_LAUNCH(VPL, true, kLnWavesBwd, true);                            \
    else if (stream) DYHIP_LN_BWD_LAUNCH(VPL, true, kLnWavesBwd, false);                                   \
    else if (full) DYHIP_LN_BWD_LAUNCH(VPL, false, kLnWavesBwd, true);                                     \
    else DYHIP_LN_BWD_LAUNCH(VPL, false, kLnWavesBwd, false);                                              \
  } while (0)
// short rows: several rows a wavefront; never more blocks than the workspace was sized for
#define DYHIP_LN_BWD_GROUP(G, VPL)                                                                          \
  do {                                                                                                      \
    const unsigned per_block = kLnWavesBwd * (64 / G);                                                      \
    if (cdiv<unsigned>(bd, per_block) < blocks) blocks = cdiv<unsigned>(bd, per_block);                     \
    const size_t glds = cols ? size_t(2) * 4 * kLnWavesBwd * n * sizeof(float) : 0;                         \
    if (stream)                                                                                             \
      hipLaunchKernelGGL((ln_bwd_group_kernel<G, VPL, true>), dim3(blocks), block, glds, dev->stream, n4, bd, x4, g4, \
                         d4, dx4, part_dg, part_db);                                                        \
    else                                                                                                    \
      hipLaunchKernelGGL((ln_bwd_group_kernel<G, VPL, false>), dim3(blocks), block, glds, dev->stream, n4, bd, x4, g4, \
                         d4, dx4, part_dg, part_db);                                                        \
  } while (0)
    if (n4 <= 4) DYHIP_LN_BWD_GROUP(4, 1);
    else if (n4 <= 8) DYHIP_LN_BWD_GROUP(8, 1);
    else if (n4 <= 16) DYHIP_LN_BWD_GROUP(16, 1);
    else if (n4 <= 32) DYHIP_LN_BWD_GROUP(16, 2);
    else if (n4 <= 64) DYHIP_LN_BWD(1);
    else if (n4 <= 128) DYHIP_LN_BWD(2);
    else if (n4 <= 256) DYHIP_LN_BWD(4);
    else DYHIP_LN_BWD(8);
#undef DYHIP_LN_BWD
#undef DYHIP_LN_BWD_GROUP
#undef DYHIP_LN_BWD_LAUNCH
#undef DYHIP_LN_BWD_LDS
    DYHIP_CHECK_LAUNCH();
    if (dg && db) launch_combine(dev, n, blocks, part_dg, dg, part_db, db, 1);
    else if (dg) launch_combine(dev, n, blocks, part_dg, dg, nullptr, nullptr, 1);
    else if (db) launch_combine(dev, n, blocks, part_db, db, nullptr, nullptr, 1);
    DYHIP_CHECK_LAUNCH();
  } else if (ln_team_ok(n, x, g, dEdf, dx)) {
    const unsigned n4 = static_cast<unsigned>(n / 4);
    const unsigned blocks = ln_bwd_blocks(n, bd);
    const int wpt = ln_team_waves(n), teams = 16 / wpt;
    float* part_dg = dg ? static_cast<float*>(ws) : nullptr;
    float* part_db = db ? static_cast<float*>(ws) + size_t(blocks) * n : nullptr;
    const size_t lds = cols && teams > 1 ? size_t(2) * teams * n * sizeof(float) : 0;  // [dg | db][team][n], <= 128 KB
    const float4 *x4 = reinterpret_cast<const float4*>(x), *g4 = reinterpret_cast<const float4*>(g),
                 *d4 = reinterpret_cast<const float4*>(dEdf);
    float4* dx4 = reinterpret_cast<float4*>(dx);
    const bool stream = n * size_t(bd) * sizeof(float) >= dev->stream_threshold;
    // 1024 rows of 4096: 8 MiB of partial rows, 21.3 -> 19.6 us with streaming stores and loads; 2 MiB (the
    // one-wave-per-row kernel's) are faster through the caches
    const int part_nt = ln_bwd_ws_fast(n, bd) >= (size_t(4) << 20) ? 1 : 0;
#define DYHIP_LN_BWD(WPT)                                                                                       \
  do {                                                                                                          \
    static bool big_lds_ok = false;                                                                             \
    if (lds > (size_t(64) << 10) && !big_lds_ok) {                                                               \
      DYHIP_CHECK_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(&ln_bwd_team_kernel<WPT, true>),        \
                                          hipFuncAttributeMaxDynamicSharedMemorySize, 128 << 10));               \
      DYHIP_CHECK_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(&ln_bwd_team_kernel<WPT, false>),       \
                                          hipFuncAttributeMaxDynamicSharedMemorySize, 128 << 10));               \
      big_lds_ok = true;                                                                                        \
    }                                                                                                           \
    if (stream)                                                                                                 \
      hipLaunchKernelGGL((ln_bwd_team_kernel<WPT, true>), dim3(blocks), dim3(1024), lds, dev->stream, n4, bd, x4, g4, \
                         d4, dx4, part_dg, part_db, part_nt);                                                   \
    else                                                                                                        \
      hipLaunchKernelGGL((ln_bwd_team_kernel<WPT, false>), dim3(blocks), dim3(1024), lds, dev->stream, n4, bd, x4, g4, \
                         d4, dx4, part_dg, part_db, part_nt);                                                   \
  } while (0)
    switch (wpt) {
      case 4: DYHIP_LN_BWD(4); break;
      case 8: DYHIP_LN_BWD(8); break;
      default: DYHIP_LN_BWD(16); break;
    }
#undef DYHIP_LN_BWD
    DYHIP_CHECK_LAUNCH();
    if (dg && db) launch_combine(dev, n, blocks, part_dg, dg, part_db, db, 1, part_nt);
    else if (dg) launch_combine(dev, n, blocks, part_dg, dg, nullptr, nullptr, 1, part_nt);
    else if (db) launch_combine(dev, n, blocks, part_db, db, nullptr, nullptr, 1, part_nt);
    DYHIP_CHECK_LAUNCH();
  } else if (n <= 1024) {
    const unsigned nn = static_cast<unsigned>(n);
    unsigned blocks = ln_bwd_blocks(n, bd);
    float* part_dg = dg ? static_cast<float*>(ws) : nullptr;
    float* part_db = db ? static_cast<float*>(ws) + size_t(blocks) * n : nullptr;  // placed for the upper bound of the block count
    const size_t lds = cols ? size_t(2) * kLnWavesBwd * n * sizeof(float) : 0;  // [dg | db][wave][n], <= 128 KB
    const dim3 grid(blocks), block(64 * kLnWavesBwd);
    const bool stream = n * size_t(bd) * sizeof(float) >= dev->stream_threshold;
    // the row after the current one is fetched ahead
#define DYHIP_LN_BWD(VS)                                                                                            \
  do {                                                                                                              \
    static bool big_lds_ok = false;                                                                                 \
    if (lds > (size_t(64) << 10) && !big_lds_ok) {                                                                   \
      DYHIP_CHECK_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(&ln_bwd_lane_kernel<VS, true, true>),  \
                                          hipFuncAttributeMaxDynamicSharedMemorySize, 128 << 10));                   \
      DYHIP_CHECK_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(&ln_bwd_lane_kernel<VS, false, true>), \
                                          hipFuncAttributeMaxDynamicSharedMemorySize, 128 << 10));                   \
      big_lds_ok = true;                                                                                            \
    }                                                                                                               \
    if (stream)                                                                                                     \
      hipLaunchKernelGGL((ln_bwd_lane_kernel<VS, true, true>), grid, block, lds, dev->stream, nn, bd, x, g, dEdf, \
                         dx, part_dg, part_db);                                                                     \
    else                                                                                                            \
      hipLaunchKernelGGL((ln_bwd_lane_kernel<VS, false, true>), grid, block, lds, dev->stream, nn, bd, x, g, dEdf, \
                         dx, part_dg, part_db);                                                                     \
  } while (0)
// short rows: several rows a wavefront; never more blocks than the workspace was sized for
#define DYHIP_LN_BWD_GROUP(G, VS)                                                                                   \
  do {                                                                                                              \
    const unsigned per_block = kLnWavesBwd * (64 / G);                                                              \
    if (cdiv<unsigned>(bd, per_block) < blocks) blocks = cdiv<unsigned>(bd, per_block);                             \
    const size_t glds = cols ? size_t(2) * (G >= 16 ? 64 / G : 4) * kLnWavesBwd * n * sizeof(float) : 0;            \
    if (stream)                                                                                                     \
      hipLaunchKernelGGL((ln_bwd_group1_kernel<G, VS, true>), dim3(blocks), block, glds, dev->stream, nn, bd, x, g, dEdf, \
                         dx, part_dg, part_db);                                                                     \
    else                                                                                                            \
      hipLaunchKernelGGL((ln_bwd_group1_kernel<G, VS, false>), dim3(blocks), block, glds, dev->stream, nn, bd, x, g, dEdf, \
                         dx, part_dg, part_db);                                                                     \
  } while (0)
    if (nn <= 4) DYHIP_LN_BWD_GROUP(4, 1);
    else if (nn <= 8) DYHIP_LN_BWD_GROUP(8, 1);
    else if (nn <= 16) DYHIP_LN_BWD_GROUP(16, 1);
    else if (nn <= 32) DYHIP_LN_BWD_GROUP(16, 2);  // 30 floats: 20.9 us, against 25.0 us with 32 lanes a row
    else if (nn <= 64) DYHIP_LN_BWD_GROUP(32, 2);  // 50 floats: 21.0 us, against 28.0 us with 16 lanes a row
    else if (nn <= 128) DYHIP_LN_BWD(2);
    else if (nn <= 256) DYHIP_LN_BWD(4);
    else if (nn <= 512) DYHIP_LN_BWD(8);
    else DYHIP_LN_BWD(16);
#undef DYHIP_LN_BWD
#undef DYHIP_LN_BWD_GROUP
    DYHIP_CHECK_LAUNCH();
    if (dg && db) launch_combine(dev, n, blocks, part_dg, dg, part_db, db, 1);
    else if (dg) launch_combine(dev, n, blocks, part_dg, dg, nullptr, nullptr, 1);
    else if (db) launch_combine(dev, n, blocks, part_db, db, nullptr, nullptr, 1);
    DYHIP_CHECK_LAUNCH();
  } else {
    float2* stats = cols ? static_cast<float2*>(ws) : nullptr;
    if (n <= 4096)
      hipLaunchKernelGGL(ln_bwd_block_kernel<256>, dim3(bd), dim3(256), 0, dev->stream, n, x, g, dEdf, dx, stats);
    else
      hipLaunchKernelGGL(ln_bwd_block_kernel<1024>, dim3(bd), dim3(1024), 0, dev->stream, n, x, g, dEdf, dx, stats);
    DYHIP_CHECK_LAUNCH();
    if (cols) {
      const unsigned splits = ln_cols_splits(n, bd), per_split = cdiv<unsigned>(bd, splits);
      float* part_dg = reinterpret_cast<float*>(static_cast<char*>(ws) + ln_stats_bytes(bd));
      float* part_db = part_dg + size_t(splits) * n;
      hipLaunchKernelGGL(ln_bwd_cols_kernel, dim3((unsigned)cdiv<size_t>(n, 64), splits), dim3(64 * kLnColsWaves), 0,
                         dev->stream, n, bd, per_split, x, dEdf, stats, dg ? part_dg : nullptr, db ? part_db : nullptr);
      DYHIP_CHECK_LAUNCH();
      if (dg && db) launch_combine(dev, n, splits, part_dg, dg, part_db, db, 1);
      else if (dg) launch_combine(dev, n, splits, part_dg, dg, nullptr, nullptr, 1);
      else launch_combine(dev, n, splits, part_db, db, nullptr, nullptr, 1);
      DYHIP_CHECK_LAUNCH();
    }
  }
  return DYHIP_OK;
}

}  // extern "C"
