// The seven scatter/gather helpers of dynet::gpu (dynet/gpu-ops.h:9-15,
// gpu-ops.cu:12-166) with their original argument lists, and the squared-norm
// reduction the trainer's gradient clipping needs (dynet/model.cc:806-848).
//
// parallel_memcpy / parallel_accumulate move the ragged per-node tensors of the
// autobatching executor (dynet/exec.cc:298-411).  The reference maps thread ->
// sequence (id % num_seqs), so neighbouring lanes touch different sequences; here
// blockIdx.y is the sequence and lanes walk consecutive floats of it, with
// 128-bit accesses when both sides are 16-byte aligned.
#include "common.h"

namespace dyhip {

constexpr int kThreads = 256;

__global__ __launch_bounds__(kThreads) void d2s_assign_kernel(int n, const unsigned* __restrict__ idx,
                                                              const float* __restrict__ src, float* __restrict__ trg) {
  const int i = blockIdx.x * kThreads + threadIdx.x;
  if (i < n) trg[idx[i]] = src[i];
}

__global__ __launch_bounds__(kThreads) void s2d_assign_kernel(int n, const unsigned* __restrict__ idx,
                                                              const float* __restrict__ src, float* __restrict__ trg) {
  const int i = blockIdx.x * kThreads + threadIdx.x;
  if (i < n) trg[i] = src[idx[i]];
}

// duplicates in idx are legal, hence the atomic (as in the reference)
__global__ __launch_bounds__(kThreads) void d2s_subtract_kernel(int n, const unsigned* __restrict__ idx,
                                                                const float* __restrict__ src,
                                                                float* __restrict__ trg) {
  const int i = blockIdx.x * kThreads + threadIdx.x;
  if (i < n) atomicAdd(trg + idx[i], -src[i]);
}

// trg[i*bsize + j] = src[idx[i]*bsize + j] * mult : block.y = i, lanes walk j
__global__ __launch_bounds__(kThreads) void s2d_block_assign_mul_kernel(int n, int bsize,
                                                                        const unsigned* __restrict__ idx, float mult,
                                                                        const float* __restrict__ src,
                                                                        float* __restrict__ trg) {
  for (size_t i = blockIdx.y; i < size_t(n); i += gridDim.y) {  // the grid's second dimension holds at most 65535 blocks
    const float* ps = src + size_t(idx[i]) * bsize;
    float* pt = trg + i * bsize;
    for (int j = blockIdx.x * kThreads + threadIdx.x; j < bsize; j += gridDim.x * kThreads) pt[j] = ps[j] * mult;
  }
}

// trg[idx[i]*bsize + j] += src[i*bsize + j] with duplicates allowed: atomic, like
// the reference.  (LookupNode gradients use the deterministic sorted path of
// dyhip_lookup_accumulate_grads instead.)
__global__ __launch_bounds__(kThreads) void d2s_block_add_kernel(int n, int bsize, const unsigned* __restrict__ idx,
                                                                 const float* __restrict__ src,
                                                                 float* __restrict__ trg) {
  for (size_t i = blockIdx.y; i < size_t(n); i += gridDim.y) {
    const float* ps = src + i * bsize;
    float* pt = trg + size_t(idx[i]) * bsize;
    for (int j = blockIdx.x * kThreads + threadIdx.x; j < bsize; j += gridDim.x * kThreads) atomicAdd(pt + j, ps[j]);
  }
}

template <bool ACC>
__global__ __launch_bounds__(kThreads) void ragged_move_kernel(int num_seqs, float* const* __restrict__ src,
                                                               float* const* __restrict__ trg,
                                                               const size_t* __restrict__ len) {
  for (unsigned s = blockIdx.y; s < unsigned(num_seqs); s += gridDim.y) {
  const float* ps = src[s];
  float* pt = trg[s];
  const size_t n = len[s];
  const size_t stride = size_t(gridDim.x) * kThreads;
  const size_t t0 = size_t(blockIdx.x) * kThreads + threadIdx.x;
  if (!ACC && aligned16(ps) && aligned16(pt)) {
    const size_t n4 = n >> 2;
    const float4* s4 = reinterpret_cast<const float4*>(ps);
    float4* t4 = reinterpret_cast<float4*>(pt);
    for (size_t i = t0; i < n4; i += stride) t4[i] = s4[i];
    for (size_t i = (n4 << 2) + t0; i < n; i += stride) pt[i] = ps[i];
  } else {
    for (size_t i = t0; i < n; i += stride) {
      if (ACC)
        atomicAdd(pt + i, ps[i]);  // several sequences may target the same gradient buffer
      else
        pt[i] = ps[i];
    }
  }
  }
}

// Equal-length segments copied one behind the other: dst[s * len, (s + 1) * len) = src_s.  The segment addresses
// travel in the kernel's argument block, not in a device table, so the call needs no staging copy, no synchronisation
// and may be recorded into a graph.  blockIdx.y = segment; a tile of 256 x 4 groups of four floats per block, all its
// loads issued before the first store.
constexpr int kGatherSegs = 32;
struct GatherArgs {
  const float* src[kGatherSegs];
};

template <bool VEC, bool NT>
__global__ __launch_bounds__(kThreads) void gather_segments_kernel(GatherArgs a, size_t len, float* __restrict__ dst) {
  const float* ps = a.src[blockIdx.y];
  float* pt = dst + size_t(blockIdx.y) * len;
  if (VEC) {
    const size_t n4 = len >> 2;
    const float4* s4 = reinterpret_cast<const float4*>(ps);
    float4* t4 = reinterpret_cast<float4*>(pt);
    const size_t i0 = size_t(blockIdx.x) * (kThreads * 4) + threadIdx.x;
    float4 v[4];
#pragma unroll
    for (int u = 0; u < 4; ++u) v[u] = ldg4<NT>(s4 + min(i0 + size_t(u) * kThreads, n4 - 1));
#pragma unroll
    for (int u = 0; u < 4; ++u)
      if (i0 + size_t(u) * kThreads < n4) stg4<NT>(t4 + i0 + size_t(u) * kThreads, v[u]);
  } else {
    for (size_t i = size_t(blockIdx.x) * (kThreads * 16) + threadIdx.x, e = min(len, (size_t(blockIdx.x) + 1) * (kThreads * 16));
         i < e; i += kThreads)
      pt[i] = ps[i];
  }
}

// stage 1: per-block partial of sum g^2 ; stage 2: one block adds the partials in order
// partial[block] = sum of squares of the block's share.  The 16-byte aligned middle of the array goes through
// 128-bit loads, four in flight per thread (plain ones: the update that follows reads the same gradient); the few floats before and after it are added by block 0.
__global__ __launch_bounds__(kThreads) void sqnorm_partial_kernel(size_t n, const float* __restrict__ g,
                                                                  float* __restrict__ partial) {
  __shared__ float red[4];
  const size_t head = min(n, (size_t(4) - ((reinterpret_cast<uintptr_t>(g) >> 2) & 3u)) & 3u);  // floats before alignment
  const size_t n4 = (n - head) / 4;
  const float4* g4 = reinterpret_cast<const float4*>(g + head);
  float s = 0.f;
  const size_t stride = size_t(gridDim.x) * kThreads;
  size_t i = size_t(blockIdx.x) * kThreads + threadIdx.x;
  for (; i + 3 * stride < n4; i += 4 * stride) {
    const float4 a = ldg4<false>(g4 + i), b = ldg4<false>(g4 + i + stride), c = ldg4<false>(g4 + i + 2 * stride),
                 d = ldg4<false>(g4 + i + 3 * stride);
    s += ((a.x * a.x + a.y * a.y) + (a.z * a.z + a.w * a.w)) + ((b.x * b.x + b.y * b.y) + (b.z * b.z + b.w * b.w));
    s += ((c.x * c.x + c.y * c.y) + (c.z * c.z + c.w * c.w)) + ((d.x * d.x + d.y * d.y) + (d.z * d.z + d.w * d.w));
  }
  for (; i < n4; i += stride) {
    const float4 a = ldg4<false>(g4 + i);
    s += (a.x * a.x + a.y * a.y) + (a.z * a.z + a.w * a.w);
  }
  if (blockIdx.x == 0) {
    const size_t tail0 = head + 4 * n4;
    for (size_t j = threadIdx.x; j < head; j += kThreads) s += g[j] * g[j];
    for (size_t j = tail0 + threadIdx.x; j < n; j += kThreads) s += g[j] * g[j];
  }
  const float t = block_sum<4>(s, red);
  if (threadIdx.x == 0) partial[blockIdx.x] = t;
}

__global__ __launch_bounds__(kThreads) void sqnorm_final_kernel(unsigned nparts, const float* __restrict__ partial,
                                                                float* __restrict__ out) {
  __shared__ float red[4];
  float s = 0.f;
  for (unsigned i = threadIdx.x; i < nparts; i += kThreads) s += partial[i];
  const float t = block_sum<4>(s, red);
  if (threadIdx.x == 0) *out = t;
}

constexpr unsigned kSqnormBlocks = 1024;

static unsigned grid1d(int n) { return static_cast<unsigned>((n + kThreads - 1) / kThreads); }

}  // namespace dyhip

using namespace dyhip;

extern "C" {

int dyhip_dense_to_sparse_assign(dyhip_device* dev, int n, const unsigned* ids, const float* src, float* trg) {
  DYHIP_CHECK_DEV(dev);
  if (n <= 0) return DYHIP_OK;
  DYHIP_REQUIRE(ids && src && trg, "null pointer");
  hipLaunchKernelGGL(d2s_assign_kernel, dim3(grid1d(n)), dim3(kThreads), 0, dev->stream, n, ids, src, trg);
  DYHIP_CHECK_LAUNCH();
  return DYHIP_OK;
}

int dyhip_sparse_to_dense_assign(dyhip_device* dev, int n, const unsigned* ids, const float* src, float* trg) {
  DYHIP_CHECK_DEV(dev);
  if (n <= 0) return DYHIP_OK;
  DYHIP_REQUIRE(ids && src && trg, "null pointer");
  hipLaunchKernelGGL(s2d_assign_kernel, dim3(grid1d(n)), dim3(kThreads), 0, dev->stream, n, ids, src, trg);
  DYHIP_CHECK_LAUNCH();
  return DYHIP_OK;
}

int dyhip_dense_to_sparse_subtract(dyhip_device* dev, int n, const unsigned* ids, const float* src, float* trg) {
  DYHIP_CHECK_DEV(dev);
  if (n <= 0) return DYHIP_OK;
  DYHIP_REQUIRE(ids && src && trg, "null pointer");
  hipLaunchKernelGGL(d2s_subtract_kernel, dim3(grid1d(n)), dim3(kThreads), 0, dev->stream, n, ids, src, trg);
  DYHIP_CHECK_LAUNCH();
  return DYHIP_OK;
}

int dyhip_sparse_to_dense_block_assign_and_multiply(dyhip_device* dev, int n, const unsigned* idx, int bsize,
                                                    float mult, const float* src, float* trg) {
  DYHIP_CHECK_DEV(dev);
  if (n <= 0 || bsize <= 0) return DYHIP_OK;
  DYHIP_REQUIRE(idx && src && trg, "null pointer");
  unsigned gx = grid1d(bsize);
  if (gx > 64) gx = 64;
  hipLaunchKernelGGL(s2d_block_assign_mul_kernel, dim3(gx, n < 65535 ? n : 65535), dim3(kThreads), 0, dev->stream, n,
                     bsize, idx, mult, src, trg);
  DYHIP_CHECK_LAUNCH();
  return DYHIP_OK;
}

int dyhip_dense_to_sparse_block_add(dyhip_device* dev, int n, const unsigned* ids, int bsize, const float* src,
                                    float* trg) {
  DYHIP_CHECK_DEV(dev);
  if (n <= 0 || bsize <= 0) return DYHIP_OK;
  DYHIP_REQUIRE(ids && src && trg, "null pointer");
  unsigned gx = grid1d(bsize);
  if (gx > 64) gx = 64;
  hipLaunchKernelGGL(d2s_block_add_kernel, dim3(gx, n < 65535 ? n : 65535), dim3(kThreads), 0, dev->stream, n, bsize, ids,
                     src, trg);
  DYHIP_CHECK_LAUNCH();
  return DYHIP_OK;
}

static int ragged_move(dyhip_device* dev, bool acc, int num_seqs, int max_len, float** src, float** trg, size_t* len) {
  DYHIP_CHECK_DEV(dev);
  if (num_seqs <= 0 || max_len <= 0) return DYHIP_OK;
  DYHIP_REQUIRE(src && trg && len, "null pointer");
  unsigned gx = static_cast<unsigned>((size_t(max_len) + size_t(kThreads) * 4 - 1) / (size_t(kThreads) * 4));
  if (gx < 1) gx = 1;
  if (gx > 256) gx = 256;
  if (acc)
    hipLaunchKernelGGL(ragged_move_kernel<true>, dim3(gx, num_seqs < 65535 ? num_seqs : 65535), dim3(kThreads), 0,
                       dev->stream, num_seqs, src, trg, len);
  else
    hipLaunchKernelGGL(ragged_move_kernel<false>, dim3(gx, num_seqs < 65535 ? num_seqs : 65535), dim3(kThreads), 0,
                       dev->stream, num_seqs, src, trg, len);
  DYHIP_CHECK_LAUNCH();
  return DYHIP_OK;
}

int dyhip_parallel_memcpy(dyhip_device* dev, int num_seqs, int max_len, float** src, float** trg, size_t* len) {
  return ragged_move(dev, false, num_seqs, max_len, src, trg, len);
}

int dyhip_parallel_accumulate(dyhip_device* dev, int num_seqs, int max_len, float** src, float** trg, size_t* len) {
  return ragged_move(dev, true, num_seqs, max_len, src, trg, len);
}

int dyhip_gather_segments(dyhip_device* dev, unsigned n_seg, size_t len, const float* const* src_host, float* dst) {
  DYHIP_CHECK_DEV(dev);
  if (n_seg == 0 || len == 0) return DYHIP_OK;
  DYHIP_REQUIRE(src_host != nullptr && dst != nullptr, "null pointer in gather_segments");
  DYHIP_REQUIRE(len < (size_t(1) << 40), "segment too long");
  bool vec = len % 4 == 0 && aligned16(dst);
  for (unsigned s2 = 0; s2 < n_seg; ++s2) {
    DYHIP_REQUIRE(src_host[s2] != nullptr, "null segment %u in gather_segments", s2);
    vec = vec && aligned16(src_host[s2]);
  }
  const bool nt = size_t(n_seg) * len * sizeof(float) >= dev->stream_threshold;
  const unsigned gx = static_cast<unsigned>(cdiv<size_t>(len, size_t(kThreads) * 16));
  for (unsigned s0 = 0; s0 < n_seg; s0 += kGatherSegs) {
    const unsigned cnt = n_seg - s0 < unsigned(kGatherSegs) ? n_seg - s0 : unsigned(kGatherSegs);
    GatherArgs a;
    for (unsigned k = 0; k < unsigned(kGatherSegs); ++k) a.src[k] = src_host[s0 + (k < cnt ? k : 0)];
    float* out = dst + size_t(s0) * len;
    const dim3 grid(gx, cnt), block(kThreads);
    if (vec && nt) hipLaunchKernelGGL((gather_segments_kernel<true, true>), grid, block, 0, dev->stream, a, len, out);
    else if (vec) hipLaunchKernelGGL((gather_segments_kernel<true, false>), grid, block, 0, dev->stream, a, len, out);
    else hipLaunchKernelGGL((gather_segments_kernel<false, false>), grid, block, 0, dev->stream, a, len, out);
    DYHIP_CHECK_LAUNCH();
  }
  return DYHIP_OK;
}

int dyhip_squared_l2norm_workspace(size_t n, size_t* ws_bytes) {
  DYHIP_REQUIRE(ws_bytes != nullptr, "null output pointer");
  (void)n;
  *ws_bytes = kSqnormBlocks * sizeof(float);
  return DYHIP_OK;
}

int dyhip_squared_l2norm(dyhip_device* dev, size_t n, const float* g, float* out, void* ws, size_t ws_bytes) {
  DYHIP_CHECK_DEV(dev);
  DYHIP_REQUIRE(out != nullptr && (n == 0 || g != nullptr), "null pointer");
  DYHIP_REQUIRE(ws != nullptr && ws_bytes >= kSqnormBlocks * sizeof(float), "squared_l2norm needs %zu workspace bytes",
                kSqnormBlocks * sizeof(float));
  unsigned blocks = static_cast<unsigned>((n + size_t(kThreads) * 16 - 1) / (size_t(kThreads) * 16));
  if (blocks < 1) blocks = 1;
  if (blocks > kSqnormBlocks) blocks = kSqnormBlocks;
  float* partial = static_cast<float*>(ws);
  hipLaunchKernelGGL(sqnorm_partial_kernel, dim3(blocks), dim3(kThreads), 0, dev->stream, n, g, partial);
  hipLaunchKernelGGL(sqnorm_final_kernel, dim3(1), dim3(kThreads), 0, dev->stream, blocks, partial, out);
  DYHIP_CHECK_LAUNCH();
  return DYHIP_OK;
}

}  // extern "C"
