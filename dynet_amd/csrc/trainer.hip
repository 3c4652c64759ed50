// Trainer kernels: gradient clipping scale on the device, the SimpleSGD rule with a
// device-resident scale, and the sparse (touched rows only) lookup update.
//
// Replaces Trainer::clip_gradients / gradient_l2_norm (dynet/training.cc:173-187,
// dynet/model.cc:806-848: one device malloc, one blocking device-to-host float copy
// and one free per parameter per update), SimpleSGDTrainer::update_rule_dev
// (dynet/training.cc:619-622), the per-row lookup updates of dynet/training.cc:215-226
// and LookupParameterStorage::clear, which on the GPU zeroes the whole gradient table
// (dynet/model.cc:175-186).
#include "common.h"

namespace dyhip {

static size_t align256(size_t n) { return (n + 255) / 256 * 256; }

// With clipping enabled (threshold > 0), a gradient norm that is NaN or infinite gives scale 0, which the update
// kernels below read as "leave the parameters alone": Trainer::clip_gradients throws in that case
// (dynet/training.cc:176-180), a kernel cannot, so the step is skipped on the device and the norm slot lets the host
// raise the error when it looks.  With clipping disabled the reference neither looks at the norm nor throws
// (dynet/training.cc:174 returns 1 before the check): the scale is 1 whatever the norm, as there.
__global__ void clip_scale_kernel(unsigned n, const float* __restrict__ sqnorms, float threshold,
                                  float* __restrict__ gscale, float* __restrict__ norm) {
  if (threadIdx.x != 0 || blockIdx.x != 0) return;
  float s = 0.f;
  for (unsigned i = 0; i < n; ++i) s += sqnorms[i];
  const float gg = sqrtf(s);
  const bool finite = gg - gg == 0.f;
  *gscale = !(threshold > 0.f) ? 1.0f : !finite ? 0.0f : gg > threshold ? threshold / gg : 1.0f;
  if (norm != nullptr) *norm = gg;
}

// p -= (lr * gscale / wd) * g over one slab, optionally clearing g in the same pass.  Four 128-bit groups per thread
// and array in flight; streaming accesses when the slab is far larger than the caches (it is read and written once).
template <bool CLEAR, bool NT>
__global__ __launch_bounds__(256) void sgd_scaled_kernel(size_t n4, size_t n, float* __restrict__ p,
                                                         float* __restrict__ g, float lr, float wd,
                                                         const float* __restrict__ gscale) {
  constexpr int U = 4;
  const float gs = *gscale;
  const bool skip = gs == 0.f;  // non-finite gradient norm: the parameters stay as they are
  const float s = lr * gs / wd;
  float4* p4 = reinterpret_cast<float4*>(p);
  float4* g4 = reinterpret_cast<float4*>(g);
  const float4 zero = make_float4(0.f, 0.f, 0.f, 0.f);
  const size_t chunks = n4 / (256 * U);  // whole chunks of 256 * U groups, dealt to the blocks in turn
  for (size_t c = blockIdx.x; c < chunks; c += gridDim.x) {
    const size_t i = c * (256 * U) + threadIdx.x;
    if (!skip) {
      float4 pv[U], gv[U];
#pragma unroll
      for (int u = 0; u < U; ++u) {
        pv[u] = ldg4<NT>(p4 + i + 256 * u);
        gv[u] = ldg4<NT>(g4 + i + 256 * u);
      }
#pragma unroll
      for (int u = 0; u < U; ++u) {
        pv[u].x -= gv[u].x * s;
        pv[u].y -= gv[u].y * s;
        pv[u].z -= gv[u].z * s;
        pv[u].w -= gv[u].w * s;
        stg4<NT>(p4 + i + 256 * u, pv[u]);
      }
    }
    if (CLEAR) {
#pragma unroll
      for (int u = 0; u < U; ++u) stg4<NT>(g4 + i + 256 * u, zero);
    }
  }
  for (size_t i = chunks * (256 * U) + size_t(blockIdx.x) * 256 + threadIdx.x; i < n4; i += size_t(gridDim.x) * 256) {
    if (!skip) {
      float4 pv = p4[i];
      const float4 gv = g4[i];
      pv.x -= gv.x * s;
      pv.y -= gv.y * s;
      pv.z -= gv.z * s;
      pv.w -= gv.w * s;
      p4[i] = pv;
    }
    if (CLEAR) g4[i] = zero;
  }
  for (size_t k = (n4 << 2) + size_t(blockIdx.x) * 256 + threadIdx.x; k < n; k += size_t(gridDim.x) * 256) {
    if (!skip) p[k] -= g[k] * s;
    if (CLEAR) g[k] = 0.f;
  }
}

// The entries of a lookup plan (lookup.hip): one 16-byte record per grouped position, .x = id (ids >= vocab replaced
// by vocab), .z = entries of its run before it (0 at the head of a run).
// One block per grouped position; only the first entry of each run of equal ids acts.
__global__ __launch_bounds__(128) void sgd_rows_kernel(unsigned n, const uint4* __restrict__ entries,
                                                       unsigned dim, unsigned vocab, float* __restrict__ values,
                                                       float* __restrict__ grads, float lr, float wd,
                                                       const float* __restrict__ gscale) {
  const unsigned k = blockIdx.x;
  const uint4 e = entries[k];
  const unsigned id = e.x;
  if (id >= vocab || e.z != 0) return;
  const float gs = *gscale;
  const float s = lr * gs / wd;
  float* pv = values + size_t(id) * dim;
  float* pg = grads + size_t(id) * dim;
  for (unsigned j = threadIdx.x; j < dim; j += 128) {
    if (gs != 0.f) pv[j] -= pg[j] * s;
    pg[j] = 0.f;
  }
}

__global__ __launch_bounds__(128) void sqnorm_rows_kernel(unsigned n, const uint4* __restrict__ entries,
                                                          unsigned dim, unsigned vocab,
                                                          const float* __restrict__ grads,
                                                          float* __restrict__ partial) {
  __shared__ float red[2];
  const unsigned k = blockIdx.x;
  const uint4 e = entries[k];
  const unsigned id = e.x;
  const bool head = id < vocab && e.z == 0;
  float s = 0.f;
  if (head) {
    const float* pg = grads + size_t(id) * dim;
    for (unsigned j = threadIdx.x; j < dim; j += 128) s += pg[j] * pg[j];
  }
  const float t = block_sum<2>(s, red);
  if (threadIdx.x == 0) partial[k] = t;
}

__global__ __launch_bounds__(256) void sum_partials_kernel(unsigned n, const float* __restrict__ partial,
                                                           float* __restrict__ out) {
  __shared__ float red[4];
  float s = 0.f;
  for (unsigned i = threadIdx.x; i < n; i += 256) s += partial[i];
  const float t = block_sum<4>(s, red);
  if (threadIdx.x == 0) *out = t;
}

}  // namespace dyhip

using namespace dyhip;

extern "C" {

int dyhip_clip_scale_norm(dyhip_device* dev, unsigned n, const float* sqnorms, float threshold, float* gscale,
                          float* norm) {
  DYHIP_CHECK_DEV(dev);
  DYHIP_REQUIRE(gscale != nullptr && (n == 0 || sqnorms != nullptr), "null pointer");
  hipLaunchKernelGGL(clip_scale_kernel, dim3(1), dim3(64), 0, dev->stream, n, sqnorms, threshold, gscale, norm);
  DYHIP_CHECK_LAUNCH();
  return DYHIP_OK;
}

int dyhip_clip_scale(dyhip_device* dev, unsigned n, const float* sqnorms, float threshold, float* gscale) {
  return dyhip_clip_scale_norm(dev, n, sqnorms, threshold, gscale, nullptr);
}

int dyhip_sgd_update_scaled(dyhip_device* dev, size_t n, float* p, float* g, float lr, const float* gscale,
                            float wd, int clear_grad) {
  DYHIP_CHECK_DEV(dev);
  if (n == 0) return DYHIP_OK;
  DYHIP_REQUIRE(p && g && gscale, "null pointer");
  DYHIP_REQUIRE(wd != 0.f, "weight decay scale must be non-zero");
  const bool vec = aligned16(p) && aligned16(g);
  const size_t n4 = vec ? n / 4 : 0;
  // a block takes whole chunks of 256 x 4 groups in turn: as many blocks as give each the same number of chunks
  const size_t chunks = cdiv<size_t>(n, size_t(256) * 16), per = cdiv<size_t>(chunks, 2048);
  const unsigned blocks = static_cast<unsigned>(cdiv<size_t>(chunks, per));
  const bool nt = n * sizeof(float) >= dev->stream_threshold;
#define DYHIP_SGD(CLEAR, NT) \
  hipLaunchKernelGGL((sgd_scaled_kernel<CLEAR, NT>), dim3(blocks), dim3(256), 0, dev->stream, n4, n, p, g, lr, wd, gscale)
  if (clear_grad) {
    if (nt) DYHIP_SGD(true, true);
    else DYHIP_SGD(true, false);
  } else {
    if (nt) DYHIP_SGD(false, true);
    else DYHIP_SGD(false, false);
  }
#undef DYHIP_SGD
  DYHIP_CHECK_LAUNCH();
  return DYHIP_OK;
}

int dyhip_sgd_update_rows(dyhip_device* dev, unsigned n_ids, const void* plan, size_t dim, unsigned vocab,
                          float* values, float* grads, float lr, const float* gscale, float wd) {
  DYHIP_CHECK_DEV(dev);
  if (n_ids == 0 || dim == 0) return DYHIP_OK;
  DYHIP_REQUIRE(plan && values && grads && gscale, "null pointer");
  DYHIP_REQUIRE(wd != 0.f && dim < (size_t(1) << 31), "bad weight decay scale or dimension");
  hipLaunchKernelGGL(sgd_rows_kernel, dim3(n_ids), dim3(128), 0, dev->stream, n_ids,
                     static_cast<const uint4*>(plan), (unsigned)dim, vocab, values, grads, lr, wd, gscale);
  DYHIP_CHECK_LAUNCH();
  return DYHIP_OK;
}

int dyhip_squared_l2norm_rows_workspace(unsigned n_ids, size_t* ws_bytes) {
  DYHIP_REQUIRE(ws_bytes != nullptr, "null output pointer");
  *ws_bytes = align256(sizeof(float) * (n_ids ? n_ids : 1));
  return DYHIP_OK;
}

int dyhip_squared_l2norm_rows(dyhip_device* dev, unsigned n_ids, const void* plan, size_t dim, unsigned vocab,
                              const float* grads, float* out, void* ws, size_t ws_bytes) {
  DYHIP_CHECK_DEV(dev);
  DYHIP_REQUIRE(out != nullptr, "null pointer");
  if (n_ids == 0 || dim == 0) return dyhip_zero(dev, out, sizeof(float));
  DYHIP_REQUIRE(plan && grads, "null pointer");
  DYHIP_REQUIRE(ws != nullptr && ws_bytes >= sizeof(float) * n_ids, "squared_l2norm_rows needs %zu workspace bytes",
                sizeof(float) * n_ids);
  float* partial = static_cast<float*>(ws);
  hipLaunchKernelGGL(sqnorm_rows_kernel, dim3(n_ids), dim3(128), 0, dev->stream, n_ids,
                     static_cast<const uint4*>(plan), (unsigned)dim, vocab, grads, partial);
  hipLaunchKernelGGL(sum_partials_kernel, dim3(1), dim3(256), 0, dev->stream, n_ids, partial, out);
  DYHIP_CHECK_LAUNCH();
  return DYHIP_OK;
}

}  // extern "C"
