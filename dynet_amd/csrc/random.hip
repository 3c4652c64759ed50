// Random tensors: TensorTools::randomize_{uniform,normal,bernoulli} (dynet/tensor.cc:261-303),
// Device_GPU::reset_rng (dynet/devices.cc:130-135) and the Dropout node
// (dynet/nodes-dropout.cc:32-47).
//
// The reference's GPU generator is cuRAND's Philox4x32-10 keyed with seed + 1.  This file
// is the same counter-based generator written out: element k of a call is word k % 4 of
// Philox(counter = {lo, hi, queue, 0}, key = {seed + 1, 0}) with the 64-bit block number
// (hi:lo) = next + k / 4, where `next` is the generator's position.  Key and position
// live in device memory and a one-thread kernel advances the position after every call,
// so a captured graph draws fresh numbers on every replay and the host never has to be
// in the loop.  Being counter-based, any element can be recomputed on the host from
// (seed, position, k): masks are reproducible host <-> device bit for bit.
//
// Conversions follow cuRAND's: u = x * 2^-32 + 2^-33 in (0, 1]; Bernoulli as the reference
// forms it, floor(u + p) * scale (dynet/tensor.cc:446-448,270-272); normals by Box-Muller
// on consecutive word pairs (sin first).
#include "common.h"

namespace dyhip {

constexpr int kRngThreads = 256;

struct U4 {
  uint32_t v[4];
};

__device__ __forceinline__ U4 philox4x32_10(uint64_t block, uint32_t queue, uint64_t key) {
  uint32_t c0 = uint32_t(block), c1 = uint32_t(block >> 32), c2 = queue, c3 = 0;
  uint32_t k0 = uint32_t(key), k1 = uint32_t(key >> 32);
#pragma unroll
  for (int r = 0; r < 10; ++r) {
    const uint64_t p0 = uint64_t(0xD2511F53u) * c0, p1 = uint64_t(0xCD9E8D57u) * c2;
    const uint32_t n0 = uint32_t(p1 >> 32) ^ c1 ^ k0, n2 = uint32_t(p0 >> 32) ^ c3 ^ k1;
    c1 = uint32_t(p1);
    c3 = uint32_t(p0);
    c0 = n0;
    c2 = n2;
    k0 += 0x9E3779B9u;
    k1 += 0xBB67AE85u;
  }
  return U4{{c0, c1, c2, c3}};
}

__device__ __forceinline__ float unit_float(uint32_t x) {  // (0, 1]
  return float(x) * 2.3283064365386963e-10f + 1.1641532182693481e-10f;
}

enum { kUniform = 0, kBernoulli = 1, kNormal = 2, kDropout = 3 };

// One thread per Philox block = 4 consecutive elements.
//   kUniform  : out = u * a + b           (a = right - left, b = left; skipped for (1, 0))
//   kBernoulli: out = floor(u + a) * b    (a = p, b = scale)
//   kNormal   : out = z * a + b           (a = stddev, b = mean)
//   kDropout  : mask = floor(u + a) * b, out = x * mask
template <int DIST>
__global__ __launch_bounds__(kRngThreads) void rng_fill_kernel(size_t n, const uint64_t* __restrict__ state,
                                                               uint32_t queue, float a, float b,
                                                               const float* __restrict__ x, float* __restrict__ mask,
                                                               float* __restrict__ out) {
  const size_t blk = size_t(blockIdx.x) * kRngThreads + threadIdx.x;
  if (blk * 4 >= n) return;
  const U4 r = philox4x32_10(state[1] + blk, queue, state[0]);
  float v[4];
  if (DIST == kNormal) {
#pragma unroll
    for (int h = 0; h < 2; ++h) {
      const float u = unit_float(r.v[2 * h]);
      const float ang = float(r.v[2 * h + 1]) * 1.4629180792671596e-9f + 7.3145903963357980e-10f;  // 2 pi * (0, 1]
      const float s = sqrtf(-2.0f * logf(u));
      v[2 * h] = s * sinf(ang) * a + b;
      v[2 * h + 1] = s * cosf(ang) * a + b;
    }
  } else {
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const float u = unit_float(r.v[e]);
      if (DIST == kUniform)
        v[e] = (a == 1.0f && b == 0.0f) ? u : u * a + b;
      else
        v[e] = floorf(u + a) * b;
    }
  }
  const size_t k = blk * 4;
  const bool whole = k + 4 <= n;
  if (DIST == kDropout) {
    // 128-bit accesses when the three tensors allow it (twelve scalar accesses a thread ran at 3.1 TB/s: 16.2 us for
    // 4M elements)
    if (whole && ((reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(mask) | reinterpret_cast<uintptr_t>(out)) & 15u) == 0) {
      const float4 xv = *reinterpret_cast<const float4*>(x + k);
      *reinterpret_cast<float4*>(mask + k) = make_float4(v[0], v[1], v[2], v[3]);
      *reinterpret_cast<float4*>(out + k) = make_float4(xv.x * v[0], xv.y * v[1], xv.z * v[2], xv.w * v[3]);
      return;
    }
#pragma unroll
    for (int e = 0; e < 4; ++e)
      if (whole || k + e < n) {
        mask[k + e] = v[e];
        out[k + e] = x[k + e] * v[e];
      }
  } else if (whole && aligned16(out)) {
    *reinterpret_cast<float4*>(out + k) = make_float4(v[0], v[1], v[2], v[3]);
  } else {
#pragma unroll
    for (int e = 0; e < 4; ++e)
      if (k + e < n) out[k + e] = v[e];
  }
}

__global__ void rng_advance_kernel(uint64_t* state, uint64_t blocks) { state[1] += blocks; }

template <int DIST>
static int fill(dyhip_device* dev, size_t n, float a, float b, const float* x, float* mask, float* out) {
  if (n == 0) return DYHIP_OK;
  const size_t blocks4 = cdiv<size_t>(n, 4);
  DYHIP_REQUIRE(cdiv<size_t>(blocks4, kRngThreads) <= 0x7fffffffu, "random tensor of %zu elements is too large", n);
  hipLaunchKernelGGL(rng_fill_kernel<DIST>, dim3(unsigned(cdiv<size_t>(blocks4, kRngThreads))), dim3(kRngThreads), 0,
                     dev->stream, n, dev->rng_state, dev->rng_stream, a, b, x, mask, out);
  DYHIP_CHECK_LAUNCH();
  hipLaunchKernelGGL(rng_advance_kernel, dim3(1), dim3(1), 0, dev->stream, dev->rng_state, uint64_t(blocks4));
  DYHIP_CHECK_LAUNCH();
  return DYHIP_OK;
}

}  // namespace dyhip

using namespace dyhip;

extern "C" {

int dyhip_reset_rng(dyhip_device* dev, unsigned seed) {
  DYHIP_CHECK_DEV(dev);
  DYHIP_CHECK_HIP(hipSetDevice(dev->ordinal));
  const uint64_t st[2] = {uint64_t(seed) + 1, 0};
  DYHIP_CHECK_HIP(hipStreamSynchronize(dev->stream));
  DYHIP_CHECK_HIP(hipMemcpy(dev->rng_state, st, sizeof(st), hipMemcpyHostToDevice));
  for (dyhip_device* q : dev->forks) {
    DYHIP_CHECK_HIP(hipStreamSynchronize(q->stream));
    DYHIP_CHECK_HIP(hipMemcpy(q->rng_state, st, sizeof(st), hipMemcpyHostToDevice));
  }
  return DYHIP_OK;
}

int dyhip_rng_state(dyhip_device* dev, unsigned long long* key, unsigned long long* position, unsigned* queue) {
  DYHIP_CHECK_DEV(dev);
  DYHIP_REQUIRE(key && position && queue, "null output pointer");
  uint64_t st[2];
  DYHIP_CHECK_HIP(hipStreamSynchronize(dev->stream));
  DYHIP_CHECK_HIP(hipMemcpy(st, dev->rng_state, sizeof(st), hipMemcpyDeviceToHost));
  *key = st[0];
  *position = st[1];
  *queue = dev->rng_stream;
  return DYHIP_OK;
}

int dyhip_rng_set_position(dyhip_device* dev, unsigned long long position) {
  DYHIP_CHECK_DEV(dev);
  const uint64_t pos = position;
  DYHIP_CHECK_HIP(hipStreamSynchronize(dev->stream));
  DYHIP_CHECK_HIP(hipMemcpy(dev->rng_state + 1, &pos, sizeof(pos), hipMemcpyHostToDevice));
  return DYHIP_OK;
}

int dyhip_randomize_uniform(dyhip_device* dev, size_t n, float left, float right, float* out) {
  DYHIP_CHECK_DEV(dev);
  DYHIP_REQUIRE(n == 0 || out, "randomize_uniform: null tensor pointer");
  return fill<kUniform>(dev, n, right - left, left, nullptr, nullptr, out);
}

int dyhip_randomize_bernoulli(dyhip_device* dev, size_t n, float p, float scale, float* out) {
  DYHIP_CHECK_DEV(dev);
  DYHIP_REQUIRE(n == 0 || out, "randomize_bernoulli: null tensor pointer");
  DYHIP_REQUIRE(p >= 0.f && p <= 1.f, "randomize_bernoulli: p = %g is not a probability", double(p));
  return fill<kBernoulli>(dev, n, p, scale, nullptr, nullptr, out);
}

int dyhip_randomize_normal(dyhip_device* dev, size_t n, float mean, float stddev, float* out) {
  DYHIP_CHECK_DEV(dev);
  DYHIP_REQUIRE(n == 0 || out, "randomize_normal: null tensor pointer");
  return fill<kNormal>(dev, n, stddev, mean, nullptr, nullptr, out);
}

int dyhip_dropout_forward(dyhip_device* dev, size_t n, float p, const float* x, float* mask, float* fx) {
  DYHIP_CHECK_DEV(dev);
  DYHIP_REQUIRE(n == 0 || (x && mask && fx), "Dropout: null tensor pointer");
  DYHIP_REQUIRE(p >= 0.f && p < 1.f, "Dropout: drop probability %g outside [0, 1)", double(p));
  return fill<kDropout>(dev, n, 1.f - p, 1.f / (1.f - p), x, mask, fx);
}

int dyhip_dropout_backward(dyhip_device* dev, size_t n, const float* mask, const float* dEdf, float* dEdxi) {
  // dEdxi += dEdf (.) mask: the first-argument gradient of a componentwise product with the mask
  DYHIP_REQUIRE(n == 0 || (mask && dEdf && dEdxi), "Dropout: null tensor pointer");
  return dyhip_cmult_backward(dev, n, 1, 1, mask, mask, dEdf, 0, dEdxi, nullptr, 0);
}

}  // extern "C"
