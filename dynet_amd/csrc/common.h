// Shared internals of libdynet_hip.so: status/error plumbing, the device and
// pool objects behind the opaque C handles, and wavefront-level primitives.
#pragma once

#include <hip/hip_runtime.h>

#include <cstdarg>
#include <cstddef>
#include <cstdint>
#include <string>
#include <vector>

#include "dynet_hip.h"

namespace dyhip {

int fail(int code, const char* fmt, ...) __attribute__((format(printf, 2, 3)));

constexpr int kWave = 64;  // CDNA wavefront width
constexpr unsigned kGemmFlagWords = 1024;  // per queue: one flag per segment of the 256x256-tile GEMM + a counter

// ceil(a / b) for positive integers
template <class T>
constexpr T cdiv(T a, T b) {
  return (a + b - 1) / b;
}

__host__ __device__ inline bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

// ---- allocators (MemAllocator of the reference: align, malloc, free, zero) --
struct MemAllocator {
  explicit MemAllocator(size_t align) : align(align) {}
  virtual ~MemAllocator() {}
  virtual void* malloc(size_t n) = 0;
  virtual void free(void* p) = 0;
  virtual bool zero(void* p, size_t n) = 0;
  size_t round_up_align(size_t n) const { return align < 2 ? n : ((n + align - 1) / align) * align; }
  const size_t align;
  const char* refusal = nullptr;  // set by malloc when it declines for a reason other than exhaustion
};

}  // namespace dyhip

// One growable bump-allocated region set: a list of blocks, allocation only
// from the newest block, consolidation on free().
struct dyhip_pool {
  struct Block {
    char* mem;
    size_t capacity;
    size_t used;
  };
  std::string name;
  std::vector<Block> blocks;
  size_t cap;             // sum of block capacities
  size_t expanding_unit;  // growth granularity (1 << 24 in the reference)
  dyhip::MemAllocator* alloc;
  bool owns_alloc;
};

struct dyhip_device {
  int ordinal;
  int num_cus;
  size_t max_lds_per_block;  // what a block may opt in to (dynamic LDS); 0 if unknown
  hipStream_t stream;
  dyhip::MemAllocator* alloc;
  dyhip_pool* pools[4];
  float* scalars;  // device: {-1, 1, 0}
  size_t stream_threshold;  // tensors at least this large are accessed with streaming (non-temporal) hints
  void* gemm_ws;   // split-K partial tiles (the analogue of a BLAS handle's workspace)
  size_t gemm_ws_bytes;
  unsigned wide_gemm_ready;  // gemm_wide.hip: kernels whose dynamic-LDS limit has been raised on this device
  unsigned* gemm_flags;      // gemm_wide.hip: kGemmFlagWords words behind gemm_ws that no other kernel touches, zero between launches
  bool gemm_flags_used;      // a launch since the last host synchronisation may have counted a wait that gave up
  unsigned gemm_spin_limit;  // polls before a block's wait for another block's partial tile gives up
  int gemm_raise_flags;      // 0 only in tests of the give-up path: producers leave their flags down
  hipEvent_t ev_start, ev_stop;
  dyhip_device* parent;                // non-null for a forked queue: pools, scalars and allocator belong to the parent
  std::vector<hipEvent_t> sync_events; // ring of events recorded on this queue for dyhip_device_wait
  size_t sync_next;
  std::vector<dyhip_device*> forks;    // live forked queues (destroyed with the device if still alive)
  uint64_t* rng_state;                 // device: {Philox key, next counter}; one per queue, see random.hip
  uint32_t rng_stream;                 // third counter word: 0 for the device, 1.. for its forked queues
  uint32_t forks_made;                 // forked queues created so far (numbers their random streams)
  void* ln_scratch;                    // this GPU's copy of the static scratch array of dyhip_layer_norm_backward_static
};

namespace dyhip {
// reduce.hip: looks up, on the current device, the address of the static scratch array (once per device handle)
int ln_static_scratch_setup(dyhip_device* dev);
// device.hip: after a host synchronisation of dev's stream, reports waits that gave up inside a large GEMM
int gemm_check_giveups(dyhip_device* dev);
}  // namespace dyhip

struct dyhip_graph {
  hipGraph_t graph;
  hipGraphExec_t exec;
};

#define DYHIP_CHECK_HIP(expr)                                                                   \
  do {                                                                                          \
    hipError_t e_ = (expr);                                                                     \
    if (e_ != hipSuccess)                                                                       \
      return dyhip::fail(DYHIP_ERR_RUNTIME, "%s failed: %s (%s:%d)", #expr, hipGetErrorString(e_), \
                         __FILE__, __LINE__);                                                   \
  } while (0)

#define DYHIP_REQUIRE(cond, ...)                                          \
  do {                                                                    \
    if (!(cond)) return dyhip::fail(DYHIP_ERR_INVALID_ARG, __VA_ARGS__);  \
  } while (0)

#define DYHIP_CHECK_DEV(dev)                                                      \
  do {                                                                            \
    if ((dev) == nullptr) return dyhip::fail(DYHIP_ERR_INVALID_ARG, "null device handle"); \
  } while (0)

#define DYHIP_CHECK_LAUNCH() DYHIP_CHECK_HIP(hipGetLastError())

#define DYHIP_CHECK_STATUS(expr) \
  do {                           \
    int s_ = (expr);             \
    if (s_ != DYHIP_OK) return s_; \
  } while (0)

#ifdef __HIPCC__
namespace dyhip {

// ---- streaming (non-temporal) global accesses ------------------------------------
// Tensors far larger than the 4 MB per-XCD L2 are read once and written once by
// these kernels; marking those accesses non-temporal keeps them from displacing
// each other in L2 / Infinity Cache and measurably raises the achieved HBM rate.
// The read half of a read-modify-write stays a normal load.
typedef float v4f __attribute__((ext_vector_type(4)));

template <bool NT>
__device__ __forceinline__ float4 ldg4(const float4* p) {
  if (NT) {
    const v4f v = __builtin_nontemporal_load(reinterpret_cast<const v4f*>(p));
    return make_float4(v.x, v.y, v.z, v.w);
  }
  return *p;
}

template <bool NT>
__device__ __forceinline__ void stg4(float4* p, const float4 r) {
  if (NT) {
    v4f v;
    v.x = r.x; v.y = r.y; v.z = r.z; v.w = r.w;
    __builtin_nontemporal_store(v, reinterpret_cast<v4f*>(p));
  } else {
    *p = r;
  }
}

template <bool NT>
__device__ __forceinline__ float ldg1(const float* p) {
  return NT ? __builtin_nontemporal_load(p) : *p;
}

template <bool NT>
__device__ __forceinline__ void stg1(float* p, const float v) {
  if (NT) __builtin_nontemporal_store(v, p);
  else *p = v;
}

// ---- wavefront reductions (64 lanes) -----------------------------------------
// Cross-lane steps are DPP modifiers of the adding instruction itself (no trip through the LDS crossbar):
// pairs, quads, half rows and rows of 16 lanes by quad permutes and row mirrors, then lane 15 of a
// row into the next row and lane 31 into the upper half; lane 63 ends up with the total, which every
// lane reads back through a scalar register.  Summation order: fixed, the same for every call.
template <int CTRL, int ROW_MASK>
__device__ __forceinline__ float dpp_move(float v, float fill) {
  return __int_as_float(__builtin_amdgcn_update_dpp(__float_as_int(fill), __float_as_int(v), CTRL, ROW_MASK, 0xF, false));
}

__device__ __forceinline__ float wave_sum(float v) {
  v += dpp_move<0xB1, 0xF>(v, 0.f);   // quad_perm [1,0,3,2]
  v += dpp_move<0x4E, 0xF>(v, 0.f);   // quad_perm [2,3,0,1]
  v += dpp_move<0x141, 0xF>(v, 0.f);  // row_half_mirror
  v += dpp_move<0x140, 0xF>(v, 0.f);  // row_mirror: every lane of a row holds the row's sum
  v += dpp_move<0x142, 0xA>(v, 0.f);  // row_bcast:15 into rows 1 and 3
  v += dpp_move<0x143, 0xC>(v, 0.f);  // row_bcast:31 into rows 2 and 3
  return __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 63));
}

__device__ __forceinline__ float wave_max(float v) {
  v = fmaxf(v, dpp_move<0xB1, 0xF>(v, v));
  v = fmaxf(v, dpp_move<0x4E, 0xF>(v, v));
  v = fmaxf(v, dpp_move<0x141, 0xF>(v, v));
  v = fmaxf(v, dpp_move<0x140, 0xF>(v, v));
  v = fmaxf(v, dpp_move<0x142, 0xA>(v, v));
  v = fmaxf(v, dpp_move<0x143, 0xC>(v, v));
  return __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 63));
}

// Block-wide sum for blockDim.x = 64 * NW.  Every thread gets the result.
// `red` is an LDS array of at least NW floats; safe to call repeatedly.
template <int NW>
__device__ __forceinline__ float block_sum(float v, float* red) {
  v = wave_sum(v);
  if (NW == 1) return v;
  const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
  __syncthreads();
  if (lane == 0) red[w] = v;
  __syncthreads();
  float t = red[0];
#pragma unroll
  for (int i = 1; i < NW; ++i) t += red[i];
  return t;
}

template <int NW>
__device__ __forceinline__ float block_max(float v, float* red) {
  v = wave_max(v);
  if (NW == 1) return v;
  const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
  __syncthreads();
  if (lane == 0) red[w] = v;
  __syncthreads();
  float t = red[0];
#pragma unroll
  for (int i = 1; i < NW; ++i) t = fmaxf(t, red[i]);
  return t;
}

// ---- scalar math shared by several kernels -----------------------------------

// scalar_logistic_sigmoid_op::packetOp of the reference (dynet/simd-functors.h:81-125):
// clamp to [-18,18], rational polynomial in Horner form with one fused
// multiply-add per pmadd, division, +0.5, clamp to [0,1].
// The reference divides with IEEE division.  Here q lies in [0.99, 500] and |p/q| <= 0.5,
// so no range scaling is needed, and the hardware reciprocal followed by one residual
// correction (4 instructions instead of ~11) gives, after the +0.5 and the clamp, the
// same bits as IEEE division for every one of the 2^32 float inputs: checked
// exhaustively on gfx950.  (The quotient alone can differ in its last bit.)
__device__ __forceinline__ float logistic_packet(float _x) {
  const float x = fmaxf(fminf(_x, 18.0f), -18.0f);
  const float x2 = x * x;
  float p = fmaf(x2, (float)4.37031012579801e-11, (float)1.15627324459942e-07);
  p = fmaf(x2, p, (float)6.08574864600143e-05);
  p = fmaf(x2, p, (float)8.51377133304701e-03);
  p = fmaf(x2, p, (float)2.48287947061529e-01);
  p = x * p;
  float q = fmaf(x2, (float)6.10247389755681e-13, (float)5.76102136993427e-09);
  q = fmaf(x2, q, (float)6.29106785017040e-06);
  q = fmaf(x2, q, (float)1.70198817374094e-03);
  q = fmaf(x2, q, (float)1.16817656904453e-01);
  q = fmaf(x2, q, (float)9.93151921023180e-01);
  const float r = __builtin_amdgcn_rcpf(q);
  float t = p * r;
  t = fmaf(fmaf(-q, t, p), r, t);
  return fmaxf(fminf(t + 0.5f, 1.0f), 0.0f);
}

// scalar operator() of the same functor (:76-79)
__device__ __forceinline__ float logistic_scalar(float x) { return 1.0f / (1.0f + expf(-x)); }

__device__ __forceinline__ float logistic(int mode, float x) {
  return mode == DYHIP_LOGISTIC_SCALAR ? logistic_scalar(x) : logistic_packet(x);
}

// tanh as a clamped odd/even rational function (the form Eigen's vectorised float
// tanh uses): p(x)/q(x) with p odd, so the result is relatively accurate for small
// |x| too; max relative error 4e-7 against fp64 tanh over the whole range.
// Branch-free: one median-of-three clamp, 9 fused multiply-adds, one hardware
// reciprocal (1 ulp; q >= 4.89e-3), and one select that hands a NaN input through
// (the clamp alone would turn it into -9, i.e. tanh(NaN) = -1; tanhf returns NaN).
__device__ __forceinline__ float tanh_accurate(float _x) {
  const float x = __builtin_amdgcn_fmed3f(_x, -9.0f, 9.0f);
  const float x2 = x * x;
  float p = fmaf(x2, -2.76076847742355e-16f, 2.00018790482477e-13f);
  p = fmaf(x2, p, -8.60467152213735e-11f);
  p = fmaf(x2, p, 5.12229709037114e-08f);
  p = fmaf(x2, p, 1.48572235717979e-05f);
  p = fmaf(x2, p, 6.37261928875436e-04f);
  p = fmaf(x2, p, 4.89352455891786e-03f);
  p = x * p;
  float q = fmaf(x2, 1.19825839466702e-06f, 1.18534705686654e-04f);
  q = fmaf(x2, q, 2.26843463243900e-03f);
  q = fmaf(x2, q, 4.89352518554385e-03f);
  const float r = p * __builtin_amdgcn_rcpf(q);
  return _x != _x ? _x : r;
}

}  // namespace dyhip
#endif  // __HIPCC__
