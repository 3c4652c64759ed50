// Elementwise launch layer: y = f(inputs) or y += f(inputs) over flat fp32
// buffers, with optional broadcast of an input over the batch dimension.
//
// Replaces the Eigen-on-GPU statements of Tanh / LogisticSigmoid / Rectify /
// Negate (dynet/nodes-trig.cc:312-326, nodes-activations.cc:31-78,
// nodes-arith-unary.cc:195-209), CwiseMultiply / CwiseSum without dimension
// broadcast (dynet/nodes-arith-cwise.cc:50-122,196-273), SumDimension's
// backward broadcast (dynet/nodes-arith-sum.cc:219-230), TensorTools::constant
// and accumulate, ParameterNode's scaled copy (dynet/param-nodes.cc:201-215),
// the SGD rule (dynet/training.cc:619-622), and takes the shape of the unused
// templated kernels of dynet/gpu-kernels.h:9-52.
//
// Layout: a tensor of n elements per batch element and bd batch elements is one
// flat buffer of n*bd floats.  A block owns one tile of 256 threads x UNROLL
// 128-bit accesses inside ONE batch element, so a broadcast input (batch 1) is
// indexed by the in-batch offset without any division per element.  All loads
// of a thread are issued before the first use to keep 4 x 16 B per lane in
// flight.  Large tensors are streamed with non-temporal loads and stores (the
// old value of an accumulating output included), which on MI355X lifts a
// 16.8 MB-per-tensor copy from about 4.6 to 5.8 TB/s and a three-read-one-write
// update from 4.7 to 5.6 TB/s.  Tensors whose n is not a multiple of 4, or whose base is not
// 16-byte aligned, take the scalar variant of the same kernel.
#include <algorithm>

#include "common.h"

namespace dyhip {

constexpr int kEwThreads = 256;

struct EwArgs {
  const float* in[3];
  float* out;
  size_t n;                 // elements per batch element (of the output)
  unsigned tiles_per_batch; // tiles covering one batch element
};

// F: struct with  __device__ float operator()(float a, float b, float c, float old) const
// NIN: number of inputs read; ACC: also read the output (old value).
// BMASK: bit k set => input k has batch 1 and is indexed by the in-batch offset.
// U: 128-bit accesses per thread and stream; NT: stream with non-temporal accesses.
// Which form a functor's kernels take for tiles that lie wholly inside the tensor, chosen per kernel by measurement
// on 4096 x 1024 floats (same GPU, same run; why the forms differ this way is not understood beyond the first point):
//   0  the bounds-checked form.  Each load sits in a branch of its own, so the compiler cannot count what is in
//      flight and waits for everything before each use: in effect every store waits for the one before it.
//   1  branch-free, in three phases: every load, all the arithmetic, every store.  Best for the three-stream backward
//      kernels (12.3 -> 12.1 us); costs the light forward kernels (rectify 6.2 -> 7.0 us, cmult 9.0 -> 9.8 us).
//   2  as 1, and each store waits for the one before it.  Brings every one-stream forward kernel to the copy's own
//      time whatever its arithmetic (tanh 6.8, logistic 7.2 (whose loads form 0 had serialised) -> 6.2 us); costs the
//      others (backward 12.5 us, cmult 9.3 us).
template <class F>
struct EwTileForm {
  static constexpr int value = 0;
};

template <int NIN, bool ACC, int BMASK, bool NT, int U, class F>
struct EwTile {
  float4 v[NIN > 0 ? NIN : 1][U];
  float4 o[U];

  // FULL: the whole tile lies inside the tensor.  Without the per-access bounds the loads are straight-line code;
  // under a bound each load sits in a branch of its own, into which the compiler may pull part of the arithmetic
  // (it did for the logistic), and then every load waits for the one before it.
  template <bool FULL>
  __device__ __forceinline__ void load(const EwArgs& a, size_t base4, size_t j0, size_t n4) {
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const size_t j = j0 + size_t(u) * kEwThreads;
      if (FULL || j < n4) {
#pragma unroll
        for (int k = 0; k < NIN; ++k) {
          const float4* p = reinterpret_cast<const float4*>(a.in[k]);
          // a broadcast input is re-read by every batch element: keep it cacheable
          if ((BMASK >> k) & 1) v[k][u] = p[j];
          else v[k][u] = ldg4<NT>(p + base4 + j);
        }
        if (ACC) o[u] = ldg4<NT>(reinterpret_cast<const float4*>(a.out) + base4 + j);
      }
    }
  }

  // Phases: every load of the tile, then all the arithmetic, then every store (scheduling barriers keep them apart:
  // left alone the compiler stores each group as soon as its loads have arrived, and a tile whose reads and writes
  // alternate measured 5-15 % slower on the one- and two-stream kernels).
  template <bool FULL>
  __device__ __forceinline__ void compute_store(const EwArgs& a, size_t base4, size_t j0, size_t n4, const F& f) {
    float4 r[U];
    if (FULL) __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const size_t j = j0 + size_t(u) * kEwThreads;
      if (FULL || j < n4) {
        const float4 z = make_float4(0.f, 0.f, 0.f, 0.f);
        const float4 x0 = NIN > 0 ? v[0][u] : z;
        const float4 x1 = NIN > 1 ? v[NIN > 1 ? 1 : 0][u] : z;
        const float4 x2 = NIN > 2 ? v[NIN > 2 ? 2 : 0][u] : z;
        const float4 od = ACC ? o[u] : z;
        r[u].x = f(x0.x, x1.x, x2.x, od.x);
        r[u].y = f(x0.y, x1.y, x2.y, od.y);
        r[u].z = f(x0.z, x1.z, x2.z, od.z);
        r[u].w = f(x0.w, x1.w, x2.w, od.w);
        if (!FULL) stg4<NT>(reinterpret_cast<float4*>(a.out) + base4 + j, r[u]);
      }
    }
    if (FULL) {
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int u = 0; u < U; ++u) {
        stg4<NT>(reinterpret_cast<float4*>(a.out) + base4 + j0 + size_t(u) * kEwThreads, r[u]);
        if (EwTileForm<F>::value == 2 && u + 1 < U) __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0)
      }
    }
  }
};

// One tile per block: every load of the tile is in flight before the first use.
template <int NIN, bool ACC, int BMASK, bool NT, int U, class F>
__global__ __launch_bounds__(kEwThreads) void ew_vec4_kernel(EwArgs a, F f) {
  const unsigned batch = blockIdx.x / a.tiles_per_batch;
  const unsigned tile = blockIdx.x - batch * a.tiles_per_batch;
  const size_t n4 = a.n >> 2;
  const size_t base4 = size_t(batch) * n4;
  const size_t j0 = size_t(tile) * (kEwThreads * U) + threadIdx.x;
  EwTile<NIN, ACC, BMASK, NT, U, F> t;
  if (EwTileForm<F>::value != 0 && size_t(tile + 1) * (kEwThreads * U) <= n4) {  // the same for every thread of the block
    t.template load<true>(a, base4, j0, n4);
    t.template compute_store<true>(a, base4, j0, n4, f);
  } else {
    t.template load<false>(a, base4, j0, n4);
    t.template compute_store<false>(a, base4, j0, n4, f);
  }
  // A flat tensor (nothing broadcast) whose length is not a multiple of four: its last one to three elements.
  if (BMASK == 0 && blockIdx.x == 0 && threadIdx.x < (a.n & 3)) {
    const size_t e = (n4 << 2) + threadIdx.x;
    const float x0 = NIN > 0 ? a.in[0][e] : 0.f;
    const float x1 = NIN > 1 ? a.in[NIN > 1 ? 1 : 0][e] : 0.f;
    const float x2 = NIN > 2 ? a.in[NIN > 2 ? 2 : 0][e] : 0.f;
    const float od = ACC ? a.out[e] : 0.f;
    a.out[e] = f(x0, x1, x2, od);
  }
}

template <int NIN, bool ACC, int BMASK, class F>
__global__ __launch_bounds__(kEwThreads) void ew_scalar_kernel(EwArgs a, F f) {
  constexpr int U = 4;
  const unsigned batch = blockIdx.x / a.tiles_per_batch;
  const unsigned tile = blockIdx.x - batch * a.tiles_per_batch;
  const size_t base = size_t(batch) * a.n;
  const size_t j0 = size_t(tile) * (kEwThreads * U) + threadIdx.x;
#pragma unroll
  for (int u = 0; u < U; ++u) {
    const size_t j = j0 + size_t(u) * kEwThreads;
    if (j < a.n) {
      const float x0 = NIN > 0 ? a.in[0][(BMASK & 1) ? j : base + j] : 0.f;
      const float x1 = NIN > 1 ? a.in[1][(BMASK & 2) ? j : base + j] : 0.f;
      const float x2 = NIN > 2 ? a.in[2][(BMASK & 4) ? j : base + j] : 0.f;
      const float od = ACC ? a.out[base + j] : 0.f;
      a.out[base + j] = f(x0, x1, x2, od);
    }
  }
}

// A batch-broadcast launch whose batch elements are shorter than a tile: a thread keeps one in-batch offset and walks
// U consecutive batch elements, so the broadcast inputs are loaded once per thread and every thread still has U
// accesses per stream in flight (with one tile per batch element a 1024-float element left three quarters of each
// tile masked off: one access per thread and 4096 blocks).  Loads are unconditional on clamped addresses; only the
// stores are guarded.
template <int NIN, bool ACC, int BMASK, bool NT, int U, class F>
__global__ __launch_bounds__(kEwThreads) void ew_bcast_vec4_kernel(EwArgs a, unsigned bd, F f) {
  const size_t n4 = a.n >> 2;
  const size_t j = size_t(blockIdx.x) * kEwThreads + threadIdx.x;
  const bool live = j < n4;
  const size_t jc = live ? j : n4 - 1;
  const unsigned b0 = blockIdx.y * U;
  float4 v[NIN > 0 ? NIN : 1][U];
  float4 o[U];
#pragma unroll
  for (int k = 0; k < NIN; ++k)
    if ((BMASK >> k) & 1) v[k][0] = reinterpret_cast<const float4*>(a.in[k])[jc];
#pragma unroll
  for (int u = 0; u < U; ++u) {
    const unsigned b = b0 + u < bd ? b0 + u : bd - 1;
    const size_t at = size_t(b) * n4 + jc;
#pragma unroll
    for (int k = 0; k < NIN; ++k)
      if (!((BMASK >> k) & 1)) v[k][u] = ldg4<NT>(reinterpret_cast<const float4*>(a.in[k]) + at);
    if (ACC) o[u] = ldg4<NT>(reinterpret_cast<const float4*>(a.out) + at);
  }
  __builtin_amdgcn_sched_barrier(0);
  float4 r[U];
#pragma unroll
  for (int u = 0; u < U; ++u) {
    const float4 z = make_float4(0.f, 0.f, 0.f, 0.f);
    const float4 x0 = NIN > 0 ? v[0][(BMASK & 1) ? 0 : u] : z;
    const float4 x1 = NIN > 1 ? v[NIN > 1 ? 1 : 0][(BMASK & 2) ? 0 : u] : z;
    const float4 x2 = NIN > 2 ? v[NIN > 2 ? 2 : 0][(BMASK & 4) ? 0 : u] : z;
    const float4 od = ACC ? o[u] : z;
    r[u].x = f(x0.x, x1.x, x2.x, od.x);
    r[u].y = f(x0.y, x1.y, x2.y, od.y);
    r[u].z = f(x0.z, x1.z, x2.z, od.z);
    r[u].w = f(x0.w, x1.w, x2.w, od.w);
  }
  __builtin_amdgcn_sched_barrier(0);
#pragma unroll
  for (int u = 0; u < U; ++u)
    if (live && b0 + u < bd) stg4<NT>(reinterpret_cast<float4*>(a.out) + size_t(b0 + u) * n4 + j, r[u]);
}

// A batch-broadcast launch over batch elements that are far shorter than a tile and cannot take 128-bit accesses (a
// scalar loss per batch element, n = 1: sum_batches backward over 100 000 of them was 100 000 blocks with one live
// thread each, 29 us): the flat tensor, four entries a thread, the in-batch offset by one division.
template <int NIN, bool ACC, int BMASK, class F>
__global__ __launch_bounds__(kEwThreads) void ew_flat_bcast_kernel(EwArgs a, size_t total, F f) {
  const size_t e0 = size_t(blockIdx.x) * (kEwThreads * 4) + threadIdx.x;
  const bool small = total <= 0xFFFFFFFFull;  // the same for every thread: 32-bit division
#pragma unroll
  for (int u = 0; u < 4; ++u) {
    const size_t e = e0 + size_t(u) * kEwThreads;
    if (e < total) {
      const size_t j = small ? size_t(unsigned(e) % unsigned(a.n)) : e % a.n;
      const float x0 = NIN > 0 ? a.in[0][(BMASK & 1) ? j : e] : 0.f;
      const float x1 = NIN > 1 ? a.in[NIN > 1 ? 1 : 0][(BMASK & 2) ? j : e] : 0.f;
      const float x2 = NIN > 2 ? a.in[NIN > 2 ? 2 : 0][(BMASK & 4) ? j : e] : 0.f;
      const float od = ACC ? a.out[e] : 0.f;
      a.out[e] = f(x0, x1, x2, od);
    }
  }
}

// Launch over an (n x bd) output.  Inputs whose bit is set in BMASK have batch 1.
template <int NIN, bool ACC, int BMASK, class F>
int ew_launch(dyhip_device* dev, size_t n, unsigned bd, const float* in0, const float* in1, const float* in2,
              float* out, F f) {
  if (n == 0 || bd == 0) return DYHIP_OK;
  if (BMASK == 0) {  // nothing is broadcast: one flat buffer
    n *= bd;
    bd = 1;
  }
  // 128-bit accesses per thread and stream: 4 for one or two streams, 2 for three or more
  constexpr int kStreams = NIN + (ACC ? 1 : 0);
  constexpr int U = kStreams >= 3 ? 2 : 4;
  EwArgs a;
  a.in[0] = in0;
  a.in[1] = in1;
  a.in[2] = in2;
  a.out = out;
  a.n = n;
  // 128-bit accesses need 16-byte aligned pointers and, when an input is broadcast, batch elements that keep that
  // alignment; a flat tensor of any length >= 4 qualifies (its last n % 4 elements are done one by one)
  bool vec = (BMASK == 0 ? n >= 4 : n % 4 == 0) && aligned16(out);
  for (int k = 0; k < NIN; ++k) vec = vec && aligned16(a.in[k]);
  const size_t per_tile = vec ? size_t(kEwThreads) * U * 4 : size_t(kEwThreads) * 4;
  const size_t tiles = cdiv(vec ? n - n % 4 : n, per_tile);
  DYHIP_REQUIRE(tiles * bd < (size_t(1) << 31), "elementwise launch too large: %zu tiles x %u batches", tiles, bd);
  a.tiles_per_batch = static_cast<unsigned>(tiles);
  const dim3 grid(static_cast<unsigned>(tiles * bd)), block(kEwThreads);
  const bool stream = n * bd * sizeof(float) >= dev->stream_threshold;
  if (BMASK != 0 && vec && n / 4 < size_t(kEwThreads) * U && cdiv<size_t>(bd, U) <= 65535) {
    const dim3 g2(static_cast<unsigned>(cdiv<size_t>(n / 4, kEwThreads)), static_cast<unsigned>(cdiv<size_t>(bd, U)));
    if (stream)
      hipLaunchKernelGGL((ew_bcast_vec4_kernel<NIN, ACC, BMASK, true, U, F>), g2, block, 0, dev->stream, a, bd, f);
    else
      hipLaunchKernelGGL((ew_bcast_vec4_kernel<NIN, ACC, BMASK, false, U, F>), g2, block, 0, dev->stream, a, bd, f);
  } else if (BMASK != 0 && !vec && n < size_t(kEwThreads) && cdiv<size_t>(n * bd, size_t(kEwThreads) * 4) < (size_t(1) << 31)) {
    const size_t total = n * bd;
    hipLaunchKernelGGL((ew_flat_bcast_kernel<NIN, ACC, BMASK, F>), dim3(static_cast<unsigned>(cdiv<size_t>(total, size_t(kEwThreads) * 4))),
                       block, 0, dev->stream, a, total, f);
  } else if (!vec) {
    hipLaunchKernelGGL((ew_scalar_kernel<NIN, ACC, BMASK, F>), grid, block, 0, dev->stream, a, f);
  } else if (stream) {
    hipLaunchKernelGGL((ew_vec4_kernel<NIN, ACC, BMASK, true, U, F>), grid, block, 0, dev->stream, a, f);
  } else {
    hipLaunchKernelGGL((ew_vec4_kernel<NIN, ACC, BMASK, false, U, F>), grid, block, 0, dev->stream, a, f);
  }
  DYHIP_CHECK_LAUNCH();
  return DYHIP_OK;
}

// ---- functors -----------------------------------------------------------------
struct TanhFwd {
  __device__ float operator()(float x, float, float, float) const { return tanh_accurate(x); }
};
struct LogisticPacketFwd {
  __device__ float operator()(float x, float, float, float) const { return logistic_packet(x); }
};
struct LogisticScalarFwd {
  __device__ float operator()(float x, float, float, float) const { return logistic_scalar(x); }
};
struct RectifyFwd { __device__ float operator()(float x, float, float, float) const { return x > 0.f ? x : 0.f; } };
struct NegateFwd { __device__ float operator()(float x, float, float, float) const { return -x; } };
struct IdentityFwd { __device__ float operator()(float x, float, float, float) const { return x; } };

// backward functors: (fx, dEdf, -, old) -> old + g(fx, dEdf); the expression
// order follows the scalar operators of dynet/simd-functors.h:509-544
struct TanhBwd { __device__ float operator()(float t, float d, float, float o) const { return o + (1.f - t * t) * d; } };
struct LogisticBwd { __device__ float operator()(float t, float d, float, float o) const { return o + (1.f - t) * t * d; } };
struct RectifyBwd { __device__ float operator()(float t, float d, float, float o) const { return o + (t != 0.f ? 1.f : 0.f) * d; } };
struct NegateBwd { __device__ float operator()(float, float d, float, float o) const { return o - d; } };

struct Mul2 { __device__ float operator()(float a, float b, float, float) const { return a * b; } };
struct Add2 { __device__ float operator()(float a, float b, float, float) const { return a + b; } };
struct AccMul2 { __device__ float operator()(float a, float b, float, float o) const { return o + a * b; } };
struct AccIn0 { __device__ float operator()(float a, float, float, float o) const { return o + a; } };
struct ConstFill {
  float c;
  __device__ float operator()(float, float, float, float) const { return c; }
};
struct ScaleCopy {
  float m;
  __device__ float operator()(float a, float, float, float) const { return a * m; }
};
struct SgdStep {  // p -= g * s
  float s;
  __device__ float operator()(float g, float, float, float p) const { return p - g * s; }
};

// Batch reduction used by the broadcast-argument backward (defined in reduce.hip):
// out[j] (+)= sum_b in0[b*n+j] * (in1 ? in1[b*n+j] : 1)
int batch_reduce(dyhip_device* dev, size_t n, unsigned bd, const float* in0, const float* in1, float* out,
                 bool accumulate, void* ws, size_t ws_bytes);

// ---- Sum node: groups of up to four arguments per launch, in the reference's association order ----
struct SumArgs {
  const float* x[32];
  unsigned bcast;    // bit i: argument i has batch size 1 and is broadcast over the batch
  unsigned cnt[8];   // members of each group (1..4)
  unsigned ngroups;  // groups in this launch (1..8)
};

// Up to eight groups per launch (a Sum over the 35 per-timestep losses of a language model was nine launches): every
// group is summed left to right, its four loads in flight together, and then added to what came before, so the
// arithmetic is that of one launch per group.
// ONE: a single group (the usual two to four arguments): its members at fixed places of the argument list (indexing
// the list by a run-time position costs more than the sum itself there).
template <bool ACC, bool ONE>
__global__ __launch_bounds__(256) void sum_group_kernel(SumArgs a, size_t n, size_t total, float* __restrict__ fx) {
  const size_t e = size_t(blockIdx.x) * 256 + threadIdx.x;
  if (e >= total) return;
  const size_t j = a.bcast != 0 ? e % n : e;
  float acc = ACC ? fx[e] : 0.f;
  if (ONE) {
    const unsigned cnt = a.cnt[0];
    float t = a.x[0][a.bcast & 1u ? j : e];
    if (cnt > 1) t = t + a.x[1][a.bcast & 2u ? j : e];
    if (cnt > 2) t = t + a.x[2][a.bcast & 4u ? j : e];
    if (cnt > 3) t = t + a.x[3][a.bcast & 8u ? j : e];
    fx[e] = ACC ? acc + t : t;
    return;
  }
  unsigned at = 0;
  for (unsigned g = 0; g < a.ngroups; ++g) {
    const unsigned cnt = a.cnt[g];
    float v[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const unsigned m = at + (unsigned(i) < cnt ? unsigned(i) : cnt - 1);  // past the group's end: its last member again
      v[i] = a.x[m][(a.bcast >> m) & 1u ? j : e];
    }
    float t = v[0];
#pragma unroll
    for (int i = 1; i < 4; ++i)
      if (unsigned(i) < cnt) t = t + v[i];
    acc = (!ACC && g == 0) ? t : acc + t;
    at += cnt;
  }
  fx[e] = acc;
}

static int check_bd(unsigned bd0, unsigned bd1) {
  DYHIP_REQUIRE(bd0 >= 1 && bd1 >= 1 && (bd0 == bd1 || bd0 == 1 || bd1 == 1),
                "batch size must match or equal 1 (got %u and %u)", bd0, bd1);
  return DYHIP_OK;
}

template <class F>
static int binary_forward(dyhip_device* dev, size_t n, unsigned bd0, unsigned bd1, const float* a, const float* b,
                          float* y, F f) {
  DYHIP_CHECK_DEV(dev);
  DYHIP_CHECK_STATUS(check_bd(bd0, bd1));
  DYHIP_REQUIRE(n == 0 || (a && b && y), "null tensor pointer");
  const unsigned bd = bd0 > bd1 ? bd0 : bd1;
  if (bd0 == bd1) return ew_launch<2, false, 0>(dev, n, bd, a, b, nullptr, y, f);
  if (bd0 == 1) return ew_launch<2, false, 1>(dev, n, bd, a, b, nullptr, y, f);
  return ew_launch<2, false, 2>(dev, n, bd, a, b, nullptr, y, f);
}

// PickRange (dynet/nodes-select.cc:230-259): slicing dimension `dim` of a column-major tensor is a
// strided copy of `outer` contiguous runs: with inner = product of the dimensions before `dim`,
// run o is src[o*inner*len + start*inner, +inner*(end-start)).  blockIdx.y walks runs, lanes walk a run.
template <bool ACC>
__global__ __launch_bounds__(256) void pick_range_kernel(size_t run, size_t small_stride, size_t big_stride,
                                                         size_t big_offset, unsigned outer,
                                                         const float* __restrict__ src, float* __restrict__ dst) {
  for (unsigned o = blockIdx.y; o < outer; o += gridDim.y) {
    // forward: dst is the slice (small), src the whole tensor (big); backward: the other way round
    const float* s = ACC ? src + o * small_stride : src + o * big_stride + big_offset;
    float* d = ACC ? dst + o * big_stride + big_offset : dst + o * small_stride;
    for (size_t e = size_t(blockIdx.x) * 256 + threadIdx.x; e < run; e += size_t(gridDim.x) * 256)
      d[e] = ACC ? d[e] + s[e] : s[e];
  }
}

// Runs shorter than a few wavefronts (a block per run left most of its lanes idle: 100 000 runs of 21 floats took
// 30 us): a thread per entry of the slice over the flat slice, four entries in flight, the run found by one 32-bit
// division.
template <bool ACC>
__global__ __launch_bounds__(256) void pick_range_flat_kernel(unsigned run, unsigned total, size_t big_stride,
                                                              size_t big_offset, const float* __restrict__ src,
                                                              float* __restrict__ dst) {
  const unsigned e0 = blockIdx.x * 1024 + threadIdx.x;
  size_t big[4];
  unsigned small[4];
  float v[4], acc[4];
#pragma unroll
  for (int k = 0; k < 4; ++k) {
    const unsigned e = e0 + 256 * k;
    small[k] = e < total ? e : total - 1;
    const unsigned o = small[k] / run;
    big[k] = size_t(o) * big_stride + big_offset + (small[k] - o * run);
    v[k] = ACC ? src[small[k]] : src[big[k]];
    acc[k] = ACC ? dst[big[k]] : 0.f;
  }
#pragma unroll
  for (int k = 0; k < 4; ++k) {
    if (e0 + 256 * k >= total) continue;
    if (ACC) dst[big[k]] = acc[k] + v[k];
    else dst[small[k]] = v[k];
  }
}

static int pick_range(dyhip_device* dev, bool backward, size_t inner, size_t len, size_t outer, size_t start,
                      size_t end, const float* src, float* dst) {
  DYHIP_REQUIRE(start < end && end <= len, "PickRange: bad range [%zu, %zu) for a dimension of %zu", start, end, len);
  if (inner == 0 || outer == 0) return DYHIP_OK;
  DYHIP_REQUIRE(src && dst, "PickRange: null tensor pointer");
  DYHIP_REQUIRE(outer <= 0xffffffffu, "PickRange: too many slices");
  const size_t run = inner * (end - start);
  if (run < 1024 && outer > 1 && run * outer <= 0xffffffffu - 1024) {
    const unsigned total = unsigned(run * outer), blocks = cdiv<unsigned>(total, 1024);
    if (backward)
      hipLaunchKernelGGL(pick_range_flat_kernel<true>, dim3(blocks), dim3(256), 0, dev->stream, unsigned(run), total,
                         inner * len, start * inner, src, dst);
    else
      hipLaunchKernelGGL(pick_range_flat_kernel<false>, dim3(blocks), dim3(256), 0, dev->stream, unsigned(run), total,
                         inner * len, start * inner, src, dst);
    DYHIP_CHECK_LAUNCH();
    return DYHIP_OK;
  }
  const dim3 grid(unsigned(std::min<size_t>(cdiv<size_t>(run, 256), 4096)), unsigned(std::min<size_t>(outer, 65535)));
  if (backward)
    hipLaunchKernelGGL(pick_range_kernel<true>, grid, dim3(256), 0, dev->stream, run, run, inner * len, start * inner,
                       unsigned(outer), src, dst);
  else
    hipLaunchKernelGGL(pick_range_kernel<false>, grid, dim3(256), 0, dev->stream, run, run, inner * len, start * inner,
                       unsigned(outer), src, dst);
  DYHIP_CHECK_LAUNCH();
  return DYHIP_OK;
}

template <> struct EwTileForm<TanhFwd> { static constexpr int value = 2; };
template <> struct EwTileForm<LogisticPacketFwd> { static constexpr int value = 2; };
template <> struct EwTileForm<LogisticScalarFwd> { static constexpr int value = 2; };
template <> struct EwTileForm<RectifyFwd> { static constexpr int value = 2; };
template <> struct EwTileForm<TanhBwd> { static constexpr int value = 1; };
template <> struct EwTileForm<LogisticBwd> { static constexpr int value = 1; };
template <> struct EwTileForm<RectifyBwd> { static constexpr int value = 1; };
template <> struct EwTileForm<AccMul2> { static constexpr int value = 1; };

}  // namespace dyhip

using namespace dyhip;

extern "C" {

int dyhip_unary_forward(dyhip_device* dev, int op, int logistic_mode, size_t n, const float* x, float* y) {
  DYHIP_CHECK_DEV(dev);
  DYHIP_REQUIRE(n == 0 || (x != nullptr && y != nullptr), "null tensor pointer");
  switch (op) {
    case DYHIP_OP_TANH: return ew_launch<1, false, 0>(dev, n, 1, x, nullptr, nullptr, y, TanhFwd());
    case DYHIP_OP_LOGISTIC:
      if (logistic_mode == DYHIP_LOGISTIC_SCALAR)
        return ew_launch<1, false, 0>(dev, n, 1, x, nullptr, nullptr, y, LogisticScalarFwd());
      DYHIP_REQUIRE(logistic_mode == DYHIP_LOGISTIC_PACKET, "unknown logistic mode %d", logistic_mode);
      return ew_launch<1, false, 0>(dev, n, 1, x, nullptr, nullptr, y, LogisticPacketFwd());
    case DYHIP_OP_RECTIFY: return ew_launch<1, false, 0>(dev, n, 1, x, nullptr, nullptr, y, RectifyFwd());
    case DYHIP_OP_NEGATE: return ew_launch<1, false, 0>(dev, n, 1, x, nullptr, nullptr, y, NegateFwd());
    case DYHIP_OP_IDENTITY: return ew_launch<1, false, 0>(dev, n, 1, x, nullptr, nullptr, y, IdentityFwd());
    default: return fail(DYHIP_ERR_INVALID_ARG, "unknown unary operator %d", op);
  }
}

int dyhip_unary_backward(dyhip_device* dev, int op, size_t n, const float* fx, const float* dEdf, float* dEdx) {
  DYHIP_CHECK_DEV(dev);
  DYHIP_REQUIRE(n == 0 || (fx != nullptr && dEdf != nullptr && dEdx != nullptr), "null tensor pointer");
  switch (op) {
    case DYHIP_OP_TANH: return ew_launch<2, true, 0>(dev, n, 1, fx, dEdf, nullptr, dEdx, TanhBwd());
    case DYHIP_OP_LOGISTIC: return ew_launch<2, true, 0>(dev, n, 1, fx, dEdf, nullptr, dEdx, LogisticBwd());
    case DYHIP_OP_RECTIFY: return ew_launch<2, true, 0>(dev, n, 1, fx, dEdf, nullptr, dEdx, RectifyBwd());
    case DYHIP_OP_NEGATE: return ew_launch<2, true, 0>(dev, n, 1, fx, dEdf, nullptr, dEdx, NegateBwd());
    case DYHIP_OP_IDENTITY: return ew_launch<1, true, 0>(dev, n, 1, dEdf, nullptr, nullptr, dEdx, AccIn0());
    default: return fail(DYHIP_ERR_INVALID_ARG, "unknown unary operator %d", op);
  }
}

int dyhip_cmult_forward(dyhip_device* dev, size_t n, unsigned bd0, unsigned bd1, const float* a, const float* b,
                        float* y) {
  return binary_forward(dev, n, bd0, bd1, a, b, y, Mul2());
}

int dyhip_csum_forward(dyhip_device* dev, size_t n, unsigned bd0, unsigned bd1, const float* a, const float* b,
                       float* y) {
  return binary_forward(dev, n, bd0, bd1, a, b, y, Add2());
}

int dyhip_cmult_backward(dyhip_device* dev, size_t n, unsigned bd0, unsigned bd1, const float* a, const float* b,
                         const float* dEdf, unsigned i, float* dEdxi, void* ws, size_t ws_bytes) {
  DYHIP_CHECK_DEV(dev);
  DYHIP_CHECK_STATUS(check_bd(bd0, bd1));
  DYHIP_REQUIRE(i < 2, "CwiseMultiply has two arguments (i = %u)", i);
  DYHIP_REQUIRE(n == 0 || (a && b && dEdf && dEdxi), "null tensor pointer");
  const unsigned bd = bd0 > bd1 ? bd0 : bd1;
  const float* other = i == 0 ? b : a;
  const unsigned bd_other = i == 0 ? bd1 : bd0;
  const unsigned bd_self = i == 0 ? bd0 : bd1;
  if (bd_self == bd) {
    if (bd_other == bd) return ew_launch<2, true, 0>(dev, n, bd, dEdf, other, nullptr, dEdxi, AccMul2());
    return ew_launch<2, true, 2>(dev, n, bd, dEdf, other, nullptr, dEdxi, AccMul2());
  }
  // this argument was broadcast over the batch: dxi += sum_b dy * other
  return batch_reduce(dev, n, bd, dEdf, other, dEdxi, true, ws, ws_bytes);
}

int dyhip_csum_backward(dyhip_device* dev, size_t n, unsigned bd0, unsigned bd1, const float* dEdf, unsigned i,
                        float* dEdxi, void* ws, size_t ws_bytes) {
  DYHIP_CHECK_DEV(dev);
  DYHIP_CHECK_STATUS(check_bd(bd0, bd1));
  DYHIP_REQUIRE(i < 2, "CwiseSum has two arguments (i = %u)", i);
  DYHIP_REQUIRE(n == 0 || (dEdf && dEdxi), "null tensor pointer");
  const unsigned bd = bd0 > bd1 ? bd0 : bd1;
  const unsigned bd_self = i == 0 ? bd0 : bd1;
  if (bd_self == bd) return ew_launch<1, true, 0>(dev, n, bd, dEdf, nullptr, nullptr, dEdxi, AccIn0());
  return batch_reduce(dev, n, bd, dEdf, nullptr, dEdxi, true, ws, ws_bytes);
}

int dyhip_sum_batches_backward(dyhip_device* dev, size_t n, unsigned bd, const float* dEdf, float* dEdx) {
  DYHIP_CHECK_DEV(dev);
  DYHIP_REQUIRE(n == 0 || bd == 0 || (dEdf && dEdx), "null tensor pointer");
  return ew_launch<1, true, 1>(dev, n, bd, dEdf, nullptr, nullptr, dEdx, AccIn0());
}

int dyhip_constant(dyhip_device* dev, size_t n, float value, float* dst) {
  DYHIP_CHECK_DEV(dev);
  DYHIP_REQUIRE(n == 0 || dst, "null tensor pointer");
  return ew_launch<0, false, 0>(dev, n, 1, nullptr, nullptr, nullptr, dst, ConstFill{value});
}

int dyhip_accumulate(dyhip_device* dev, size_t n, const float* src, float* dst) {
  DYHIP_CHECK_DEV(dev);
  DYHIP_REQUIRE(n == 0 || (src && dst), "null tensor pointer");
  return ew_launch<1, true, 0>(dev, n, 1, src, nullptr, nullptr, dst, AccIn0());
}

int dyhip_scale_copy(dyhip_device* dev, size_t n, const float* src, float mult, float* dst) {
  DYHIP_CHECK_DEV(dev);
  DYHIP_REQUIRE(n == 0 || (src && dst), "null tensor pointer");
  if (mult == 1.0f) return ew_launch<1, false, 0>(dev, n, 1, src, nullptr, nullptr, dst, IdentityFwd());
  return ew_launch<1, false, 0>(dev, n, 1, src, nullptr, nullptr, dst, ScaleCopy{mult});
}

int dyhip_sgd_update(dyhip_device* dev, size_t n, float* p, const float* g, float lr, float gscale, float wd) {
  DYHIP_CHECK_DEV(dev);
  DYHIP_REQUIRE(n == 0 || (p && g), "null tensor pointer");
  DYHIP_REQUIRE(wd != 0.f, "weight decay scale must be non-zero");
  return ew_launch<1, true, 0>(dev, n, 1, g, nullptr, nullptr, p, SgdStep{lr * gscale / wd});
}

int dyhip_sum_forward(dyhip_device* dev, unsigned k, size_t n, unsigned bd, const float* const* xs_host,
                      const unsigned* bds_host, float* fx) {
  DYHIP_CHECK_DEV(dev);
  DYHIP_REQUIRE(k >= 1 && xs_host && bds_host && fx, "Sum needs at least one argument");
  const size_t total = n * size_t(bd);
  if (total == 0) return DYHIP_OK;
  bool same = true;
  for (unsigned i = 0; i < k; ++i) {
    DYHIP_REQUIRE(xs_host[i] != nullptr, "null argument %u of Sum", i);
    DYHIP_REQUIRE(bds_host[i] == bd || bds_host[i] == 1, "Mismatched batch dimension in Sum (argument %u)", i);
    same = same && bds_host[i] == bds_host[0];
  }
  DYHIP_REQUIRE(!same || bds_host[0] == bd, "Sum: output batch size %u but every argument has batch size 1", bd);
  const dim3 grid((unsigned)cdiv<size_t>(total, 256)), block(256);
  // equal batch sizes: (first four) then the remainder (k - 4) % 4 then groups of four, each group summed
  // left to right before it is added; mixed batch sizes: one argument at a time onto a zeroed output
  unsigned at = 0;
  bool first = true;
  while (at < k) {
    SumArgs a;
    a.bcast = 0;
    a.ngroups = 0;
    unsigned used = 0;
    const bool launch_first = first;
    while (at < k && a.ngroups < 8 && used + 4 <= 32) {
      unsigned cnt;
      if (!same) cnt = 1;
      else if (first) cnt = k < 4 ? k : 4;
      else if (at == 4 && (k - 4) % 4 != 0) cnt = (k - 4) % 4;
      else cnt = 4;
      for (unsigned i = 0; i < cnt; ++i) {
        a.x[used + i] = xs_host[at + i];
        if (bds_host[at + i] != bd) a.bcast |= 1u << (used + i);
      }
      a.cnt[a.ngroups++] = cnt;
      used += cnt;
      at += cnt;
      first = false;
    }
    for (unsigned i = used; i < 32; ++i) a.x[i] = nullptr;
    for (unsigned g = a.ngroups; g < 8; ++g) a.cnt[g] = 0;
    const bool one = a.ngroups == 1;
    if (launch_first && same) {
      if (one) hipLaunchKernelGGL((sum_group_kernel<false, true>), grid, block, 0, dev->stream, a, n, total, fx);
      else hipLaunchKernelGGL((sum_group_kernel<false, false>), grid, block, 0, dev->stream, a, n, total, fx);
    } else {
      if (launch_first) DYHIP_CHECK_STATUS(dyhip_zero(dev, fx, total * sizeof(float)));
      if (one) hipLaunchKernelGGL((sum_group_kernel<true, true>), grid, block, 0, dev->stream, a, n, total, fx);
      else hipLaunchKernelGGL((sum_group_kernel<true, false>), grid, block, 0, dev->stream, a, n, total, fx);
    }
  }
  DYHIP_CHECK_LAUNCH();
  return DYHIP_OK;
}

int dyhip_pick_range_forward(dyhip_device* dev, size_t inner, size_t len, size_t outer, size_t start, size_t end,
                             const float* x, float* fx) {
  DYHIP_CHECK_DEV(dev);
  return pick_range(dev, false, inner, len, outer, start, end, x, fx);
}

int dyhip_pick_range_backward(dyhip_device* dev, size_t inner, size_t len, size_t outer, size_t start, size_t end,
                              const float* dEdf, float* dEdxi) {
  DYHIP_CHECK_DEV(dev);
  return pick_range(dev, true, inner, len, outer, start, end, dEdf, dEdxi);
}

}  // extern "C"
