// fp32 MFMA GEMM for large outputs: a 512-thread block (8 wavefronts, 2 x 4) owns a 256 x 256 tile of C, one block
// per CU, operands streamed from memory straight into LDS.  Same three forms and the same arithmetic
// (v_mfma_f32_32x32x2_f32, fp32 in and out) as gemm.hip, which keeps the small, skinny, ragged, segmented and batched
// problems (dynet/matrix-multiply.h:16-37,97-117,162-180 are the callers this replaces cublasSgemm for).
//
// Why a second kernel.  A 128 x 128 tile needs 32 KiB of operands per MFLOP, and gemm.hip stages them through
// registers into LDS: the loads, the LDS writes and the address arithmetic share issue slots with the MFMAs, and the
// staging registers are what limits its tile.  A 256 x 256 tile halves the bytes per flop, and `global_load_lds_dwordx4`
// moves them without passing through registers: the main loop is MFMAs, 24 LDS reads and 8 load issues per 128 MFMAs.
//
// LDS.  Two stages of 64 KiB.  A stage holds the 256 x 32 tiles of both operands as 64 chunks of 1 KiB, one per
// wave-wide load (64 lanes x 16 bytes; lane j fills bytes 16 j.. of its chunk).  Wave w issues chunks 4w..4w+3 of each
// operand and owns the 8 KiB [A chunks 4w..4w+3][B chunks 4w..4w+3], so that ONE LDS base (M0) serves its eight loads
// and the instruction offset picks the chunk: a write to M0 waits for the wave's loads in flight, which costs ~250
// cycles apiece when every load has a base of its own.
//   * chunk q of an operand stored along mn ([k][mn] in LDS) is row k = q;
//   * chunk q of an operand stored along k ([mn][k] in LDS) is rows 8q..8q+7, 128 bytes each, and lane j (row 8q + j/8,
//     position j%8) fetches k-group (j%8) ^ ((row/2)%8): the 128-bit fragment reads of 16 consecutive rows then cover
//     all 64 banks without padding.
// Within a group of 8 k, MFMA step s takes k = 4*lhi + s from lane half lhi (any bijection works as long as both
// operands use it), so a lane's four steps are one 128-bit read of a k-contiguous row, and for an mn-contiguous
// operand one 128-bit read per step yields the values of its four row tiles (rows interleaved: tile t owns 4*l + t).
//
// Schedule of a k-tile (128 MFMAs per wave): fragments of group kg+1 are fetched after the first 8 MFMAs of group kg.
// Before the last group every wave waits for its own loads and meets the others at the one barrier of the k-tile:
// from there the stage just consumed is refilled two k-tiles ahead and the next k-tile's first fragments are fetched,
// both under the remaining MFMAs.
//
// Work distribution.  Tiles beyond the last full round of one tile per CU would leave most CUs idle for a whole
// round, so the k-tiles of those remaining tiles are dealt to the CUs in equal runs; a run that does not cover a
// whole tile leaves a partial tile in the workspace, and a second kernel adds the partial tiles of each tile in run
// order (deterministic, no atomics) and applies the epilogue.
#include "gemm.h"

namespace dyhip {

namespace {

typedef float floatx16 __attribute__((ext_vector_type(16)));
typedef float fvec2 __attribute__((ext_vector_type(2)));
typedef const __attribute__((address_space(1))) void* global_ptr_t;
typedef __attribute__((address_space(3))) void* lds_ptr_t;

constexpr int kWideThreads = 512;
constexpr int kWT = 256;                  // tile extent along m and along n
constexpr int kWK = 32;                   // k-tile
constexpr int kStageFloats = 16384;       // 64 KiB
constexpr size_t kWideLdsBytes = sizeof(float) * 2 * kStageFloats;
constexpr size_t kSlotFloats = size_t(kWT) * kWT;

struct WideArgs {
  const float* A;
  const float* B;
  float* C;
  const float* bias;      // C = bias[m] + sum when set (beta unused)
  float* slots;           // partial tiles [slot][256 n][256 m]
  unsigned lda, ldb;
  unsigned M, N;
  unsigned nt;            // k-tiles
  unsigned tiles_m;
  unsigned direct_tiles;  // tiles [0, direct_tiles) are computed whole, one per block
  unsigned rem_units;     // k-tiles of the remaining tiles, dealt to the blocks that follow in runs of `per`
  unsigned per;
  float beta;
};

// offsets (floats) of this lane's four loads from the tile's first k; rows and groups of four past the matrix edge are
// clamped to the last one inside (their values only reach outputs the epilogue masks)
template <bool KMAJOR>
__device__ __forceinline__ void load_offsets(unsigned (&off)[4], unsigned ld, unsigned mn0, unsigned MN) {
  const unsigned lane = threadIdx.x & 63, w = threadIdx.x >> 6;
#pragma unroll
  for (int u = 0; u < 4; ++u) {
    const unsigned q = 4 * w + u;
    if (!KMAJOR) {
      unsigned mn = mn0 + lane * 4;
      mn = mn < MN ? mn : MN - 4;
      off[u] = mn + q * ld;
    } else {
      const unsigned row = 8 * q + lane / 8;
      unsigned mn = mn0 + row;
      mn = mn < MN ? mn : MN - 1;
      off[u] = ((lane % 8) ^ ((row / 2) % 8)) * 4 + mn * ld;
    }
  }
}

// wave_stage = the wave's 8 KiB of a stage + 4 KiB (the boundary between its A and B chunks).  The instruction offset
// is added to the LDS and to the global address, so the latter is biased back.
template <int OP>
__device__ __forceinline__ void load_chunks(const float* __restrict__ base, const unsigned (&off)[4],
                                            float* wave_stage) {
  constexpr int I0 = OP == 0 ? -4096 : 0;
#define DYHIP_LOAD_CHUNK(u)                                                                                        \
  __builtin_amdgcn_global_load_lds((global_ptr_t)(base + off[u] - (I0 + u * 1024) / 4), (lds_ptr_t)wave_stage, 16, \
                                   I0 + u * 1024, 0);
  DYHIP_LOAD_CHUNK(0) DYHIP_LOAD_CHUNK(1) DYHIP_LOAD_CHUNK(2) DYHIP_LOAD_CHUNK(3)
#undef DYHIP_LOAD_CHUNK
}

// fragments of one group of 8 k: a[s][t] (t = 4 row tiles of the wave's 128 m), b[s][u] (u = 2 column tiles of its
// 64 n).  la / lb: the lane's origin in the stage; sw[kg]: float offset of its k-group 2 kg + lhi in a swizzled row
template <bool AK>
__device__ __forceinline__ void read_a(float (&a)[4][4], const float* __restrict__ la, int kg, const int (&sw)[4]) {
  if (!AK) {
#pragma unroll
    for (int s = 0; s < 4; ++s) {
      const float4 v = *reinterpret_cast<const float4*>(la + kg * 4096 + s * 256);
      a[s][0] = v.x; a[s][1] = v.y; a[s][2] = v.z; a[s][3] = v.w;
    }
  } else {
#pragma unroll
    for (int t = 0; t < 4; ++t) {
      const float4 v = *reinterpret_cast<const float4*>(la + t * 2048 + sw[kg]);
      a[0][t] = v.x; a[1][t] = v.y; a[2][t] = v.z; a[3][t] = v.w;
    }
  }
}
template <bool BKM>
__device__ __forceinline__ void read_b(float (&b)[4][2], const float* __restrict__ lb, int kg, const int (&sw)[4]) {
  if (!BKM) {
#pragma unroll
    for (int s = 0; s < 4; ++s) {
      const fvec2 v = *reinterpret_cast<const fvec2*>(lb + kg * 4096 + s * 256);
      b[s][0] = v[0]; b[s][1] = v[1];
    }
  } else {
#pragma unroll
    for (int u = 0; u < 2; ++u) {
      const float4 v = *reinterpret_cast<const float4*>(lb + u * 2048 + sw[kg]);
      b[0][u] = v.x; b[1][u] = v.y; b[2][u] = v.z; b[3][u] = v.w;
    }
  }
}

// AK: A(m,k) = A[k + m*lda], else A[m + k*lda].  BKM: B(k,n) = B[k + n*ldb], else B[n + k*ldb].
template <bool AK, bool BKM>
__global__ __launch_bounds__(kWideThreads, 1) void gemm_wide_kernel(WideArgs g) {
  extern __shared__ __attribute__((aligned(16))) float lds[];
  const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
  const int wm = w & 1, wn = w >> 1;
  const int l32 = lane & 31, lhi = lane >> 5;
  const int oa = AK ? wm * 8192 + l32 * 32 : lhi * 2048 + wm * 128 + 4 * l32;
  const int ob = 1024 + (BKM ? wn * 4096 + l32 * 32 : lhi * 2048 + wn * 64 + 2 * l32);
  float* const wave_stage = lds + w * 2048 + 1024;
  int sw[4];
#pragma unroll
  for (int kg = 0; kg < 4; ++kg) sw[kg] = 4 * ((2 * kg + lhi) ^ ((l32 / 2) % 8));
  const unsigned nt = g.nt;
  const size_t stepa = AK ? kWK : size_t(kWK) * g.lda, stepb = BKM ? kWK : size_t(kWK) * g.ldb;

  // work of this block: one whole tile, or a run of k-tiles that may cross from one tile into the next
  unsigned u0, u1, tile_base, run = 0;
  if (blockIdx.x < g.direct_tiles) {
    tile_base = blockIdx.x;
    u0 = 0;
    u1 = nt;
  } else {
    run = blockIdx.x - g.direct_tiles;
    tile_base = g.direct_tiles;
    u0 = run * g.per;
    u1 = min(g.rem_units, u0 + g.per);
  }
  for (unsigned ti = u0 / nt; ti * nt < u1; ++ti) {
    const unsigned tile = tile_base + ti;
    const unsigned kt0 = max(u0, ti * nt) - ti * nt, kt1 = min(u1, (ti + 1) * nt) - ti * nt;
    const unsigned tm = tile % g.tiles_m, tn = tile / g.tiles_m;
    const unsigned m0 = tm * kWT, n0 = tn * kWT;
    floatx16 acc[2][4];
#pragma unroll
    for (int u = 0; u < 2; ++u)
#pragma unroll
      for (int t = 0; t < 4; ++t)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[u][t][r] = 0.f;
    unsigned offa[4], offb[4];
    load_offsets<AK>(offa, g.lda, m0, g.M);
    load_offsets<BKM>(offb, g.ldb, n0, g.N);
    __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0): loads of the previous tile still on their way into LDS
    __syncthreads();                     // and every wave has left its stages
    {
      const unsigned second = kt0 + 1 < kt1 ? kt0 + 1 : kt0;
      load_chunks<0>(g.A + kt0 * stepa, offa, wave_stage);
      load_chunks<1>(g.B + kt0 * stepb, offb, wave_stage);
      load_chunks<0>(g.A + second * stepa, offa, wave_stage + kStageFloats);
      load_chunks<1>(g.B + second * stepb, offb, wave_stage + kStageFloats);
    }
    __builtin_amdgcn_s_waitcnt(0x0F70);
    __syncthreads();
    float a[2][4][4], b[2][4][2];
    read_a<AK>(a[0], lds + oa, 0, sw);
    read_b<BKM>(b[0], lds + ob, 0, sw);
    for (unsigned i = kt0; i < kt1; ++i) {
      const int buf = (i - kt0) & 1;
      const float* la = lds + buf * kStageFloats + oa;
      const float* lb = lds + buf * kStageFloats + ob;
#pragma unroll
      for (int kg = 0; kg < 4; ++kg) {
        const int cur = kg & 1;
        if (kg == 3) {
          // every wave holds its last fragments of this stage, and the loads into the other stage (issued one k-tile
          // ago) have landed
          __builtin_amdgcn_s_waitcnt(0x0F70);
          __syncthreads();
        }
#pragma unroll
        for (int u = 0; u < 2; ++u)
#pragma unroll
          for (int t = 0; t < 4; ++t)
            acc[u][t] = __builtin_amdgcn_mfma_f32_32x32x2f32(b[cur][0][u], a[cur][0][t], acc[u][t], 0, 0, 0);
        __builtin_amdgcn_sched_barrier(0);
        if (kg < 3) {
          read_a<AK>(a[cur ^ 1], la, kg + 1, sw);
          read_b<BKM>(b[cur ^ 1], lb, kg + 1, sw);
        } else {
          // refill this stage two k-tiles ahead (the last two iterations reload the last k-tile, unconditional loads
          // keep the loop free of branches) and fetch the next k-tile's first fragments
          const unsigned nx = i + 2 < kt1 ? i + 2 : kt1 - 1;
          load_chunks<0>(g.A + nx * stepa, offa, wave_stage + buf * kStageFloats);
          load_chunks<1>(g.B + nx * stepb, offb, wave_stage + buf * kStageFloats);
          read_a<AK>(a[0], lds + (buf ^ 1) * kStageFloats + oa, 0, sw);
          read_b<BKM>(b[0], lds + (buf ^ 1) * kStageFloats + ob, 0, sw);
        }
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int s = 1; s < 4; ++s)
#pragma unroll
          for (int u = 0; u < 2; ++u)
#pragma unroll
            for (int t = 0; t < 4; ++t)
              acc[u][t] = __builtin_amdgcn_mfma_f32_32x32x2f32(b[cur][s][u], a[cur][s][t], acc[u][t], 0, 0, 0);
        __builtin_amdgcn_sched_barrier(0);
      }
    }

    // write back.  acc[u][t][r] of lane l: m = AK ? 32 t + l%32 : 4 (l%32) + t (+ 128 wm),
    // n = BKM ? 32 u + i : 2 i + u (+ 64 wn) with i = 8 (r/4) + 4 (l/32) + r%4
    const bool whole = kt0 == 0 && kt1 == nt;
    float* out = whole ? g.C + m0 + size_t(n0) * g.M : g.slots + size_t(run + ti) * kSlotFloats;
    const unsigned ldo = whole ? g.M : kWT;
    const unsigned mlim = whole ? g.M - m0 : kWT, nlim = whole ? g.N - n0 : kWT;
    const float beta = whole && g.bias == nullptr ? g.beta : 0.f;
    const bool add_bias = whole && g.bias != nullptr;
#pragma unroll
    for (int u = 0; u < 2; ++u)
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int i = 8 * (r / 4) + 4 * lhi + (r % 4);
        const unsigned n = wn * 64 + (BKM ? 32 * u + i : 2 * i + u);
        if (n >= nlim) continue;
        if (!AK) {
          const unsigned m = wm * 128 + 4 * l32;
          if (m >= mlim) continue;
          float* p = out + m + size_t(n) * ldo;
          float4 v = make_float4(acc[u][0][r], acc[u][1][r], acc[u][2][r], acc[u][3][r]);
          if (add_bias) {
            const float4 o = *reinterpret_cast<const float4*>(g.bias + m0 + m);
            v.x += o.x; v.y += o.y; v.z += o.z; v.w += o.w;
          } else if (beta != 0.f) {
            const float4 o = *reinterpret_cast<const float4*>(p);
            v.x += beta * o.x; v.y += beta * o.y; v.z += beta * o.z; v.w += beta * o.w;
          }
          *reinterpret_cast<float4*>(p) = v;
        } else {
#pragma unroll
          for (int t = 0; t < 4; ++t) {
            const unsigned m = wm * 128 + 32 * t + l32;
            if (m >= mlim) continue;
            float* p = out + m + size_t(n) * ldo;
            float v = acc[u][t][r];
            if (add_bias) v += g.bias[m0 + m];
            else if (beta != 0.f) v += beta * *p;
            *p = v;
          }
        }
      }
  }
}

// C tile = epilogue(sum of the partial tiles of its runs, in run order).  Block (x, y): 16 columns y of remaining
// tile x, one thread per four consecutive m (scalar when M is not a multiple of 4).
__global__ __launch_bounds__(256) void gemm_wide_fixup_kernel(WideArgs g) {
  const unsigned nt = g.nt, ti = blockIdx.x;
  const unsigned r0 = (ti * nt) / g.per, r1 = min(((ti + 1) * nt - 1) / g.per, (g.rem_units - 1) / g.per);
  if (r0 == r1) return;  // one run had the whole tile and wrote it itself
  const unsigned tile = g.direct_tiles + ti, tm = tile % g.tiles_m, tn = tile / g.tiles_m;
  const unsigned ml = (threadIdx.x % 64) * 4, m = tm * kWT + ml;
  const bool vec = g.M % 4 == 0;
#pragma unroll
  for (int c = 0; c < 4; ++c) {
    const unsigned nl = blockIdx.y * 16 + (threadIdx.x / 64) * 4 + c, n = tn * kWT + nl;
    if (m >= g.M || n >= g.N) continue;
    const size_t e = ml + size_t(nl) * kWT;
    float4 s = *reinterpret_cast<const float4*>(g.slots + size_t(r0 + ti) * kSlotFloats + e);
    for (unsigned r = r0 + 1; r <= r1; ++r) {
      const float4 v = *reinterpret_cast<const float4*>(g.slots + size_t(r + ti) * kSlotFloats + e);
      s.x += v.x; s.y += v.y; s.z += v.z; s.w += v.w;
    }
    float* p = g.C + m + size_t(n) * g.M;
    float sv[4] = {s.x, s.y, s.z, s.w};
    if (vec) {
      if (g.bias != nullptr) {
        const float4 o = *reinterpret_cast<const float4*>(g.bias + m);
        s.x += o.x; s.y += o.y; s.z += o.z; s.w += o.w;
      } else if (g.beta != 0.f) {
        const float4 o = *reinterpret_cast<const float4*>(p);
        s.x += g.beta * o.x; s.y += g.beta * o.y; s.z += g.beta * o.z; s.w += g.beta * o.w;
      }
      *reinterpret_cast<float4*>(p) = s;
    } else {
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        if (m + j >= g.M) break;
        float v = sv[j];
        if (g.bias != nullptr) v += g.bias[m + j];
        else if (g.beta != 0.f) v += g.beta * p[j];
        p[j] = v;
      }
    }
  }
}

// ---- shallow products: C[M x N] = beta*C + A[M x K] * B[N x K]^T with K <= 128 (the weight gradient of one timestep:
// K is the batch) -----------------------------------------------------------------------------------------------
// With four k-tiles a pipelined loop never fills: set-up, the exposed latency of each k-tile and the read-modify-write
// of C add up to more than the MFMAs.  Here a 512-thread block owns a 128 x 128 tile and fetches BOTH operand tiles
// whole (2 x 64 KiB, straight into LDS) plus its part of the old C in one burst at the start, so the block pays one
// memory latency, then 128 MFMAs per wave, then stores.  Wave w (2 x 4 over the tile) owns 64 m x 32 n.
// LDS: [half h of the depth][wave w][A 4 KiB][B 4 KiB]; the 1 KiB chunk u of wave w in half h holds rows
// k = 64h + 8w + 2u + {0, 1} of the operand tile (128 floats each), so that each half is one M0 window per wave.
struct ShallowArgs {
  const float* A;
  const float* B;
  float* C;
  unsigned lda, ldb;
  unsigned M, N, K;
  unsigned tiles_m;
  float beta;
};

constexpr size_t kShallowLdsBytes = sizeof(float) * 2 * kStageFloats;

__global__ __launch_bounds__(kWideThreads, 1) void gemm_shallow_nt_kernel(ShallowArgs g) {
  extern __shared__ __attribute__((aligned(16))) float lds[];
  const unsigned lane = threadIdx.x & 63, w = threadIdx.x >> 6;
  const unsigned wm = w & 1, wn = w >> 1, l32 = lane & 31, lhi = lane >> 5;
  const unsigned tm = blockIdx.x % g.tiles_m, tn = blockIdx.x / g.tiles_m;
  const unsigned m0 = tm * 128, n0 = tn * 128;

  // old C of this lane's outputs: m = m0 + 64 wm + 2 l32 + {0, 1}, n = n0 + 32 wn + i, i = 8 (r/4) + 4 lhi + r%4
  const unsigned m = m0 + wm * 64 + 2 * l32;
  fvec2 cold[16];
  if (g.beta != 0.f) {
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      const unsigned n = n0 + wn * 32 + 8 * (r / 4) + 4 * lhi + (r % 4);
      cold[r] = fvec2{0.f, 0.f};
      if (m < g.M && n < g.N) cold[r] = *reinterpret_cast<const fvec2*>(g.C + m + size_t(n) * g.M);
    }
  }
  // operand tiles: rows past the depth are not fetched (nor read), groups of four past the edge are clamped
  unsigned am = m0 + 4 * l32, bn = n0 + 4 * l32;
  am = am < g.M ? am : g.M - 4;
  bn = bn < g.N ? bn : g.N - 4;
#define DYHIP_SHALLOW_LOADS(h)                                                                                     \
  {                                                                                                                \
    float* window = lds + (h) * kStageFloats + w * 2048 + 1024;                                                    \
    const unsigned k0 = 64 * (h) + 8 * w + lhi;                                                                    \
    const float* pa = g.A + am + size_t(k0) * g.lda;                                                               \
    const float* pb = g.B + bn + size_t(k0) * g.ldb;                                                               \
    if (64 * (h) + 8 * w + 0 < g.K) {                                                                              \
      __builtin_amdgcn_global_load_lds((global_ptr_t)(pa + 1024), (lds_ptr_t)window, 16, -4096, 0);                \
      __builtin_amdgcn_global_load_lds((global_ptr_t)(pb), (lds_ptr_t)window, 16, 0, 0);                           \
    }                                                                                                              \
    if (64 * (h) + 8 * w + 2 < g.K) {                                                                              \
      __builtin_amdgcn_global_load_lds((global_ptr_t)(pa + 2 * size_t(g.lda) + 768), (lds_ptr_t)window, 16, -3072, 0); \
      __builtin_amdgcn_global_load_lds((global_ptr_t)(pb + 2 * size_t(g.ldb) - 256), (lds_ptr_t)window, 16, 1024, 0);  \
    }                                                                                                              \
    if (64 * (h) + 8 * w + 4 < g.K) {                                                                              \
      __builtin_amdgcn_global_load_lds((global_ptr_t)(pa + 4 * size_t(g.lda) + 512), (lds_ptr_t)window, 16, -2048, 0); \
      __builtin_amdgcn_global_load_lds((global_ptr_t)(pb + 4 * size_t(g.ldb) - 512), (lds_ptr_t)window, 16, 2048, 0);  \
    }                                                                                                              \
    if (64 * (h) + 8 * w + 6 < g.K) {                                                                              \
      __builtin_amdgcn_global_load_lds((global_ptr_t)(pa + 6 * size_t(g.lda) + 256), (lds_ptr_t)window, 16, -1024, 0); \
      __builtin_amdgcn_global_load_lds((global_ptr_t)(pb + 6 * size_t(g.ldb) - 768), (lds_ptr_t)window, 16, 3072, 0);  \
    }                                                                                                              \
  }
  DYHIP_SHALLOW_LOADS(0)
  DYHIP_SHALLOW_LOADS(1)
#undef DYHIP_SHALLOW_LOADS

  floatx16 acc[2];
#pragma unroll
  for (int t = 0; t < 2; ++t)
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[t][r] = 0.f;
  // group kg (8 k) of half h: step s of lane half lhi is row k = 8 kg + 4 lhi + s, i.e. chunk 2 lhi + s/2 of wave kg%8
  const float* la = lds + lhi * 512 + wm * 64 + 2 * l32;
  const float* lb = lds + 1024 + lhi * 512 + wn * 32 + l32;
  const unsigned groups = g.K / 8;
  fvec2 a[2][4];
  float b[2][4];
#define DYHIP_SHALLOW_READ(buf, kg)                                                        \
  _Pragma("unroll") for (int s = 0; s < 4; ++s) {                                          \
    const unsigned o = ((kg) / 8) * kStageFloats + ((kg) % 8) * 2048 + (s / 2) * 256 + (s % 2) * 128; \
    a[buf][s] = *reinterpret_cast<const fvec2*>(la + o);                                   \
    b[buf][s] = lb[o];                                                                     \
  }
#define DYHIP_SHALLOW_MMA(buf)                                                                          \
  __builtin_amdgcn_sched_barrier(0);                                                                    \
  _Pragma("unroll") for (int s = 0; s < 4; ++s) {                                                       \
    acc[0] = __builtin_amdgcn_mfma_f32_32x32x2f32(b[buf][s], a[buf][s][0], acc[0], 0, 0, 0);            \
    acc[1] = __builtin_amdgcn_mfma_f32_32x32x2f32(b[buf][s], a[buf][s][1], acc[1], 0, 0, 0);            \
  }                                                                                                     \
  __builtin_amdgcn_sched_barrier(0);
  // the first half of the depth can start while the second is still on its way (only when the whole second half
  // was asked for, so that every wave has the same number of loads in flight)
  const bool two_phase = g.K == 128;
  if (two_phase) __builtin_amdgcn_s_waitcnt(0x0F78);  // vmcnt(8): the eight loads of the second half may be in flight
  else __builtin_amdgcn_s_waitcnt(0x0F70);
  __syncthreads();
  const unsigned first = two_phase ? 8 : groups;
  DYHIP_SHALLOW_READ(0, 0u)
  for (unsigned kg = 0; kg < first; kg += 2) {
    const unsigned k1 = kg + 1 < first ? kg + 1 : kg, k2 = kg + 2 < first ? kg + 2 : kg;
    DYHIP_SHALLOW_READ(1, k1)
    DYHIP_SHALLOW_MMA(0)
    DYHIP_SHALLOW_READ(0, k2)
    if (kg + 1 < first) { DYHIP_SHALLOW_MMA(1) }
  }
  if (two_phase) {
    __builtin_amdgcn_s_waitcnt(0x0F70);
    __syncthreads();
    DYHIP_SHALLOW_READ(0, 8u)
    for (unsigned kg = 8; kg < 16; kg += 2) {
      const unsigned k2 = kg + 2 < 16 ? kg + 2 : kg;
      DYHIP_SHALLOW_READ(1, kg + 1)
      DYHIP_SHALLOW_MMA(0)
      DYHIP_SHALLOW_READ(0, k2)
      DYHIP_SHALLOW_MMA(1)
    }
  }
#undef DYHIP_SHALLOW_READ
#undef DYHIP_SHALLOW_MMA
  if (m >= g.M) return;
#pragma unroll
  for (int r = 0; r < 16; ++r) {
    const unsigned n = n0 + wn * 32 + 8 * (r / 4) + 4 * lhi + (r % 4);
    if (n >= g.N) continue;
    fvec2 v = fvec2{acc[0][r], acc[1][r]};
    if (g.beta != 0.f) v += g.beta * cold[r];
    *reinterpret_cast<fvec2*>(g.C + m + size_t(n) * g.M) = v;
  }
}

template <bool AK, bool BKM>
int launch_wide(dyhip_device* dev, const WideArgs& g, unsigned blocks, unsigned bit) {
  const void* fn = reinterpret_cast<const void*>(&gemm_wide_kernel<AK, BKM>);
  if ((dev->wide_gemm_ready & (1u << bit)) == 0) {  // 128 KiB of LDS need the opt-in, once per device
    DYHIP_CHECK_HIP(hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, int(kWideLdsBytes)));
    dev->wide_gemm_ready |= 1u << bit;
  }
  hipLaunchKernelGGL((gemm_wide_kernel<AK, BKM>), dim3(blocks), dim3(kWideThreads), kWideLdsBytes, dev->stream, g);
  return DYHIP_OK;
}

}  // namespace

// How the tiles are dealt to the blocks.  ok = false: leave the problem to the 128-wide kernel.
struct WidePlan {
  bool ok;
  unsigned tiles_m, nt, direct_tiles, rem, per, runs;
};

static WidePlan plan_wide(const dyhip_device* dev, size_t M, size_t N, size_t K32) {
  const unsigned cus = dev->num_cus > 0 ? unsigned(dev->num_cus) : 256;
  WidePlan p{};
  p.tiles_m = unsigned(cdiv<size_t>(M, kWT));
  p.nt = unsigned(K32 / kWK);
  const unsigned tiles = p.tiles_m * unsigned(cdiv<size_t>(N, kWT));
  p.direct_tiles = tiles / cus * cus;
  p.rem = tiles - p.direct_tiles;
  p.per = p.nt;
  p.runs = p.rem;
  if (p.rem > 0) {
    const unsigned units = p.rem * p.nt, per = cdiv<unsigned>(units, cus), runs = cdiv<unsigned>(units, per);
    // a run costs `per` k-tiles (~7.5 us each); a partial tile is written and read once more (~0.2 us over the GPU)
    if (per + (runs + p.rem) / 40 < p.nt) {
      p.per = per;
      p.runs = runs;
    }
  }
  // Measured against the 128-wide kernel: a block's set-up, its 256 KiB of output and the second kernel cost about
  // three k-tiles, so runs must be long (a problem of fewer tiles than CUs is nothing but runs), and a cut remainder
  // after full rounds pays only under deep tiles.
  // A last round of whole tiles is only worth a round when it is mostly full.
  const bool split = p.per < p.nt;
  if (p.direct_tiles == 0) p.ok = split ? p.per >= 16 : p.nt >= 16 && p.rem * 4 >= cus * 3;
  else p.ok = split ? p.nt >= 16 : p.nt >= 8 && (p.rem == 0 || p.rem * 4 >= cus * 3);
  return p;
}

bool gemm_wide_eligible(const dyhip_device* dev, bool a_kmajor, bool b_kmajor, size_t M, size_t N, size_t K,
                        const float* A, size_t lda, const float* B, size_t ldb, const float* C) {
  const size_t K32 = K / kWK * kWK;
  if (K32 < 256 || M < 192 || N < 192 || dev->max_lds_per_block < kWideLdsBytes) return false;
  if (!aligned16(A) || !aligned16(B) || !aligned16(C) || lda % 4 != 0 || ldb % 4 != 0) return false;
  if ((!a_kmajor && M % 4 != 0) || (!b_kmajor && N % 4 != 0)) return false;
  // 32-bit element offsets inside the kernel
  const size_t span_a = a_kmajor ? M * lda : K * lda, span_b = b_kmajor ? N * ldb : K * ldb;
  if (span_a >= (size_t(1) << 31) || span_b >= (size_t(1) << 31) || M * N >= (size_t(1) << 31)) return false;
  const size_t tiles = cdiv<size_t>(M, kWT) * cdiv<size_t>(N, kWT);
  const size_t cus = dev->num_cus > 0 ? size_t(dev->num_cus) : 256;
  // edge tiles compute whole 256 x 256 tiles: ragged shapes stay with the 128-wide kernel
  if (double(M) * double(N) < 0.8 * double(tiles) * double(kSlotFloats)) return false;
  if (dev->gemm_ws == nullptr || dev->gemm_ws_bytes < (2 * cus) * kSlotFloats * sizeof(float)) return false;
  return plan_wide(dev, M, N, K32).ok;
}

size_t gemm_wide_whole_rounds_columns(const dyhip_device* dev, bool a_kmajor, bool b_kmajor, size_t M, size_t N, size_t K,
                                      const float* A, size_t lda, const float* B, size_t ldb, const float* C) {
  const size_t cus = dev->num_cus > 0 ? size_t(dev->num_cus) : 256;
  const size_t tiles_m = cdiv<size_t>(M, kWT), tiles = tiles_m * cdiv<size_t>(N, kWT);
  const size_t direct = tiles / cus * cus;
  if (direct == 0 || direct == tiles || direct % tiles_m != 0) return 0;
  const size_t cols = direct / tiles_m * kWT;
  return cols < N && gemm_wide_eligible(dev, a_kmajor, b_kmajor, M, cols, K, A, lda, B, ldb, C) ? cols : 0;
}

int gemm_wide_run(dyhip_device* dev, bool a_kmajor, bool b_kmajor, size_t M, size_t N, size_t K32, const float* A,
                  size_t lda, const float* B, size_t ldb, float* C, float beta, const float* bias) {
  const WidePlan p = plan_wide(dev, M, N, K32);
  WideArgs g;
  g.A = A;
  g.B = B;
  g.C = C;
  g.bias = bias;
  g.slots = static_cast<float*>(dev->gemm_ws);
  g.lda = unsigned(lda);
  g.ldb = unsigned(ldb);
  g.M = unsigned(M);
  g.N = unsigned(N);
  g.nt = p.nt;
  g.tiles_m = p.tiles_m;
  g.beta = beta;
  g.direct_tiles = p.direct_tiles;
  g.rem_units = p.rem * p.nt;
  g.per = p.per;
  const unsigned blocks = p.direct_tiles + p.runs;
  int st;
  if (a_kmajor && b_kmajor) st = launch_wide<true, true>(dev, g, blocks, 0);
  else if (a_kmajor) st = launch_wide<true, false>(dev, g, blocks, 1);
  else if (b_kmajor) st = launch_wide<false, true>(dev, g, blocks, 2);
  else st = launch_wide<false, false>(dev, g, blocks, 3);
  DYHIP_CHECK_STATUS(st);
  DYHIP_CHECK_LAUNCH();
  if (g.per < g.nt) {
    hipLaunchKernelGGL(gemm_wide_fixup_kernel, dim3(p.rem, kWT / 16), dim3(256), 0, dev->stream, g);
    DYHIP_CHECK_LAUNCH();
  }
  return DYHIP_OK;
}

bool gemm_shallow_nt_eligible(const dyhip_device* dev, size_t M, size_t N, size_t K, const float* A, size_t lda,
                              const float* B, size_t ldb, const float* C) {
  if (K < 32 || K > 128 || K % 8 != 0 || M % 4 != 0 || N % 4 != 0 || M < 128 || N < 128) return false;
  if (dev->max_lds_per_block < kShallowLdsBytes) return false;
  if (!aligned16(A) || !aligned16(B) || lda % 4 != 0 || ldb % 4 != 0 || (reinterpret_cast<uintptr_t>(C) & 7u) != 0)
    return false;
  if (K * lda >= (size_t(1) << 31) || K * ldb >= (size_t(1) << 31) || M * N >= (size_t(1) << 31)) return false;
  const size_t cus = dev->num_cus > 0 ? size_t(dev->num_cus) : 256;
  return cdiv<size_t>(M, 128) * cdiv<size_t>(N, 128) * 2 >= cus;  // fewer tiles: the 128-wide kernel cuts the depth
}

int gemm_shallow_nt_run(dyhip_device* dev, size_t M, size_t N, size_t K, const float* A, size_t lda, const float* B,
                        size_t ldb, float* C, float beta) {
  ShallowArgs g;
  g.A = A;
  g.B = B;
  g.C = C;
  g.lda = unsigned(lda);
  g.ldb = unsigned(ldb);
  g.M = unsigned(M);
  g.N = unsigned(N);
  g.K = unsigned(K);
  g.tiles_m = unsigned(cdiv<size_t>(M, 128));
  g.beta = beta;
  if ((dev->wide_gemm_ready & (1u << 4)) == 0) {
    DYHIP_CHECK_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(&gemm_shallow_nt_kernel),
                                        hipFuncAttributeMaxDynamicSharedMemorySize, int(kShallowLdsBytes)));
    dev->wide_gemm_ready |= 1u << 4;
  }
  const unsigned blocks = g.tiles_m * unsigned(cdiv<size_t>(N, 128));
  hipLaunchKernelGGL(gemm_shallow_nt_kernel, dim3(blocks), dim3(kWideThreads), kShallowLdsBytes, dev->stream, g);
  DYHIP_CHECK_LAUNCH();
  return DYHIP_OK;
}

}  // namespace dyhip
