// Small products C = A * B in any of the three layouts (l*r, l^T*r, l*r^T), single or strided-batched, in one launch.
//
// The 128 x 128-tile kernel with its split over the depth and a second launch to sum the slices costs 9..18 us on
// products whose operands are a few hundred KB (128 x 128 x 128 as l^T*r: 9.4 us; 200 x 100 x 50: 13 us; 7 x 5 x 9
// times 1000 items: 11 us): that is launch and pipeline latency, not arithmetic.  Here a wavefront owns a 32 x 32
// tile of C and feeds v_mfma_f32_32x32x2_f32 straight from global memory (the operands stay in the L2s): lane l
// fetches, for row l % 32 of A and column l % 32 of B, the four depth indices 4 * (l / 32) .. + 3 of every group of
// eight, as one 128-bit load where the operand is contiguous along the depth and aligned, as four loads (adjacent
// lanes on adjacent floats when the operand is contiguous along its rows or columns) otherwise; two groups are in
// flight.  With KW = 4 the four wavefronts of a block split the depth of one tile and meet in LDS; with KW = 1 (a
// shallow depth) each takes a tile of its own.  B goes in as the first matrix-core operand: a lane's sixteen results
// then share the row l % 32 of the tile, and adjacent lanes store adjacent floats of C.
//
// Follows the products of dynet/nodes-matrixmultiply.cc:51-135 and nodes-affinetransform.cc:78-160 (cuBLAS sgemm and
// sgemmStridedBatched there); rows and columns past the matrix are computed on clamped addresses and not stored,
// depth indices past the end are zeroed in both operands.
#include <hip/hip_runtime.h>

#include <algorithm>

#include "gemm.h"

namespace dyhip {

typedef float smallx16 __attribute__((ext_vector_type(16)));

struct SmallGemmArgs {
  const float* A;
  const float* B;
  float* C;
  const float* bias;  // bias[m] replaces beta * C when set
  size_t sam, sak;    // A(m, k) = A[m * sam + k * sak]
  size_t sbk, sbn;    // B(k, n) = B[k * sbk + n * sbn]
  size_t stride_a, stride_b, stride_c;  // between the items of a batch
  unsigned M, N, K;
  unsigned kw;  // depth a wavefront takes (KW = 4), a multiple of 8
  float beta;
};

// the four depth indices base .. base + 3 of one row (or column) of an operand; `base + i >= kend` gives 0.
// VEC: floats a load along the depth (4 or 2: the operand is contiguous along the depth and aligned to that; 1: any
// stride).  Chunk ends are multiples of VEC, so a vector lies inside or outside as a whole.
template <int VEC>
__device__ __forceinline__ void small_fetch(const float* __restrict__ p, size_t sk, unsigned base, unsigned kbeg,
                                            unsigned kend, float (&v)[4]) {
  if (VEC == 4) {
    const bool in = base < kend;
    const float4 t = *reinterpret_cast<const float4*>(p + (in ? base : kbeg));
    v[0] = in ? t.x : 0.f;
    v[1] = in ? t.y : 0.f;
    v[2] = in ? t.z : 0.f;
    v[3] = in ? t.w : 0.f;
  } else if (VEC == 2) {
#pragma unroll
    for (int i = 0; i < 4; i += 2) {
      const bool in = base + i < kend;
      const float2 t = *reinterpret_cast<const float2*>(p + (in ? base + i : kbeg));
      v[i] = in ? t.x : 0.f;
      v[i + 1] = in ? t.y : 0.f;
    }
  } else {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const bool in = base + i < kend;
      const float t = p[size_t(in ? base + i : kbeg) * sk];
      v[i] = in ? t : 0.f;
    }
  }
}

constexpr int kSmallGroups = 4;  // groups of eight depth indices a stage: 32 indices, 16 values of each operand a lane

// KW: wavefronts that split the depth of one tile (8 or 4; the block has KW wavefronts), or 1: four wavefronts, a tile
// each.  The next stage's loads are issued before the current stage's matrix-core steps.
template <int AVEC, int BVEC, int KW>
__global__ __launch_bounds__(KW == 1 ? 256 : 64 * KW) void gemm_small_kernel(SmallGemmArgs g) {
  __shared__ float red[KW > 1 ? KW * 16 * 64 : 1];
  constexpr int T = kSmallGroups;
  const unsigned lane = threadIdx.x & 63, w = threadIdx.x >> 6, h = lane >> 5, q = lane & 31;
  const unsigned mt = KW > 1 ? blockIdx.x : blockIdx.x * 4 + w, nt = blockIdx.y;
  if (KW == 1 && mt * 32 >= g.M) return;  // whole wavefronts; this form has no barrier
  const unsigned kbeg = KW > 1 ? w * g.kw : 0, kend = KW > 1 ? min(g.K, kbeg + g.kw) : g.K;
  const unsigned m = mt * 32 + q, n = nt * 32 + q;
  const float* pa = g.A + size_t(blockIdx.z) * g.stride_a + size_t(m < g.M ? m : g.M - 1) * g.sam;
  const float* pb = g.B + size_t(blockIdx.z) * g.stride_b + size_t(n < g.N ? n : g.N - 1) * g.sbn;
  smallx16 acc = {0};
  float a0[T][4], b0[T][4], a1[T][4], b1[T][4];
  auto fetch = [&](float (&a)[T][4], float (&b)[T][4], unsigned k0) {
    if (k0 < kend) {
#pragma unroll
      for (int t = 0; t < T; ++t) {
        small_fetch<AVEC>(pa, g.sak, k0 + 8 * t + 4 * h, kbeg, kend, a[t]);
        small_fetch<BVEC>(pb, g.sbk, k0 + 8 * t + 4 * h, kbeg, kend, b[t]);
      }
    }
  };
  auto steps = [&](const float (&a)[T][4], const float (&b)[T][4], unsigned k0) {
    if (k0 < kend) {
#pragma unroll
      for (int t = 0; t < T; ++t)
#pragma unroll
        for (int i = 0; i < 4; ++i) acc = __builtin_amdgcn_mfma_f32_32x32x2f32(b[t][i], a[t][i], acc, 0, 0, 0);
    }
  };
  fetch(a0, b0, kbeg);
  for (unsigned k0 = kbeg; k0 < kend; k0 += 16 * T) {
    fetch(a1, b1, k0 + 8 * T);
    steps(a0, b0, k0);
    fetch(a0, b0, k0 + 16 * T);
    steps(a1, b1, k0 + 8 * T);
  }
  // register r of lane l: column 8 * (r / 4) + 4 * (l / 32) + r % 4 of the tile, row l % 32
  float* pc = g.C + size_t(blockIdx.z) * g.stride_c;
  const float add = g.bias != nullptr && m < g.M ? g.bias[m] : 0.f;
  if (KW > 1) {
#pragma unroll
    for (int r = 0; r < 16; ++r) red[(w * 16 + r) * 64 + lane] = acc[r];
    __syncthreads();
    constexpr int PER = 16 / KW;  // registers a wavefront finishes
#pragma unroll
    for (int rr = 0; rr < PER; ++rr) {
      const unsigned r = w * PER + rr;
      float v = red[r * 64 + lane];
#pragma unroll
      for (int x = 1; x < KW; ++x) v += red[(x * 16 + r) * 64 + lane];
      const unsigned col = nt * 32 + 8 * (r / 4) + 4 * h + r % 4;
      if (m < g.M && col < g.N) {
        float* out = pc + size_t(col) * g.M + m;
        *out = g.bias != nullptr ? add + v : (g.beta == 0.f ? v : g.beta * *out + v);
      }
    }
  } else {
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      const unsigned col = nt * 32 + 8 * (r / 4) + 4 * h + r % 4;
      if (m < g.M && col < g.N) {
        float* out = pc + size_t(col) * g.M + m;
        *out = g.bias != nullptr ? add + acc[r] : (g.beta == 0.f ? acc[r] : g.beta * *out + acc[r]);
      }
    }
  }
}

// wavefronts that split the depth of a tile: all four (or eight) of a block unless the depth is shallow and there are
// tiles enough for every CU; eight when each still gets two stages and the tiles do not fill the device
static int small_depth_waves(size_t K, size_t tiles, size_t cus) {
  if (!(K > 64 || (K > 16 && tiles < 2 * cus))) return 1;
  return K >= 512 && tiles <= 2 * cus ? 8 : 4;
}

// Which products come here instead of the 128 x 128-tile kernel (measured on 60 shapes in the three layouts).  A
// wavefront's depth costs one memory round trip per stage of 32 indices, hidden only by other blocks on the CU, and
// nothing is reused through LDS: the tile kernel wins from about four stages per wavefront on, unless it would run
// its scalar-load form (operands not 16-byte aligned or leading dimensions not multiples of four), which is two to
// ten times slower on narrow outputs.
bool gemm_small_eligible(const dyhip_device* dev, size_t M, size_t N, size_t K, const GemmEpiParams& epi, unsigned batch,
                         bool tile_kernel_vectorizes) {
  if (epi.kind != kEpiAxpby && !(epi.kind == kEpiBias && epi.bias != nullptr)) return false;
  if (M == 0 || N == 0 || K == 0 || M > (size_t(1) << 20) || N > (size_t(1) << 20) || K > 65536 || batch > 65535u) return false;
  const size_t cus = dev->num_cus > 0 ? size_t(dev->num_cus) : 256;
  const size_t tiles = cdiv<size_t>(M, 32) * cdiv<size_t>(N, 32) * (batch > 0 ? batch : 1);
  const size_t work = tiles * cdiv<size_t>(K, 32);  // in units of one tile x one stage
  if (tiles > 16 * cus || work > 64 * cus) return false;
  const size_t stages = cdiv<size_t>(cdiv<size_t>(K, small_depth_waves(K, tiles, cus)), 8 * kSmallGroups);
  if (stages <= 3 || (stages <= 4 && tiles <= cus / 2)) return true;
  if (batch > 1) return true;  // the tile kernel does not split the depth of batch items
  if (tile_kernel_vectorizes) return false;
  return N <= 4 || (stages <= 6 && tiles >= cus);
}

int gemm_small_run(dyhip_device* dev, bool a_kmajor, bool b_kmajor, size_t M, size_t N, const GemmSeg& s, float* C,
                   const GemmEpiParams& epi, const GemmBatch* batch) {
  SmallGemmArgs g;
  g.A = s.A;
  g.B = s.B;
  g.C = C;
  g.bias = epi.kind == kEpiBias ? epi.bias : nullptr;
  g.beta = epi.kind == kEpiAxpby ? epi.beta : 0.f;
  g.sam = a_kmajor ? s.lda : 1;
  g.sak = a_kmajor ? 1 : s.lda;
  g.sbk = b_kmajor ? 1 : s.ldb;
  g.sbn = b_kmajor ? s.ldb : 1;
  const unsigned items = batch != nullptr && batch->count > 1 ? batch->count : 1;
  g.stride_a = items > 1 ? batch->stride_a : 0;
  g.stride_b = items > 1 ? batch->stride_b : 0;
  g.stride_c = items > 1 ? batch->stride_c : 0;
  g.M = static_cast<unsigned>(M);
  g.N = static_cast<unsigned>(N);
  g.K = static_cast<unsigned>(s.K);
  const unsigned tm = cdiv<unsigned>(g.M, 32), tn = cdiv<unsigned>(g.N, 32);
  const size_t cus = dev->num_cus > 0 ? size_t(dev->num_cus) : 256;
  const size_t tiles = size_t(tm) * tn * items;
  const int kwaves = small_depth_waves(g.K, tiles, cus);
  g.kw = kwaves > 1 ? cdiv<unsigned>(cdiv<unsigned>(g.K, kwaves), 8) * 8 : g.K;
  auto width = [&](bool kmajor, const float* p, size_t ld, size_t stride) {
    if (!kmajor) return 1;
    if (g.K % 4 == 0 && ld % 4 == 0 && stride % 4 == 0 && aligned16(p)) return 4;
    if (g.K % 2 == 0 && ld % 2 == 0 && stride % 2 == 0 && reinterpret_cast<uintptr_t>(p) % 8 == 0) return 2;
    return 1;
  };
  const int av = width(a_kmajor, s.A, s.lda, g.stride_a), bv = width(b_kmajor, s.B, s.ldb, g.stride_b);
  const dim3 grid(kwaves > 1 ? tm : cdiv<unsigned>(tm, 4), tn, items);
#define DYHIP_SMALL_KW(AV, BV)                                                                                       \
  do {                                                                                                               \
    if (kwaves == 8) hipLaunchKernelGGL((gemm_small_kernel<AV, BV, 8>), grid, dim3(512), 0, dev->stream, g);         \
    else if (kwaves == 4) hipLaunchKernelGGL((gemm_small_kernel<AV, BV, 4>), grid, dim3(256), 0, dev->stream, g);    \
    else hipLaunchKernelGGL((gemm_small_kernel<AV, BV, 1>), grid, dim3(256), 0, dev->stream, g);                     \
  } while (0)
#define DYHIP_SMALL_B(AV)                     \
  do {                                        \
    if (bv == 4) DYHIP_SMALL_KW(AV, 4);       \
    else if (bv == 2) DYHIP_SMALL_KW(AV, 2);  \
    else DYHIP_SMALL_KW(AV, 1);               \
  } while (0)
  if (av == 4) DYHIP_SMALL_B(4);
  else if (av == 2) DYHIP_SMALL_B(2);
  else DYHIP_SMALL_B(1);
#undef DYHIP_SMALL_B
#undef DYHIP_SMALL_KW
  DYHIP_CHECK_LAUNCH();
  return DYHIP_OK;
}

}  // namespace dyhip
