// fp32 GEMM on the CDNA matrix cores (v_mfma_f32_32x32x2_f32: fp32 inputs,
// fp32 accumulate, no reduced-precision shortcut), in the three forms DyNet's
// GEMM shim needs (dynet/matrix-multiply.h:16-37,97-117,162-180), replacing its
// cublasSgemm calls.
//
// Tiling: a 256-thread block (4 wavefronts) owns a 128 x (32*TN) tile of C.
// Wavefront w owns rows [32w, 32w+32) and TN accumulators of 32x32 (16 VGPRs
// each).  K advances in steps of 16 through a double-buffered LDS stage: while
// the matrix cores work on stage s, the global loads of stage s+1 are already
// in flight in registers.  Operand tiles are kept in LDS in whichever of two
// layouts makes both the 128-bit global load and the per-lane MFMA operand read
// conflict-free:
//   "MN-major" operand (contiguous along the C row/column index):  lds[k][mn]
//   "K-major"  operand (contiguous along K, i.e. a transposed one): lds[mn][k], pitch 17
// MFMA 32x32x2 operand mapping: lane l supplies A(i = l%32, k = l/32) and
// B(k = l/32, j = l%32); accumulator register r of lane l is
// C(i = 8*(r/4) + 4*(l/32) + r%4, j = l%32).
//
// Skinny problems (the LSTM gate GEMMs have N = batch) do not have enough
// tiles to fill 256 CUs, so K is split across blocks; each split writes its
// partial tile to a device-owned workspace and a second kernel adds the splits
// in ascending order (deterministic, no atomics) and applies the epilogue:
// either C = beta*C + sum, or the fused LSTM gate epilogue (bias, +1 forget
// bias, logistic / tanh).
#include "gemm.h"

namespace dyhip {

typedef float floatx16 __attribute__((ext_vector_type(16)));

constexpr int kBM = 128;
constexpr int kBK = 16;
constexpr int kGemmThreads = 256;
constexpr int kKPitch = kBK + 1;  // row pitch of the K-major LDS layout

struct GemmArgs {
  GemmSeg seg[kGemmMaxSeg];
  int nseg;
  unsigned ktiles[kGemmMaxSeg];  // k-tiles per segment
  unsigned ktiles_total;
  unsigned ktiles_per_split;
  size_t M, N;
  float* C;         // used when partial == nullptr
  float beta;       // used when partial == nullptr
  const float* bias;  // when set (and partial == nullptr): C = bias[i] + sum
  float* partial;   // [splits][M*N] or nullptr
};

// ---- global -> register tile loads ------------------------------------------------
// A tile is W (mn extent) x 16 (k extent) floats = W*4 float4.  Thread t loads
// float4 number f = t + 256*u.
template <int W>
struct TileRegs {
  static constexpr int NV = (W * 4 + kGemmThreads - 1) / kGemmThreads;
  float4 v[NV];
};

template <bool KMAJOR, int W>
__device__ __forceinline__ void load_tile(TileRegs<W>& r, const float* __restrict__ p, size_t ld, size_t mn0,
                                          size_t k0, size_t MN, size_t K, bool vec_ok) {
#pragma unroll
  for (int u = 0; u < TileRegs<W>::NV; ++u) {
    const int f = threadIdx.x + kGemmThreads * u;
    float4 val = make_float4(0.f, 0.f, 0.f, 0.f);
    if (f < W * 4) {
      if (!KMAJOR) {
        // float4 along mn at fixed k: W/4 float4 per k row
        const int k = f / (W / 4), m4 = f % (W / 4);
        const size_t mn = mn0 + size_t(m4) * 4, kk = k0 + k;
        if (kk < K && mn < MN) {
          const float* q = p + mn + kk * ld;
          if (vec_ok && mn + 3 < MN) {
            val = *reinterpret_cast<const float4*>(q);
          } else {
            val.x = q[0];
            if (mn + 1 < MN) val.y = q[1];
            if (mn + 2 < MN) val.z = q[2];
            if (mn + 3 < MN) val.w = q[3];
          }
        }
      } else {
        // float4 along k at fixed mn: 4 float4 per mn row
        const int mn_l = f / 4, k4 = f % 4;
        const size_t mn = mn0 + mn_l, kk = k0 + size_t(k4) * 4;
        if (mn < MN && kk < K) {
          const float* q = p + kk + mn * ld;
          if (vec_ok && kk + 3 < K) {
            val = *reinterpret_cast<const float4*>(q);
          } else {
            val.x = q[0];
            if (kk + 1 < K) val.y = q[1];
            if (kk + 2 < K) val.z = q[2];
            if (kk + 3 < K) val.w = q[3];
          }
        }
      }
    }
    r.v[u] = val;
  }
}

template <bool KMAJOR, int W>
__device__ __forceinline__ void store_tile(const TileRegs<W>& r, float* __restrict__ lds) {
#pragma unroll
  for (int u = 0; u < TileRegs<W>::NV; ++u) {
    const int f = threadIdx.x + kGemmThreads * u;
    if (f < W * 4) {
      if (!KMAJOR) {
        const int k = f / (W / 4), m4 = f % (W / 4);
        *reinterpret_cast<float4*>(lds + k * W + m4 * 4) = r.v[u];
      } else {
        const int mn_l = f / 4, k4 = f % 4;
        float* q = lds + mn_l * kKPitch + k4 * 4;
        q[0] = r.v[u].x;
        q[1] = r.v[u].y;
        q[2] = r.v[u].z;
        q[3] = r.v[u].w;
      }
    }
  }
}

template <bool KMAJOR, int W>
__device__ __forceinline__ float lds_operand(const float* __restrict__ lds, int mn, int k) {
  return KMAJOR ? lds[mn * kKPitch + k] : lds[k * W + mn];
}

template <bool KMAJOR, int W>
constexpr int tile_floats() {
  return KMAJOR ? W * kKPitch : W * kBK;
}

template <bool A_KMAJOR, bool B_KMAJOR, int TN>
__global__ __launch_bounds__(kGemmThreads) void gemm_tile_kernel(GemmArgs g, unsigned tiles_m, int a_vec, int b_vec) {
  constexpr int BN = 32 * TN;
  constexpr int A_FLOATS = tile_floats<A_KMAJOR, kBM>();
  constexpr int B_FLOATS = tile_floats<B_KMAJOR, BN>();
  __shared__ __attribute__((aligned(16))) float lds_a[2][A_FLOATS];
  __shared__ __attribute__((aligned(16))) float lds_b[2][B_FLOATS];

  const unsigned tm = blockIdx.x % tiles_m, tn = blockIdx.x / tiles_m;
  const unsigned split = blockIdx.y;
  const size_t m0 = size_t(tm) * kBM, n0 = size_t(tn) * BN;
  const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
  const int l32 = lane & 31, lhi = lane >> 5;

  floatx16 acc[TN];
#pragma unroll
  for (int t = 0; t < TN; ++t)
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[t][r] = 0.f;

  const unsigned kt_begin = split * g.ktiles_per_split;
  const unsigned kt_end = min(g.ktiles_total, kt_begin + g.ktiles_per_split);

  unsigned seg_first = 0;
  for (int s = 0; s < g.nseg; ++s) {
    const unsigned seg_last = seg_first + g.ktiles[s];
    const unsigned lo = max(kt_begin, seg_first), hi = min(kt_end, seg_last);
    if (lo < hi) {
      const GemmSeg sg = g.seg[s];
      const unsigned nt = hi - lo;
      TileRegs<kBM> ra;
      TileRegs<BN> rb;
      size_t k0 = size_t(lo - seg_first) * kBK;
      load_tile<A_KMAJOR, kBM>(ra, sg.A, sg.lda, m0, k0, g.M, sg.K, a_vec);
      load_tile<B_KMAJOR, BN>(rb, sg.B, sg.ldb, n0, k0, g.N, sg.K, b_vec);
      __syncthreads();  // previous segment's readers are done with buffer 0
      store_tile<A_KMAJOR, kBM>(ra, lds_a[0]);
      store_tile<B_KMAJOR, BN>(rb, lds_b[0]);
      __syncthreads();
      for (unsigned t = 0; t < nt; ++t) {
        const int buf = t & 1;
        if (t + 1 < nt) {
          k0 += kBK;
          load_tile<A_KMAJOR, kBM>(ra, sg.A, sg.lda, m0, k0, g.M, sg.K, a_vec);
          load_tile<B_KMAJOR, BN>(rb, sg.B, sg.ldb, n0, k0, g.N, sg.K, b_vec);
        }
        const float* la = lds_a[buf];
        const float* lb = lds_b[buf];
#pragma unroll
        for (int kk = 0; kk < kBK; kk += 2) {
          const float a = lds_operand<A_KMAJOR, kBM>(la, 32 * w + l32, kk + lhi);
#pragma unroll
          for (int t2 = 0; t2 < TN; ++t2) {
            const float b = lds_operand<B_KMAJOR, BN>(lb, 32 * t2 + l32, kk + lhi);
            acc[t2] = __builtin_amdgcn_mfma_f32_32x32x2f32(a, b, acc[t2], 0, 0, 0);
          }
        }
        if (t + 1 < nt) {
          // buffer buf^1 was last read in iteration t-1, which every wave has left
          store_tile<A_KMAJOR, kBM>(ra, lds_a[buf ^ 1]);
          store_tile<B_KMAJOR, BN>(rb, lds_b[buf ^ 1]);
        }
        __syncthreads();
      }
    }
    seg_first = seg_last;
  }

  // ---- write back --------------------------------------------------------------
  float* out = g.partial ? g.partial + size_t(split) * g.M * g.N : g.C;
  const bool direct = g.partial == nullptr;
  const bool vec_store = (g.M % 4 == 0) && aligned16(out);
#pragma unroll
  for (int t2 = 0; t2 < TN; ++t2) {
    const size_t j = n0 + 32 * t2 + l32;
    if (j >= g.N) continue;
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      const size_t i = m0 + 32 * w + 8 * q + 4 * lhi;
      if (i >= g.M) continue;
      float* p = out + i + j * g.M;
      float4 v = make_float4(acc[t2][4 * q], acc[t2][4 * q + 1], acc[t2][4 * q + 2], acc[t2][4 * q + 3]);
      if (direct && g.bias != nullptr) {
        v.x += g.bias[i];
        if (i + 1 < g.M) v.y += g.bias[i + 1];
        if (i + 2 < g.M) v.z += g.bias[i + 2];
        if (i + 3 < g.M) v.w += g.bias[i + 3];
      }
      if (vec_store && i + 3 < g.M) {
        if (direct && g.beta != 0.f) {
          const float4 o = *reinterpret_cast<const float4*>(p);
          v.x = g.beta * o.x + v.x;
          v.y = g.beta * o.y + v.y;
          v.z = g.beta * o.z + v.z;
          v.w = g.beta * o.w + v.w;
        }
        *reinterpret_cast<float4*>(p) = v;
      } else {
        const float vv[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
        for (int c = 0; c < 4; ++c)
          if (i + c < g.M) p[c] = (direct && g.beta != 0.f) ? g.beta * p[c] + vv[c] : vv[c];
      }
    }
  }
}

// C[e] = epilogue(sum_s partial[s][e]), splits added in ascending order
template <int EPI>
__global__ __launch_bounds__(256) void gemm_splitk_reduce_kernel(size_t M, size_t total, unsigned splits,
                                                                 const float* __restrict__ partial,
                                                                 float* __restrict__ C, GemmEpiParams ep) {
  const size_t e = size_t(blockIdx.x) * 256 + threadIdx.x;
  if (e >= total) return;
  if (EPI == kEpiAxpby) {
    float s = partial[e];
    for (unsigned k = 1; k < splits; ++k) s += partial[size_t(k) * total + e];
    C[e] = ep.beta != 0.f ? ep.beta * C[e] + s : s;
  } else if (EPI == kEpiBias) {
    float s = ep.bias[e % M];
    for (unsigned k = 0; k < splits; ++k) s += partial[size_t(k) * total + e];
    C[e] = s;
  } else {
    const unsigned i = static_cast<unsigned>(e % M);
    float pre = ep.bias[i];
    if (i >= ep.H && i < 2 * ep.H) pre += 1.0f;  // forget-gate bias
    for (unsigned k = 0; k < splits; ++k) pre += partial[size_t(k) * total + e];
    C[e] = i < 3 * ep.H ? logistic(ep.logistic_mode, pre) : tanh_accurate(pre);
  }
}

template <bool A_KMAJOR, bool B_KMAJOR>
static void launch_tiles(dyhip_device* dev, const GemmArgs& g, unsigned tiles_m, unsigned tiles_n, unsigned splits,
                         int tn, int a_vec, int b_vec) {
  const dim3 grid(tiles_m * tiles_n, splits), block(kGemmThreads);
  if (tn == 1)
    hipLaunchKernelGGL((gemm_tile_kernel<A_KMAJOR, B_KMAJOR, 1>), grid, block, 0, dev->stream, g, tiles_m, a_vec, b_vec);
  else if (tn == 2)
    hipLaunchKernelGGL((gemm_tile_kernel<A_KMAJOR, B_KMAJOR, 2>), grid, block, 0, dev->stream, g, tiles_m, a_vec, b_vec);
  else
    hipLaunchKernelGGL((gemm_tile_kernel<A_KMAJOR, B_KMAJOR, 4>), grid, block, 0, dev->stream, g, tiles_m, a_vec, b_vec);
}

int gemm_run(dyhip_device* dev, bool a_kmajor, bool b_kmajor, size_t M, size_t N, int nseg, const GemmSeg* segs,
             float* C, const GemmEpiParams& epi) {
  if (M == 0 || N == 0) return DYHIP_OK;
  DYHIP_REQUIRE(nseg >= 1 && nseg <= kGemmMaxSeg, "GEMM supports 1..%d K segments", kGemmMaxSeg);
  DYHIP_REQUIRE(C != nullptr, "null GEMM output");
  GemmArgs g;
  g.nseg = nseg;
  g.M = M;
  g.N = N;
  g.C = C;
  g.beta = epi.kind == kEpiBias ? 0.f : epi.beta;
  g.bias = epi.kind == kEpiBias ? epi.bias : nullptr;
  g.ktiles_total = 0;
  bool a_vec = true, b_vec = true;
  for (int s = 0; s < nseg; ++s) {
    DYHIP_REQUIRE(segs[s].A != nullptr && segs[s].B != nullptr, "null GEMM operand");
    g.seg[s] = segs[s];
    g.ktiles[s] = static_cast<unsigned>(cdiv<size_t>(segs[s].K, kBK));
    g.ktiles_total += g.ktiles[s];
    a_vec = a_vec && aligned16(segs[s].A) && segs[s].lda % 4 == 0;
    b_vec = b_vec && aligned16(segs[s].B) && segs[s].ldb % 4 == 0;
  }
  const int tn = N <= 32 ? 1 : (N <= 64 ? 2 : 4);
  const size_t tiles_m = cdiv<size_t>(M, kBM), tiles_n = cdiv<size_t>(N, size_t(32) * tn);
  DYHIP_REQUIRE(tiles_m * tiles_n < (size_t(1) << 31), "GEMM too large");
  const size_t tiles = tiles_m * tiles_n;
  const size_t out_bytes = M * N * sizeof(float);
  // split K only when the tiles alone cannot fill the device
  unsigned splits = 1;
  if (g.ktiles_total == 0) {
    splits = 1;
  } else if (tiles < size_t(dev->num_cus)) {
    size_t want = cdiv<size_t>(size_t(2) * dev->num_cus, tiles);
    const size_t by_k = g.ktiles_total >= 8 ? g.ktiles_total / 4 : 1;
    const size_t by_ws = dev->gemm_ws_bytes / out_bytes;
    if (want > by_k) want = by_k;
    if (want > by_ws) want = by_ws;
    if (want > 65535) want = 65535;
    splits = want < 1 ? 1u : static_cast<unsigned>(want);
  }
  const bool fused_epi = epi.kind == kEpiLstmGates;  // needs the whole sum before the activation
  const bool use_partial = splits > 1 || fused_epi;
  if (use_partial)
    DYHIP_REQUIRE(dev->gemm_ws_bytes >= out_bytes * splits,
                  "GEMM output of %zu bytes does not fit the %zu-byte split-K workspace", out_bytes,
                  dev->gemm_ws_bytes);
  g.ktiles_per_split = g.ktiles_total == 0 ? 1 : cdiv<unsigned>(g.ktiles_total, splits);
  splits = g.ktiles_total == 0 ? 1 : cdiv<unsigned>(g.ktiles_total, g.ktiles_per_split);
  g.partial = use_partial ? static_cast<float*>(dev->gemm_ws) : nullptr;
  const int av = a_vec ? 1 : 0, bv = b_vec ? 1 : 0;
  if (a_kmajor && b_kmajor) launch_tiles<true, true>(dev, g, (unsigned)tiles_m, (unsigned)tiles_n, splits, tn, av, bv);
  else if (a_kmajor && !b_kmajor) launch_tiles<true, false>(dev, g, (unsigned)tiles_m, (unsigned)tiles_n, splits, tn, av, bv);
  else if (!a_kmajor && b_kmajor) launch_tiles<false, true>(dev, g, (unsigned)tiles_m, (unsigned)tiles_n, splits, tn, av, bv);
  else launch_tiles<false, false>(dev, g, (unsigned)tiles_m, (unsigned)tiles_n, splits, tn, av, bv);
  DYHIP_CHECK_LAUNCH();
  if (use_partial) {
    const size_t total = M * N;
    const dim3 grid((unsigned)cdiv<size_t>(total, 256));
    if (fused_epi)
      hipLaunchKernelGGL(gemm_splitk_reduce_kernel<kEpiLstmGates>, grid, dim3(256), 0, dev->stream, M, total, splits,
                         g.partial, C, epi);
    else if (epi.kind == kEpiBias)
      hipLaunchKernelGGL(gemm_splitk_reduce_kernel<kEpiBias>, grid, dim3(256), 0, dev->stream, M, total, splits,
                         g.partial, C, epi);
    else
      hipLaunchKernelGGL(gemm_splitk_reduce_kernel<kEpiAxpby>, grid, dim3(256), 0, dev->stream, M, total, splits,
                         g.partial, C, epi);
    DYHIP_CHECK_LAUNCH();
  }
  return DYHIP_OK;
}

}  // namespace dyhip

using namespace dyhip;

extern "C" {

int dyhip_gemm_nn(dyhip_device* dev, size_t M, size_t N, size_t K, const float* l, const float* r, float beta,
                  float* y) {
  DYHIP_CHECK_DEV(dev);
  GemmSeg s{l, M, r, K, K};
  GemmEpiParams ep{kEpiAxpby, beta, nullptr, 0, 0};
  return gemm_run(dev, false, true, M, N, 1, &s, y, ep);
}

int dyhip_affine_forward(dyhip_device* dev, size_t M, size_t N, size_t K, const float* bias, const float* W,
                         const float* x, float* fx) {
  DYHIP_CHECK_DEV(dev);
  DYHIP_REQUIRE(bias != nullptr, "AffineTransform: null bias");
  GemmSeg s{W, M, x, K, K};
  GemmEpiParams ep{kEpiBias, 0.f, bias, 0, 0};
  return gemm_run(dev, false, true, M, N, 1, &s, fx, ep);
}

int dyhip_gemm_tn_acc(dyhip_device* dev, size_t M, size_t N, size_t K, const float* l, const float* r, float* y) {
  DYHIP_CHECK_DEV(dev);
  GemmSeg s{l, K, r, K, K};
  GemmEpiParams ep{kEpiAxpby, 1.0f, nullptr, 0, 0};
  return gemm_run(dev, true, true, M, N, 1, &s, y, ep);
}

int dyhip_gemm_nt_acc(dyhip_device* dev, size_t M, size_t N, size_t K, const float* l, const float* r, float* y) {
  DYHIP_CHECK_DEV(dev);
  GemmSeg s{l, M, r, N, K};
  GemmEpiParams ep{kEpiAxpby, 1.0f, nullptr, 0, 0};
  return gemm_run(dev, false, false, M, N, 1, &s, y, ep);
}

}  // extern "C"
