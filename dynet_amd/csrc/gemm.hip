// fp32 GEMM on the CDNA matrix cores (v_mfma_f32_32x32x2_f32: fp32 inputs,
// fp32 accumulate, no reduced-precision shortcut), in the three forms DyNet's
// GEMM shim needs (dynet/matrix-multiply.h:16-37,97-117,162-180), replacing its
// cublasSgemm calls.
//
// Tiling.  A 256-thread block (4 wavefronts, 2 x 2) owns a 128 x (64*WN) tile of
// C; each wavefront owns 64 x (32*WN) of it as 2 x WN accumulators of 32x32.  K
// advances in steps of 32 through a double-buffered LDS stage.  Both operand
// tiles sit in LDS as lds[k][mn], whatever their orientation in memory, so one
// lane fetches the operand values of two (WN) neighbouring rows with a single
// 64-bit LDS read: the rows of a wave's tile are interleaved over its MFMA
// blocks (tile row 2*i + b belongs to block b), which is only a relabelling of
// the output rows.  The row pitch is W+4 floats for an operand stored along mn
// (128-bit LDS writes) and W+2 for one stored along k (transposing 32-bit writes
// land on 32 distinct banks).
//
// The MFMA "row" index is fed from B and the "column" index (lane % 32) from A,
// so a lane ends up holding two consecutive rows m of C for each of its columns
// and a wavefront stores 256 contiguous bytes per column.
//
// Schedule per K-tile: issue the global loads of the next tile, run the 16 MFMA
// steps with the LDS reads of step s+1 in flight under the MFMAs of step s
// (pinned with scheduling barriers: left alone the compiler waits for every read
// right before its use), park the next tile in the other LDS buffer three
// quarters of the way through, barrier.  Two blocks per CU (LDS-limited) cover
// each other's barrier bubbles; more resident wavefronts per SIMD lower the
// matrix-core issue rate, fewer expose the bubbles.
//
// Tile count rarely divides the 256 CUs, and skinny problems (the LSTM gate
// GEMMs have N = batch) have far too few tiles, so K is split across blocks when
// the estimate says it pays: each split writes its partial tile to a workspace
// and a second kernel adds the splits in ascending order (deterministic, no
// atomics) and applies the epilogue: C = beta*C + sum, + bias, or the fused LSTM
// gate epilogue.  The fused LSTM cell kernels consume the unreduced slices.
#include "gemm.h"

namespace dyhip {

typedef float floatx16 __attribute__((ext_vector_type(16)));
typedef float fvec2 __attribute__((ext_vector_type(2)));

constexpr int kBM = 128;
constexpr int kBK = 32;
constexpr int kGemmThreads = 256;
constexpr int kWritePos = (kBK / 2) * 3 / 4;  // MFMA step after which the next tile goes to LDS

struct GemmArgs {
  GemmSeg seg[kGemmMaxSeg];
  int nseg;
  unsigned ktiles0;  // k-tiles of segment 0
  unsigned ktiles_total;
  unsigned ktiles_per_split;
  size_t M, N;
  float* C;           // used when partial == nullptr
  float beta;         // used when partial == nullptr
  const float* bias;  // when set (and partial == nullptr): C = bias[i] + sum
  float* partial;     // [splits][M*N] or nullptr
  size_t stride_a, stride_b, stride_c;  // floats between consecutive batch items (blockIdx.z); 0 = shared operand
  int vec_ok;         // every operand 16-byte aligned with a leading dimension that is a multiple of 4
  int edge4_ok;       // vec_ok, and no 128-bit group of any operand straddles the matrix edge
};

// ---- global -> register tile loads ------------------------------------------------
// An operand tile is W (mn extent) x 32 (k extent) floats; thread t loads float4 number t + 256*u.
template <int W>
struct TileRegs {
  static constexpr int NV = (W * kBK / 4) / kGemmThreads;
  float4 v[NV];
};

// EDGE == 0: the whole tile lies inside the matrix and is 16-byte aligned.
// EDGE == 1: 16-byte aligned operands whose extent along the vectorised direction is a multiple of 4,
//            so every 128-bit group is wholly inside or wholly outside: branch-free clamped 128-bit loads.
// EDGE == 2: branch-free clamped scalar loads, zeros outside the matrix.
template <bool KMAJOR, int W, int EDGE>
__device__ __forceinline__ void load_tile(TileRegs<W>& r, const float* __restrict__ p, size_t ld, size_t mn0,
                                          size_t k0, size_t MN, size_t K) {
#pragma unroll
  for (int u = 0; u < TileRegs<W>::NV; ++u) {
    const int f = threadIdx.x + kGemmThreads * u;
    size_t mn, kk;
    if (!KMAJOR) {
      mn = mn0 + size_t(f % (W / 4)) * 4;
      kk = k0 + f / (W / 4);
    } else {
      mn = mn0 + f / (kBK / 4);
      kk = k0 + size_t(f % (kBK / 4)) * 4;
    }
    if (EDGE == 0) {
      r.v[u] = *reinterpret_cast<const float4*>(KMAJOR ? p + kk + mn * ld : p + mn + kk * ld);
    } else if (EDGE == 1) {
      const bool ok = mn < MN && kk < K;
      const size_t mc = ok ? mn : 0, kc = ok ? kk : 0;
      const float4 x = *reinterpret_cast<const float4*>(KMAJOR ? p + kc + mc * ld : p + mc + kc * ld);
      r.v[u] = make_float4(ok ? x.x : 0.f, ok ? x.y : 0.f, ok ? x.z : 0.f, ok ? x.w : 0.f);
    } else {
      float e[4];
#pragma unroll
      for (int c = 0; c < 4; ++c) {
        const size_t mi = KMAJOR ? mn : mn + c, ki = KMAJOR ? kk + c : kk;
        const bool ok = mi < MN && ki < K;
        const size_t mc = mi < MN ? mi : MN - 1, kc = ki < K ? ki : K - 1;
        const float x = KMAJOR ? p[kc + mc * ld] : p[mc + kc * ld];
        e[c] = ok ? x : 0.f;
      }
      r.v[u] = make_float4(e[0], e[1], e[2], e[3]);
    }
  }
}

template <bool KMAJOR, int W>
constexpr int lds_pitch() {
  return KMAJOR ? W + 2 : W + 4;
}

template <bool KMAJOR, int W>
__device__ __forceinline__ void store_tile(const TileRegs<W>& r, float* __restrict__ lds) {
  constexpr int P = lds_pitch<KMAJOR, W>();
#pragma unroll
  for (int u = 0; u < TileRegs<W>::NV; ++u) {
    const int f = threadIdx.x + kGemmThreads * u;
    if (!KMAJOR) {
      const int k = f / (W / 4), m4 = f % (W / 4);
      *reinterpret_cast<float4*>(lds + k * P + m4 * 4) = r.v[u];
    } else {
      const int k4 = f % (kBK / 4), mn_l = f / (kBK / 4);
      float* q = lds + (k4 * 4) * P + mn_l;
      q[0] = r.v[u].x;
      q[P] = r.v[u].y;
      q[2 * P] = r.v[u].z;
      q[3 * P] = r.v[u].w;
    }
  }
}

template <int V>
__device__ __forceinline__ void lds_read(const float* p, float (&out)[V]) {
  if constexpr (V == 1) {
    out[0] = *p;
  } else {
    const fvec2 t = *reinterpret_cast<const fvec2*>(p);
    out[0] = t[0];
    out[1] = t[1];
  }
}

// k-tile kt of the (up to two) concatenated K segments -> its segment and offset
__device__ __forceinline__ void locate_ktile(const GemmArgs& g, unsigned kt, GemmSeg& sg, size_t& k0) {
  if (g.nseg > 1 && kt >= g.ktiles0) {
    sg = g.seg[1];
    k0 = size_t(kt - g.ktiles0) * kBK;
  } else {
    sg = g.seg[0];
    k0 = size_t(kt) * kBK;
  }
}

template <bool A_KMAJOR, bool B_KMAJOR, int WN>
__device__ __forceinline__ void load_pair(const GemmArgs& g, unsigned kt, bool interior, size_t m0, size_t n0,
                                          TileRegs<kBM>& ra, TileRegs<64 * WN>& rb) {
  constexpr int BN = 64 * WN;
  GemmSeg sg;
  size_t k0;
  locate_ktile(g, kt, sg, k0);
  if (interior && k0 + kBK <= sg.K) {
    load_tile<A_KMAJOR, kBM, 0>(ra, sg.A, sg.lda, m0, k0, g.M, sg.K);
    load_tile<B_KMAJOR, BN, 0>(rb, sg.B, sg.ldb, n0, k0, g.N, sg.K);
  } else if (g.edge4_ok) {
    load_tile<A_KMAJOR, kBM, 1>(ra, sg.A, sg.lda, m0, k0, g.M, sg.K);
    load_tile<B_KMAJOR, BN, 1>(rb, sg.B, sg.ldb, n0, k0, g.N, sg.K);
  } else {
    load_tile<A_KMAJOR, kBM, 2>(ra, sg.A, sg.lda, m0, k0, g.M, sg.K);
    load_tile<B_KMAJOR, BN, 2>(rb, sg.B, sg.ldb, n0, k0, g.N, sg.K);
  }
}

// One K-tile of the main loop: MFMA steps on LDS buffer `buf`, with the global loads of
// tile i+PF issued first (into register slot S) and the tile i+1 (register slot S^1 for
// PF == 2, S for PF == 1) parked in the other LDS buffer three quarters of the way through.
template <bool A_KMAJOR, bool B_KMAJOR, int WN, int PF, int S>
__device__ __forceinline__ void ktile_iter(const GemmArgs& g, unsigned kt_begin, unsigned n_tiles, unsigned i,
                                           bool interior, size_t m0, size_t n0, TileRegs<kBM> (&ra)[PF],
                                           TileRegs<64 * WN> (&rb)[PF], float* lds_a, float* lds_b,
                                           floatx16 (&acc)[WN][2], int wm, int wn, int l32, int lhi) {
  constexpr int BN = 64 * WN;
  constexpr int PA = lds_pitch<A_KMAJOR, kBM>(), PB = lds_pitch<B_KMAJOR, BN>();
  constexpr int NEXT = PF == 2 ? (S ^ 1) : S;  // register slot holding tile i+1
  const int buf = i & 1;
  if (i + PF < n_tiles) load_pair<A_KMAJOR, B_KMAJOR, WN>(g, kt_begin + i + PF, interior, m0, n0, ra[S], rb[S]);
  const bool more = i + 1 < n_tiles;
  const float* la = lds_a + buf * (kBK * PA) + wm * 64 + 2 * l32 + lhi * PA;
  const float* lb = lds_b + buf * (kBK * PB) + wn * 32 * WN + WN * l32 + lhi * PB;
  float av[2][2], bv[2][WN];
  lds_read<2>(la, av[0]);
  lds_read<WN>(lb, bv[0]);
#pragma unroll
  for (int s = 0; s < kBK / 2; ++s) {
    const int cur = s & 1;
    if (s + 1 < kBK / 2) {
      lds_read<2>(la + (2 * s + 2) * PA, av[cur ^ 1]);
      lds_read<WN>(lb + (2 * s + 2) * PB, bv[cur ^ 1]);
    }
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int a = 0; a < WN; ++a)
#pragma unroll
      for (int b = 0; b < 2; ++b)
        acc[a][b] = __builtin_amdgcn_mfma_f32_32x32x2f32(bv[cur][a], av[cur][b], acc[a][b], 0, 0, 0);
    __builtin_amdgcn_sched_barrier(0);
    if (s == kWritePos && more) {
      // the other buffer was last read in the previous iteration, which every wave has left
      store_tile<A_KMAJOR, kBM>(ra[NEXT], lds_a + (buf ^ 1) * (kBK * PA));
      store_tile<B_KMAJOR, BN>(rb[NEXT], lds_b + (buf ^ 1) * (kBK * PB));
      __builtin_amdgcn_sched_barrier(0);
    }
  }
  __syncthreads();
}

// PF = how many K-tiles ahead the global loads run (register stages).  Two for the 64-wide
// tile: its blocks are the skinny, split-K ones whose few K-tiles are bound by load latency.
template <bool A_KMAJOR, bool B_KMAJOR, int WN, int PF>
__global__ __launch_bounds__(kGemmThreads, 2) void gemm_tile_kernel(GemmArgs g, unsigned tiles_m) {
  constexpr int BN = 64 * WN;
  if (gridDim.z > 1) {  // strided batch: item blockIdx.z of every operand (single K segment, no split)
    g.seg[0].A += size_t(blockIdx.z) * g.stride_a;
    g.seg[0].B += size_t(blockIdx.z) * g.stride_b;
    g.C += size_t(blockIdx.z) * g.stride_c;
  }
  constexpr int PA = lds_pitch<A_KMAJOR, kBM>(), PB = lds_pitch<B_KMAJOR, BN>();
  __shared__ __attribute__((aligned(16))) float lds_a[2 * kBK * PA];
  __shared__ __attribute__((aligned(16))) float lds_b[2 * kBK * PB];

  const unsigned tm = blockIdx.x % tiles_m, tn = blockIdx.x / tiles_m;
  const unsigned split = blockIdx.y;
  const size_t m0 = size_t(tm) * kBM, n0 = size_t(tn) * BN;
  const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
  const int wm = w & 1, wn = w >> 1;
  const int l32 = lane & 31, lhi = lane >> 5;

  floatx16 acc[WN][2];
#pragma unroll
  for (int a = 0; a < WN; ++a)
#pragma unroll
    for (int b = 0; b < 2; ++b)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[a][b][r] = 0.f;

  const unsigned kt_begin = split * g.ktiles_per_split;
  const unsigned kt_end = min(g.ktiles_total, kt_begin + g.ktiles_per_split);
  const bool interior = g.vec_ok && (m0 + kBM <= g.M) && (n0 + BN <= g.N);

  if (kt_begin < kt_end) {
    const unsigned n_tiles = kt_end - kt_begin;
    TileRegs<kBM> ra[PF];
    TileRegs<BN> rb[PF];
    load_pair<A_KMAJOR, B_KMAJOR, WN>(g, kt_begin, interior, m0, n0, ra[0], rb[0]);
    if (PF == 2 && n_tiles > 1)
      load_pair<A_KMAJOR, B_KMAJOR, WN>(g, kt_begin + 1, interior, m0, n0, ra[PF - 1], rb[PF - 1]);
    store_tile<A_KMAJOR, kBM>(ra[0], lds_a);
    store_tile<B_KMAJOR, BN>(rb[0], lds_b);
    __syncthreads();
    if (PF == 1) {
      for (unsigned i = 0; i < n_tiles; ++i)
        ktile_iter<A_KMAJOR, B_KMAJOR, WN, PF, 0>(g, kt_begin, n_tiles, i, interior, m0, n0, ra, rb, lds_a, lds_b, acc,
                                                   wm, wn, l32, lhi);
    } else {
      for (unsigned i = 0; i < n_tiles; i += 2) {
        ktile_iter<A_KMAJOR, B_KMAJOR, WN, PF, 0>(g, kt_begin, n_tiles, i, interior, m0, n0, ra, rb, lds_a, lds_b, acc,
                                                   wm, wn, l32, lhi);
        if (i + 1 < n_tiles)
          ktile_iter<A_KMAJOR, B_KMAJOR, WN, PF, PF - 1>(g, kt_begin, n_tiles, i + 1, interior, m0, n0, ra, rb, lds_a,
                                                          lds_b, acc, wm, wn, l32, lhi);
      }
    }
  }

  // ---- write back ----------------------------------------------------------------
  // acc[a][b][r] of lane l: row m = m0 + 64*wm + 2*(l%32) + b,
  //                         column n = n0 + 32*WN*wn + WN*i + a with i = 8*(r/4) + 4*(l/32) + r%4
  float* out = g.partial ? g.partial + size_t(split) * g.M * g.N : g.C;
  const bool direct = g.partial == nullptr;
  const size_t m = m0 + wm * 64 + 2 * l32;
  if (m >= g.M) return;
  const bool pair = (m + 1 < g.M) && (g.M % 2 == 0) && ((reinterpret_cast<uintptr_t>(out) & 7u) == 0);
  float bias0 = 0.f, bias1 = 0.f;
  if (direct && g.bias != nullptr) {
    bias0 = g.bias[m];
    if (m + 1 < g.M) bias1 = g.bias[m + 1];
  }
#pragma unroll
  for (int a = 0; a < WN; ++a)
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      const int i = 8 * (r / 4) + 4 * lhi + (r % 4);
      const size_t n = n0 + wn * 32 * WN + WN * i + a;
      if (n >= g.N) continue;
      float* p = out + m + n * g.M;
      float v0 = acc[a][0][r] + bias0, v1 = acc[a][1][r] + bias1;
      if (pair) {
        if (direct && g.beta != 0.f) {
          const fvec2 o = *reinterpret_cast<const fvec2*>(p);
          v0 = g.beta * o[0] + v0;
          v1 = g.beta * o[1] + v1;
        }
        *reinterpret_cast<fvec2*>(p) = fvec2{v0, v1};
      } else {
        p[0] = (direct && g.beta != 0.f) ? g.beta * p[0] + v0 : v0;
        if (m + 1 < g.M) p[1] = (direct && g.beta != 0.f) ? g.beta * p[1] + v1 : v1;
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
  // eight slices in flight (a loop of one load and one add per slice waits a memory round trip per slice)
  float s = 0.f;
  for (unsigned k0 = 0; k0 < splits; k0 += 8) {
    float v[8];
#pragma unroll
    for (int u = 0; u < 8; ++u) v[u] = partial[size_t(min(k0 + u, splits - 1)) * total + e];
#pragma unroll
    for (int u = 0; u < 8; ++u)
      if (k0 + u < splits) s += v[u];
  }
  if (EPI == kEpiAxpby) {
    C[e] = ep.beta != 0.f ? ep.beta * C[e] + s : s;
  } else if (EPI == kEpiBias) {
    C[e] = ep.bias[e % M] + s;
  } else {
    const unsigned i = static_cast<unsigned>(e % M);
    float pre = ep.bias[i];
    if (i >= ep.H && i < 2 * ep.H) pre += 1.0f;  // forget-gate bias
    pre += s;
    C[e] = i < 3 * ep.H ? logistic(ep.logistic_mode, pre) : tanh_accurate(pre);
  }
}

template <bool A_KMAJOR, bool B_KMAJOR>
static void launch_tiles(dyhip_device* dev, const GemmArgs& g, unsigned tiles_m, unsigned tiles_n, unsigned splits,
                         int wn, unsigned batch = 1) {
  const dim3 grid(tiles_m * tiles_n, splits, batch), block(kGemmThreads);
  if (wn == 1)
    hipLaunchKernelGGL((gemm_tile_kernel<A_KMAJOR, B_KMAJOR, 1, 2>), grid, block, 0, dev->stream, g, tiles_m);
  else
    hipLaunchKernelGGL((gemm_tile_kernel<A_KMAJOR, B_KMAJOR, 2, 1>), grid, block, 0, dev->stream, g, tiles_m);
}

// Tile width and split count by a small cost model.  Measured on MI355X: the matrix cores
// sustain ~2.0 GHz under this kernel (131 TFLOP/s over 256 CUs); a CU running two blocks
// keeps them ~95 % busy, a lone block ~77 %; the 64-wide tile reads more LDS per MFMA.
struct GemmPlan {
  int wn;
  unsigned splits;
};

static GemmPlan plan_gemm(const dyhip_device* dev, size_t M, size_t N, unsigned ktiles, size_t max_splits_ws,
                          bool must_use_partials) {
  const double cus = dev->num_cus > 0 ? dev->num_cus : 256;
  const double peak = cus * 256.0 * 2.0e9, ws_bw = 3.0e12;
  GemmPlan best{2, 1};
  double best_t = 1e30;
  for (int wn = 2; wn >= 1; --wn) {
    if (wn == 2 && N <= 64) continue;
    const double tiles = double(cdiv<size_t>(M, kBM)) * double(cdiv<size_t>(N, size_t(64) * wn));
    // a tile costs its full multiply-adds whatever part of it lies inside the matrix (a 650 x 1 product priced by
    // its own multiply-adds was never split over the depth: one block per 128 rows walked all k-tiles, 53 us)
    const double flops = 2.0 * tiles * double(kBM) * 64.0 * wn * double(ktiles) * kBK;
    for (unsigned s = 1; s <= 32; ++s) {
      if (s > 1 && (ktiles / s < 2 || s > max_splits_ws)) break;
      const double blocks = tiles * s;
      const double rounds = blocks <= cus ? 1.0 : double(cdiv<size_t>(size_t(blocks), size_t(cus)));
      const double eff = blocks / (rounds * cus);
      double inloop = blocks >= 2 * cus ? 0.95 : (blocks > cus ? 0.85 : 0.77);
      if (wn == 1) inloop *= 0.9;
      double t = flops / (peak * eff * inloop) + rounds * 1.0e-6;
      if (s > 1 || must_use_partials) t += 2.0 * double(M) * double(N) * 4.0 * s / ws_bw + 2.0e-6;
      if (t < best_t) {
        best_t = t;
        best = GemmPlan{wn, s};
      }
    }
  }
  return best;
}

// ---- C (+)= A * B^T with a depth of at most 32: the weight gradient of one timestep at a small batch ---------------
// (A = dpre, M x K with M = 4H; B = x or h, N x K; K = the batch size.)  This is a rank-K update of a matrix that is
// read and written once: memory work, not matrix-core work.  A thread owns four consecutive rows and kThinCols columns
// of C: its K fragments of A stay in registers (128-bit loads along the contiguous rows), the entries of B it needs
// are the same for the whole block and come through scalar loads, the old C values are all requested before the first
// multiply.  A 128 x 128-tile kernel gives an output of 1024 x 128 (the cell of the baseline's smallest
// configuration) to eight blocks.
// (Sixteen columns per thread, for half the re-reads of A from the L2, measured no better or worse: 10.4 against
// 10.3 us at 4096 x 1024 x 20, 34.3 against 26.3 us at 8192 x 2048 x 16.)
// Four or two columns per thread while the wider form would leave fewer than two blocks per CU (a small output: more
// blocks, fewer multiply-adds per thread; 1024 x 128 x 32: 6.8 us with eight, 5.0 with four).
template <int KT, int kThinCols>  // KT: depth rounded up to a multiple of four
__global__ __launch_bounds__(256) void gemm_nt_thin_kernel(unsigned M4, unsigned N, unsigned K, const float* __restrict__ A,
                                                           size_t lda, const float* __restrict__ B, size_t ldb,
                                                           float* __restrict__ C, float beta, size_t stride_a,
                                                           size_t stride_b, size_t stride_c) {
  __shared__ __attribute__((aligned(16))) float bt[KT][kThinCols];  // the block's entries of B, zero past the ends
  // item blockIdx.z of a strided batch (the gradient of a batch of matrices times vectors: a rank-one update each)
  A += size_t(blockIdx.z) * stride_a;
  B += size_t(blockIdx.z) * stride_b;
  C += size_t(blockIdx.z) * stride_c;
  const unsigned j0 = blockIdx.y * kThinCols;
  for (unsigned e = threadIdx.x; e < unsigned(KT * kThinCols); e += 256) {
    const unsigned k = e / kThinCols, jj = e % kThinCols;
    bt[k][jj] = k < K && j0 + jj < N ? B[j0 + jj + size_t(k) * ldb] : 0.f;
  }
  __syncthreads();
  const unsigned m4 = blockIdx.x * 256 + threadIdx.x;
  if (m4 >= M4) return;
  float4 c[kThinCols];
#pragma unroll
  for (int jj = 0; jj < kThinCols; ++jj) {
    const unsigned j = min(j0 + jj, N - 1);  // columns past the end repeat the last one and are not stored
    c[jj] = beta != 0.f ? *reinterpret_cast<const float4*>(C + (size_t(j) * M4 + m4) * 4) : make_float4(0.f, 0.f, 0.f, 0.f);
  }
  // depth outermost: one fragment of A at a time (unconditional loads on a clamped depth index; B is zero past the end)
#pragma unroll
  for (int k = 0; k < KT; ++k) {
    const unsigned kc = unsigned(k) < K ? unsigned(k) : K - 1;
    const float4 a = *reinterpret_cast<const float4*>(A + size_t(kc) * lda + size_t(m4) * 4);
#pragma unroll
    for (int jj = 0; jj < kThinCols; ++jj) {
      const float b = bt[k][jj];  // the same address in every lane: a broadcast read
      c[jj].x = fmaf(a.x, b, c[jj].x);
      c[jj].y = fmaf(a.y, b, c[jj].y);
      c[jj].z = fmaf(a.z, b, c[jj].z);
      c[jj].w = fmaf(a.w, b, c[jj].w);
    }
  }
#pragma unroll
  for (int jj = 0; jj < kThinCols; ++jj) {
    const unsigned j = j0 + jj;
    if (j < N) *reinterpret_cast<float4*>(C + (size_t(j) * M4 + m4) * 4) = c[jj];
  }
}

static bool gemm_nt_thin_eligible(size_t M, size_t N, size_t K, const float* A, size_t lda, const float* B, float* C,
                                  float beta) {
  return K >= 1 && K <= 32 && M % 4 == 0 && lda % 4 == 0 && M >= 256 && N >= 1 && N <= 0xFFFFFFFFull / 2 &&
         M / 4 <= 0xFFFFFFFFull && cdiv<size_t>(N, 2) <= 65535 && aligned16(A) && aligned16(C) && B != nullptr &&
         (beta == 0.f || beta == 1.f);
}

static int gemm_nt_thin_run(dyhip_device* dev, size_t M, size_t N, size_t K, const float* A, size_t lda, const float* B,
                            size_t ldb, float* C, float beta, const GemmBatch* batch = nullptr) {
  const unsigned M4 = static_cast<unsigned>(M / 4);
  const unsigned items = batch != nullptr && batch->count > 1 ? batch->count : 1;
  const size_t sa = items > 1 ? batch->stride_a : 0, sb = items > 1 ? batch->stride_b : 0, sc = items > 1 ? batch->stride_c : 0;
  // columns per thread: eight, or four, or two while the wider form would leave fewer than two blocks per CU
  const size_t want = 2 * size_t(dev->num_cus), bxm = size_t(cdiv<unsigned>(M4, 256)) * items;
  const int cols = bxm * cdiv<size_t>(N, 8) >= want ? 8 : bxm * cdiv<size_t>(N, 4) >= want ? 4 : 2;
  const dim3 grid(cdiv<unsigned>(M4, 256), static_cast<unsigned>(cdiv<size_t>(N, size_t(cols))), items), block(256);
#define DYHIP_THIN_C(KT, COLS)                                                                                        \
  hipLaunchKernelGGL((gemm_nt_thin_kernel<KT, COLS>), grid, block, 0, dev->stream, M4, static_cast<unsigned>(N),      \
                     static_cast<unsigned>(K), A, lda, B, ldb, C, beta, sa, sb, sc)
#define DYHIP_THIN(KT)                     \
  do {                                     \
    if (cols == 8) DYHIP_THIN_C(KT, 8);    \
    else if (cols == 4) DYHIP_THIN_C(KT, 4); \
    else DYHIP_THIN_C(KT, 2);              \
  } while (0)
  switch ((K + 3) / 4) {  // the depth rounded up to a multiple of four: a padded step costs as much as a real one
    case 1: DYHIP_THIN(4); break;
    case 2: DYHIP_THIN(8); break;
    case 3: DYHIP_THIN(12); break;
    case 4: DYHIP_THIN(16); break;
    case 5: DYHIP_THIN(20); break;
    case 6: DYHIP_THIN(24); break;
    case 7: DYHIP_THIN(28); break;
    default: DYHIP_THIN(32); break;
  }
#undef DYHIP_THIN
#undef DYHIP_THIN_C
  DYHIP_CHECK_LAUNCH();
  return DYHIP_OK;
}


// ---- C = beta * C (or bias) + A * B with at most 8 columns of B: matrix times vector(s), the un-batched graph's
// product (affine layers, output projections, one sentence at a time) -----------------------------------------------
// Memory work: A (M x K, rows contiguous inside a column) is read once in kilobyte runs, lane l owning rows 4l..4l+3 of
// a 256-row slab for every depth index of its wavefront's range; the depth is split over the block's four wavefronts
// (combined through LDS) and, to fill the GPU, over gridDim.y blocks, whose slabs of partial sums a second small
// kernel adds (with the epilogue).  The tile kernel gives a one-column product to M / 128 blocks that each walk the
// whole depth: 60 us for 4096 x 1024, 117 us for 4096 x 2048.
constexpr int kGemvWaves = 4;
constexpr unsigned kGemvMaxChunk = 4096;  // depth indices per block
template <int NB>  // columns padded to 1, 2, 4 or 8
__global__ __launch_bounds__(64 * kGemvWaves) void gemm_nn_thin_kernel(unsigned M4, unsigned N, unsigned chunk,
                                                                      GemmSeg seg0, GemmSeg seg1, unsigned slabs0,
                                                                      float* __restrict__ C, float beta,
                                                                      const float* __restrict__ bias,
                                                                      float* __restrict__ partial, size_t stride_a,
                                                                      size_t stride_b, size_t stride_c) {
  __shared__ float4 red[kGemvWaves - 1][64][NB];
  // a product over two depth segments (the gates node: Wx x + Wh h) is one sequence of slabs: the first slabs0 walk
  // the first segment, the others the second; the choice is the same for the whole block
  const bool second = blockIdx.y >= slabs0;
  // blockIdx.z: the item of a strided batch (one segment, one slab; the strides are 0 otherwise)
  const float* __restrict__ A = (second ? seg1.A : seg0.A) + size_t(blockIdx.z) * stride_a;
  const float* __restrict__ B = (second ? seg1.B : seg0.B) + size_t(blockIdx.z) * stride_b;
  C += size_t(blockIdx.z) * stride_c;
  const size_t lda = second ? seg1.lda : seg0.lda, ldb = second ? seg1.ldb : seg0.ldb;
  const unsigned K = static_cast<unsigned>(second ? seg1.K : seg0.K);
  const unsigned k0 = (second ? blockIdx.y - slabs0 : blockIdx.y) * chunk, k1 = min(K, k0 + chunk);
  const unsigned lane = threadIdx.x & 63, w = threadIdx.x >> 6;
  const unsigned m4 = blockIdx.x * 64 + lane;
  const bool live = m4 < M4;
  const float4* a4 = reinterpret_cast<const float4*>(A) + (live ? m4 : M4 - 1);
  const size_t lda4 = lda / 4;
  // wavefront w takes the depth indices k0 + w, k0 + w + 4, ..., eight at a time: eight 128-bit loads of A in flight
  // and, beside them, the entries of B for those eight indices, one index per lane (lane l fetches index l % 8; the
  // multiply reads them back lane by lane through scalar registers), so that nothing is staged and waited for first
  float4 acc[NB];
#pragma unroll
  for (int n = 0; n < NB; ++n) acc[n] = make_float4(0.f, 0.f, 0.f, 0.f);
  for (unsigned k = k0 + w; k < k1; k += 8 * kGemvWaves) {
    float4 a[8];
#pragma unroll
    for (int u = 0; u < 8; ++u) a[u] = ldg4<true>(a4 + size_t(min(k + u * kGemvWaves, k1 - 1)) * lda4);
    const unsigned kmine = k + (lane & 7u) * kGemvWaves;
    float xv[NB];
#pragma unroll
    for (int n = 0; n < NB; ++n) xv[n] = kmine < k1 && unsigned(n) < N ? B[size_t(kmine) + size_t(n) * ldb] : 0.f;
#pragma unroll
    for (int u = 0; u < 8; ++u) {
#pragma unroll
      for (int n = 0; n < NB; ++n) {
        const float b = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, xv[n]), u));  // 0 past the end
        acc[n].x = fmaf(a[u].x, b, acc[n].x);
        acc[n].y = fmaf(a[u].y, b, acc[n].y);
        acc[n].z = fmaf(a[u].z, b, acc[n].z);
        acc[n].w = fmaf(a[u].w, b, acc[n].w);
      }
    }
  }
  if (w > 0) {
#pragma unroll
    for (int n = 0; n < NB; ++n) red[w - 1][lane][n] = acc[n];
  }
  __syncthreads();
  if (w != 0 || !live) return;
#pragma unroll
  for (int n = 0; n < NB; ++n) {
    if (unsigned(n) >= N) break;
    float4 t = acc[n];
#pragma unroll
    for (int v = 0; v < kGemvWaves - 1; ++v) {
      const float4 o = red[v][lane][n];
      t.x += o.x; t.y += o.y; t.z += o.z; t.w += o.w;
    }
    if (partial != nullptr) {
      reinterpret_cast<float4*>(partial)[(size_t(blockIdx.y) * N + n) * M4 + m4] = t;
    } else {
      float4* out = reinterpret_cast<float4*>(C) + size_t(n) * M4 + m4;
      if (bias != nullptr) {
        const float4 bb = reinterpret_cast<const float4*>(bias)[m4];
        t.x += bb.x; t.y += bb.y; t.z += bb.z; t.w += bb.w;
      } else if (beta != 0.f) {
        const float4 o = *out;
        t.x += beta * o.x; t.y += beta * o.y; t.z += beta * o.z; t.w += beta * o.w;
      }
      *out = t;
    }
  }
}

// C = beta * C (or bias) + the slabs' sum, slabs in ascending order
// GATES: C = act(bias + (forget rows: 1) + sum), the epilogue of the gates node (kEpiLstmGates)
constexpr int kCombineFlight = 16;  // slabs a thread has in flight (8: +0.5 us at 16 slabs)
constexpr unsigned kCombineThreads = 256;
template <bool GATES>
__global__ __launch_bounds__(256) void gemm_nn_thin_combine_kernel(unsigned M4, unsigned N, unsigned slabs,
                                                                   const float4* __restrict__ partial,
                                                                   float4* __restrict__ C, float beta,
                                                                   const float* __restrict__ bias, unsigned H,
                                                                   int logistic_mode) {
  const size_t e = size_t(blockIdx.x) * blockDim.x + threadIdx.x, total = size_t(M4) * N;
  if (e >= total) return;
  float4 t = make_float4(0.f, 0.f, 0.f, 0.f);
  for (unsigned s0 = 0; s0 < slabs; s0 += kCombineFlight) {  // slabs in flight together, added in ascending order
    float4 o[kCombineFlight];
#pragma unroll
    for (int u = 0; u < kCombineFlight; ++u) o[u] = partial[size_t(min(s0 + u, slabs - 1)) * total + e];
#pragma unroll
    for (int u = 0; u < kCombineFlight; ++u) {
      if (s0 + u < slabs) {
        t.x += o[u].x; t.y += o[u].y; t.z += o[u].z; t.w += o[u].w;
      }
    }
  }
  if (GATES) {
    const unsigned i0 = static_cast<unsigned>(e % M4) * 4;
    float v[4] = {t.x, t.y, t.z, t.w};
#pragma unroll
    for (int c = 0; c < 4; ++c) {
      const unsigned i = i0 + c;
      float pre = bias[i];
      if (i >= H && i < 2 * H) pre += 1.0f;  // forget-gate bias
      pre += v[c];
      v[c] = i < 3 * H ? logistic(logistic_mode, pre) : tanh_accurate(pre);
    }
    C[e] = make_float4(v[0], v[1], v[2], v[3]);
    return;
  }
  if (bias != nullptr) {
    const float4 bb = reinterpret_cast<const float4*>(bias)[e % M4];
    t.x += bb.x; t.y += bb.y; t.z += bb.z; t.w += bb.w;
  } else if (beta != 0.f) {
    const float4 o = C[e];
    t.x += beta * o.x; t.y += beta * o.y; t.z += beta * o.z; t.w += beta * o.w;
  }
  C[e] = t;
}

// One launch for the same product when the rows alone fill the GPU: a block owns 32 rows and the whole depth.
// A read in 128-byte runs streams at 3.9 of the 4.2 TB/s that kilobyte runs reach on this part (64-byte runs: 2.5), so
// 32 rows a block cost little bandwidth and M / 32 blocks need no second kernel (whose launch gap and dependent trips
// are 4.8 us of the slab form's 9).  The wavefronts of a block split the depth; lane l of a wavefront owns rows
// 4 (l % 8)..+3 for the depth indices l / 8, l / 8 + 8, ... of its range, so one load instruction is eight 128-byte
// runs; B is staged in LDS once per block by coalesced loads; the lanes' sums cross the wavefront by three
// exchange steps and the block through LDS in ascending wavefront order, then the epilogue.
constexpr unsigned kRowsMaxBBytes = 64u << 10;  // B staged in LDS
constexpr int kRowsWavesN = 8;  // 16 wavefronts: 4096 x 1 x 1024 7.0 against 6.8 us, 10 000 x 4 x 1024 19.0 against 15.5
constexpr int kRowsFlight = 4;  // loads of A in flight a lane, and as many behind them (8: 7.2 us)
template <int NB, int kRowsWaves, int U>  // columns padded to 1, 2, 4 or 8
__global__ __launch_bounds__(64 * kRowsWaves) void gemm_nn_rows_kernel(unsigned M4, unsigned N, GemmSeg seg0, GemmSeg seg1,
                                                                      unsigned per_wave, float* __restrict__ C, float beta,
                                                                      const float* __restrict__ bias, int gates, unsigned H,
                                                                      int logistic_mode) {
  extern __shared__ float bs[];  // [n][K0 + K1]
  __shared__ float4 red[kRowsWaves][NB][8];
  const unsigned K0 = static_cast<unsigned>(seg0.K), K1 = static_cast<unsigned>(seg1.K), Kt = K0 + K1;
  const unsigned lane = threadIdx.x & 63, w = threadIdx.x >> 6, rq = lane & 7, kk = lane >> 3;
  const unsigned m4 = blockIdx.x * 8 + rq;
  const bool live = m4 < M4;
  const float4* a0 = reinterpret_cast<const float4*>(seg0.A) + (live ? m4 : M4 - 1);
  const float4* a1 = reinterpret_cast<const float4*>(seg1.A) + (live ? m4 : M4 - 1);
  const size_t lda0 = seg0.lda / 4, lda1 = seg1.lda / 4;
  // depth index kc of the two segments laid end to end
  auto a_at = [&](unsigned kc) __attribute__((always_inline)) {
    return kc < K0 ? a0 + size_t(kc) * lda0 : a1 + size_t(kc - K0) * lda1;
  };
  const unsigned kw0 = w * per_wave, kw1 = min(Kt, kw0 + per_wave);
  float4 acc[NB];
#pragma unroll
  for (int n = 0; n < NB; ++n) acc[n] = make_float4(0.f, 0.f, 0.f, 0.f);
  // U loads of A in flight and the next U behind them (fetched before the current ones are used; past the range
  // they all fall on the range's last column, one cached line); the first leave before B is staged
  float4 a[U], nxt[U];
  const unsigned klast = (kw1 > kw0 ? kw1 : Kt) - 1;  // a wavefront without a range fetches the matrix's last column
#pragma unroll
  for (int u = 0; u < U; ++u) a[u] = ldg4<true>(a_at(min(kw0 + kk + 8 * u, klast)));
  for (unsigned n = 0; n < N; ++n) {
    for (unsigned k = threadIdx.x; k < K0; k += 64 * kRowsWaves) bs[n * Kt + k] = seg0.B[k + size_t(n) * seg0.ldb];
    for (unsigned k = threadIdx.x; k < K1; k += 64 * kRowsWaves) bs[n * Kt + K0 + k] = seg1.B[k + size_t(n) * seg1.ldb];
  }
  __syncthreads();
  for (unsigned k = kw0; k < kw1; k += 8 * U) {
#pragma unroll
    for (int u = 0; u < U; ++u) nxt[u] = ldg4<true>(a_at(min(k + 8 * U + kk + 8 * u, klast)));
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const unsigned kc = k + kk + 8 * u;
      const bool in = kc < kw1;
#pragma unroll
      for (int n = 0; n < NB; ++n) {
        const float b = in && unsigned(n) < N ? bs[min(unsigned(n), N - 1) * Kt + min(kc, Kt - 1)] : 0.f;
        acc[n].x = fmaf(a[u].x, b, acc[n].x);
        acc[n].y = fmaf(a[u].y, b, acc[n].y);
        acc[n].z = fmaf(a[u].z, b, acc[n].z);
        acc[n].w = fmaf(a[u].w, b, acc[n].w);
      }
    }
#pragma unroll
    for (int u = 0; u < U; ++u) a[u] = nxt[u];
  }
  // across the eight depth classes of the wavefront: lanes 8 apart in a DPP row, then the rows
#pragma unroll
  for (int n = 0; n < NB; ++n) {
#define DYHIP_ROWS_ACROSS(c)                            \
  {                                                     \
    float v = acc[n].c;                                 \
    v += dpp_move<0x128, 0xF>(v, 0.f); /* row_ror:8 */  \
    v += __shfl_xor(v, 16);                             \
    v += __shfl_xor(v, 32);                             \
    acc[n].c = v;                                       \
  }
    DYHIP_ROWS_ACROSS(x) DYHIP_ROWS_ACROSS(y) DYHIP_ROWS_ACROSS(z) DYHIP_ROWS_ACROSS(w)
#undef DYHIP_ROWS_ACROSS
  }
  if (lane < 8) {
#pragma unroll
    for (int n = 0; n < NB; ++n) red[w][n][lane] = acc[n];
  }
  __syncthreads();
  if (threadIdx.x >= 8 * N) return;
  const unsigned n = threadIdx.x >> 3, r = threadIdx.x & 7, mo = blockIdx.x * 8 + r;
  if (mo >= M4) return;
  float4 t = red[0][n][r];
#pragma unroll
  for (int v = 1; v < kRowsWaves; ++v) {
    const float4 o = red[v][n][r];
    t.x += o.x; t.y += o.y; t.z += o.z; t.w += o.w;
  }
  float4* out = reinterpret_cast<float4*>(C) + size_t(n) * M4 + mo;
  if (gates) {
    float v[4] = {t.x, t.y, t.z, t.w};
#pragma unroll
    for (int c = 0; c < 4; ++c) {
      const unsigned i = mo * 4 + c;
      float pre = bias[i];
      if (i >= H && i < 2 * H) pre += 1.0f;  // forget-gate bias
      pre += v[c];
      v[c] = i < 3 * H ? logistic(logistic_mode, pre) : tanh_accurate(pre);
    }
    *out = make_float4(v[0], v[1], v[2], v[3]);
    return;
  }
  if (bias != nullptr) {
    const float4 bb = reinterpret_cast<const float4*>(bias)[mo];
    t.x += bb.x; t.y += bb.y; t.z += bb.z; t.w += bb.w;
  } else if (beta != 0.f) {
    const float4 o = *out;
    t.x += beta * o.x; t.y += beta * o.y; t.z += beta * o.z; t.w += beta * o.w;
  }
  *out = t;
}

// Taken where it measured faster than the slab form (4096 x 1 x 1024: 6.8 against 8.0 us, 8192 x 1 x 1024: 8.5 against
// 10.8, 16384 x 8 x 256: 10.1 against 11.6): at least 32 blocks, a depth one block walks in a few microseconds
// (4096 x 1 x 2048: 11.2 against 10.6 us; 1024 x 1 x 4096: 18.0 against 13.9), and a block count that fills the
// CUs evenly (10 000 rows = 313 blocks on 256 CUs: 13.9 against 11.9 us).
static bool gemm_nn_rows_fit(const dyhip_device* dev, size_t M, size_t N, int nseg, const GemmSeg* segs) {
  const size_t Kt = segs[0].K + (nseg > 1 ? segs[1].K : 0);
  const size_t nb = N == 1 ? 1 : N == 2 ? 2 : N <= 4 ? 4 : 8;
  const size_t bx = cdiv<size_t>(M, 32), cus = dev->num_cus > 0 ? size_t(dev->num_cus) : 256;
  return M >= 1024 && Kt <= 1536 && Kt * nb * sizeof(float) <= kRowsMaxBBytes && (bx <= cus || bx >= 3 * cus);
}

static int gemm_nn_rows_run(dyhip_device* dev, size_t M, size_t N, int nseg, const GemmSeg* segs, float* C,
                            const GemmEpiParams& epi) {
  const unsigned M4 = static_cast<unsigned>(M / 4), bx = cdiv<unsigned>(M4, 8);
  GemmSeg s0 = segs[0], s1 = segs[0];
  s1.K = 0;
  if (nseg > 1) s1 = segs[1];
  const unsigned Kt = static_cast<unsigned>(s0.K + s1.K);
  const unsigned waves = kRowsWavesN;
  unsigned per_wave = cdiv<unsigned>(Kt, waves);
  per_wave = (per_wave + 7) / 8 * 8;
  const bool gates = epi.kind == kEpiLstmGates;
  const float beta = epi.kind == kEpiAxpby ? epi.beta : 0.f;
  const float* bias = epi.kind == kEpiAxpby ? nullptr : epi.bias;
  const size_t lds = sizeof(float) * Kt * N;
  const dim3 grid(bx), block(64 * waves);
#define DYHIP_ROWS(NB, W, U)                                                                                        \
  do {                                                                                                              \
    static bool big_lds_ok = false;                                                                                 \
    if (lds > (size_t(32) << 10) && !big_lds_ok) {                                                                   \
      DYHIP_CHECK_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(&gemm_nn_rows_kernel<NB, W, U>),            \
                                          hipFuncAttributeMaxDynamicSharedMemorySize, int(kRowsMaxBBytes)));        \
      big_lds_ok = true;                                                                                            \
    }                                                                                                               \
    hipLaunchKernelGGL((gemm_nn_rows_kernel<NB, W, U>), grid, block, lds, dev->stream, M4, static_cast<unsigned>(N), s0, s1, \
                       per_wave, C, beta, bias, gates ? 1 : 0, epi.H, epi.logistic_mode);                           \
  } while (0)
  if (N == 1) DYHIP_ROWS(1, kRowsWavesN, kRowsFlight);
  else if (N == 2) DYHIP_ROWS(2, kRowsWavesN, kRowsFlight);
  else if (N <= 4) DYHIP_ROWS(4, kRowsWavesN, kRowsFlight);
  else DYHIP_ROWS(8, kRowsWavesN, kRowsFlight);
#undef DYHIP_ROWS
  DYHIP_CHECK_LAUNCH();
  return DYHIP_OK;
}

static bool gemm_nn_thin_eligible(const dyhip_device* dev, size_t M, size_t N, int nseg, const GemmSeg* segs,
                                  const float* C, const GemmEpiParams& epi) {
  if (!(epi.kind == kEpiAxpby || (epi.kind == kEpiBias && epi.bias != nullptr && aligned16(epi.bias)) ||
        (epi.kind == kEpiLstmGates && epi.bias != nullptr)))
    return false;
  if (nseg < 1 || nseg > 2 || (nseg == 2 && epi.kind != kEpiLstmGates)) return false;
  for (int q = 0; q < nseg; ++q)
    if (segs[q].A == nullptr || segs[q].B == nullptr || segs[q].K < 1 || segs[q].K > 0x3FFFFFFFull || segs[q].lda % 4 != 0 ||
        !aligned16(segs[q].A))
      return false;
  return N >= 1 && N <= 8 && M >= 256 && M % 4 == 0 && M / 4 <= 0x7FFFFFFFull && aligned16(C) && dev->gemm_ws != nullptr;
}

static int gemm_nn_thin_run(dyhip_device* dev, size_t M, size_t N, int nseg, const GemmSeg* segs, float* C,
                            const GemmEpiParams& epi, const GemmBatch* batch = nullptr) {
  const unsigned items = batch != nullptr && batch->count > 1 ? batch->count : 1;
  if (items == 1 && gemm_nn_rows_fit(dev, M, N, nseg, segs)) return gemm_nn_rows_run(dev, M, N, nseg, segs, C, epi);
  const unsigned M4 = static_cast<unsigned>(M / 4), bx = cdiv<unsigned>(M4, 64);
  const unsigned K0 = static_cast<unsigned>(segs[0].K), K1 = nseg > 1 ? static_cast<unsigned>(segs[1].K) : 0u;
  const unsigned K = K0 + K1;
  // depth slabs: enough blocks for two per CU, each with at least 32 and at most kGemvMaxChunk depth indices, and
  // partial sums that fit the workspace
  unsigned slabs = cdiv<unsigned>(2 * dev->num_cus, bx);
  const unsigned max_by_depth = cdiv<unsigned>(K, 32);
  if (slabs > max_by_depth) slabs = max_by_depth;
  if (slabs < cdiv<unsigned>(K, kGemvMaxChunk)) slabs = cdiv<unsigned>(K, kGemvMaxChunk);
  if (items > 1) slabs = 1;  // the items fill the GPU; the caller has checked that one slab holds the depth
  unsigned chunk = cdiv<unsigned>(K, slabs);
  chunk = (chunk + 7) / 8 * 8;
  const unsigned slabs0 = cdiv<unsigned>(K0, chunk), slabs1 = K1 ? cdiv<unsigned>(K1, chunk) : 0u;
  slabs = slabs0 + slabs1;
  DYHIP_REQUIRE(slabs <= 65535 && chunk <= kGemvMaxChunk, "matrix-vector product: depth %u needs too many slabs", K);
  const bool gates = epi.kind == kEpiLstmGates;
  float* partial = nullptr;
  if (slabs > 1 || gates) {  // the gates epilogue lives in the second kernel
    DYHIP_REQUIRE(dev->gemm_ws_bytes >= sizeof(float) * M * N * slabs, "matrix-vector product: workspace too small");
    partial = static_cast<float*>(dev->gemm_ws);
  }
  const float beta = epi.kind == kEpiAxpby ? epi.beta : 0.f;
  const float* bias = epi.kind == kEpiAxpby ? nullptr : epi.bias;
  const GemmSeg s0 = segs[0], s1 = nseg > 1 ? segs[1] : segs[0];
  const dim3 grid(bx, slabs, items), block(64 * kGemvWaves);
  const size_t sa = items > 1 ? batch->stride_a : 0, sb = items > 1 ? batch->stride_b : 0, sc = items > 1 ? batch->stride_c : 0;
#define DYHIP_GEMV(NB)                                                                                             \
  hipLaunchKernelGGL(gemm_nn_thin_kernel<NB>, grid, block, 0, dev->stream, M4, static_cast<unsigned>(N), chunk, s0, s1, \
                     slabs0, C, beta, bias, partial, sa, sb, sc)
  if (N == 1) DYHIP_GEMV(1);
  else if (N == 2) DYHIP_GEMV(2);
  else if (N <= 4) DYHIP_GEMV(4);
  else DYHIP_GEMV(8);
#undef DYHIP_GEMV
  DYHIP_CHECK_LAUNCH();
  if (partial != nullptr) {
    const size_t total = size_t(M4) * N;
    const dim3 g2(static_cast<unsigned>(cdiv<size_t>(total, kCombineThreads)));
    if (gates)
      hipLaunchKernelGGL(gemm_nn_thin_combine_kernel<true>, g2, dim3(kCombineThreads), 0, dev->stream, M4, static_cast<unsigned>(N),
                         slabs, reinterpret_cast<const float4*>(partial), reinterpret_cast<float4*>(C), 0.f, bias, epi.H,
                         epi.logistic_mode);
    else
      hipLaunchKernelGGL(gemm_nn_thin_combine_kernel<false>, g2, dim3(kCombineThreads), 0, dev->stream, M4, static_cast<unsigned>(N),
                         slabs, reinterpret_cast<const float4*>(partial), reinterpret_cast<float4*>(C), beta, bias, 0u, 0);
    DYHIP_CHECK_LAUNCH();
  }
  return DYHIP_OK;
}


// ---- C = beta * C (or bias) + A * B with 9..32 columns of B: the affine layers and the gates node of a small batch ---
// Still memory work (the weights are read once, the batch is 16-32 sequences), but too many columns for one lane's
// registers on the vector ALUs, so the sums run on the matrix cores.  A wavefront owns 128 rows: lane l feeds rows
// 4(l % 32)..+3 by 128-bit loads (512-byte runs of a column of A) for four depth indices of the lower (l < 32) or upper
// half of an 8-index group, and column l % 32 of B for the same indices; one v_mfma_f32_32x32x2_f32 per row component
// pairs a depth index of each half.  The result lands with a lane's four rows in the four accumulators' same
// register, so a column's 128 rows are stored as one 512-byte run.  The block's four wavefronts split its depth range
// (combined through LDS), gridDim.y blocks split the depth further, and gemm_nn_thin_combine_kernel adds their slabs.
constexpr int kMidWaves = 4;
constexpr unsigned kMidBlocksPerCu = 2;  // eight wavefronts a block and one block a CU halves the slabs: -1.5 us at 4096 rows, +1 to +6 us elsewhere
constexpr unsigned kMidSub = 256;             // depth indices of B staged in LDS at a time
constexpr unsigned kMidPitch = kMidSub + 4;  // floats between B's columns in LDS
template <bool BVEC>  // B's columns can be read by 128-bit loads (16-byte aligned, depths a multiple of four)
__global__ __launch_bounds__(64 * kMidWaves) void gemm_nn_mid_kernel(unsigned M4, unsigned N, unsigned chunk, GemmSeg seg0,
                                                                     GemmSeg seg1, unsigned slabs0, float* __restrict__ C,
                                                                     float beta, const float* __restrict__ bias,
                                                                     float* __restrict__ partial) {
  // B's staged entries during the products, then the wavefronts' sums: 48 KB, so that two blocks fit a CU
  __shared__ float4 red[kMidWaves - 1][16][64];
  static_assert(sizeof(float) * 32 * kMidPitch <= sizeof(float4) * (kMidWaves - 1) * 16 * 64, "B's staging area fits");
  float* bs = reinterpret_cast<float*>(&red[0][0][0]);
  const bool second = blockIdx.y >= slabs0;
  const float* __restrict__ A = second ? seg1.A : seg0.A;
  const float* __restrict__ B = second ? seg1.B : seg0.B;
  const size_t lda4 = (second ? seg1.lda : seg0.lda) / 4, ldb = second ? seg1.ldb : seg0.ldb;
  const unsigned K = static_cast<unsigned>(second ? seg1.K : seg0.K);
  const unsigned k0 = (second ? blockIdx.y - slabs0 : blockIdx.y) * chunk, k1 = min(K, k0 + chunk);
  const unsigned lane = threadIdx.x & 63, w = threadIdx.x >> 6, l32 = lane & 31, hi = lane >> 5;
  const unsigned m4 = blockIdx.x * 32 + l32;
  const bool live = m4 < M4;
  const float4* a4 = reinterpret_cast<const float4*>(A) + (live ? m4 : M4 - 1);
  const bool ncol = l32 < N;
  floatx16 acc[4];
#pragma unroll
  for (int c = 0; c < 4; ++c)
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[c][r] = 0.f;
  // B's entries for up to kMidSub depth indices are staged in LDS by coalesced loads (a lane reading its own column
  // of B from memory made every load 64 separate lines); a wavefront's first loads of A are issued before that.
  // 16 depth indices a step: two groups of eight, lanes below 32 the first four of a group, the others the last four.
  for (unsigned kc = k0; kc < k1; kc += kMidSub) {
    const unsigned kend = min(kc + kMidSub, k1), len = kend - kc;
    unsigned kb = kc + 16 * w;
    bool have = kb < kend;
    float4 a[2][4];
    auto load_a = [&]() {
#pragma unroll
      for (int g = 0; g < 2; ++g)
#pragma unroll
        for (int j = 0; j < 4; ++j) a[g][j] = ldg4<true>(a4 + size_t(min(kb + 8 * g + 4 * hi + j, k1 - 1)) * lda4);
    };
    if (have) load_a();
    if (kc > k0) __syncthreads();  // the last range's readers are done
    if (BVEC) {
      const unsigned q4 = len / 4;  // kc and k1 are multiples of four
      for (unsigned e = threadIdx.x; e < N * q4; e += 64 * kMidWaves) {
        const unsigned n = e / q4, q = e - n * q4;
        *reinterpret_cast<float4*>(bs + n * kMidPitch + 4 * q) = *reinterpret_cast<const float4*>(B + size_t(n) * ldb + kc + 4 * q);
      }
    } else {
      for (unsigned e = threadIdx.x; e < N * len; e += 64 * kMidWaves) {
        const unsigned n = e / len, k = e - n * len;
        bs[n * kMidPitch + k] = B[size_t(n) * ldb + kc + k];
      }
    }
    __syncthreads();
    while (have) {
      float b[2][4];
#pragma unroll
      for (int g = 0; g < 2; ++g) {
        const unsigned off = kb - kc + 8 * g + 4 * hi;
        const float4 t = *reinterpret_cast<const float4*>(bs + l32 * kMidPitch + off);
        b[g][0] = ncol && kc + off < kend ? t.x : 0.f;
        b[g][1] = ncol && kc + off + 1 < kend ? t.y : 0.f;
        b[g][2] = ncol && kc + off + 2 < kend ? t.z : 0.f;
        b[g][3] = ncol && kc + off + 3 < kend ? t.w : 0.f;
      }
#pragma unroll
      for (int g = 0; g < 2; ++g)
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          acc[0] = __builtin_amdgcn_mfma_f32_32x32x2f32(b[g][j], a[g][j].x, acc[0], 0, 0, 0);
          acc[1] = __builtin_amdgcn_mfma_f32_32x32x2f32(b[g][j], a[g][j].y, acc[1], 0, 0, 0);
          acc[2] = __builtin_amdgcn_mfma_f32_32x32x2f32(b[g][j], a[g][j].z, acc[2], 0, 0, 0);
          acc[3] = __builtin_amdgcn_mfma_f32_32x32x2f32(b[g][j], a[g][j].w, acc[3], 0, 0, 0);
        }
      kb += 16 * kMidWaves;
      have = kb < kend;
      if (have) load_a();
    }
  }
  // acc[c][r] of lane l: row 4 * m4 + c, column 8 * (r / 4) + 4 * (l / 32) + r % 4
  __syncthreads();  // B's entries have been read
  if (w > 0) {
#pragma unroll
    for (int r = 0; r < 16; ++r) red[w - 1][r][lane] = make_float4(acc[0][r], acc[1][r], acc[2][r], acc[3][r]);
  }
  __syncthreads();
  if (w != 0 || !live) return;
  // the slab of partial sums, or the output itself when the depth was not split over blocks
  float4* out = partial != nullptr ? reinterpret_cast<float4*>(partial) + size_t(blockIdx.y) * N * M4 + m4
                                   : reinterpret_cast<float4*>(C) + m4;
  float4 bb = make_float4(0.f, 0.f, 0.f, 0.f);
  if (partial == nullptr && bias != nullptr) bb = reinterpret_cast<const float4*>(bias)[m4];
  const bool old = partial == nullptr && bias == nullptr && beta != 0.f;
#pragma unroll
  for (int r = 0; r < 16; ++r) {
    const unsigned n = 8 * (r / 4) + 4 * hi + (r % 4);
    if (n >= N) continue;
    float4 t = make_float4(acc[0][r], acc[1][r], acc[2][r], acc[3][r]);
#pragma unroll
    for (int v = 0; v < kMidWaves - 1; ++v) {
      const float4 o = red[v][r][lane];
      t.x += o.x; t.y += o.y; t.z += o.z; t.w += o.w;
    }
    t.x += bb.x; t.y += bb.y; t.z += bb.z; t.w += bb.w;
    float4* q = out + size_t(n) * M4;
    if (old) {
      const float4 o = *q;
      t.x += beta * o.x; t.y += beta * o.y; t.z += beta * o.z; t.w += beta * o.w;
    }
    *q = t;
  }
}

static bool gemm_nn_mid_eligible(const dyhip_device* dev, size_t M, size_t N, int nseg, const GemmSeg* segs,
                                 const float* C, const GemmEpiParams& epi) {
  if (!(epi.kind == kEpiAxpby || (epi.kind == kEpiBias && epi.bias != nullptr && aligned16(epi.bias)) ||
        (epi.kind == kEpiLstmGates && epi.bias != nullptr)))
    return false;
  if (nseg < 1 || nseg > 2 || (nseg == 2 && epi.kind != kEpiLstmGates)) return false;
  for (int q = 0; q < nseg; ++q)
    if (segs[q].A == nullptr || segs[q].B == nullptr || segs[q].K < 16 || segs[q].K > 0x3FFFFFFFull || segs[q].lda % 4 != 0 ||
        !aligned16(segs[q].A))
      return false;
  return N >= 9 && N <= 32 && M >= 128 && M % 4 == 0 && M / 4 <= 0x7FFFFFFFull && aligned16(C) && dev->gemm_ws != nullptr;
}

static int gemm_nn_mid_run(dyhip_device* dev, size_t M, size_t N, int nseg, const GemmSeg* segs, float* C,
                           const GemmEpiParams& epi) {
  const unsigned M4 = static_cast<unsigned>(M / 4), bx = cdiv<unsigned>(M4, 32);
  const unsigned K0 = static_cast<unsigned>(segs[0].K), K1 = nseg > 1 ? static_cast<unsigned>(segs[1].K) : 0u;
  const unsigned K = K0 + K1;
  // depth slabs: enough blocks to fill the GPU, each with at least one 16-index step per wavefront
  unsigned slabs = cdiv<unsigned>(kMidBlocksPerCu * dev->num_cus, bx);
  const unsigned max_by_depth = cdiv<unsigned>(K, 16 * kMidWaves);
  if (slabs > max_by_depth) slabs = max_by_depth;
  if (slabs < 1) slabs = 1;
  unsigned chunk = cdiv<unsigned>(K, slabs);
  chunk = (chunk + 16 * kMidWaves - 1) / (16 * kMidWaves) * (16 * kMidWaves);  // whole steps for every wavefront
  const unsigned slabs0 = cdiv<unsigned>(K0, chunk), slabs1 = K1 ? cdiv<unsigned>(K1, chunk) : 0u;
  slabs = slabs0 + slabs1;
  DYHIP_REQUIRE(slabs <= 65535, "small-batch product: depth %u needs too many slabs", K);
  const bool gates = epi.kind == kEpiLstmGates;
  float* partial = nullptr;
  if (slabs > 1 || gates) {  // the gates epilogue lives in the second kernel
    DYHIP_REQUIRE(dev->gemm_ws_bytes >= sizeof(float) * M * N * slabs, "small-batch product: workspace too small");
    partial = static_cast<float*>(dev->gemm_ws);
  }
  const float beta = epi.kind == kEpiAxpby ? epi.beta : 0.f;
  const float* bias = epi.kind == kEpiAxpby ? nullptr : epi.bias;
  const GemmSeg s0 = segs[0], s1 = nseg > 1 ? segs[1] : segs[0];
  bool bvec = true;
  for (int q = 0; q < nseg; ++q) bvec = bvec && segs[q].K % 4 == 0 && segs[q].ldb % 4 == 0 && aligned16(segs[q].B);
  const dim3 grid(bx, slabs), block(64 * kMidWaves);
  if (bvec)
    hipLaunchKernelGGL(gemm_nn_mid_kernel<true>, grid, block, 0, dev->stream, M4, static_cast<unsigned>(N), chunk, s0, s1,
                       slabs0, C, beta, bias, partial);
  else
    hipLaunchKernelGGL(gemm_nn_mid_kernel<false>, grid, block, 0, dev->stream, M4, static_cast<unsigned>(N), chunk, s0, s1,
                       slabs0, C, beta, bias, partial);
  DYHIP_CHECK_LAUNCH();
  if (partial != nullptr) {
    const size_t total = size_t(M4) * N;
    const dim3 g2(static_cast<unsigned>(cdiv<size_t>(total, kCombineThreads)));
    if (gates)
      hipLaunchKernelGGL(gemm_nn_thin_combine_kernel<true>, g2, dim3(kCombineThreads), 0, dev->stream, M4, static_cast<unsigned>(N),
                         slabs, reinterpret_cast<const float4*>(partial), reinterpret_cast<float4*>(C), 0.f, bias, epi.H,
                         epi.logistic_mode);
    else
      hipLaunchKernelGGL(gemm_nn_thin_combine_kernel<false>, g2, dim3(kCombineThreads), 0, dev->stream, M4, static_cast<unsigned>(N),
                         slabs, reinterpret_cast<const float4*>(partial), reinterpret_cast<float4*>(C), beta, bias, 0u, 0);
    DYHIP_CHECK_LAUNCH();
  }
  return DYHIP_OK;
}


// ---- C (+)= A * B^T with at most 32 rows of C and a deep sum: the weight gradient of an output layer with a handful
// of classes over thousands of tokens (A = dy, 20 x 4480; B = x, 512 x 4480).  Memory work on B, which is read once:
// a thread owns a column of C (adjacent threads adjacent rows of B: every load of a wavefront is one run), keeps its
// M sums in registers, and takes A's entries, the same for the whole block, from LDS; the depth is cut over
// gridDim.y blocks whose slices the split reduce kernel adds.  The 128-row tile kernel ran 20 live rows of 128 and
// took 17 us for 9.6 MB.
constexpr unsigned kFewRowsChunk = 128;  // depth indices a block takes (its part of A in LDS: 16 KB at 32 rows)
template <int MP>  // M rounded up to a multiple of four
__global__ __launch_bounds__(256) void gemm_nt_fewrows_kernel(unsigned M, unsigned N, unsigned K, unsigned chunk,
                                                              const float* __restrict__ A, size_t lda,
                                                              const float* __restrict__ B, size_t ldb,
                                                              float* __restrict__ partial) {
  // a block: 64 columns of C (lanes) x four wavefronts that take a quarter of the block's depth range each and meet in
  // LDS, so that the slices left for the reduce kernel stay few
  __shared__ __attribute__((aligned(16))) float as[kFewRowsChunk][MP];
  __shared__ float red[3][MP][64];
  const unsigned k0 = blockIdx.y * chunk, k1 = min(K, k0 + chunk);
  for (unsigned e = threadIdx.x; e < (k1 - k0) * MP; e += 256) {
    const unsigned k = e / MP, m = e % MP;
    as[k][m] = m < M ? A[m + size_t(k0 + k) * lda] : 0.f;
  }
  __syncthreads();
  const unsigned lane = threadIdx.x & 63, w = threadIdx.x >> 6;
  const unsigned n = blockIdx.x * 64 + lane, nc = n < N ? n : N - 1;
  const unsigned sub = chunk / 4, w0 = min(k1, k0 + w * sub), w1 = min(k1, w0 + sub);
  float acc[MP];
#pragma unroll
  for (int m = 0; m < MP; ++m) acc[m] = 0.f;
  // eight loads of B in flight, the next eight requested before the current eight are used
  auto fetch = [&](float (&b)[8], unsigned k) {
    if (k < w1) {  // uniform
#pragma unroll
      for (int u = 0; u < 8; ++u) b[u] = B[nc + size_t(min(k + u, w1 - 1)) * ldb];  // clamped; the extra terms are not added
    }
  };
  auto use = [&](const float (&b)[8], unsigned k) {
#pragma unroll
    for (int u = 0; u < 8; ++u) {
      if (k + u >= w1) break;  // uniform
#pragma unroll
      for (int m4 = 0; m4 < MP / 4; ++m4) {
        const float4 a = *reinterpret_cast<const float4*>(&as[k + u - k0][4 * m4]);  // the same address in every lane
        acc[4 * m4] = fmaf(a.x, b[u], acc[4 * m4]);
        acc[4 * m4 + 1] = fmaf(a.y, b[u], acc[4 * m4 + 1]);
        acc[4 * m4 + 2] = fmaf(a.z, b[u], acc[4 * m4 + 2]);
        acc[4 * m4 + 3] = fmaf(a.w, b[u], acc[4 * m4 + 3]);
      }
    }
  };
  float b0[8], b1[8];
  fetch(b0, w0);
  for (unsigned k = w0; k < w1; k += 16) {
    fetch(b1, k + 8);
    use(b0, k);
    fetch(b0, k + 16);
    use(b1, k + 8);
  }
  if (w > 0) {
#pragma unroll
    for (int m = 0; m < MP; ++m) red[w - 1][m][lane] = acc[m];
  }
  __syncthreads();
  if (w != 0 || n >= N) return;
  float* out = partial + size_t(blockIdx.y) * M * N + size_t(n) * M;
#pragma unroll
  for (int m = 0; m < MP; ++m)
    if (unsigned(m) < M) out[m] = ((acc[m] + red[0][m][lane]) + red[1][m][lane]) + red[2][m][lane];
}

static bool gemm_nt_fewrows_eligible(const dyhip_device* dev, size_t M, size_t N, size_t K, const GemmEpiParams& epi) {
  if (epi.kind != kEpiAxpby || M < 1 || M > 32 || N < 256 || K < 256 || N > 0xFFFFFF00ull || K > 0x7FFFFFFFull) return false;
  const size_t splits = cdiv<size_t>(K, kFewRowsChunk);
  return splits <= 65535 && dev->gemm_ws != nullptr && dev->gemm_ws_bytes >= sizeof(float) * M * N * splits;
}

static int gemm_nt_fewrows_run(dyhip_device* dev, size_t M, size_t N, size_t K, const float* A, size_t lda, const float* B,
                               size_t ldb, float* C, const GemmEpiParams& epi) {
  // as few depth ranges as give every CU a block, each at most kFewRowsChunk long (a multiple of 32: the block's four
  // wavefronts take whole groups of eight)
  const size_t bx = cdiv<size_t>(N, 64), cus = dev->num_cus > 0 ? size_t(dev->num_cus) : 256;
  size_t splits = std::max(cdiv<size_t>(K, kFewRowsChunk), std::min(cdiv<size_t>(cus, bx), cdiv<size_t>(K, 32)));
  const unsigned chunk = static_cast<unsigned>(cdiv<size_t>(cdiv<size_t>(K, splits), 32) * 32);
  splits = cdiv<size_t>(K, chunk);
  DYHIP_REQUIRE(chunk <= kFewRowsChunk && dev->gemm_ws_bytes >= sizeof(float) * M * N * splits,
                "few-row product: %zu slices of %zu x %zu floats do not fit the workspace", splits, M, N);
  float* partial = static_cast<float*>(dev->gemm_ws);
  const dim3 grid(static_cast<unsigned>(bx), static_cast<unsigned>(splits)), block(256);
#define DYHIP_FEWROWS(MP)                                                                                         \
  hipLaunchKernelGGL(gemm_nt_fewrows_kernel<MP>, grid, block, 0, dev->stream, static_cast<unsigned>(M),           \
                     static_cast<unsigned>(N), static_cast<unsigned>(K), chunk, A, lda, B, ldb, partial)
  switch ((M + 3) / 4) {
    case 1: DYHIP_FEWROWS(4); break;
    case 2: DYHIP_FEWROWS(8); break;
    case 3: DYHIP_FEWROWS(12); break;
    case 4: DYHIP_FEWROWS(16); break;
    case 5: DYHIP_FEWROWS(20); break;
    case 6: DYHIP_FEWROWS(24); break;
    case 7: DYHIP_FEWROWS(28); break;
    default: DYHIP_FEWROWS(32); break;
  }
#undef DYHIP_FEWROWS
  DYHIP_CHECK_LAUNCH();
  const size_t total = M * N;
  // many slices of a small output: the combine kernel that spreads the slices over a block's threads (a thread per
  // output walking 35 slices eight at a time was half of the product's time)
  if (epi.beta == 0.f || epi.beta == 1.f)
    return combine_partial_rows(dev, total, static_cast<unsigned>(splits), partial, C, epi.beta == 1.f);
  hipLaunchKernelGGL(gemm_splitk_reduce_kernel<kEpiAxpby>, dim3(static_cast<unsigned>(cdiv<size_t>(total, 256))), dim3(256), 0,
                     dev->stream, M, total, static_cast<unsigned>(splits), partial, C, epi);
  DYHIP_CHECK_LAUNCH();
  return DYHIP_OK;
}

int gemm_run(dyhip_device* dev, bool a_kmajor, bool b_kmajor, size_t M, size_t N, int nseg, const GemmSeg* segs,
             float* C, const GemmEpiParams& epi, const GemmBatch* batch) {
  const bool to_caller = epi.kind == kEpiPartials;
  if (to_caller) {
    DYHIP_REQUIRE(epi.partials != nullptr && epi.splits_out != nullptr, "null split-K output");
    *epi.splits_out = 0;
  }
  if (M == 0 || N == 0) return DYHIP_OK;
  DYHIP_REQUIRE(nseg >= 1 && nseg <= kGemmMaxSeg, "GEMM supports 1..%d K segments", kGemmMaxSeg);
  DYHIP_REQUIRE(to_caller || C != nullptr, "null GEMM output");
  // large outputs: the 256 x 256-tile kernel over the depth's multiple of 32, the rest of the depth added by the
  // kernel below; when only the leading columns form full rounds of tiles, those columns, and the rest as a product
  // of its own
  if (nseg == 1 && (batch == nullptr || batch->count <= 1) && segs[0].A != nullptr && segs[0].B != nullptr &&
      (epi.kind == kEpiAxpby || (epi.kind == kEpiBias && epi.bias != nullptr && aligned16(epi.bias)))) {
    const GemmSeg& s0 = segs[0];
    // leading full rounds first: the 128-wide kernel finishes a few remaining tile columns (96 of its tiles) sooner
    // than one sequence of k-tiles over all tiles does (4096x4480x1024: 335 against 349 us)
    size_t cols = gemm_wide_whole_rounds_columns(dev, a_kmajor, b_kmajor, M, N, s0.K, s0.A, s0.lda, s0.B, s0.ldb, C);
    if (cols == 0 && gemm_wide_eligible(dev, a_kmajor, b_kmajor, M, N, s0.K, s0.A, s0.lda, s0.B, s0.ldb, C)) cols = N;
    if (cols > 0) {
      const size_t K32 = s0.K / kBK * kBK;
      DYHIP_CHECK_STATUS(gemm_wide_run(dev, a_kmajor, b_kmajor, M, cols, K32, s0.A, s0.lda, s0.B, s0.ldb, C,
                                       epi.kind == kEpiAxpby ? epi.beta : 0.f,
                                       epi.kind == kEpiBias ? epi.bias : nullptr));
      if (K32 < s0.K) {
        GemmSeg tail{s0.A + (a_kmajor ? K32 : K32 * s0.lda), s0.lda, s0.B + (b_kmajor ? K32 : K32 * s0.ldb), s0.ldb,
                     s0.K - K32};
        GemmEpiParams acc{};
        acc.kind = kEpiAxpby;
        acc.beta = 1.f;
        DYHIP_CHECK_STATUS(gemm_run(dev, a_kmajor, b_kmajor, M, cols, 1, &tail, C, acc, nullptr));
      }
      if (cols == N) return DYHIP_OK;
      GemmSeg rest{s0.A, s0.lda, s0.B + (b_kmajor ? cols * s0.ldb : cols), s0.ldb, s0.K};
      return gemm_run(dev, a_kmajor, b_kmajor, M, N - cols, 1, &rest, C + cols * M, epi, nullptr);
    }
  }
  // 5..256 columns with a depth that is a multiple of four: the one-launch fragment-order product on the operands as
  // they lie (4096 x 20 x 1024: 8.4 us against 13.7 us for the two-launch 9..32-column product below, 4096 x 128 x 1024:
  // 14.2 against 22.9 us for the tile kernel with split depth, 4096 x 8 x 1024: 8.2 against 10.7 us for the
  // matrix-times-vector kernels, which keep one to four columns: 4096 x 1 x 1024 6.9 against 8.0 us)
  if ((batch == nullptr || batch->count <= 1) && !a_kmajor && b_kmajor && C != nullptr && N >= 5 && N <= 256) {
    bool taken = false;
    DYHIP_CHECK_STATUS(skinny_nn_gemm(dev, M, N, nseg, segs, C, epi, &taken));
    if (taken) return DYHIP_OK;
  }
  if ((batch == nullptr || batch->count <= 1) && !a_kmajor && b_kmajor && C != nullptr &&
      gemm_nn_thin_eligible(dev, M, N, nseg, segs, C, epi))
    return gemm_nn_thin_run(dev, M, N, nseg, segs, C, epi);
  // a batch of matrices times their own vector(s) (the context vector of an attention over a batch: 1024 x 1 x 35
  // times 128 items 11.1 us with a matrix-core tile per wavefront): the items in gridDim.z, one slab each
  if (batch != nullptr && batch->count > 1 && batch->count <= 65535u && nseg == 1 && epi.kind == kEpiAxpby && !a_kmajor &&
      b_kmajor && C != nullptr && segs[0].K <= kGemvMaxChunk && batch->stride_a % 4 == 0 && batch->stride_c % 4 == 0 &&
      batch->stride_c >= M * N && gemm_nn_thin_eligible(dev, M, N, nseg, segs, C, epi))
    return gemm_nn_thin_run(dev, M, N, nseg, segs, C, epi, batch);
  if ((batch == nullptr || batch->count <= 1) && !a_kmajor && b_kmajor && C != nullptr &&
      gemm_nn_mid_eligible(dev, M, N, nseg, segs, C, epi))
    return gemm_nn_mid_run(dev, M, N, nseg, segs, C, epi);
  // a depth of at most 32: the rank-K update, except for outputs above 4 MB at a depth of 24 or 32, where its
  // re-reads of the left operand (once per eight columns, from the L2s) cost more than the burst-fetch kernel's
  // matrix-core tiles (4096 x 1024: depth 16 8.9 against 9.1 us, depth 24 13.2 against 9.6 us, depth 32 15.4 against
  // 10.1 us; 1024 x 1024 x 32: 5.3 against 7.7 us)
  if (nseg == 1 && batch != nullptr && batch->count > 1 && a_kmajor && b_kmajor && epi.kind == kEpiAxpby &&
      segs[0].A != nullptr && segs[0].B != nullptr && C != nullptr) {
    bool taken = false;
    DYHIP_CHECK_STATUS(thin_tn_batched(dev, M, N, segs[0].K, segs[0].A, segs[0].lda, segs[0].B, segs[0].ldb, epi.beta, C,
                                       batch, &taken));
    if (taken) return DYHIP_OK;
  }
  // the same for the items of a strided batch whose operands stay on the 16-byte grid (dH += dctx * a^T of an attention
  // over a batch: 1024 x 35 x 1 times 128 items 22.8 us with a 32 x 32 matrix-core tile per wavefront)
  if (nseg == 1 && batch != nullptr && batch->count > 1 && batch->count <= 65535u && !a_kmajor && !b_kmajor &&
      epi.kind == kEpiAxpby && segs[0].A != nullptr && segs[0].B != nullptr && C != nullptr &&
      batch->stride_a % 4 == 0 && batch->stride_c % 4 == 0 && batch->stride_c >= M * N &&
      gemm_nt_thin_eligible(M, N, segs[0].K, segs[0].A, segs[0].lda, segs[0].B, C, epi.beta))
    return gemm_nt_thin_run(dev, M, N, segs[0].K, segs[0].A, segs[0].lda, segs[0].B, segs[0].ldb, C, epi.beta, batch);
  if (nseg == 1 && (batch == nullptr || batch->count <= 1) && !a_kmajor && !b_kmajor && epi.kind == kEpiAxpby &&
      segs[0].A != nullptr && segs[0].B != nullptr && C != nullptr &&
      gemm_nt_thin_eligible(M, N, segs[0].K, segs[0].A, segs[0].lda, segs[0].B, C, epi.beta) &&
      !(segs[0].K >= 24 && M * N * sizeof(float) > (size_t(4) << 20) &&
        gemm_shallow_nt_eligible(dev, M, N, segs[0].K, segs[0].A, segs[0].lda, segs[0].B, segs[0].ldb, C)))
    return gemm_nt_thin_run(dev, M, N, segs[0].K, segs[0].A, segs[0].lda, segs[0].B, segs[0].ldb, C, epi.beta);
  if (nseg == 1 && (batch == nullptr || batch->count <= 1) && !a_kmajor && !b_kmajor && !to_caller && C != nullptr &&
      segs[0].A != nullptr && segs[0].B != nullptr && gemm_nt_fewrows_eligible(dev, M, N, segs[0].K, epi))
    return gemm_nt_fewrows_run(dev, M, N, segs[0].K, segs[0].A, segs[0].lda, segs[0].B, segs[0].ldb, C, epi);
  if (nseg == 1 && (batch == nullptr || batch->count <= 1) && !a_kmajor && !b_kmajor && epi.kind == kEpiAxpby &&
      segs[0].A != nullptr && segs[0].B != nullptr &&
      gemm_shallow_nt_eligible(dev, M, N, segs[0].K, segs[0].A, segs[0].lda, segs[0].B, segs[0].ldb, C))
    return gemm_shallow_nt_run(dev, M, N, segs[0].K, segs[0].A, segs[0].lda, segs[0].B, segs[0].ldb, C, epi.beta);
  const bool batched = batch != nullptr && batch->count > 1;
  const bool tile_vec = nseg == 1 && aligned16(segs[0].A) && segs[0].lda % 4 == 0 && aligned16(segs[0].B) &&
                        segs[0].ldb % 4 == 0 && (!batched || (batch->stride_a % 4 == 0 && batch->stride_b % 4 == 0));
  if (nseg == 1 && !to_caller && C != nullptr && segs[0].A != nullptr && segs[0].B != nullptr &&
      gemm_small_eligible(dev, M, N, segs[0].K, epi, batch ? batch->count : 1, tile_vec)) {
    if (batch != nullptr && batch->count > 1)
      DYHIP_REQUIRE(batch->stride_c >= M * N, "batch items of the GEMM output overlap");
    return gemm_small_run(dev, a_kmajor, b_kmajor, M, N, segs[0], C, epi, batch);
  }
  GemmArgs g;
  g.nseg = nseg;
  g.M = M;
  g.N = N;
  g.C = C;
  g.beta = epi.kind == kEpiAxpby ? epi.beta : 0.f;
  g.bias = epi.kind == kEpiBias ? epi.bias : nullptr;
  g.ktiles_total = 0;
  g.ktiles0 = 0;
  g.seg[1] = GemmSeg{nullptr, 0, nullptr, 0, 0};
  const unsigned items = batch ? batch->count : 1;
  g.stride_a = g.stride_b = g.stride_c = 0;
  bool vec = true;
  if (items > 1) {
    DYHIP_REQUIRE(nseg == 1 && epi.kind == kEpiAxpby, "a strided-batched GEMM has one K segment and the axpby epilogue");
    DYHIP_REQUIRE(batch->stride_c >= M * N, "batch items of the GEMM output overlap");
    g.stride_a = batch->stride_a;
    g.stride_b = batch->stride_b;
    g.stride_c = batch->stride_c;
    vec = g.stride_a % 4 == 0 && g.stride_b % 4 == 0;
  }
  for (int s = 0; s < nseg; ++s) {
    DYHIP_REQUIRE(segs[s].A != nullptr && segs[s].B != nullptr, "null GEMM operand");
    g.seg[s] = segs[s];
    const unsigned kt = static_cast<unsigned>(cdiv<size_t>(segs[s].K, kBK));
    if (s == 0) g.ktiles0 = kt;
    g.ktiles_total += kt;
    vec = vec && aligned16(segs[s].A) && segs[s].lda % 4 == 0 && aligned16(segs[s].B) && segs[s].ldb % 4 == 0;
  }
  g.vec_ok = vec ? 1 : 0;
  // a group of four runs along k for a k-major operand and along m (or n) otherwise
  bool edge4 = vec && (a_kmajor || M % 4 == 0) && (b_kmajor || N % 4 == 0);
  for (int s = 0; s < nseg; ++s) edge4 = edge4 && (!(a_kmajor || b_kmajor) || segs[s].K % 4 == 0);
  g.edge4_ok = edge4 ? 1 : 0;
  const size_t out_bytes = M * N * sizeof(float);
  const size_t ws_bytes = to_caller ? epi.partials_bytes : dev->gemm_ws_bytes;
  void* ws = to_caller ? static_cast<void*>(epi.partials) : dev->gemm_ws;
  const bool fused_epi = epi.kind == kEpiLstmGates;  // needs the whole sum before the activation
  const bool must_partial = fused_epi || to_caller;
  GemmPlan plan{N <= 64 ? 1 : 2, 1};
  if (g.ktiles_total > 0)
    plan = plan_gemm(dev, M, N, g.ktiles_total, items > 1 ? 1 : ws_bytes / out_bytes, must_partial);
  unsigned splits = plan.splits;
  const size_t tiles_m = cdiv<size_t>(M, kBM), tiles_n = cdiv<size_t>(N, size_t(64) * plan.wn);
  DYHIP_REQUIRE(tiles_m * tiles_n < (size_t(1) << 31), "GEMM too large");
  g.ktiles_per_split = g.ktiles_total == 0 ? 1 : cdiv<unsigned>(g.ktiles_total, splits);
  splits = g.ktiles_total == 0 ? 1 : cdiv<unsigned>(g.ktiles_total, g.ktiles_per_split);
  const bool use_partial = splits > 1 || must_partial;
  if (use_partial)
    DYHIP_REQUIRE(ws != nullptr && ws_bytes >= out_bytes * splits,
                  "GEMM output of %zu bytes x %u splits does not fit the %zu-byte split-K workspace", out_bytes,
                  splits, ws_bytes);
  g.partial = use_partial ? static_cast<float*>(ws) : nullptr;
  // grid z holds at most 65535 batch items per launch
  for (unsigned first = 0; first < items; first += 65535u) {
    const unsigned nb = items - first < 65535u ? items - first : 65535u;
    GemmArgs h = g;
    h.seg[0].A += size_t(first) * g.stride_a;
    h.seg[0].B += size_t(first) * g.stride_b;
    if (h.C != nullptr) h.C += size_t(first) * g.stride_c;
    if (a_kmajor && b_kmajor) launch_tiles<true, true>(dev, h, (unsigned)tiles_m, (unsigned)tiles_n, splits, plan.wn, nb);
    else if (a_kmajor && !b_kmajor) launch_tiles<true, false>(dev, h, (unsigned)tiles_m, (unsigned)tiles_n, splits, plan.wn, nb);
    else if (!a_kmajor && b_kmajor) launch_tiles<false, true>(dev, h, (unsigned)tiles_m, (unsigned)tiles_n, splits, plan.wn, nb);
    else launch_tiles<false, false>(dev, h, (unsigned)tiles_m, (unsigned)tiles_n, splits, plan.wn, nb);
  }
  DYHIP_CHECK_LAUNCH();
  if (to_caller) {
    *epi.splits_out = splits;
    return DYHIP_OK;
  }
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

static GemmEpiParams axpby(float beta) {
  GemmEpiParams ep{};
  ep.kind = kEpiAxpby;
  ep.beta = beta;
  return ep;
}

}  // namespace dyhip

using namespace dyhip;

extern "C" {

int dyhip_gemm_nn(dyhip_device* dev, size_t M, size_t N, size_t K, const float* l, const float* r, float beta,
                  float* y) {
  DYHIP_CHECK_DEV(dev);
  // A row vector times a matrix (v^T * X of an attention's scores) is X^T * v with the same bytes on both sides:
  // the streaming transposed product instead of a matrix-core tile with one live row (1 x 4480 x 512: 20.2 -> 4.7 us)
  if (M == 1 && N > 1 && l != nullptr && r != nullptr && y != nullptr) {
    bool taken = false;
    DYHIP_CHECK_STATUS(skinny_tn_gemm(dev, N, 1, K, r, K, l, K, beta, y, &taken));
    if (taken) return DYHIP_OK;
  }
  GemmSeg s{l, M, r, K, K};
  return gemm_run(dev, false, true, M, N, 1, &s, y, axpby(beta));
}

int dyhip_affine_forward(dyhip_device* dev, size_t M, size_t N, size_t K, const float* bias, const float* W,
                         const float* x, float* fx) {
  DYHIP_CHECK_DEV(dev);
  DYHIP_REQUIRE(bias != nullptr, "AffineTransform: null bias");
  GemmSeg s{W, M, x, K, K};
  GemmEpiParams ep{};
  ep.kind = kEpiBias;
  ep.bias = bias;
  return gemm_run(dev, false, true, M, N, 1, &s, fx, ep);
}

int dyhip_gemm_tn(dyhip_device* dev, size_t M, size_t N, size_t K, const float* l, const float* r, float beta,
                  float* y) {
  DYHIP_CHECK_DEV(dev);
  // A depth of one (the gradient of X in v^T * X: v * dy): both operands are vectors, and the outer product is the
  // rank-one update of the l * r^T form
  if (K == 1 && l != nullptr && r != nullptr && y != nullptr &&
      gemm_nt_thin_eligible(M, N, 1, l, M, r, y, beta))
    return gemm_nt_thin_run(dev, M, N, 1, l, M, r, N, y, beta);
  if (l != nullptr && r != nullptr && y != nullptr) {
    bool taken = false;
    DYHIP_CHECK_STATUS(skinny_tn_gemm(dev, M, N, K, l, K, r, K, beta, y, &taken));
    if (taken) return DYHIP_OK;
  }
  GemmSeg s{l, K, r, K, K};
  return gemm_run(dev, true, true, M, N, 1, &s, y, axpby(beta));
}

int dyhip_gemm_nt(dyhip_device* dev, size_t M, size_t N, size_t K, const float* l, const float* r, float beta,
                  float* y) {
  DYHIP_CHECK_DEV(dev);
  // A row vector times a transposed matrix (the gradient of v in v^T * X) is that matrix times the vector
  if (M == 1 && N >= 256 && N % 4 == 0 && l != nullptr && r != nullptr && y != nullptr) {
    GemmSeg t{r, N, l, K, K};
    const GemmEpiParams ep = axpby(beta);
    if (gemm_nn_thin_eligible(dev, N, 1, 1, &t, y, ep)) return gemm_nn_thin_run(dev, N, 1, 1, &t, y, ep);
  }
  GemmSeg s{l, M, r, N, K};
  return gemm_run(dev, false, false, M, N, 1, &s, y, axpby(beta));
}

int dyhip_gemm_strided_batched(dyhip_device* dev, int trans_l, int trans_r, size_t M, size_t N, size_t K,
                               const float* l, size_t stride_l, const float* r, size_t stride_r, float beta, float* y,
                               size_t stride_y, unsigned batch) {
  DYHIP_CHECK_DEV(dev);
  DYHIP_REQUIRE(!(trans_l && trans_r), "the strided-batched GEMM has the forms l*r, l^T*r and l*r^T");
  if (batch == 0) return DYHIP_OK;
  GemmSeg s{l, trans_l ? K : M, r, trans_r ? N : K, K};
  GemmBatch b{batch, stride_l, stride_r, stride_y};
  return gemm_run(dev, trans_l != 0, trans_r == 0, M, N, 1, &s, y, axpby(beta), &b);
}

int dyhip_gemm_uses_wide_tiles(dyhip_device* dev, int trans_l, int trans_r, size_t M, size_t N, size_t K,
                               int* wide_tiles) {
  DYHIP_CHECK_DEV(dev);
  DYHIP_REQUIRE(wide_tiles != nullptr, "null output");
  DYHIP_REQUIRE(!(trans_l && trans_r), "the GEMM has the forms l*r, l^T*r and l*r^T");
  // any 16-byte aligned address stands for the operands: only alignment is looked at
  const float* aligned = reinterpret_cast<const float*>(uintptr_t(256));
  const size_t lda = trans_l ? K : M, ldb = trans_r ? N : K;
  if (gemm_wide_whole_rounds_columns(dev, trans_l != 0, trans_r == 0, M, N, K, aligned, lda, aligned, ldb, aligned) > 0)
    *wide_tiles = 2;
  else if (gemm_wide_eligible(dev, trans_l != 0, trans_r == 0, M, N, K, aligned, lda, aligned, ldb, aligned)) *wide_tiles = 1;
  else *wide_tiles = 0;
  return DYHIP_OK;
}

int dyhip_gemm_wide_segments(size_t M, size_t N, size_t K, unsigned segments, unsigned* starts,
                             unsigned* k_tiles_per_tile, int* finish_in_kernel) {
  DYHIP_REQUIRE(starts && k_tiles_per_tile && finish_in_kernel, "null output");
  DYHIP_REQUIRE(segments >= 1 && segments <= 65536 && M >= 1 && N >= 1 && K >= 32, "bad shape or segment count");
  DYHIP_REQUIRE(cdiv<size_t>(M, 256) * cdiv<size_t>(N, 256) * (K / 32) < (size_t(1) << 31), "too many k-tiles");
  gemm_wide_describe(M, N, K, segments, starts, k_tiles_per_tile, finish_in_kernel);
  return DYHIP_OK;
}

int dyhip_gemm_tn_acc(dyhip_device* dev, size_t M, size_t N, size_t K, const float* l, const float* r, float* y) {
  return dyhip_gemm_tn(dev, M, N, K, l, r, 1.0f, y);
}

int dyhip_gemm_nt_acc(dyhip_device* dev, size_t M, size_t N, size_t K, const float* l, const float* r, float* y) {
  return dyhip_gemm_nt(dev, M, N, K, l, r, 1.0f, y);
}

}  // extern "C"
