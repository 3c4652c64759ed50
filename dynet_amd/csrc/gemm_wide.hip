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
// Work distribution.  The tile count rarely divides the CU count, and a round of one tile per CU that is not full
// leaves CUs idle for the whole round.  So the units of work are k-tiles: all k-tiles of all tiles, tile by tile, form
// one sequence that is cut into one equal segment per CU, and a block walks its segment, loads running two k-tiles
// ahead of the MFMAs straight across tile boundaries (the next tile's operands arrive under the stores of the one
// just finished).  A tile that lies wholly inside a segment is written out by that block.  A tile cut by segment
// boundaries is completed in one of two ways:
//   * segments at least a tile long (more tiles than CUs): a tile is cut at most once.  The block that holds its later
//     k-tiles (the start of its segment) leaves a partial tile in the workspace and raises a flag; the block that
//     holds its first k-tiles (the end of its segment, hundreds of microseconds later) adds that partial tile to its
//     own, applies the epilogue and stores.  No second kernel, no float atomics, a fixed order of additions.
//     Segments are dealt in descending block order, so a block only ever waits for a block dispatched before it,
//     which itself waits for nobody before it raises its flag; the wait is bounded anyway, and a wait that gave up is
//     counted and reported by dyhip_device_sync.
//   * shorter segments (fewer tiles than CUs, or little more): a tile spans several segments, one CU adding all their
//     partial tiles would take longer than its share of the product (256 KiB per partial tile at one CU's ~30 GB/s
//     from beyond its L2), so every part goes to the workspace and a second kernel, 16 blocks per tile, adds them in
//     segment order and applies the epilogue.
// When the tiles are a whole number of rounds plus a few tile columns, the caller gives this kernel the leading
// columns (whole rounds, nothing cut) and the rest to the 128-wide kernel.
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
  const float* bias;    // C = bias[m] + sum when set (beta unused)
  float* slots;         // partial tiles, [32][512 threads][4] in the order the threads hold them: slot = segment when
                        // tiles are finished in the kernel, else 2 x segment + (0: the segment's first item, 1: its last)
  unsigned* flags;      // one per segment, zero between launches; the last of the kGemmFlagWords counts waits that gave up
  unsigned lda, ldb;
  unsigned M, N;
  unsigned nt;          // k-tiles of a tile
  unsigned tiles_m;
  unsigned units;       // tiles x nt, dealt to the blocks in equal segments
  unsigned spin_limit;  // polls (about a microsecond apart) before a wait for another block gives up
  int raise_flags;      // 1; 0 only in tests of the give-up path (the partial tile is stored, its flag stays down)
  int finish_in_kernel; // a cut tile is finished by the block that holds its first k-tiles; else by the second kernel
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

// the same with the four global addresses formed ahead of time (biased back by the instruction offset already)
template <int OP>
__device__ __forceinline__ void load_chunks_at(const float* const (&ptr)[4], float* wave_stage) {
  constexpr int I0 = OP == 0 ? -4096 : 0;
#define DYHIP_LOAD_CHUNK(u) \
  __builtin_amdgcn_global_load_lds((global_ptr_t)(ptr[u]), (lds_ptr_t)wave_stage, 16, I0 + u * 1024, 0);
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

// Values that blocks on different L2s hand to each other inside one launch go past those caches (each L2 serves one
// eighth of the chip and does not see the others' lines): relaxed system-scope atomic accesses, which the compiler
// offers up to 64 bits, two per 128-bit group.  They are ordinary accesses to the compiler: it counts them, waits for
// them before their values are used and pads the stores' data registers itself.
typedef float wide_v4 __attribute__((ext_vector_type(4)));
__device__ __forceinline__ unsigned long long pack_through(float lo, float hi) {
  return (unsigned long long)__float_as_uint(lo) | ((unsigned long long)__float_as_uint(hi) << 32);
}
__device__ __forceinline__ void store_through(float* p, float x, float y, float z, float w) {
  unsigned long long* q = reinterpret_cast<unsigned long long*>(p);
  __hip_atomic_store(q, pack_through(x, y), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
  __hip_atomic_store(q + 1, pack_through(z, w), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
}
__device__ __forceinline__ wide_v4 load_through(const float* p) {
  const unsigned long long* q = reinterpret_cast<const unsigned long long*>(p);
  const unsigned long long lo = __hip_atomic_load(q, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
  const unsigned long long hi = __hip_atomic_load(q + 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
  const wide_v4 v = {__uint_as_float(unsigned(lo)), __uint_as_float(unsigned(lo >> 32)), __uint_as_float(unsigned(hi)),
                     __uint_as_float(unsigned(hi >> 32))};
  return v;
}

// first unit of segment s when `units` k-tiles are dealt to `segments` blocks: floor(s * units / segments) in 32-bit
// arithmetic (segments <= 65536)
__host__ __device__ __forceinline__ unsigned segment_start(unsigned s, unsigned units, unsigned segments) {
  const unsigned q = units / segments, rm = units - q * segments;
  return s * q + s * rm / segments;
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

  // this block's segment of the unit sequence (tile-major, k-tiles ascending inside a tile).  Segments are handed out
  // in descending order of block index: the blocks that a block may have to wait for (below) have lower indices and
  // were therefore dispatched before it.
  const unsigned segments = gridDim.x, seg = segments - 1 - blockIdx.x;
  const unsigned u0 = segment_start(seg, g.units, segments), u1 = segment_start(seg + 1, g.units, segments);
  if (u0 == u1) return;

  // Loads run two units ahead of the product, across tile boundaries (a unit two ahead lies in this tile or the next:
  // a tile has at least two k-tiles), and repeat the segment's last unit at its end: unconditional loads and selects
  // keep the loop one basic block.
  const unsigned last = u1 - 1, tiles = g.units / nt;
  unsigned offa[4], offb[4], offa_n[4], offb_n[4];
  {
    const unsigned t0 = u0 / nt;
    load_offsets<AK>(offa_n, g.lda, (t0 % g.tiles_m) * kWT, g.M);
    load_offsets<BKM>(offb_n, g.ldb, (t0 / g.tiles_m) * kWT, g.N);
  }
  // DYHIP_WIDE_AIM forms the eight addresses of a unit's loads (early in a k-tile, under its MFMAs: in front of the
  // loads themselves the arithmetic would hold up both wavefronts of a SIMD right after their barrier),
  // DYHIP_WIDE_FIRE issues the loads.
  const float *pa_[4], *pb_[4];
#define DYHIP_WIDE_AIM(unit, ub)                                                        \
  {                                                                                     \
    const unsigned p_ = min((unit), last);                                              \
    const bool nxt_ = p_ >= (ub) + nt;                                                  \
    const unsigned kk_ = p_ - (ub) - (nxt_ ? nt : 0u);                                  \
    _Pragma("unroll") for (int u_ = 0; u_ < 4; ++u_) {                                  \
      pa_[u_] = g.A + kk_ * stepa + (nxt_ ? offa_n[u_] : offa[u_]) - (-4096 + u_ * 1024) / 4; \
      pb_[u_] = g.B + kk_ * stepb + (nxt_ ? offb_n[u_] : offb[u_]) - (u_ * 1024) / 4;   \
      asm volatile("" : "+v"(pa_[u_]), "+v"(pb_[u_]));                                  \
    }                                                                                   \
  }
#define DYHIP_WIDE_FIRE(stage)         \
  load_chunks_at<0>(pa_, (stage));     \
  load_chunks_at<1>(pb_, (stage));
  float a[2][4][4], b[2][4][2];
  int buf = 0;

  for (unsigned pos = u0; pos < u1;) {
    const unsigned tile = pos / nt, ub = tile * nt, kt0 = pos - ub, kt1 = min(nt, u1 - ub);
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      offa[u] = offa_n[u];
      offb[u] = offb_n[u];
    }
    {
      const unsigned tn_ = min(tile + 1, tiles - 1);
      load_offsets<AK>(offa_n, g.lda, (tn_ % g.tiles_m) * kWT, g.M);
      load_offsets<BKM>(offb_n, g.ldb, (tn_ / g.tiles_m) * kWT, g.N);
    }
    if (pos == u0) {
      DYHIP_WIDE_AIM(pos, ub)
      DYHIP_WIDE_FIRE(wave_stage)
      DYHIP_WIDE_AIM(pos + 1, ub)
      DYHIP_WIDE_FIRE(wave_stage + kStageFloats)
      __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0)
      __syncthreads();
      read_a<AK>(a[0], lds + oa, 0, sw);
      read_b<BKM>(b[0], lds + ob, 0, sw);
    }
    pos += kt1 - kt0;
    floatx16 acc[2][4];
#pragma unroll
    for (int u = 0; u < 2; ++u)
#pragma unroll
      for (int t = 0; t < 4; ++t)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[u][t][r] = 0.f;
    for (unsigned i = kt0; i < kt1; ++i, buf ^= 1) {
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
          if (kg == 0) DYHIP_WIDE_AIM(ub + i + 2, ub)
        } else {
          // refill this stage two units ahead and fetch the next unit's first fragments (after the block's last unit
          // both are idle repeats)
          DYHIP_WIDE_FIRE(wave_stage + buf * kStageFloats)
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

    // the thread index as the compiler cannot see through: the addresses below are formed here, after the loop,
    // instead of being computed ahead of it and parked in scratch memory
    unsigned tid_e = threadIdx.x;
    asm volatile("" : "+v"(tid_e));
    // acc[u][t][r] of lane l: m = AK ? 32 t + l%32 : 4 (l%32) + t (+ 128 wm),
    // n = BKM ? 32 u + i : 2 i + u (+ 64 wn) with i = 8 (r/4) + 4 (l/32) + r%4.
    // A partial tile is stored as [u][r][thread][t]: one 128-bit access per thread and (u, r), whoever reads it.
    if (kt0 > 0 || (kt1 < nt && !g.finish_in_kernel)) {
      // Not the whole tile, and not this block's to finish: leave the partial tile in a slot.
      if (g.finish_in_kernel) {
        // past the L2, for a block on another one; the segment's flag goes up once memory has acknowledged every store
        float* slot = g.slots + size_t(seg) * kSlotFloats + 4 * tid_e;
#pragma unroll
        for (int u = 0; u < 2; ++u)
#pragma unroll
          for (int r = 0; r < 16; ++r)
            store_through(slot + size_t(u * 16 + r) * (4 * kWideThreads), acc[u][0][r], acc[u][1][r], acc[u][2][r],
                          acc[u][3][r]);
        __builtin_amdgcn_s_waitcnt(0);
        __syncthreads();
        if (tid_e == 0 && g.raise_flags) __hip_atomic_store(g.flags + seg, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      } else {
        float* slot = g.slots + size_t(2 * seg + (tile == u0 / nt ? 0 : 1)) * kSlotFloats + 4 * tid_e;
#pragma unroll
        for (int u = 0; u < 2; ++u)
#pragma unroll
          for (int r = 0; r < 16; ++r)
            *reinterpret_cast<float4*>(slot + size_t(u * 16 + r) * (4 * kWideThreads)) =
                make_float4(acc[u][0][r], acc[u][1][r], acc[u][2][r], acc[u][3][r]);
      }
      continue;
    }
    // This block holds the tile's first k-tiles (or all of them) and finishes the tile.  The segments that start inside
    // the tile computed their partial tiles first thing, long ago by now; the wait is bounded all the same, and a wait
    // that gives up is counted for the host to report.  Partial tiles are added in segment order.
    unsigned s_end = seg + 1;
    if (kt1 < nt) {
      while (s_end < segments && segment_start(s_end, g.units, segments) < ub + nt) ++s_end;
      if (tid_e == 0) {
        for (unsigned s2 = seg + 1; s2 < s_end; ++s2) {
          unsigned spins = 0;
          while (__hip_atomic_load(g.flags + s2, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) == 0u) {
            if (spins++ >= g.spin_limit) {
              atomicAdd(g.flags + kGemmFlagWords - 1, 1u);
              break;
            }
            __builtin_amdgcn_s_sleep(32);
          }
          __hip_atomic_store(g.flags + s2, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);  // for the next launch
        }
      }
      __syncthreads();
    }
    const unsigned lane_e = tid_e & 63, wm_e = (tid_e >> 6) & 1, wn_e = tid_e >> 7, l32_e = lane_e & 31, lhi_e = lane_e >> 5;
    const unsigned m0 = (tile % g.tiles_m) * kWT, n0 = (tile / g.tiles_m) * kWT;
    float* out = g.C + m0 + size_t(n0) * g.M;
    const unsigned mlim = g.M - m0, nlim = g.N - n0;
    const float beta = g.bias == nullptr ? g.beta : 0.f;
    const bool add_bias = g.bias != nullptr;
#pragma unroll
    for (int u = 0; u < 2; ++u)
#pragma unroll
      for (int r0 = 0; r0 < 16; r0 += 8) {
        float4 v[8];
#pragma unroll
        for (int q = 0; q < 8; ++q) v[q] = make_float4(acc[u][0][r0 + q], acc[u][1][r0 + q], acc[u][2][r0 + q], acc[u][3][r0 + q]);
        for (unsigned s2 = seg + 1; s2 < s_end; ++s2) {  // eight loads in flight
          const float* slot = g.slots + size_t(s2) * kSlotFloats + 4 * tid_e + size_t(u * 16 + r0) * (4 * kWideThreads);
          wide_v4 o[8];
#pragma unroll
          for (int q = 0; q < 8; ++q) o[q] = load_through(slot + size_t(q) * (4 * kWideThreads));
#pragma unroll
          for (int q = 0; q < 8; ++q) {
            v[q].x += o[q][0]; v[q].y += o[q][1]; v[q].z += o[q][2]; v[q].w += o[q][3];
          }
        }
#pragma unroll
        for (int q = 0; q < 8; ++q) {
          const int r = r0 + q;
          const int i = 8 * (r / 4) + 4 * lhi_e + (r % 4);
          const unsigned n = wn_e * 64 + (BKM ? 32 * u + i : 2 * i + u);
          if (n >= nlim) continue;
          if (!AK) {
            const unsigned m = wm_e * 128 + 4 * l32_e;
            if (m >= mlim) continue;
            float* p = out + m + size_t(n) * g.M;
            float4 x = v[q];
            if (add_bias) {
              const float4 o = *reinterpret_cast<const float4*>(g.bias + m0 + m);
              x.x += o.x; x.y += o.y; x.z += o.z; x.w += o.w;
            } else if (beta != 0.f) {
              const float4 o = *reinterpret_cast<const float4*>(p);
              x.x += beta * o.x; x.y += beta * o.y; x.z += beta * o.z; x.w += beta * o.w;
            }
            *reinterpret_cast<float4*>(p) = x;
          } else {
            const float xs[4] = {v[q].x, v[q].y, v[q].z, v[q].w};
#pragma unroll
            for (int t = 0; t < 4; ++t) {
              const unsigned m = wm_e * 128 + 32 * t + l32_e;
              if (m >= mlim) continue;
              float* p = out + m + size_t(n) * g.M;
              float x = xs[t];
              if (add_bias) x += g.bias[m0 + m];
              else if (beta != 0.f) x += beta * *p;
              *p = x;
            }
          }
        }
      }
  }
#undef DYHIP_WIDE_AIM
#undef DYHIP_WIDE_FIRE
}

// Second kernel for products whose tiles span several segments each (fewer tiles than CUs, or little more): C tile =
// epilogue(sum of the tile's partial tiles in segment order).  Block (x, y) takes tile x and two of its 32 (u, r)
// groups, its threads standing for the threads of the main kernel (a partial tile is stored in their order).
template <bool AK, bool BKM>
__global__ __launch_bounds__(kWideThreads) void gemm_wide_fixup_kernel(WideArgs g, unsigned segments) {
  const unsigned nt = g.nt, tile = blockIdx.x, ub = tile * nt;
  // segments that hold k-tiles of this tile: s_lo holds its first, s_hi its last
  unsigned s_lo = min(ub / (g.units / segments), segments - 1);
  while (s_lo + 1 < segments && segment_start(s_lo + 1, g.units, segments) <= ub) ++s_lo;
  while (segment_start(s_lo, g.units, segments) > ub) --s_lo;
  unsigned s_hi = s_lo;
  while (s_hi + 1 < segments && segment_start(s_hi + 1, g.units, segments) < ub + nt) ++s_hi;
  if (s_lo == s_hi) return;  // one block had the whole tile and wrote it itself
  const unsigned tid = threadIdx.x, lane = tid & 63, wm = (tid >> 6) & 1, wn = tid >> 7, l32 = lane & 31, lhi = lane >> 5;
  const unsigned m0 = (tile % g.tiles_m) * kWT, n0 = (tile / g.tiles_m) * kWT;
  float* out = g.C + m0 + size_t(n0) * g.M;
  const unsigned mlim = g.M - m0, nlim = g.N - n0;
#pragma unroll
  for (int j = 0; j < 2; ++j) {
    const unsigned ur = blockIdx.y * 2 + j, u = ur / 16, r = ur % 16;
    float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
    for (unsigned s2 = s_lo; s2 <= s_hi; ++s2) {
      // the tile is the first item of every segment but the one that holds its first k-tiles (unless that segment
      // starts with it)
      const unsigned first_tile = segment_start(s2, g.units, segments) / nt;
      const float4 o = *reinterpret_cast<const float4*>(g.slots + size_t(2 * s2 + (first_tile == tile ? 0 : 1)) * kSlotFloats +
                                                        size_t(ur) * (4 * kWideThreads) + 4 * tid);
      v.x += o.x; v.y += o.y; v.z += o.z; v.w += o.w;
    }
    const unsigned i = 8 * (r / 4) + 4 * lhi + (r % 4);
    const unsigned n = wn * 64 + (BKM ? 32 * u + i : 2 * i + u);
    if (n >= nlim) continue;
    if (!AK) {
      const unsigned m = wm * 128 + 4 * l32;
      if (m >= mlim) continue;
      float* p = out + m + size_t(n) * g.M;
      if (g.bias != nullptr) {
        const float4 o = *reinterpret_cast<const float4*>(g.bias + m0 + m);
        v.x += o.x; v.y += o.y; v.z += o.z; v.w += o.w;
      } else if (g.beta != 0.f) {
        const float4 o = *reinterpret_cast<const float4*>(p);
        v.x += g.beta * o.x; v.y += g.beta * o.y; v.z += g.beta * o.z; v.w += g.beta * o.w;
      }
      *reinterpret_cast<float4*>(p) = v;
    } else {
      const float xs[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
      for (int t = 0; t < 4; ++t) {
        const unsigned m = wm * 128 + 32 * t + l32;
        if (m >= mlim) continue;
        float* p = out + m + size_t(n) * g.M;
        float x = xs[t];
        if (g.bias != nullptr) x += g.bias[m0 + m];
        else if (g.beta != 0.f) x += g.beta * *p;
        *p = x;
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

// How the k-tiles are dealt to the blocks.  ok = false: leave the problem to the 128-wide kernel.
struct WidePlan {
  bool ok;
  bool finish_in_kernel;  // segments at least a tile long: a tile is cut at most once, and finished inside the kernel
  unsigned tiles_m, tiles, nt, units, segments;
};

static WidePlan plan_wide(const dyhip_device* dev, size_t M, size_t N, size_t K32) {
  const unsigned cus = dev->num_cus > 0 ? unsigned(dev->num_cus) : 256;
  WidePlan p{};
  p.tiles_m = unsigned(cdiv<size_t>(M, kWT));
  p.nt = unsigned(K32 / kWK);
  const size_t tiles = size_t(p.tiles_m) * cdiv<size_t>(N, kWT), units = tiles * p.nt;
  p.tiles = unsigned(tiles);
  p.units = unsigned(units);
  p.segments = cus;
  const size_t per = units / cus;
  p.finish_in_kernel = per >= p.nt;
  // Measured against the 128-wide kernel: a block's set-up, its share of partial tiles and of the second kernel cost
  // about three k-tiles, so a problem of fewer tiles than CUs (nothing but cut tiles) needs long segments.
  p.ok = units < (size_t(1) << 31) && (p.finish_in_kernel ? p.nt >= 8 : per >= 16);
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
  if (dev->gemm_ws == nullptr || dev->gemm_flags == nullptr || dev->gemm_ws_bytes < (2 * cus) * kSlotFloats * sizeof(float) ||
      cus + 1 > size_t(kGemmFlagWords))
    return false;
  return plan_wide(dev, M, N, K32).ok;
}

size_t gemm_wide_whole_rounds_columns(const dyhip_device* dev, bool a_kmajor, bool b_kmajor, size_t M, size_t N, size_t K,
                                      const float* A, size_t lda, const float* B, size_t ldb, const float* C) {
  const size_t cus = dev->num_cus > 0 ? size_t(dev->num_cus) : 256;
  const size_t tiles_m = cdiv<size_t>(M, kWT), tiles = tiles_m * cdiv<size_t>(N, kWT);
  const size_t direct = tiles / cus * cus;
  if (direct == 0 || direct == tiles || direct % tiles_m != 0 || tiles - direct > cus / 4) return 0;
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
  g.flags = dev->gemm_flags;
  g.lda = unsigned(lda);
  g.ldb = unsigned(ldb);
  g.M = unsigned(M);
  g.N = unsigned(N);
  g.nt = p.nt;
  g.tiles_m = p.tiles_m;
  g.units = p.units;
  g.finish_in_kernel = p.finish_in_kernel ? 1 : 0;
  g.spin_limit = dev->gemm_spin_limit;  // seconds by default; a partial tile is normally there hundreds of microseconds before it is asked for
  g.raise_flags = dev->gemm_raise_flags;
  g.beta = beta;
  int st;
  if (a_kmajor && b_kmajor) st = launch_wide<true, true>(dev, g, p.segments, 0);
  else if (a_kmajor) st = launch_wide<true, false>(dev, g, p.segments, 1);
  else if (b_kmajor) st = launch_wide<false, true>(dev, g, p.segments, 2);
  else st = launch_wide<false, false>(dev, g, p.segments, 3);
  DYHIP_CHECK_STATUS(st);
  DYHIP_CHECK_LAUNCH();
  if (p.finish_in_kernel) {
    dev->gemm_flags_used = true;
  } else {
    const dim3 grid(p.tiles, 16);
    if (a_kmajor && b_kmajor) hipLaunchKernelGGL((gemm_wide_fixup_kernel<true, true>), grid, dim3(kWideThreads), 0, dev->stream, g, p.segments);
    else if (a_kmajor) hipLaunchKernelGGL((gemm_wide_fixup_kernel<true, false>), grid, dim3(kWideThreads), 0, dev->stream, g, p.segments);
    else if (b_kmajor) hipLaunchKernelGGL((gemm_wide_fixup_kernel<false, true>), grid, dim3(kWideThreads), 0, dev->stream, g, p.segments);
    else hipLaunchKernelGGL((gemm_wide_fixup_kernel<false, false>), grid, dim3(kWideThreads), 0, dev->stream, g, p.segments);
    DYHIP_CHECK_LAUNCH();
  }
  return DYHIP_OK;
}

bool gemm_shallow_nt_eligible(const dyhip_device* dev, size_t M, size_t N, size_t K, const float* A, size_t lda,
                              const float* B, size_t ldb, const float* C) {
  if (K < 24 || K > 128 || K % 8 != 0 || M % 4 != 0 || N % 4 != 0 || M < 128 || N < 128) return false;
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

// For tests of the hand-off between blocks without a GPU: the first unit of every segment (segments + 1 values, the
// last one = units) when the k-tiles of an M x N x K product are dealt to `segments` blocks, and how cut tiles are
// finished.  The same function as the kernels use.
void gemm_wide_describe(size_t M, size_t N, size_t K, unsigned segments, unsigned* starts, unsigned* k_tiles_per_tile,
                        int* finish_in_kernel) {
  const unsigned nt = unsigned(K / kWK);
  const size_t units = cdiv<size_t>(M, kWT) * cdiv<size_t>(N, kWT) * nt;
  for (unsigned s2 = 0; s2 <= segments; ++s2) starts[s2] = segment_start(s2, unsigned(units), segments);
  *k_tiles_per_tile = nt;
  *finish_in_kernel = units / segments >= nt ? 1 : 0;
}

}  // namespace dyhip
