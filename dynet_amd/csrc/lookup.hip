// LookupNode: embedding gather and sorted-index segmented scatter-add.
//
// Replaces LookupNode::forward_dev_impl (dynet/param-nodes.cc:304-329) with its
// one-thread-per-float gather (dynet/gpu-ops.cu:72-90, a division and a modulo
// per element) and LookupParameterStorage::accumulate_grads_dev
// (dynet/model.cc:728-743) with its float atomicAdd scatter
// (dynet/gpu-ops.cu:148-166, order-dependent and serialising on hot rows).
//
// Layout: the table is dim x vocab column-major, i.e. row r of the embedding is
// the contiguous run table[r*dim, (r+1)*dim); fx and g are dim x n_ids.
//
// Scatter-add: the ids are grouped by value (a "plan": equal ids consecutive, ascending
// position inside each run, see below) and one kernel sums each run: short runs by one
// thread group in the CPU path's order, long runs split by columns over several thread
// groups.  No atomics on floats and no partial rows: the result is deterministic, each
// gradient row is read and written exactly once, and rows with short runs are bit-identical
// to the sequential CPU sum.
#include <algorithm>
#include <cstring>

#include "common.h"

namespace dyhip {

constexpr unsigned kNone = 0xFFFFFFFFu;
constexpr int kLkThreads = 256;
constexpr int kGatherRowsUnroll = 4;

template <class V>
__device__ __forceinline__ V vzero();
template <>
__device__ __forceinline__ float4 vzero<float4>() { return make_float4(0.f, 0.f, 0.f, 0.f); }
template <>
__device__ __forceinline__ float vzero<float>() { return 0.f; }
__device__ __forceinline__ float4 vadd(const float4 a, const float4 b) {
  return make_float4(a.x + b.x, a.y + b.y, a.z + b.z, a.w + b.w);
}
__device__ __forceinline__ float vadd(const float a, const float b) { return a + b; }
__device__ __forceinline__ float4 vscale(const float4 a, const float m) {
  return make_float4(a.x * m, a.y * m, a.z * m, a.w * m);
}
__device__ __forceinline__ float vscale(const float a, const float m) { return a * m; }
template <bool NT>
__device__ __forceinline__ float4 vload(const float4* p) { return ldg4<NT>(p); }
template <bool NT>
__device__ __forceinline__ float vload(const float* p) { return ldg1<NT>(p); }
template <bool NT>
__device__ __forceinline__ void vstore(float4* p, const float4 v) { stg4<NT>(p, v); }
template <bool NT>
__device__ __forceinline__ void vstore(float* p, const float v) { stg1<NT>(p, v); }
// Stores and loads that bypass the caches that are private to a part of the chip (used for the few values that
// thread groups on different L2s hand to each other inside one kernel).
__device__ __forceinline__ void vstore_through(float* p, const float v) {
  __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
}
__device__ __forceinline__ void vstore_through(float4* p, const float4 v) {
  unsigned long long* q = reinterpret_cast<unsigned long long*>(p);
  const unsigned long long lo = (unsigned long long)__float_as_uint(v.x) | ((unsigned long long)__float_as_uint(v.y) << 32);
  const unsigned long long hi = (unsigned long long)__float_as_uint(v.z) | ((unsigned long long)__float_as_uint(v.w) << 32);
  __hip_atomic_store(q, lo, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
  __hip_atomic_store(q + 1, hi, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
}
__device__ __forceinline__ float vload_through(const float* p) {
  return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
}
__device__ __forceinline__ float4 vload_through(const float4* p) {
  const unsigned long long* q = reinterpret_cast<const unsigned long long*>(p);
  const unsigned long long lo = __hip_atomic_load(q, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
  const unsigned long long hi = __hip_atomic_load(q + 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
  return make_float4(__uint_as_float(unsigned(lo)), __uint_as_float(unsigned(lo >> 32)), __uint_as_float(unsigned(hi)),
                     __uint_as_float(unsigned(hi >> 32)));
}
__device__ __forceinline__ float vshfl(const float v, int src) { return __shfl(v, src, kWave); }
__device__ __forceinline__ float4 vshfl(const float4 v, int src) {
  return make_float4(__shfl(v.x, src, kWave), __shfl(v.y, src, kWave), __shfl(v.z, src, kWave), __shfl(v.w, src, kWave));
}

// ---- gather ---------------------------------------------------------------------
// A group of `tpr` threads owns one id at a time; a block holds 256/tpr groups and
// each group processes kGatherRowsUnroll ids with all loads issued first.
template <class V, bool SCALE, bool NT>
__global__ __launch_bounds__(kLkThreads) void lookup_gather_kernel(unsigned n_ids, unsigned dimv, unsigned tpr,
                                                                   unsigned vocab, const unsigned* __restrict__ ids,
                                                                   const V* __restrict__ table, float mult,
                                                                   V* __restrict__ fx) {
  const unsigned groups = kLkThreads / tpr;
  const unsigned grp = threadIdx.x / tpr, t = threadIdx.x - grp * tpr;
  const unsigned row0 = (blockIdx.x * groups + grp) * kGatherRowsUnroll;
  unsigned id[kGatherRowsUnroll];
#pragma unroll
  for (int u = 0; u < kGatherRowsUnroll; ++u) id[u] = row0 + u < n_ids ? ids[row0 + u] : kNone;
  for (unsigned c = t; c < dimv; c += tpr) {
    V v[kGatherRowsUnroll];
#pragma unroll
    for (int u = 0; u < kGatherRowsUnroll; ++u)
      v[u] = (row0 + u < n_ids && id[u] < vocab) ? table[size_t(id[u]) * dimv + c] : vzero<V>();
#pragma unroll
    for (int u = 0; u < kGatherRowsUnroll; ++u)
      if (row0 + u < n_ids) vstore<NT>(fx + size_t(row0 + u) * dimv + c, SCALE ? vscale(v[u], mult) : v[u]);
  }
}

// ---- the plan: ids grouped by value ------------------------------------------------
// plan = [entries | arrivals | status], each part padded to 256 bytes.  Entry k of the grouped order is one
// 16-byte record, so that a consumer's first (and only) dependent load per entry is a single 128-bit access:
//   .x  id of the entry: entries of one id are consecutive (a "run"); ids >= vocab are replaced by vocab
//       (one run that the reduction skips)
//   .y  position of that entry in the caller's id vector; ascending inside a run
//   .z  entries of the run before k        (0 at the head of a run)
//   .w  entries of the run from k onwards  (1 at its last entry)
//   arrivals one counter per 8 entries, zero whenever no reduction is running: the groups that share one
//            slice of a very long run count themselves here so that the last one adds their partial sums up
//   status   [0] = number of ids >= vocab
// The order of the runs does not matter to anything that consumes a plan (the segmented sum below and
// the trainer's row kernels), so the ids are grouped, not fully sorted:
// bucket = id mod 256, inside a bucket ascending id / 256, inside a run ascending position.
struct Plan {
  uint4* ent;
  unsigned* arrivals;
  unsigned* status;
};

constexpr int kChunk = 8;  // entries per thread group of the segmented sum (see there)

static size_t align256(size_t n) { return (n + 255) / 256 * 256; }

static size_t plan_bytes(unsigned n) {
  return align256(sizeof(uint4) * size_t(n)) + align256(sizeof(unsigned) * cdiv<unsigned>(n, kChunk)) + 256;
}

static void plan_parts(const void* plan, unsigned n, Plan* w) {
  char* p = const_cast<char*>(static_cast<const char*>(plan));
  const size_t b = align256(sizeof(uint4) * size_t(n));
  w->ent = reinterpret_cast<uint4*>(p);
  w->arrivals = reinterpret_cast<unsigned*>(p + b);
  w->status = reinterpret_cast<unsigned*>(p + b + align256(sizeof(unsigned) * cdiv<unsigned>(n, kChunk)));
}

static unsigned key_bits(unsigned max_key) {
  unsigned bits = 1;
  while (bits < 32 && (1ull << bits) <= (unsigned long long)max_key) ++bits;
  return bits;
}

// ---- one-launch plan for up to 65535 ids -----------------------------------------------
// 256 blocks, one per bucket (id mod 256).  Every block reads the whole id vector (64 KB at
// 16384 ids, from L2 after the first block of an XCD), so no block waits for another.
// Two kernels: plan_direct_kernel (further down) when the keys fit 16 bits, which needs neither a
// compaction nor sort passes, and this general one for wider keys:
//   1. thread t owns a contiguous piece of the positions and counts, in registers, the ids of smaller
//      buckets (their sum is where this bucket starts in the output) and of this bucket (their prefix
//      over the threads is where the thread's matches go: the bucket is compacted in ascending position);
//   2. stable counting sort of the bucket by the higher id bits, 8 bits per pass, in LDS: wave-private
//      digit counters, ranks inside a 64-entry step from ballots, so no atomic decides an order;
//   3. run offsets: head flags per 64-entry step, the last head before / first head after each step from
//      a scan over the steps, written out together with ids and positions in coalesced order.
// A bucket of more than kPlanCap entries (a heavily skewed id vector) takes the same steps in a
// global-memory buffer instead of LDS.
constexpr int kPlanThreads = 1024;
constexpr int kPlanWaves = kPlanThreads / 64;
constexpr unsigned kPlanSmallMax = 65535;
constexpr int kPlanMaxQuads = (kPlanSmallMax + 4 * kPlanThreads - 1) / (4 * kPlanThreads);  // 128-bit loads per thread: 16
constexpr unsigned kPlanCap = 8192;
constexpr unsigned kPlanBuckets = 256;
constexpr unsigned kPlanMaxSteps = (kPlanSmallMax + 63) / 64;  // 64-entry steps of the largest bucket: 1024
// LDS words: digit counters [256][16] | scratch [128] | per-step last / first head [2][1024] | four buffers of kPlanCap
constexpr unsigned kPlanLdsCnt = 0;
constexpr unsigned kPlanLdsTmp = kPlanLdsCnt + 256 * kPlanWaves;
constexpr unsigned kPlanLdsStep = kPlanLdsTmp + 128;
constexpr unsigned kPlanLdsBuf = kPlanLdsStep + 2 * kPlanMaxSteps;
constexpr unsigned kPlanLdsWords = kPlanLdsBuf + 4 * kPlanCap;

__device__ __forceinline__ unsigned long long lanes_below(int lane) { return (1ull << lane) - 1ull; }

// Inclusive prefix sum over the lanes of a wavefront.  The cross-lane steps are DPP modifiers (shifts inside a row of
// 16 lanes, then lane 15 of a row into the next row and lane 31 into the upper half), not trips through the LDS
// crossbar: six dependent adds of a few cycles each instead of six round trips.
template <int CTRL, int ROW_MASK>
__device__ __forceinline__ unsigned dpp_from(unsigned v) {  // 0 where the source lane does not exist or the row is masked
  return unsigned(__builtin_amdgcn_update_dpp(0, int(v), CTRL, ROW_MASK, 0xF, false));
}
__device__ __forceinline__ unsigned wave_scan_add(unsigned v, int lane) {
  (void)lane;
  v += dpp_from<0x111, 0xF>(v);  // row_shr:1
  v += dpp_from<0x112, 0xF>(v);  // row_shr:2
  v += dpp_from<0x114, 0xF>(v);  // row_shr:4
  v += dpp_from<0x118, 0xF>(v);  // row_shr:8: every row holds its own inclusive prefix
  v += dpp_from<0x142, 0xA>(v);  // row_bcast:15 into rows 1 and 3
  v += dpp_from<0x143, 0xC>(v);  // row_bcast:31 into rows 2 and 3
  return v;
}

// Exclusive prefix sum of one value per thread over the whole block (1024 threads), and the total.
// tmp = kPlanWaves LDS words; a barrier separates the call from earlier uses of tmp.
__device__ __forceinline__ unsigned block_scan_excl(unsigned v, unsigned* tmp, unsigned* total) {
  const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
  const unsigned inc = wave_scan_add(v, lane);
  if (lane == 63) tmp[w] = inc;
  __syncthreads();
  unsigned before = 0, all = 0;
#pragma unroll
  for (int k = 0; k < kPlanWaves; ++k) {
    const unsigned x = tmp[k];
    all += x;
    if (k < w) before += x;
  }
  *total = all;
  return before + inc - v;
}

// lanes of the wavefront (among `valid` ones) that hold the same 8-bit digit as this lane
__device__ __forceinline__ unsigned long long same_digit_lanes(unsigned dig, bool valid) {
  // One ballot per distinct digit for the first few digits: a step mostly holds the odd id of a bucket, or many
  // copies of one hot id and little else.  Lanes left after that (many distinct digits in one step) are matched bit
  // by bit, eight ballots whatever their number.
  unsigned long long todo = __ballot(valid), mine = 0ull;
#pragma unroll 1
  for (int it = 0; it < 4 && todo != 0ull; ++it) {  // uniform
    const unsigned d0 = unsigned(__builtin_amdgcn_readlane(int(dig), __ffsll((long long)todo) - 1));
    const unsigned long long eq = __ballot(valid && dig == d0);
    if (valid && dig == d0) mine = eq;
    todo &= ~eq;
  }
  if (todo != 0ull) {
    const bool rest = valid && ((todo >> (threadIdx.x & 63)) & 1ull) != 0ull;
    unsigned long long same = todo;
#pragma unroll
    for (int b = 0; b < 8; ++b) {
      const bool bit = (dig >> b) & 1u;
      const unsigned long long bal = __ballot(rest && bit);
      same &= bit ? bal : ~bal;
    }
    if (rest) mine = same;
  }
  return mine;
}

// One stable counting-sort pass over the m entries (key, pos) of a bucket on digit (key >> shift) & 255.
// cnt[digit * 16 + wave] must be zero on entry and is zero again on return.  Wavefront w owns a contiguous
// piece of the input.  A: it counts its digits; B: exclusive prefix over (digit, wavefront) in that
// order; C: it walks its piece 64 entries at a time, ranks equal digits inside the step with ballots and
// advances its own counters, so entries with equal digits keep their input order.
__device__ __forceinline__ void plan_sort_pass(unsigned m, unsigned shift, const unsigned* kin, const unsigned* pin,
                                               unsigned* kout, unsigned* pout, unsigned* cnt, unsigned* tmp) {
  const int t = threadIdx.x, lane = t & 63, w = t >> 6;
  const unsigned per_wave = cdiv<unsigned>(cdiv<unsigned>(m, kPlanWaves), 64u) * 64u;
  const unsigned wb = min(m, w * per_wave), we = min(m, wb + per_wave);
  for (unsigned j0 = wb; j0 < we; j0 += 64) {  // uniform over the wavefront
    const unsigned j = j0 + lane;
    const bool valid = j < we;
    const unsigned dig = valid ? (kin[j] >> shift) & 255u : 0u;
    const unsigned long long same = same_digit_lanes(dig, valid);
    if (valid && (same & lanes_below(lane)) == 0) cnt[dig * kPlanWaves + w] += __popcll(same);
  }
  __syncthreads();
  // B: thread t scans counters [4t, 4t + 4)
  uint4 c4 = reinterpret_cast<uint4*>(cnt)[t];
  unsigned tot_unused;
  const unsigned sum4 = c4.x + c4.y + c4.z + c4.w;
  const unsigned base = block_scan_excl(sum4, tmp, &tot_unused);
  uint4 e4;
  e4.x = base;
  e4.y = e4.x + c4.x;
  e4.z = e4.y + c4.y;
  e4.w = e4.z + c4.z;
  reinterpret_cast<uint4*>(cnt)[t] = e4;
  __syncthreads();
  for (unsigned j0 = wb; j0 < we; j0 += 64) {
    const unsigned j = j0 + lane;
    const bool valid = j < we;
    const unsigned key = valid ? kin[j] : 0u;
    const unsigned pos = valid ? pin[j] : 0u;
    const unsigned dig = (key >> shift) & 255u;
    const unsigned long long same = same_digit_lanes(dig, valid);
    const unsigned rank = __popcll(same & lanes_below(lane));
    // every lane reads its digit's counter before the first lane of each digit advances it: the
    // wavefront issues the load for all its lanes, then the store, and LDS keeps that order
    unsigned at = 0;
    if (valid) at = cnt[dig * kPlanWaves + w];
    __builtin_amdgcn_wave_barrier();
    if (valid && rank == 0) cnt[dig * kPlanWaves + w] = at + __popcll(same);
    __builtin_amdgcn_wave_barrier();
    if (valid) {
      kout[at + rank] = key;
      pout[at + rank] = pos;
    }
  }
  __syncthreads();
  reinterpret_cast<uint4*>(cnt)[t] = make_uint4(0u, 0u, 0u, 0u);
  __syncthreads();
}

// Steps 2 and 3 on buffers in LDS or in global memory (same code, two address spaces).
__device__ __forceinline__ void plan_finish_bucket(unsigned m, unsigned passes, unsigned bstart, unsigned* kA,
                                                   unsigned* pA, unsigned* kB, unsigned* pB, unsigned* cnt,
                                                   unsigned* tmp, int* step_last, int* step_first, const Plan out) {
  const int t = threadIdx.x, lane = t & 63, w = t >> 6;
  for (unsigned p = 0; p < passes; ++p) {
    plan_sort_pass(m, 8u + 8u * p, kA, pA, kB, pB, cnt, tmp);
    unsigned* s;
    s = kA; kA = kB; kB = s;
    s = pA; pA = pB; pB = s;
  }
  // grouped entries are in (kA, pA).  Step q = entries [64q, 64q + 64), taken by wavefront q mod 16.
  const unsigned steps = cdiv<unsigned>(m, 64u);
  for (unsigned q = w; q < steps; q += kPlanWaves) {
    const unsigned j = q * 64 + lane;
    const bool head = j < m && (j == 0 || kA[j - 1] != kA[j]);
    const unsigned long long hm = __ballot(head);
    if (lane == 0) {
      step_last[q] = hm ? int(q * 64) + 63 - __clzll(hm) : -1;
      step_first[q] = hm ? int(q * 64) + __ffsll((long long)hm) - 1 : int(m);
    }
  }
  __syncthreads();
  // running maximum of step_last (ascending) and running minimum of step_first (descending), by wavefront 0:
  // afterwards step_last[q] = last head in steps <= q, step_first[q] = first head in steps >= q (m if none)
  if (w == 0) {
    int carry_l = -1, carry_f = int(m);
    for (unsigned q0 = 0; q0 < steps; q0 += 64) {
      const unsigned q = q0 + lane;
      int l = q < steps ? step_last[q] : -1;
#pragma unroll
      for (int off = 1; off < 64; off <<= 1) {
        const int u = __shfl_up(l, off, kWave);
        if (lane >= off) l = max(l, u);
      }
      l = max(l, carry_l);
      if (q < steps) step_last[q] = l;
      carry_l = __shfl(l, 63, kWave);
    }
    for (unsigned r0 = 0; r0 < steps; r0 += 64) {  // from the top step down
      const unsigned r = r0 + lane;                // reversed index
      const bool in = r < steps;
      const unsigned q = in ? steps - 1 - r : 0;
      int f = in ? step_first[q] : int(m);
#pragma unroll
      for (int off = 1; off < 64; off <<= 1) {
        const int u = __shfl_up(f, off, kWave);
        if (lane >= off) f = min(f, u);
      }
      f = min(f, carry_f);
      if (in) step_first[q] = f;
      carry_f = __shfl(f, 63, kWave);
    }
  }
  __syncthreads();
  for (unsigned q = w; q < steps; q += kPlanWaves) {
    const unsigned j = q * 64 + lane;
    const bool in = j < m;
    const unsigned key = in ? kA[j] : 0u;
    const bool head = in && (j == 0 || kA[j - 1] != key);
    const unsigned long long hm = __ballot(head);
    // last head at or before j: inside this step, else carried from the steps before
    const unsigned long long le = hm & (lanes_below(lane) | (1ull << lane));
    const int lh = le ? int(q * 64) + 63 - __clzll(le) : (q > 0 ? step_last[q - 1] : 0);
    // first head after j: inside this step, else carried from the steps after
    const unsigned long long gt = lane == 63 ? 0ull : hm & ~(lanes_below(lane + 1));
    const int nh = gt ? int(q * 64) + __ffsll((long long)gt) - 1 : (q + 1 < steps ? step_first[q + 1] : int(m));
    if (in) {
      out.ent[bstart + j] = make_uint4(key, pA[j], j - unsigned(lh), unsigned(nh) - j);
      if ((bstart + j) % kChunk == 0) out.arrivals[(bstart + j) / kChunk] = 0;
    }
  }
}

template <bool VEC>
__global__ __launch_bounds__(kPlanThreads) void plan_group_kernel(unsigned n, unsigned vocab, unsigned passes,
                                                                  const unsigned* __restrict__ ids, const Plan out,
                                                                  unsigned* __restrict__ gbuf) {
  extern __shared__ __attribute__((aligned(16))) unsigned plan_lds[];
  unsigned* cnt = plan_lds + kPlanLdsCnt;
  unsigned* tmp = plan_lds + kPlanLdsTmp;
  int* step_last = reinterpret_cast<int*>(plan_lds + kPlanLdsStep);
  int* step_first = step_last + kPlanMaxSteps;
  const unsigned d = blockIdx.x;
  const int t = threadIdx.x;
  reinterpret_cast<uint4*>(cnt)[t] = make_uint4(0u, 0u, 0u, 0u);  // 4096 counters, 4 per thread
  // ---- 1. thread t reads positions [t * 4 * quads, (t + 1) * 4 * quads); keys stay in registers ------
  const unsigned quads = cdiv<unsigned>(n, 4u * kPlanThreads);  // 128-bit loads per thread (uniform)
  const unsigned p_first = unsigned(t) * 4u * quads;
  unsigned key[kPlanMaxQuads][4];
  unsigned lt = 0, eq = 0, bad = 0;
#pragma unroll
  for (int i = 0; i < kPlanMaxQuads; ++i) {
    if (unsigned(i) < quads) {  // uniform
      const unsigned p0 = p_first + 4u * i;
      unsigned raw[4] = {kNone, kNone, kNone, kNone};
      if (VEC && p0 + 3 < n) {
        const uint4 v = *reinterpret_cast<const uint4*>(ids + p0);
        raw[0] = v.x; raw[1] = v.y; raw[2] = v.z; raw[3] = v.w;
      } else {
#pragma unroll
        for (int c = 0; c < 4; ++c)
          if (p0 + c < n) raw[c] = ids[p0 + c];
      }
#pragma unroll
      for (int c = 0; c < 4; ++c) {
        const bool in = p0 + c < n;
        const unsigned k = in ? min(raw[c], vocab) : kNone;
        key[i][c] = k;
        const unsigned dg = k & 255u;
        lt += in && dg < d ? 1u : 0u;
        eq += in && dg == d ? 1u : 0u;
        bad += in && raw[c] >= vocab ? 1u : 0u;
      }
    } else {
#pragma unroll
      for (int c = 0; c < 4; ++c) key[i][c] = kNone;
    }
  }
  // one scan for both counts: eq in the low half (its total is at most 65535), lt in the high half
  unsigned both = 0, nbad = 0;
  const unsigned my_at = block_scan_excl(eq | (lt << 16), tmp, &both) & 0xFFFFu;
  const unsigned m = both & 0xFFFFu, bstart = both >> 16;
  if (d == kPlanBuckets - 1) {  // the ids >= vocab are counted by one block, not the one of the (often hottest) bucket 0
    (void)block_scan_excl(bad, tmp + 32, &nbad);
    if (t == 0) out.status[0] = nbad;
  }
  if (m == 0) return;  // uniform over the block
  const bool in_lds = m <= kPlanCap;
  unsigned* kA = in_lds ? plan_lds + kPlanLdsBuf : gbuf + bstart;
  unsigned* pA = in_lds ? plan_lds + kPlanLdsBuf + kPlanCap : gbuf + size_t(n) + bstart;
  // ---- compaction of this bucket's entries, ascending position ------------------------------
  if (eq) {
    unsigned at = my_at;
#pragma unroll
    for (int i = 0; i < kPlanMaxQuads; ++i) {
#pragma unroll
      for (int c = 0; c < 4; ++c) {
        if (unsigned(i) < quads && key[i][c] != kNone && (key[i][c] & 255u) == d) {
          if (in_lds) {
            plan_lds[kPlanLdsBuf + at] = key[i][c];
            plan_lds[kPlanLdsBuf + kPlanCap + at] = p_first + 4u * i + c;
          } else {
            kA[at] = key[i][c];
            pA[at] = p_first + 4u * i + c;
          }
          ++at;
        }
      }
    }
  }
  __syncthreads();
  if (in_lds)
    plan_finish_bucket(m, passes, bstart, plan_lds + kPlanLdsBuf, plan_lds + kPlanLdsBuf + kPlanCap,
                       plan_lds + kPlanLdsBuf + 2 * kPlanCap, plan_lds + kPlanLdsBuf + 3 * kPlanCap, cnt, tmp,
                       step_last, step_first, out);
  else
    plan_finish_bucket(m, passes, bstart, kA, pA, gbuf + 2 * size_t(n) + bstart, gbuf + 3 * size_t(n) + bstart, cnt,
                       tmp, step_last, step_first, out);
}

// ---- one-launch plan when the keys fit 16 bits (vocab <= 65535): no compaction, no sort passes -------------
// The bucket digit is the low byte, and what is left of a key is one more byte, which names the id inside its
// bucket: a run IS a bin of that byte.  Wavefront w owns the positions [w * per_wave, (w + 1) * per_wave), 64 at a
// step, and keeps their keys in registers.
//   pass 1  counts per (high byte, wavefront) in LDS: the lanes of a step that hold the same byte are found with
//           ballots, the first of them adds their number to the wavefront's own counter (no atomics, nothing
//           depends on timing); also the ids of smaller buckets (where this bucket starts in the output);
//   scan    exclusive prefix over the 4096 counters in (byte, wavefront) order: counter (b, w) becomes the place of
//           the first entry with byte b that wavefront w holds, and (b, 0) the start of the run;
//   pass 2  the same walk again: an entry's place is its wavefront's counter plus its rank among the equal bytes of
//           its step, the counter advances by the step's count; place, run start and run end give the whole record,
//           which goes straight to global memory.
// Entries of a run end up in ascending position because wavefronts own ascending position ranges and walk them in
// ascending order.  A bucket of any size takes the same path (nothing is staged in LDS but the counters).
template <int STEPS>
__global__ __launch_bounds__(kPlanThreads) void plan_direct_kernel(unsigned n, unsigned vocab,
                                                                   const unsigned* __restrict__ ids, const Plan out) {
  __shared__ __attribute__((aligned(16))) unsigned cnt[256 * kPlanWaves];  // [high byte][wavefront]
  __shared__ unsigned run_start[257];
  __shared__ unsigned tmp[kPlanWaves], lt_tot[kPlanWaves], bad_tot[kPlanWaves];
  const unsigned d = blockIdx.x;
  const int t = threadIdx.x, lane = t & 63, w = t >> 6;
  reinterpret_cast<uint4*>(cnt)[t] = make_uint4(0u, 0u, 0u, 0u);
  const unsigned per_wave = cdiv<unsigned>(cdiv<unsigned>(n, kPlanWaves), 64u) * 64u;
  const unsigned base = unsigned(w) * per_wave;
  // A slot (wavefront, step, lane) that stands for no position holds a key that is in no bucket's way: its low byte
  // is not d, so it never counts as this bucket's; it may count as a smaller bucket's, which is taken off again below.
  // What a wavefront-step costs is its vector instructions (16 wavefronts share 4 SIMDs): the first walk is kept to
  // six per step.
  const unsigned none_key = 0x80000000u | ((d + 1u) & 255u);
  const unsigned slots = unsigned(kPlanWaves) * 64u * unsigned(STEPS);
  const unsigned left = n > base + lane ? n - base - lane : 0u;          // positions from this lane's first one on
  const unsigned lim = min(cdiv<unsigned>(left, 64u), per_wave / 64u);   // steps in which this lane holds a position
  unsigned key[STEPS];
#pragma unroll
  for (int i = 0; i < STEPS; ++i) {
    // unconditional loads (a slot past the end reads the last id and is masked): loads inside branches are waited
    // for one by one
    const unsigned p = base + 64u * i + lane;
    key[i] = ids[min(p, n - 1u)];
  }
  __syncthreads();  // the counters are zero
  // Each wavefront "tracks" one high byte, the first of this bucket that it meets: in the bucket of a hot id that is
  // the hot id.  Entries with the tracked byte are counted and ranked in scalar registers (one ballot a step); only
  // the others go through the wavefront's LDS counters, a round trip per step that holds any.
  unsigned lt = 0;
  unsigned tracked = kNone, run = 0;  // uniform over the wavefront
  // which steps hold an id of this bucket at all: both walks skip the other steps (most of them) with a scalar test
  unsigned long long active = 0ull;  // uniform; STEPS <= 64
#pragma unroll
  for (int i = 0; i < STEPS; ++i) {
    const unsigned k = unsigned(i) < lim ? min(key[i], vocab) : none_key;
    key[i] = k;
    lt += (k & 255u) < d ? 1u : 0u;
    active |= __ballot((k & 255u) == d) != 0ull ? 1ull << i : 0ull;
  }
  unsigned bad = 0;
  if (d == kPlanBuckets - 1) {  // one block counts the ids >= vocab (not the one of the often hottest bucket 0)
#pragma unroll
    for (int i = 0; i < STEPS; ++i) bad += key[i] == vocab ? 1u : 0u;
  }
#pragma unroll
  for (int i = 0; i < STEPS; ++i) {
    if (((active >> i) & 1ull) != 0ull) {  // uniform over the wavefront
      unsigned k = key[i];
      asm volatile("" : "+v"(k));  // a value of its own: the lane masks of the loop above are recomputed, not kept
      const bool mine = (k & 255u) == d;
      unsigned long long todo = __ballot(mine);
      const unsigned hi = mine ? k >> 8 : kNone;
      if (tracked == kNone) tracked = unsigned(__builtin_amdgcn_readlane(int(hi), __ffsll((long long)todo) - 1));
      const unsigned long long eq = __ballot(hi == tracked);
      run += unsigned(__popcll(eq));
      todo &= ~eq;
      if (todo != 0ull) {
        // the wavefront's own counters: LDS adds that return nothing, so the walk does not wait for them
        const bool rest = mine && hi != tracked;
        if ((todo & (todo - 1ull)) == 0ull) {  // one more entry, the usual case in a sparse bucket: nothing to match
          if (rest) atomicAdd(&cnt[hi * kPlanWaves + w], 1u);
        } else {
          const unsigned long long same = same_digit_lanes(hi, rest);
          if (rest && (same & lanes_below(lane)) == 0) atomicAdd(&cnt[hi * kPlanWaves + w], unsigned(__popcll(same)));
        }
      }
    }
  }
  if (tracked != kNone && lane == 0) atomicAdd(&cnt[tracked * kPlanWaves + w], run);
  lt = wave_scan_add(lt, lane);
  bad = wave_scan_add(bad, lane);
  if (lane == 63) {
    lt_tot[w] = lt;
    bad_tot[w] = bad;
  }
  __syncthreads();
  // thread t scans counters [4t, 4t + 4): bytes in ascending order, wavefronts in ascending order inside a byte
  uint4 c4 = reinterpret_cast<uint4*>(cnt)[t];
  unsigned m = 0;
  const unsigned e0 = block_scan_excl(c4.x + c4.y + c4.z + c4.w, tmp, &m);
  uint4 e4;
  e4.x = e0;
  e4.y = e4.x + c4.x;
  e4.z = e4.y + c4.y;
  e4.w = e4.z + c4.z;
  reinterpret_cast<uint4*>(cnt)[t] = e4;
  if ((t & 3) == 0) run_start[t >> 2] = e0;  // counter (byte, wavefront 0)
  if (t == 0) run_start[256] = m;
  unsigned bstart = 0, nbad = 0;
#pragma unroll
  for (int k = 0; k < kPlanWaves; ++k) {
    bstart += lt_tot[k];
    nbad += bad_tot[k];
  }
  if ((none_key & 255u) < d) bstart -= slots - n;  // the slots that stand for no position were counted as a smaller bucket's
  if (d == kPlanBuckets - 1 && t == 0) out.status[0] = nbad;
  if (m == 0) return;  // uniform over the block
  __syncthreads();
  unsigned at_tracked = 0, first_tracked = 0, end_tracked = 0;
  if (tracked != kNone) {
    at_tracked = unsigned(__builtin_amdgcn_readfirstlane(int(cnt[tracked * kPlanWaves + w])));
    first_tracked = unsigned(__builtin_amdgcn_readfirstlane(int(run_start[tracked])));
    end_tracked = unsigned(__builtin_amdgcn_readfirstlane(int(run_start[tracked + 1])));
  }
#pragma unroll
  for (int i = 0; i < STEPS; ++i) {
    if (((active >> i) & 1ull) != 0ull) {
      unsigned k = key[i];
      asm volatile("" : "+v"(k));  // a value of its own: the first walk's lane masks are recomputed, not kept in registers
      const bool mine = (k & 255u) == d;
      unsigned long long todo = __ballot(mine);
      const unsigned hi = mine ? k >> 8 : kNone;
      const unsigned pos = base + 64u * i + lane;
      const unsigned long long eq = __ballot(hi == tracked);
      if (hi == tracked) {
        const unsigned j = at_tracked + __builtin_amdgcn_mbcnt_hi(unsigned(eq >> 32), __builtin_amdgcn_mbcnt_lo(unsigned(eq), 0u));
        out.ent[bstart + j] = make_uint4(k, pos, j - first_tracked, end_tracked - j);
      }
      at_tracked += unsigned(__popcll(eq));
      todo &= ~eq;
      if (todo != 0ull && (todo & (todo - 1ull)) == 0ull) {  // one more entry: its counter is its place
        if (mine && hi != tracked) {
          const unsigned j = atomicAdd(&cnt[hi * kPlanWaves + w], 1u);
          out.ent[bstart + j] = make_uint4(k, pos, j - run_start[hi], run_start[hi + 1] - j);
        }
      } else if (todo != 0ull) {
        const bool rest = mine && hi != tracked;
        const unsigned long long same = same_digit_lanes(hi, rest);
        const unsigned rank = __popcll(same & lanes_below(lane));
        // every lane reads its byte's counter before the first lane of each byte advances it: the wavefront issues
        // the load for all its lanes, then the store, and LDS keeps that order
        unsigned at = 0;
        if (rest) at = cnt[hi * kPlanWaves + w];
        __builtin_amdgcn_wave_barrier();
        if (rest && rank == 0) cnt[hi * kPlanWaves + w] = at + __popcll(same);
        __builtin_amdgcn_wave_barrier();
        if (rest) {
          const unsigned j = at + rank;
          out.ent[bstart + j] = make_uint4(k, pos, j - run_start[hi], run_start[hi + 1] - j);
        }
      }
    }
  }
  // the arrival counters of the chunks that start inside this bucket's part of the output
  for (unsigned c = cdiv<unsigned>(bstart, kChunk) + t; c * kChunk < bstart + m; c += kPlanThreads) out.arrivals[c] = 0;
}

// ---- plan for more ids than that: a stable radix sort over all blocks, then the run offsets by binary search -----
// Least significant digit first, 8 bits a pass, three launches a pass:
//   count    a block of 16 wavefronts owns a piece of consecutive entries, a wavefront a contiguous part of it; the
//            block leaves how many of its entries hold each digit (wave-private LDS counters fed by ballots, as in
//            plan_sort_pass: no atomic, nothing depends on timing);
//   scan     one block turns the counts, in (digit, block) order, into where each block's entries of each digit start;
//   scatter  the block counts again per wavefront, adds the prefix over its wavefronts to its start, and every
//            wavefront walks its part 64 entries at a step, ranking equal digits inside a step with ballots: entries
//            with equal digits keep their order, so after the last pass equal ids are in ascending position.
// The first pass reads the ids themselves (clamped to the vocabulary size) and takes the index as the position.
// (The library sort this replaces took 58 us for 100 000 ids and 104 us for 262 144.)
constexpr unsigned kRadixMaxBlocks = 256;  // pieces grow beyond 2048 entries to keep the count table at 256 x 256

static unsigned radix_piece(unsigned n) {
  const unsigned per = cdiv<unsigned>(n, kRadixMaxBlocks);
  return std::max(2048u, cdiv<unsigned>(per, 1024u) * 1024u);  // a multiple of 16 wavefronts x 64 lanes
}

// digit counts of the block's piece per (digit, wavefront) into cnt (zero on entry); returns after a barrier
template <bool FIRST>
__device__ __forceinline__ void radix_count_piece(unsigned n, unsigned vocab, unsigned piece, unsigned shift,
                                                  const unsigned* __restrict__ kin, unsigned* cnt) {
  const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
  const unsigned per_wave = piece / kPlanWaves;
  const unsigned wb = min(n, blockIdx.x * piece + w * per_wave), we = min(n, wb + per_wave);
  for (unsigned j0 = wb; j0 < we; j0 += 64) {  // uniform over the wavefront
    const unsigned j = j0 + lane;
    const bool valid = j < we;
    const unsigned raw = valid ? kin[j] : 0u;
    const unsigned dig = ((FIRST ? min(raw, vocab) : raw) >> shift) & 255u;
    const unsigned long long same = same_digit_lanes(dig, valid);
    if (valid && (same & lanes_below(lane)) == 0) cnt[dig * kPlanWaves + w] += __popcll(same);
  }
  __syncthreads();
}

template <bool FIRST>
__global__ __launch_bounds__(kPlanThreads) void radix_count_kernel(unsigned n, unsigned vocab, unsigned piece,
                                                                  unsigned shift, const unsigned* __restrict__ kin,
                                                                  unsigned* __restrict__ gcount, unsigned* status) {
  __shared__ __attribute__((aligned(16))) unsigned cnt[256 * kPlanWaves];
  const int t = threadIdx.x;
  reinterpret_cast<uint4*>(cnt)[t] = make_uint4(0u, 0u, 0u, 0u);
  if (FIRST && blockIdx.x == 0 && t == 0) *status = 0;  // the count itself is taken by plan_runs_sorted_kernel
  __syncthreads();
  radix_count_piece<FIRST>(n, vocab, piece, shift, kin, cnt);
  if (t < 256) {
    unsigned sum = 0;
#pragma unroll
    for (int w = 0; w < kPlanWaves; ++w) sum += cnt[t * kPlanWaves + w];
    gcount[size_t(t) * gridDim.x + blockIdx.x] = sum;
  }
}

// Exclusive prefix sum over `total` counts (a multiple of 4, at most 65536, 16-byte aligned) in place: thread t owns
// a contiguous run of at most 16 quads, all fetched before the first add (a loop of dependent single loads took 57 us).
constexpr int kRadixScanQuads = 16;
__global__ __launch_bounds__(kPlanThreads) void radix_scan_kernel(unsigned total, unsigned* __restrict__ gcount) {
  __shared__ unsigned tmp[kPlanWaves];
  uint4* g4 = reinterpret_cast<uint4*>(gcount);
  const unsigned quads = total / 4, per = cdiv<unsigned>(quads, kPlanThreads);  // per <= kRadixScanQuads
  const unsigned b = min(quads, threadIdx.x * per), e = min(quads, b + per);
  uint4 v[kRadixScanQuads];
#pragma unroll
  for (int q = 0; q < kRadixScanQuads; ++q) v[q] = b + q < e ? g4[b + q] : make_uint4(0u, 0u, 0u, 0u);
  unsigned sum = 0;
#pragma unroll
  for (int q = 0; q < kRadixScanQuads; ++q) sum += v[q].x + v[q].y + v[q].z + v[q].w;
  unsigned all = 0;
  unsigned run = block_scan_excl(sum, tmp, &all);
#pragma unroll
  for (int q = 0; q < kRadixScanQuads; ++q) {
    if (b + q < e) {
      uint4 o;
      o.x = run;
      o.y = o.x + v[q].x;
      o.z = o.y + v[q].y;
      o.w = o.z + v[q].z;
      run = o.w + v[q].w;
      g4[b + q] = o;
    }
  }
}

template <bool FIRST>
__global__ __launch_bounds__(kPlanThreads) void radix_scatter_kernel(unsigned n, unsigned vocab, unsigned piece,
                                                                    unsigned shift, const unsigned* __restrict__ kin,
                                                                    const unsigned* __restrict__ pin,
                                                                    const unsigned* __restrict__ gstart,
                                                                    unsigned* __restrict__ kout,
                                                                    unsigned* __restrict__ pout) {
  __shared__ __attribute__((aligned(16))) unsigned cnt[256 * kPlanWaves];
  const int t = threadIdx.x, lane = t & 63, w = t >> 6;
  reinterpret_cast<uint4*>(cnt)[t] = make_uint4(0u, 0u, 0u, 0u);
  __syncthreads();
  radix_count_piece<FIRST>(n, vocab, piece, shift, kin, cnt);
  if (t < 256) {  // counter (digit, wavefront) becomes the place of the wavefront's first entry with that digit
    unsigned run = gstart[size_t(t) * gridDim.x + blockIdx.x];
#pragma unroll
    for (int k = 0; k < kPlanWaves; ++k) {
      const unsigned v = cnt[t * kPlanWaves + k];
      cnt[t * kPlanWaves + k] = run;
      run += v;
    }
  }
  __syncthreads();
  const unsigned per_wave = piece / kPlanWaves;
  const unsigned wb = min(n, blockIdx.x * piece + w * per_wave), we = min(n, wb + per_wave);
  for (unsigned j0 = wb; j0 < we; j0 += 64) {
    const unsigned j = j0 + lane;
    const bool valid = j < we;
    const unsigned raw = valid ? kin[j] : 0u;
    const unsigned key = FIRST ? min(raw, vocab) : raw;
    const unsigned pos = FIRST ? j : (valid ? pin[j] : 0u);
    const unsigned dig = (key >> shift) & 255u;
    const unsigned long long same = same_digit_lanes(dig, valid);
    const unsigned rank = __popcll(same & lanes_below(lane));
    // every lane reads its digit's counter before the first lane of each digit advances it (see plan_sort_pass)
    unsigned at = 0;
    if (valid) at = cnt[dig * kPlanWaves + w];
    __builtin_amdgcn_wave_barrier();
    if (valid && rank == 0) cnt[dig * kPlanWaves + w] = at + __popcll(same);
    __builtin_amdgcn_wave_barrier();
    if (valid) {
      kout[at + rank] = key;
      pout[at + rank] = pos;
    }
  }
}

__global__ __launch_bounds__(256) void plan_runs_sorted_kernel(unsigned n, unsigned vocab,
                                                               const unsigned* __restrict__ sid,
                                                               const unsigned* __restrict__ spos, const Plan out) {
  const unsigned k = blockIdx.x * 256 + threadIdx.x;
  if (k >= n) return;
  const unsigned id = sid[k];
  // Both ends of the run by doubling steps away from k, then bisection inside the last step: most runs are short,
  // and two bisections over the whole vector were 2 x 18 dependent loads for every entry at 262 144 ids.
  unsigned off = 1;
  while (off <= k && sid[k - off] == id) off <<= 1;
  unsigned lo = off <= k ? k - off + 1 : 0, hi = k - off / 2;  // first index holding id lies in [lo, hi]
  while (lo < hi) {
    const unsigned mid = lo + (hi - lo) / 2;
    if (sid[mid] < id) lo = mid + 1;
    else hi = mid;
  }
  const unsigned first = lo;
  off = 1;
  while (off < n - k && sid[k + off] == id) off <<= 1;
  lo = k + off / 2 + 1, hi = off < n - k ? k + off : n;  // first index holding a larger id lies in [lo, hi]
  while (lo < hi) {
    const unsigned mid = lo + (hi - lo) / 2;
    if (sid[mid] <= id) lo = mid + 1;
    else hi = mid;
  }
  out.ent[k] = make_uint4(id, spos[k], k - first, lo - k);
  if (k % kChunk == 0) out.arrivals[k / kChunk] = 0;
  if (id >= vocab && k == first) out.status[0] = lo - first;  // one writer: the head of the run of clamped ids
}

static int plan_ws_bytes(unsigned n, unsigned vocab, size_t* bytes) {
  if (n <= kPlanSmallMax) {
    // only a bucket too large for LDS on the route for keys wider than 16 bits uses it
    *bytes = align256(4 * sizeof(unsigned) * size_t(n));
    return DYHIP_OK;
  }
  (void)vocab;
  // two (key, position) buffers and the count table
  *bytes = 4 * align256(sizeof(unsigned) * size_t(n)) + align256(sizeof(unsigned) * 256 * cdiv<unsigned>(n, radix_piece(n)));
  return DYHIP_OK;
}

static int build_plan(dyhip_device* dev, unsigned n, const unsigned* ids_dev, unsigned vocab, void* plan,
                      size_t plan_size, void* ws, size_t ws_bytes) {
  DYHIP_REQUIRE(vocab >= 1 && vocab < 0x7FFFFFFFu, "lookup vocabulary size %u out of range", vocab);
  size_t need = 0;
  DYHIP_CHECK_STATUS(plan_ws_bytes(n, vocab, &need));
  DYHIP_REQUIRE(plan != nullptr && plan_size >= plan_bytes(n) && aligned16(plan),
                "lookup plan needs %zu bytes (16-byte aligned), got %zu", plan_bytes(n), plan_size);
  DYHIP_REQUIRE(ws != nullptr && ws_bytes >= need && aligned16(ws), "lookup plan needs %zu workspace bytes, got %zu", need,
                ws_bytes);
  Plan out;
  plan_parts(plan, n, &out);
  const unsigned bits = key_bits(vocab);  // keys are min(id, vocab) <= vocab
  // 64-entry steps of a wavefront; a wavefront keeps its keys in registers, and 64 of them do not fit beside the
  // rest (the 64-step form spilled and took 122 us for 32 768 ids): beyond 32 steps the route below takes over
  const unsigned per_wave = cdiv<unsigned>(cdiv<unsigned>(n, kPlanWaves), 64u);
  if (n <= kPlanSmallMax && bits <= 16 && per_wave <= 32) {
    const dim3 grid(kPlanBuckets), block(kPlanThreads);
    if (per_wave <= 4) hipLaunchKernelGGL(plan_direct_kernel<4>, grid, block, 0, dev->stream, n, vocab, ids_dev, out);
    else if (per_wave <= 8) hipLaunchKernelGGL(plan_direct_kernel<8>, grid, block, 0, dev->stream, n, vocab, ids_dev, out);
    else if (per_wave <= 16) hipLaunchKernelGGL(plan_direct_kernel<16>, grid, block, 0, dev->stream, n, vocab, ids_dev, out);
    else hipLaunchKernelGGL(plan_direct_kernel<32>, grid, block, 0, dev->stream, n, vocab, ids_dev, out);
    DYHIP_CHECK_LAUNCH();
    return DYHIP_OK;
  }
  if (n <= kPlanSmallMax) {
    const unsigned passes = bits <= 8 ? 0u : (bits - 8 + 7) / 8;
    const size_t lds = sizeof(unsigned) * kPlanLdsWords;
    static bool attr_set[2] = {false, false};
    const bool vec = aligned16(ids_dev);
    if (!attr_set[vec]) {
      if (vec)
        DYHIP_CHECK_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(&plan_group_kernel<true>),
                                            hipFuncAttributeMaxDynamicSharedMemorySize, int(lds)));
      else
        DYHIP_CHECK_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(&plan_group_kernel<false>),
                                            hipFuncAttributeMaxDynamicSharedMemorySize, int(lds)));
      attr_set[vec] = true;
    }
    if (vec)
      hipLaunchKernelGGL(plan_group_kernel<true>, dim3(kPlanBuckets), dim3(kPlanThreads), lds, dev->stream, n, vocab,
                         passes, ids_dev, out, static_cast<unsigned*>(ws));
    else
      hipLaunchKernelGGL(plan_group_kernel<false>, dim3(kPlanBuckets), dim3(kPlanThreads), lds, dev->stream, n, vocab,
                         passes, ids_dev, out, static_cast<unsigned*>(ws));
    DYHIP_CHECK_LAUNCH();
    return DYHIP_OK;
  }
  const size_t keys_b = align256(sizeof(unsigned) * size_t(n));
  char* base = static_cast<char*>(ws);
  unsigned* kbuf[2] = {reinterpret_cast<unsigned*>(base), reinterpret_cast<unsigned*>(base + 2 * keys_b)};
  unsigned* pbuf[2] = {reinterpret_cast<unsigned*>(base + keys_b), reinterpret_cast<unsigned*>(base + 3 * keys_b)};
  unsigned* gcount = reinterpret_cast<unsigned*>(base + 4 * keys_b);
  const unsigned piece = radix_piece(n), nblocks = cdiv<unsigned>(n, piece), passes = cdiv<unsigned>(bits, 8u);
  const dim3 rgrid(nblocks), rblock(kPlanThreads);
  for (unsigned p = 0; p < passes; ++p) {
    const unsigned* kin = p == 0 ? ids_dev : kbuf[(p - 1) & 1];
    const unsigned* pin = p == 0 ? nullptr : pbuf[(p - 1) & 1];
    if (p == 0) {
      hipLaunchKernelGGL(radix_count_kernel<true>, rgrid, rblock, 0, dev->stream, n, vocab, piece, 0u, kin, gcount, out.status);
      hipLaunchKernelGGL(radix_scan_kernel, dim3(1), rblock, 0, dev->stream, 256u * nblocks, gcount);
      hipLaunchKernelGGL(radix_scatter_kernel<true>, rgrid, rblock, 0, dev->stream, n, vocab, piece, 0u, kin, pin, gcount,
                         kbuf[0], pbuf[0]);
    } else {
      hipLaunchKernelGGL(radix_count_kernel<false>, rgrid, rblock, 0, dev->stream, n, vocab, piece, 8u * p, kin, gcount,
                         out.status);
      hipLaunchKernelGGL(radix_scan_kernel, dim3(1), rblock, 0, dev->stream, 256u * nblocks, gcount);
      hipLaunchKernelGGL(radix_scatter_kernel<false>, rgrid, rblock, 0, dev->stream, n, vocab, piece, 8u * p, kin, pin,
                         gcount, kbuf[p & 1], pbuf[p & 1]);
    }
    DYHIP_CHECK_LAUNCH();
  }
  const unsigned* sid = kbuf[(passes - 1) & 1];
  const unsigned* spos = pbuf[(passes - 1) & 1];
  const dim3 grid(cdiv<unsigned>(n, 256)), block(256);
  hipLaunchKernelGGL(plan_runs_sorted_kernel, grid, block, 0, dev->stream, n, vocab, sid, spos, out);
  DYHIP_CHECK_LAUNCH();
  return DYHIP_OK;
}

// ---- segmented sum over the runs of a plan -----------------------------------------
// One thread group per chunk of kChunk consecutive grouped entries; a group is `tpr` threads that
// cover the row width (one block = one group when tpr >= 64, else 64 / tpr groups inside one wavefront).
//   * A run of fewer than kHeavyMin entries is summed by the group whose chunk holds its head, to its
//     end (into the following chunks if need be): acc = old row, += each gradient row in ascending
//     position, store.  That is the CPU path's order, so such rows come out bit-identical to it.
//     A group's runs hold at most kItemMax entries together.
//   * A run of kHeavyMin or more entries covers at least one whole chunk; the groups of the chunks
//     it covers entirely have no run of their own and share the run by COLUMNS: each sums every entry
//     of the run for a slice of the row, entry slots in parallel across the group's threads, slots
//     added in ascending order.  A slice is at least one 128-byte line wide; a run long enough to give
//     every slice several groups is also cut into parts of consecutive entries, whose sums the last
//     group to finish adds up in ascending order (arrival counters in the plan, partial sums in the
//     workspace).  Either way a thread's share of a run is one batch of loads at the usual row widths.
// The kernel keeps few enough registers for every block of the grid to be resident at once.  Updated rows are
// written with streaming stores, so they drain while the kernel runs instead of when it ends; the old rows are read
// with streaming loads (each is read once, and a line left in the L2 would only stand in the store's way).
// No second launch, no float atomics, and no group ever waits for another: the result does not depend on timing.
constexpr int kBatch = 11;                              // narrow groups: rows per thread and batch
constexpr int kBatchLong = 16;                          // wide groups inside a long run: rows per thread and batch
constexpr unsigned kHeavyMin = 2 * kChunk - 1;         // shortest run that must contain a whole chunk
constexpr int kItemMax = 3 * kChunk - 2;               // own chunk after its first entry (7) + the longest short run (14) <= 22
constexpr int kItemBatches = (kItemMax + kBatch - 1) / kBatch;
static_assert(kChunk - 1 + int(kHeavyMin) - 1 <= kItemMax, "a group's short runs fit kItemBatches batches");
static_assert(3 * kChunk <= 64 && kItemMax <= 32 && kBatch >= kChunk, "plan entries of an item sit in the lanes of one "
              "wavefront / two 16-lane rounds; every head of an item is in its first batch");

// Wide groups sum the short runs of their item as one stream of rows per thread, straight-line code without a
// branch around any load: the old rows of the (at most kChunk) runs that start in the chunk and the first kBatch
// gradient rows are requested at once; an item of more than kBatch entries refills the register of each row it has
// consumed with the row kBatch further on, so its later rows never wait for a whole batch to come back.  A slot
// without an entry loads a row that is in flight anyway and is not added.  Because nothing is conditional the compiler
// can count the loads in flight and waits for exactly the row it needs; loads issued inside per-entry branches made
// it wait for everything before every use.
constexpr unsigned kSlotValid = 1u, kSlotHead = 2u, kSlotLast = 4u;

__device__ __forceinline__ unsigned lane_get(unsigned v, unsigned src_lane) {
  return unsigned(__builtin_amdgcn_readlane(int(v), int(src_lane)));
}
__device__ __forceinline__ float4 vsel(bool c, const float4 a, const float4 b) {
  return make_float4(c ? a.x : b.x, c ? a.y : b.y, c ? a.z : b.z, c ? a.w : b.w);
}
__device__ __forceinline__ float vsel(bool c, const float a, const float b) { return c ? a : b; }

// Entry j of the item sits in lane first_l + j: e_pos its position (row of g), e_id its id (row of grads), e_fl its
// kSlot* flags (0 = no such entry, or an entry of the run of ids >= vocab, which is skipped).  NE = entries walked.
template <class V, int NE>
__device__ __forceinline__ void stream_item(unsigned e_pos, unsigned e_id, unsigned e_fl, unsigned first_l,
                                            unsigned dimv, unsigned c, bool cok, const V* __restrict__ g,
                                            V* __restrict__ grads) {
  const unsigned cc = cok ? c : 0u;
  const unsigned dummy_pos = lane_get(e_pos, first_l);  // a row of g that exists and is requested anyway
  V old[kChunk], v[kBatch];
#pragma unroll
  for (int j = 0; j < kChunk; ++j) {  // a run of the item starts inside the chunk
    const unsigned fl = lane_get(e_fl, first_l + j);
    const bool head = (fl & kSlotHead) != 0;
    const V* src = head ? grads + size_t(lane_get(e_id, first_l + j)) * dimv : g + size_t(dummy_pos) * dimv;
    old[j] = vload<true>(src + cc);
  }
#define DYHIP_ENTRY_LOAD(dst, j2)                                                                  \
  do {                                                                                             \
    const unsigned fl_ = lane_get(e_fl, first_l + (j2));                                           \
    const unsigned row_ = (fl_ & kSlotValid) ? lane_get(e_pos, first_l + (j2)) : dummy_pos;        \
    (dst) = vload<false>(g + size_t(row_) * dimv + cc);                                            \
  } while (0)
#pragma unroll
  for (int j = 0; j < kBatch; ++j) DYHIP_ENTRY_LOAD(v[j], j);
  V acc = vzero<V>();
#pragma unroll
  for (int j = 0; j < NE; ++j) {
    const unsigned fl = lane_get(e_fl, first_l + j);
    const V x = v[j % kBatch];
    if (j + kBatch < NE) DYHIP_ENTRY_LOAD(v[j % kBatch], j + kBatch);
    const V from = j < kChunk ? vsel((fl & kSlotHead) != 0, old[j < kChunk ? j : 0], acc) : acc;
    acc = vsel((fl & kSlotValid) != 0, vadd(from, x), acc);
    if ((fl & kSlotLast) && cok) vstore<true>(grads + size_t(lane_get(e_id, first_l + j)) * dimv + c, acc);
  }
#undef DYHIP_ENTRY_LOAD
}

template <class V, bool WIDE>
__global__ __launch_bounds__(256) void scatter_runs_kernel(unsigned n, unsigned dimv, unsigned tpr, unsigned vocab,
                                                           const Plan p, const V* __restrict__ g,
                                                           V* __restrict__ grads, V* partials) {
  extern __shared__ __attribute__((aligned(16))) char scatter_lds_raw[];
  V* lds = reinterpret_cast<V*>(scatter_lds_raw);
  const unsigned groups = blockDim.x / tpr;
  const unsigned grp = threadIdx.x / tpr, t = threadIdx.x - grp * tpr;
  const unsigned ch = blockIdx.x * groups + grp;
  const unsigned k0 = ch * kChunk;
  if (k0 >= n) return;  // whole groups leave; with tpr >= 64 the group is the block
  const int lane = threadIdx.x & 63;
  // Plan entries k0 + l, one per lane.  WIDE: lanes 0..23 of every wavefront of the group hold the chunk and
  // the two after it (as far as a short run that starts here can reach).  Narrow groups (16 or 32
  // threads) hold entries k0 .. k0+15 in each 16-lane cluster and fetch an item's entries afterwards.
  const unsigned l = WIDE ? unsigned(lane) : (threadIdx.x & 15u);
  const bool l_in = (WIDE ? l < 3u * kChunk : true) && k0 + l < n;
  const uint4 ent = l_in ? p.ent[k0 + l] : make_uint4(kNone, kNone, 1u, 0u);
  const unsigned e_id = ent.x, e_pos = ent.y, e_off = ent.z, e_rem = ent.w;
  const unsigned o0 = WIDE ? __builtin_amdgcn_readfirstlane(e_off) : __shfl(e_off, 0, 16);
  const unsigned r0 = WIDE ? __builtin_amdgcn_readfirstlane(e_rem) : __shfl(e_rem, 0, 16);
  if (o0 + r0 >= kHeavyMin && r0 >= unsigned(kChunk)) {
    // ---- this chunk lies inside a long run: take a slice of its columns --------------------
    constexpr int kB = WIDE ? kBatchLong : kBatch;
    const unsigned start = k0 - o0, R = o0 + r0;
    const unsigned cf = (start + kChunk - 1) / kChunk;       // first chunk the run covers entirely
    const unsigned W = (start + R) / kChunk - cf;            // how many it covers entirely (>= 1)
    const unsigned idx = ch - cf;
    const unsigned row = WIDE ? __builtin_amdgcn_readfirstlane(e_id) : __shfl(e_id, 0, 16);
    if (row >= vocab) return;
    // Slice width w in vector elements: whole 128-byte lines (narrower slices make several L2s fetch
    // the same line), wider if the run covers too few chunks to give every line-wide slice a group.
    const unsigned line = min(128u / unsigned(sizeof(V)), dimv);
    const unsigned w = min(tpr, max(cdiv<unsigned>(dimv, W), line));
    const unsigned S = cdiv<unsigned>(dimv, w), E = tpr / w;  // slices; entry slots per slice (threads >= E * w idle)
    const unsigned slot = t / w, cin = t - slot * w;
    const bool busy = slot < E;
    // A run that covers at least two groups per slice is also cut into P parts of consecutive entries: group
    // idx takes slice idx mod S of part idx / S.  The parts of a slice meet through `partials` (one 128-byte
    // line per chunk): each writes its sum there, counts itself in the slice's arrival counter, and the one
    // that arrives last adds all P up in ascending part order: the same sum whoever is last.
    const unsigned P = (WIDE && w * unsigned(sizeof(V)) <= 128u && W >= 2 * S) ? W / S : 1u;
    const unsigned per_part = cdiv<unsigned>(R, P);
    for (unsigned s0 = idx; s0 < S * P; s0 += W) {            // uniform over the group; one trip unless dimv > tpr * W
      const unsigned s = s0 % S, q = s0 / S;
      const unsigned eb = q * per_part, ee = min(R, eb + per_part);  // this part's entries of the run
      const unsigned c = s * w + cin;
      const bool cok = busy && c < dimv;
      V old = vzero<V>();
      if (cok && slot == 0) old = vload<true>(grads + size_t(row) * dimv + c);
      V acc = vzero<V>();
      for (unsigned e0 = eb + slot; e0 < ee; e0 += E * kB) {
        unsigned pos[kB];
#pragma unroll
        for (int u = 0; u < kB; ++u) {
          const unsigned e = e0 + u * E;
          pos[u] = (cok && e < ee) ? p.ent[start + e].y : kNone;
        }
        V v[kB];
#pragma unroll
        for (int u = 0; u < kB; ++u)
          v[u] = pos[u] != kNone ? g[size_t(pos[u]) * dimv + c] : vzero<V>();
#pragma unroll
        for (int u = 0; u < kB; ++u) acc = vadd(acc, v[u]);
      }
      if (WIDE) {
        // slots are added in ascending order: first every eighth slot by eight threads per column, then those
        __syncthreads();
        lds[t] = acc;
        __syncthreads();
        const unsigned fan = E >= 16 ? 8u : 1u;
        V part = vzero<V>();
        if (slot < fan && cok) {
          part = acc;
          for (unsigned qq = slot + fan; qq < E; qq += fan) part = vadd(part, lds[qq * w + cin]);
        }
        if (fan > 1) {
          __syncthreads();
          if (slot < fan) lds[slot * w + cin] = part;
          __syncthreads();
          if (slot == 0)
            for (unsigned qq = 1; qq < fan; ++qq) part = vadd(part, lds[qq * w + cin]);
        }
        if (P == 1) {
          if (slot == 0 && cok) vstore<true>(grads + size_t(row) * dimv + c, vadd(old, part));
        } else {
          // The partial sum goes to memory past the L2 of this block (each L2 serves one eighth of the chip
          // and does not see the others' lines); when the stores have been acknowledged the group counts
          // itself.  Nobody waits for anybody: whichever group finds P - 1 arrivals before it does the rest.
          const unsigned line_v = 128u / unsigned(sizeof(V));
          if (slot == 0 && cok) vstore_through(partials + size_t(ch) * line_v + cin, part);
          // every store of this wavefront has been acknowledged by memory before the barrier lets thread 0 count
          // (a workgroup-scope fence does not wait for global stores, an agent-scope one would also write the L2 back)
          __builtin_amdgcn_s_waitcnt(0);
          __syncthreads();
          unsigned* flag = reinterpret_cast<unsigned*>(lds);
          if (t == 0)
            *flag = __hip_atomic_fetch_add(p.arrivals + cf + s, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) == P - 1;
          __syncthreads();
          const bool last = *flag != 0;
          __syncthreads();
          if (last) {
            if (slot == 0 && cok) {
              // sixteen partial sums in flight at a time (the loads go past the caches; issued one by one between
              // the additions, each would be a round trip of its own), added in ascending part order
              V tot = vzero<V>();
              for (unsigned q0 = 0; q0 < P; q0 += 16) {
                V part16[16];
#pragma unroll
                for (int u = 0; u < 16; ++u)
                  part16[u] = vload_through(partials + size_t(cf + min(q0 + u, P - 1) * S + s) * line_v + cin);
#pragma unroll
                for (int u = 0; u < 16; ++u)
                  if (q0 + u < P) tot = q0 + u == 0 ? part16[u] : vadd(tot, part16[u]);
              }
              vstore<true>(grads + size_t(row) * dimv + c, vadd(old, tot));
            }
            if (t == 0) __hip_atomic_store(p.arrivals + cf + s, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
          }
        }
      } else {
        // the group sits inside one wavefront: slots are fetched from their lanes in ascending order
        const int lane0 = lane - int(t);
        V tot = acc;
        for (unsigned qq = 1; qq < E; ++qq) {
          const V o = vshfl(acc, lane0 + int(qq * w + cin));
          tot = vadd(tot, o);
        }
        if (slot == 0 && cok) vstore<true>(grads + size_t(row) * dimv + c, vadd(old, tot));
      }
    }
    return;
  }
  // ---- short runs whose head lies in this chunk ------------------------------------------------
  // first such head and the end of the last such run (a long run that starts here takes the rest of the chunk)
  const bool own = l < unsigned(kChunk) && l_in && e_off == 0 && e_rem < kHeavyMin;
  unsigned long long own_mask = __ballot(own);
  if (!WIDE) own_mask = (own_mask >> (lane & 48)) & 0xFFFFull;  // this group's 16-lane cluster
  if (own_mask == 0) return;
  const unsigned first_l = __ffsll((long long)own_mask) - 1, last_l = 63 - __clzll(own_mask);
  const unsigned ks = k0 + first_l;
  const unsigned ke = k0 + last_l + (WIDE ? __builtin_amdgcn_readlane(e_rem, last_l) : __shfl(e_rem, last_l, 16));
  if constexpr (WIDE) {
    // entry ks + j sits in lane first_l + j (< 24) of every wavefront of the group
    const bool live = l >= first_l && k0 + l < ke && e_id < vocab;  // ids >= vocab form one run that is skipped
    const unsigned e_fl = live ? (kSlotValid | (e_off == 0 ? kSlotHead : 0u) | (e_rem == 1 ? kSlotLast : 0u)) : 0u;
    for (unsigned c0 = 0; c0 < dimv; c0 += tpr) {
      const unsigned c = c0 + t;
      if (ke - ks <= unsigned(kBatch)) stream_item<V, kBatch>(e_pos, e_id, e_fl, first_l, dimv, c, c < dimv, g, grads);
      else stream_item<V, kItemMax>(e_pos, e_id, e_fl, first_l, dimv, c, c < dimv, g, grads);
    }
  } else {
    // Narrow groups fetch entry ks + j with lane j mod 16 of their 16-lane cluster (two rounds) and hand it around.
    unsigned b_pos[2] = {kNone, kNone}, b_id[2] = {kNone, kNone}, b_fl[2] = {0u, 0u};
#pragma unroll
    for (int r = 0; r < 2; ++r) {
      const unsigned k = ks + 16u * r + (threadIdx.x & 15u);
      const bool in = k < ke;
      const uint4 e2 = in ? p.ent[k] : make_uint4(kNone, kNone, 1u, 0u);
      b_pos[r] = e2.y;
      b_id[r] = e2.x;
      b_fl[r] = in ? (e2.z == 0 ? 1u : 0u) | (e2.w == 1 ? 2u : 0u) : 0u;
    }
    for (unsigned c0 = 0; c0 < dimv; c0 += tpr) {
      const unsigned c = c0 + t;
      const bool cok = c < dimv;
      V acc = vzero<V>();
#pragma unroll
      for (int r = 0; r < kItemBatches; ++r) {
        if (ks + unsigned(r * kBatch) >= ke) break;  // uniform over the group
        unsigned id[kBatch], pos[kBatch];
        bool head[kBatch], tail[kBatch];
#pragma unroll
        for (int u = 0; u < kBatch; ++u) {
          const int j = r * kBatch + u;
          if (j >= kItemMax) {
            pos[u] = kNone; id[u] = kNone; head[u] = false; tail[u] = false;
          } else {
            pos[u] = __shfl(b_pos[j / 16], j % 16, 16);
            id[u] = __shfl(b_id[j / 16], j % 16, 16);
            const unsigned fl = __shfl(b_fl[j / 16], j % 16, 16);
            head[u] = fl & 1u;
            tail[u] = fl & 2u;
          }
        }
        // every load of the batch is issued before the first add; heads lie in the own chunk, i.e. in batch 0
        V v[kBatch], old[kChunk];
#pragma unroll
        for (int u = 0; u < kBatch; ++u) {
          v[u] = (cok && pos[u] != kNone) ? g[size_t(pos[u]) * dimv + c] : vzero<V>();
          if (r == 0 && u < kChunk)
            old[u] = (cok && head[u] && id[u] < vocab) ? vload<true>(grads + size_t(id[u]) * dimv + c) : vzero<V>();
        }
        __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0): one explicit wait for the batch
#pragma unroll
        for (int u = 0; u < kBatch; ++u) {
          if (pos[u] != kNone) {
            if (r == 0 && u < kChunk && head[u]) acc = old[u];
            acc = vadd(acc, v[u]);
            if (cok && tail[u] && id[u] < vocab) vstore<true>(grads + size_t(id[u]) * dimv + c, acc);
          }
        }
      }
    }
  }
}

static unsigned threads_per_row(size_t dimv) {
  unsigned t = 16;
  while (t < kLkThreads && t < dimv) t <<= 1;
  return t;
}

// scratch of the segmented sum: one 128-byte line per chunk (partial sums of the parts of very long runs)
static size_t reduce_ws_bytes(unsigned n) { return size_t(128) * cdiv<unsigned>(n, kChunk); }

static int reduce_planned(dyhip_device* dev, unsigned n, const void* plan, size_t dim, unsigned vocab, const float* g,
                          float* all_grads, void* ws, size_t ws_bytes) {
  DYHIP_REQUIRE(ws != nullptr && ws_bytes >= reduce_ws_bytes(n) && aligned16(ws),
                "lookup scatter-add needs %zu workspace bytes (16-byte aligned), got %zu", reduce_ws_bytes(n), ws_bytes);
  Plan w;
  plan_parts(plan, n, &w);
  const bool vec = dim % 4 == 0 && aligned16(g) && aligned16(all_grads);
  const unsigned dimv = static_cast<unsigned>(vec ? dim / 4 : dim);
  const unsigned tpr = threads_per_row(dimv);
  const unsigned threads = tpr >= 64 ? tpr : 64;
  const unsigned chunks = cdiv<unsigned>(n, kChunk);
  const dim3 grid(cdiv<unsigned>(chunks, threads / tpr)), block(threads);
  const size_t lds = tpr >= 64 ? size_t(threads) * (vec ? sizeof(float4) : sizeof(float)) : 0;
#define DYHIP_SCATTER(V, WIDE)                                                                                    \
  hipLaunchKernelGGL((scatter_runs_kernel<V, WIDE>), grid, block, lds, dev->stream, n, dimv, tpr, vocab, w,     \
                     reinterpret_cast<const V*>(g), reinterpret_cast<V*>(all_grads), reinterpret_cast<V*>(ws))
  if (vec) {
    if (tpr >= 64) DYHIP_SCATTER(float4, true); else DYHIP_SCATTER(float4, false);
  } else {
    if (tpr >= 64) DYHIP_SCATTER(float, true); else DYHIP_SCATTER(float, false);
  }
#undef DYHIP_SCATTER
  DYHIP_CHECK_LAUNCH();
  return DYHIP_OK;
}

}  // namespace dyhip

using namespace dyhip;

extern "C" {

int dyhip_lookup_forward(dyhip_device* dev, unsigned n_ids, const unsigned* ids_host, unsigned* ids_dev, size_t dim,
                         unsigned vocab, const float* table, float mult, float* fx) {
  DYHIP_CHECK_DEV(dev);
  if (n_ids == 0 || dim == 0) return DYHIP_OK;
  DYHIP_REQUIRE(ids_dev && table && fx, "null pointer in lookup");
  DYHIP_REQUIRE(dim < (size_t(1) << 31), "lookup dimension too large");
  if (ids_host != nullptr) {
    for (unsigned b = 0; b < n_ids; ++b)
      DYHIP_REQUIRE(ids_host[b] < vocab, "Out-of-bounds attempt to access index %u for LookupParameter of size %u",
                    ids_host[b], vocab);
    DYHIP_CHECK_HIP(hipMemcpyAsync(ids_dev, ids_host, sizeof(unsigned) * n_ids, hipMemcpyHostToDevice, dev->stream));
    DYHIP_CHECK_HIP(hipStreamSynchronize(dev->stream));  // ids_host may be released by the caller on return
  }
  const bool vec = dim % 4 == 0 && aligned16(table) && aligned16(fx);
  const unsigned dimv = static_cast<unsigned>(vec ? dim / 4 : dim);
  const unsigned tpr = threads_per_row(dimv);
  const unsigned rows_per_block = (kLkThreads / tpr) * kGatherRowsUnroll;
  const dim3 grid(cdiv<unsigned>(n_ids, rows_per_block)), block(kLkThreads);
  // the table is read through the caches (hot rows repeat); the output is streamed when large
  const bool stream = size_t(n_ids) * dim * sizeof(float) >= dev->stream_threshold;
#define DYHIP_GATHER(V, SCALE, NT)                                                                                \
  hipLaunchKernelGGL((lookup_gather_kernel<V, SCALE, NT>), grid, block, 0, dev->stream, n_ids, dimv, tpr, vocab, \
                     ids_dev, reinterpret_cast<const V*>(table), mult, reinterpret_cast<V*>(fx))
  if (vec && stream) {
    if (mult == 1.0f) DYHIP_GATHER(float4, false, true); else DYHIP_GATHER(float4, true, true);
  } else if (vec) {
    if (mult == 1.0f) DYHIP_GATHER(float4, false, false); else DYHIP_GATHER(float4, true, false);
  } else {
    if (mult == 1.0f) DYHIP_GATHER(float, false, false); else DYHIP_GATHER(float, true, false);
  }
#undef DYHIP_GATHER
  DYHIP_CHECK_LAUNCH();
  return DYHIP_OK;
}

int dyhip_lookup_plan_bytes(unsigned n_ids, size_t* bytes) {
  DYHIP_REQUIRE(bytes != nullptr, "null output pointer");
  *bytes = n_ids ? plan_bytes(n_ids) : 0;
  return DYHIP_OK;
}

int dyhip_lookup_plan_workspace(unsigned n_ids, unsigned vocab, size_t* ws_bytes) {
  DYHIP_REQUIRE(ws_bytes != nullptr, "null output pointer");
  *ws_bytes = 0;
  if (n_ids == 0) return DYHIP_OK;
  return plan_ws_bytes(n_ids, vocab, ws_bytes);
}

int dyhip_lookup_build_plan(dyhip_device* dev, unsigned n_ids, const unsigned* ids_dev, unsigned vocab, void* plan,
                            size_t plan_size, void* ws, size_t ws_bytes) {
  DYHIP_CHECK_DEV(dev);
  if (n_ids == 0) return DYHIP_OK;
  DYHIP_REQUIRE(ids_dev != nullptr, "null pointer in lookup plan");
  return build_plan(dev, n_ids, ids_dev, vocab, plan, plan_size, ws, ws_bytes);
}

int dyhip_lookup_plan_invalid_ids(dyhip_device* dev, unsigned n_ids, const void* plan, unsigned* count) {
  DYHIP_CHECK_DEV(dev);
  DYHIP_REQUIRE(count != nullptr, "null output pointer");
  *count = 0;
  if (n_ids == 0) return DYHIP_OK;
  DYHIP_REQUIRE(plan != nullptr, "null pointer in lookup plan");
  Plan w;
  plan_parts(plan, n_ids, &w);
  DYHIP_CHECK_HIP(hipMemcpyAsync(count, w.status, sizeof(unsigned), hipMemcpyDeviceToHost, dev->stream));
  DYHIP_CHECK_HIP(hipStreamSynchronize(dev->stream));
  return gemm_check_giveups(dev);
}

int dyhip_lookup_accumulate_grads_planned_workspace(unsigned n_ids, size_t dim, size_t* ws_bytes) {
  DYHIP_REQUIRE(ws_bytes != nullptr, "null output pointer");
  (void)dim;
  *ws_bytes = n_ids ? reduce_ws_bytes(n_ids) : 0;
  return DYHIP_OK;
}

int dyhip_lookup_accumulate_grads_planned(dyhip_device* dev, unsigned n_ids, const void* plan, size_t dim,
                                          unsigned vocab, const float* g, float* all_grads, void* ws, size_t ws_bytes) {
  DYHIP_CHECK_DEV(dev);
  if (n_ids == 0 || dim == 0) return DYHIP_OK;
  DYHIP_REQUIRE(plan && g && all_grads, "null pointer in lookup accumulate_grads");
  DYHIP_REQUIRE(dim < (size_t(1) << 31), "lookup dimension too large");
  return reduce_planned(dev, n_ids, plan, dim, vocab, g, all_grads, ws, ws_bytes);
}

int dyhip_lookup_accumulate_grads_workspace(unsigned n_ids, size_t dim, unsigned vocab, size_t* ws_bytes) {
  DYHIP_REQUIRE(ws_bytes != nullptr, "null output pointer");
  *ws_bytes = 0;
  if (n_ids == 0 || dim == 0) return DYHIP_OK;
  size_t plan_ws = 0;
  DYHIP_CHECK_STATUS(plan_ws_bytes(n_ids, vocab, &plan_ws));
  *ws_bytes = plan_bytes(n_ids) + align256(reduce_ws_bytes(n_ids)) + plan_ws;
  return DYHIP_OK;
}

int dyhip_lookup_accumulate_grads(dyhip_device* dev, unsigned n_ids, const unsigned* ids_dev, size_t dim,
                                  unsigned vocab, const float* g, float* all_grads, void* ws, size_t ws_bytes) {
  DYHIP_CHECK_DEV(dev);
  if (n_ids == 0 || dim == 0) return DYHIP_OK;
  DYHIP_REQUIRE(ids_dev && g && all_grads, "null pointer in lookup accumulate_grads");
  DYHIP_REQUIRE(dim < (size_t(1) << 31), "lookup dimension too large");
  size_t need = 0;
  DYHIP_CHECK_STATUS(dyhip_lookup_accumulate_grads_workspace(n_ids, dim, vocab, &need));
  DYHIP_REQUIRE(ws != nullptr && ws_bytes >= need && aligned16(ws),
                "lookup scatter-add needs %zu workspace bytes (16-byte aligned), got %zu", need, ws_bytes);
  char* base = static_cast<char*>(ws);
  const size_t pb = plan_bytes(n_ids), rb = align256(reduce_ws_bytes(n_ids));
  DYHIP_CHECK_STATUS(build_plan(dev, n_ids, ids_dev, vocab, base, pb, base + pb + rb, ws_bytes - pb - rb));
  return reduce_planned(dev, n_ids, base, dim, vocab, g, all_grads, base + pb, rb);
}

}  // extern "C"
