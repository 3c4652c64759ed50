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
// Scatter-add: (id, position) pairs are radix-sorted by id (stable, so equal
// ids keep ascending position).  The sorted sequence is cut into chunks of
// kChunk entries; one thread group per chunk walks its entries in order and
// sums runs of equal ids in registers.  A run that lies inside one chunk is
// added straight into its gradient row (the chunk is the only writer of that
// row).  A run that crosses chunk boundaries leaves one partial row per chunk
// in the workspace, and a second kernel adds the partials of each such run in
// a fixed order.  No atomics anywhere: the result is deterministic and
// each gradient row is read and written exactly once.
#include <cstring>

#include <rocprim/rocprim.hpp>

#include "common.h"

namespace dyhip {

constexpr unsigned kNone = 0xFFFFFFFFu;
constexpr int kChunk = 16;
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

// ---- segmented scatter-add --------------------------------------------------------
struct ScatterWs {
  unsigned* sorted_ids;
  unsigned* sorted_pos;
  uint4* fix_list;       // part of the plan: {first chunk, last chunk, row, -} of every run that crosses a chunk
                         // boundary, in no particular order
  unsigned* fix_count;   // part of the plan: how many
  float* part_first;     // [chunks][dim]
  float* part_last;      // [chunks][dim]
  unsigned chunks;
};

template <class V, bool NT>
__global__ __launch_bounds__(kLkThreads) void scatter_chunk_kernel(unsigned n, unsigned dimv, unsigned tpr,
                                                                   unsigned vocab, ScatterWs w,
                                                                   const V* __restrict__ g, V* __restrict__ grads) {
  const unsigned groups = kLkThreads / tpr;
  const unsigned grp = threadIdx.x / tpr, t = threadIdx.x - grp * tpr;
  const unsigned ch = blockIdx.x * groups + grp;
  if (ch >= w.chunks) return;
  const unsigned k0 = ch * kChunk;
  const unsigned cnt = min(n - k0, (unsigned)kChunk);
  unsigned id[kChunk], pos[kChunk];
#pragma unroll
  for (int k = 0; k < kChunk; ++k) {
    id[k] = k < (int)cnt ? w.sorted_ids[k0 + k] : kNone;
    pos[k] = k < (int)cnt ? w.sorted_pos[k0 + k] : 0u;
  }
  const unsigned prev_id = k0 > 0 ? w.sorted_ids[k0 - 1] : kNone;
  const unsigned next_id = k0 + cnt < n ? w.sorted_ids[k0 + cnt] : kNone;
  const unsigned first = id[0], last = id[cnt - 1];
  const bool open_left = prev_id == first;
  const bool open_right = next_id == last;
  V* part_first = reinterpret_cast<V*>(w.part_first) + size_t(ch) * dimv;
  V* part_last = reinterpret_cast<V*>(w.part_last) + size_t(ch) * dimv;
  // run_end[k]: entry k is the last of its run inside this chunk; direct[k]: that run
  // lies wholly inside the chunk, so this thread group is the only writer of the row
  bool run_end[kChunk], direct[kChunk];
#pragma unroll
  for (int k = 0; k < kChunk; ++k) {
    const bool last_k = k + 1 >= (int)cnt;
    run_end[k] = k < (int)cnt && (last_k || id[k + 1 < kChunk ? k + 1 : k] != id[k]);
    const bool ol = open_left && id[k] == first;
    const bool orr = open_right && last_k;
    direct[k] = run_end[k] && !ol && !orr && id[k] < vocab;
  }
  for (unsigned c = t; c < dimv; c += tpr) {
    V v[kChunk], old[kChunk];
    // every load of the chunk is issued up front: the 16 gradient columns and the
    // old value of each row that will be updated in place
#pragma unroll
    for (int k = 0; k < kChunk; ++k) {
      v[k] = k < (int)cnt ? vload<NT>(g + size_t(pos[k]) * dimv + c) : vzero<V>();
      if (direct[k]) old[k] = grads[size_t(id[k]) * dimv + c];
    }
    V acc = vzero<V>();
#pragma unroll
    for (int k = 0; k < kChunk; ++k) {
      if (k < (int)cnt) {
        acc = vadd(acc, v[k]);
        if (run_end[k]) {
          if (direct[k])
            grads[size_t(id[k]) * dimv + c] = vadd(old[k], acc);
          else if (open_left && id[k] == first)
            part_first[c] = acc;
          else if (id[k] < vocab)
            part_last[c] = acc;
          acc = vzero<V>();
        }
      }
    }
  }
}

// One block per boundary-crossing run (the plan lists the chunks in which such runs start and
// where each ends).  The run's partial rows (one per chunk it touches) are split over
// kFixThreads / tpr thread slices that each add every slices-th partial in ascending order with
// four loads in flight, and the slices are then added in ascending order: deterministic, and a
// run of thousands of entries costs a handful of memory round trips instead of one per partial.
constexpr int kFixThreads = 1024;

template <class V>
__global__ __launch_bounds__(kFixThreads) void scatter_fixup_kernel(unsigned n, unsigned dimv, unsigned tpr,
                                                                    unsigned vocab, ScatterWs w,
                                                                    V* __restrict__ grads) {
  extern __shared__ __attribute__((aligned(16))) char fix_lds_raw[];
  V* lds = reinterpret_cast<V*>(fix_lds_raw);
  const unsigned slices = kFixThreads / tpr;
  const unsigned q = threadIdx.x / tpr, t = threadIdx.x - q * tpr;
  const V* pf = reinterpret_cast<const V*>(w.part_first);
  // count and the block's first entry are fetched together (entries past count are never used)
  uint4 e = w.fix_list[blockIdx.x];
  const unsigned count = *w.fix_count;
  for (unsigned i = blockIdx.x; i < count; i += gridDim.x) {  // uniform over the block
    if (i != blockIdx.x) e = w.fix_list[i];
    const unsigned c0 = e.x, c_last = e.y, row = e.z;
    if (row >= vocab) continue;
    const V* pl = reinterpret_cast<const V*>(w.part_last) + size_t(c0) * dimv;
    for (unsigned cb = 0; cb < dimv; cb += tpr) {
      const unsigned c = cb + t;
      V acc = vzero<V>(), old = vzero<V>();
      if (q == 0 && c < dimv) old = grads[size_t(row) * dimv + c];  // in flight beside the partials
      if (c < dimv) {
        // partial index p = 0 is part_last[c0]; p >= 1 is part_first[c0 + p]
        const unsigned np = c_last - c0 + 1;
        unsigned p = q;
        for (; p + 3 * slices < np; p += 4 * slices) {
          const V a0 = p == 0 ? pl[c] : pf[size_t(c0 + p) * dimv + c];
          const V a1 = pf[size_t(c0 + p + slices) * dimv + c];
          const V a2 = pf[size_t(c0 + p + 2 * slices) * dimv + c];
          const V a3 = pf[size_t(c0 + p + 3 * slices) * dimv + c];
          acc = vadd(vadd(vadd(vadd(acc, a0), a1), a2), a3);
        }
        for (; p < np; p += slices) acc = vadd(acc, p == 0 ? pl[c] : pf[size_t(c0 + p) * dimv + c]);
      }
      __syncthreads();
      lds[q * tpr + t] = acc;
      __syncthreads();
      if (q == 0 && c < dimv) {
        V tot = lds[t];
        for (unsigned k = 1; k < slices; ++k) tot = vadd(tot, lds[k * tpr + t]);
        grads[size_t(row) * dimv + c] = vadd(old, tot);
      }
    }
  }
}

static unsigned threads_per_row(size_t dimv) {
  unsigned t = 16;
  while (t < kLkThreads && t < dimv) t <<= 1;
  return t;
}

static unsigned key_bits(unsigned vocab) {
  unsigned bits = 1;
  while (bits < 32 && (1ull << bits) < (unsigned long long)vocab) ++bits;
  return bits;
}

static size_t align256(size_t n) { return (n + 255) / 256 * 256; }

static int sort_tmp_bytes(unsigned n, unsigned vocab, size_t* bytes) {
  size_t tmp = 0;
  unsigned* k = nullptr;
  hipError_t e = rocprim::radix_sort_pairs(nullptr, tmp, static_cast<const unsigned*>(k), k,
                                           rocprim::counting_iterator<unsigned>(0), k, n, 0, key_bits(vocab));
  if (e != hipSuccess) return fail(DYHIP_ERR_RUNTIME, "radix sort size query failed: %s", hipGetErrorString(e));
  *bytes = tmp;
  return DYHIP_OK;
}

__global__ void plan_reset_kernel(unsigned* fix_count) { *fix_count = 0; }

// Per chunk of the sorted ids: does a run start here (not continuing from the previous chunk,
// or filling this chunk only partly) and continue into the next chunk?  If so, in which chunk
// does it end (binary search for the upper bound of its id)?  Every such run becomes one entry
// of the plan's fix-up list, so the search is paid when the plan is built, not in the backward pass.

__global__ __launch_bounds__(256) void plan_runs_kernel(unsigned n, unsigned chunks,
                                                        const unsigned* __restrict__ sorted_ids,
                                                        uint4* __restrict__ fix_list, unsigned* fix_count) {
  const unsigned ch = blockIdx.x * 256 + threadIdx.x;
  if (ch >= chunks) return;
  const unsigned k0 = ch * kChunk, cnt = min(n - k0, (unsigned)kChunk);
  const unsigned first = sorted_ids[k0], last = sorted_ids[k0 + cnt - 1];
  const bool open_left = k0 > 0 && sorted_ids[k0 - 1] == first;
  const bool open_right = k0 + cnt < n && sorted_ids[k0 + cnt] == last;
  unsigned out = kNone;
  if (open_right && !(first == last && open_left)) {
    unsigned lo = k0 + cnt, hi = n;
    while (lo < hi) {
      const unsigned mid = lo + (hi - lo) / 2;
      if (sorted_ids[mid] <= last) lo = mid + 1;
      else hi = mid;
    }
    out = (lo - 1) / kChunk;
  }
  // the order of the list does not matter: the runs are independent of each other
  if (out != kNone) fix_list[atomicAdd(fix_count, 1u)] = make_uint4(ch, out, last, 0u);
}

// plan = [sorted_ids (n u32) | sorted_pos (n u32) | fix_list (chunks uint4) | fix_count], each part padded to 256 bytes
static size_t plan_bytes(unsigned n) {
  return 2 * align256(sizeof(unsigned) * n) + align256(sizeof(uint4) * cdiv<unsigned>(n, kChunk)) + 256;
}

static void plan_parts(const void* plan, unsigned n, ScatterWs* w) {
  char* p = const_cast<char*>(static_cast<const char*>(plan));
  const size_t ids_b = align256(sizeof(unsigned) * n);
  w->chunks = cdiv<unsigned>(n, kChunk);
  w->sorted_ids = reinterpret_cast<unsigned*>(p);
  w->sorted_pos = reinterpret_cast<unsigned*>(p + ids_b);
  w->fix_list = reinterpret_cast<uint4*>(p + 2 * ids_b);
  w->fix_count = reinterpret_cast<unsigned*>(p + 2 * ids_b + align256(sizeof(uint4) * w->chunks));
}

// scratch of the reduction kernels = [part_first | part_last]
static size_t reduce_ws_bytes(unsigned n, size_t dim) {
  const unsigned chunks = cdiv<unsigned>(n, kChunk);
  return 2 * align256(sizeof(float) * dim * chunks);
}

static int build_plan(dyhip_device* dev, unsigned n, const unsigned* ids_dev, unsigned vocab, void* plan,
                      size_t plan_size, void* ws, size_t ws_bytes) {
  size_t sort_bytes = 0;
  DYHIP_CHECK_STATUS(sort_tmp_bytes(n, vocab, &sort_bytes));
  DYHIP_REQUIRE(plan != nullptr && plan_size >= plan_bytes(n) && aligned16(plan),
                "lookup plan needs %zu bytes (16-byte aligned), got %zu", plan_bytes(n), plan_size);
  DYHIP_REQUIRE(sort_bytes == 0 || (ws != nullptr && ws_bytes >= sort_bytes),
                "lookup plan needs %zu workspace bytes, got %zu", sort_bytes, ws_bytes);
  unsigned* sorted_ids = static_cast<unsigned*>(plan);
  unsigned* sorted_pos = reinterpret_cast<unsigned*>(static_cast<char*>(plan) + align256(sizeof(unsigned) * n));
  DYHIP_CHECK_HIP(rocprim::radix_sort_pairs(ws, sort_bytes, ids_dev, sorted_ids,
                                            rocprim::counting_iterator<unsigned>(0), sorted_pos, n, 0, key_bits(vocab),
                                            dev->stream));
  ScatterWs w;
  plan_parts(plan, n, &w);
  hipLaunchKernelGGL(plan_reset_kernel, dim3(1), dim3(1), 0, dev->stream, w.fix_count);
  hipLaunchKernelGGL(plan_runs_kernel, dim3(cdiv<unsigned>(w.chunks, 256)), dim3(256), 0, dev->stream, n, w.chunks,
                     sorted_ids, w.fix_list, w.fix_count);
  DYHIP_CHECK_LAUNCH();
  return DYHIP_OK;
}

static int reduce_planned(dyhip_device* dev, unsigned n, const void* plan, size_t dim, unsigned vocab, const float* g,
                          float* all_grads, void* ws, size_t ws_bytes) {
  const size_t need = reduce_ws_bytes(n, dim);
  DYHIP_REQUIRE(ws != nullptr && ws_bytes >= need && aligned16(ws),
                "lookup scatter-add needs %zu workspace bytes (16-byte aligned), got %zu", need, ws_bytes);
  ScatterWs w;
  plan_parts(plan, n, &w);
  char* base = static_cast<char*>(ws);
  w.part_first = reinterpret_cast<float*>(base);
  w.part_last = reinterpret_cast<float*>(base + align256(sizeof(float) * dim * w.chunks));
  const bool vec = dim % 4 == 0 && aligned16(g) && aligned16(all_grads);
  const unsigned dimv = static_cast<unsigned>(vec ? dim / 4 : dim);
  const unsigned tpr = threads_per_row(dimv);
  const dim3 grid(cdiv<unsigned>(w.chunks, kLkThreads / tpr)), block(kLkThreads);
  // enough blocks for every CU; a block walks the plan's list of boundary-crossing runs
  const dim3 fgrid(std::min<unsigned>(w.chunks, 2u * unsigned(dev->num_cus))), fblock(kFixThreads);
  const size_t flds = size_t(kFixThreads) * (vec ? sizeof(float4) : sizeof(float));
  if (vec) {
    float4* gr = reinterpret_cast<float4*>(all_grads);
    const float4* g4 = reinterpret_cast<const float4*>(g);
    // plain loads: streaming (non-temporal) hints make this random-row gather slower, not faster
    hipLaunchKernelGGL((scatter_chunk_kernel<float4, false>), grid, block, 0, dev->stream, n, dimv, tpr, vocab, w, g4, gr);
    hipLaunchKernelGGL(scatter_fixup_kernel<float4>, fgrid, fblock, flds, dev->stream, n, dimv, tpr, vocab, w, gr);
  } else {
    hipLaunchKernelGGL((scatter_chunk_kernel<float, false>), grid, block, 0, dev->stream, n, dimv, tpr, vocab, w, g,
                       all_grads);
    hipLaunchKernelGGL(scatter_fixup_kernel<float>, fgrid, fblock, flds, dev->stream, n, dimv, tpr, vocab, w, all_grads);
  }
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
  size_t b = 0;
  DYHIP_CHECK_STATUS(sort_tmp_bytes(n_ids, vocab, &b));
  *ws_bytes = align256(b);
  return DYHIP_OK;
}

int dyhip_lookup_build_plan(dyhip_device* dev, unsigned n_ids, const unsigned* ids_dev, unsigned vocab, void* plan,
                            size_t plan_size, void* ws, size_t ws_bytes) {
  DYHIP_CHECK_DEV(dev);
  if (n_ids == 0) return DYHIP_OK;
  DYHIP_REQUIRE(ids_dev != nullptr, "null pointer in lookup plan");
  return build_plan(dev, n_ids, ids_dev, vocab, plan, plan_size, ws, ws_bytes);
}

int dyhip_lookup_accumulate_grads_planned_workspace(unsigned n_ids, size_t dim, size_t* ws_bytes) {
  DYHIP_REQUIRE(ws_bytes != nullptr, "null output pointer");
  *ws_bytes = (n_ids == 0 || dim == 0) ? 0 : reduce_ws_bytes(n_ids, dim);
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
  size_t sort_ws = 0;
  DYHIP_CHECK_STATUS(dyhip_lookup_plan_workspace(n_ids, vocab, &sort_ws));
  *ws_bytes = plan_bytes(n_ids) + reduce_ws_bytes(n_ids, dim) + sort_ws;
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
  const size_t pb = plan_bytes(n_ids), rb = reduce_ws_bytes(n_ids, dim);
  DYHIP_CHECK_STATUS(build_plan(dev, n_ids, ids_dev, vocab, base, pb, base + pb + rb, ws_bytes - pb - rb));
  return reduce_planned(dev, n_ids, base, dim, vocab, g, all_grads, base + pb, rb);
}

}  // extern "C"
