// Device object, memory pools, copies and stream timing.
//
// Replaces Device_GPU (dynet/devices.cc:91-121), GPUAllocator (dynet/mem.cc:71-90)
// and AlignedMemoryPool (dynet/aligned-mem-pool.cc:8-91) of the reference.  The
// pool keeps the reference's observable behaviour: bump allocation rounded to
// the allocator's alignment, growth in multiples of the expanding unit when the
// newest block overflows, consolidation into one block of the total capacity
// on free(), zero-fill at block creation, used()/set_used() only meaningful
// while there is a single block.
#include <cstdio>
#include <cstdlib>
#include <cstring>

#include "common.h"

namespace dyhip {

static thread_local char g_last_error[1024] = "";

int fail(int code, const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_last_error, sizeof(g_last_error), fmt, ap);
  va_end(ap);
  return code;
}

// Zero-fill as a kernel rather than a memset node, so that callers may capture
// it into a HIP graph.  Handles any address and byte count: byte head up to the
// first 16-byte boundary, 16-byte body, byte tail.
__global__ __launch_bounds__(256) void zero_fill_kernel(char* p, size_t nbytes) {
  const size_t gid = size_t(blockIdx.x) * blockDim.x + threadIdx.x;
  const size_t stride = size_t(gridDim.x) * blockDim.x;
  size_t head = (16 - (reinterpret_cast<uintptr_t>(p) & 15u)) & 15u;
  if (head > nbytes) head = nbytes;
  if (gid < head) p[gid] = 0;
  char* body = p + head;
  const size_t rest = nbytes - head, n16 = rest >> 4;
  uint4* p16 = reinterpret_cast<uint4*>(body);
  for (size_t i = gid; i < n16; i += stride) p16[i] = make_uint4(0u, 0u, 0u, 0u);
  for (size_t i = (n16 << 4) + gid; i < rest; i += stride) body[i] = 0;
}

hipError_t zero_fill(void* p, size_t nbytes, hipStream_t stream) {
  if (nbytes == 0) return hipSuccess;
  size_t blocks = cdiv<size_t>(nbytes >> 4, 256 * 8);
  if (blocks < 1) blocks = 1;
  if (blocks > 4096) blocks = 4096;
  hipLaunchKernelGGL(zero_fill_kernel, dim3((unsigned)blocks), dim3(256), 0, stream, static_cast<char*>(p), nbytes);
  return hipGetLastError();
}

// hipMalloc-backed allocator, 256-byte alignment like the reference's GPUAllocator.
struct HipAllocator : MemAllocator {
  HipAllocator(int ordinal, hipStream_t stream) : MemAllocator(256), ordinal(ordinal), stream(stream) {}
  void* malloc(size_t n) override {
    void* p = nullptr;
    refusal = nullptr;
    if (hipSetDevice(ordinal) != hipSuccess) return nullptr;
    // A block allocated while a graph is being recorded would be zeroed and freed outside the recorded
    // order (and the queues forked from this device record into the same capture): pools are sized before
    // a capture begins, growth inside one is refused.
    hipStreamCaptureStatus cap = hipStreamCaptureStatusNone;
    if (hipStreamIsCapturing(stream, &cap) != hipSuccess) (void)hipGetLastError();
    if (cap != hipStreamCaptureStatusNone) {
      refusal = "a memory pool cannot grow while a graph capture is in progress; allocate before the capture";
      return nullptr;
    }
    if (hipMalloc(&p, n) != hipSuccess) {
      (void)hipGetLastError();
      return nullptr;
    }
    return p;
  }
  void free(void* p) override { (void)hipFree(p); }
  // The fill runs on the device's own stream; queues forked from the device share the pools, so the call
  // returns only once the block is zero: whatever any queue launches afterwards finds it cleared.
  bool zero(void* p, size_t n) override {
    if (zero_fill(p, n, stream) != hipSuccess) return false;
    hipStreamCaptureStatus cap = hipStreamCaptureStatusNone;
    if (hipStreamIsCapturing(stream, &cap) != hipSuccess) (void)hipGetLastError();
    if (cap != hipStreamCaptureStatusNone) return true;  // pool_zero_allocated inside a capture: recorded in order
    return hipStreamSynchronize(stream) == hipSuccess;
  }
  int ordinal;
  hipStream_t stream;
};

// Host allocator, 32-byte alignment like the reference's CPUAllocator.
struct HostAllocator : MemAllocator {
  HostAllocator() : MemAllocator(32) {}
  void* malloc(size_t n) override {
    void* p = nullptr;
    if (posix_memalign(&p, 32, n ? n : 32) != 0) return nullptr;
    return p;
  }
  void free(void* p) override { ::free(p); }
  bool zero(void* p, size_t n) override {
    memset(p, 0, n);
    return true;
  }
};

static int pool_add_block(dyhip_pool* pool, size_t cap) {
  dyhip_pool::Block blk;
  blk.capacity = pool->alloc->round_up_align(cap);
  blk.mem = static_cast<char*>(pool->alloc->malloc(blk.capacity));
  blk.used = 0;
  if (blk.mem == nullptr) {
    if (pool->alloc->refusal != nullptr) return fail(DYHIP_ERR_RUNTIME, "%s: %s", pool->name.c_str(), pool->alloc->refusal);
    return fail(DYHIP_ERR_OUT_OF_MEMORY, "%s failed to allocate %zu bytes", pool->name.c_str(), blk.capacity);
  }
  if (!pool->alloc->zero(blk.mem, blk.capacity)) {
    pool->alloc->free(blk.mem);
    return fail(DYHIP_ERR_RUNTIME, "%s failed to zero %zu bytes", pool->name.c_str(), blk.capacity);
  }
  pool->blocks.push_back(blk);
  return DYHIP_OK;
}

static int pool_new(const char* name, size_t cap, size_t expanding_unit, MemAllocator* alloc, bool owns_alloc,
                    dyhip_pool** out) {
  if (cap == 0) {
    if (owns_alloc) delete alloc;
    return fail(DYHIP_ERR_INVALID_ARG, "Attempt to allocate memory of size 0 in AlignedMemoryPool");
  }
  dyhip_pool* pool = new dyhip_pool();
  pool->name = name ? name : "pool";
  pool->cap = cap;
  pool->expanding_unit = expanding_unit ? expanding_unit : (size_t(1) << 24);
  pool->alloc = alloc;
  pool->owns_alloc = owns_alloc;
  int st = pool_add_block(pool, cap);
  if (st != DYHIP_OK) {
    if (owns_alloc) delete alloc;
    delete pool;
    return st;
  }
  *out = pool;
  return DYHIP_OK;
}

static void pool_delete(dyhip_pool* pool) {
  for (auto& b : pool->blocks) pool->alloc->free(b.mem);
  if (pool->owns_alloc) delete pool->alloc;
  delete pool;
}

}  // namespace dyhip

using namespace dyhip;

// The flag words of the 256 x 256-tile GEMM sit behind the split-K workspace, outside the size that other kernels
// are told, and start out zero.
// The fill runs on the queue's own stream (a non-blocking stream is not ordered against the null stream) and has
// finished when the call returns.
static int gemm_flags_clear(dyhip_device* dev) {
  DYHIP_CHECK_HIP(hipMemsetAsync(dev->gemm_flags, 0, kGemmFlagWords * sizeof(unsigned), dev->stream));
  DYHIP_CHECK_HIP(hipStreamSynchronize(dev->stream));
  return DYHIP_OK;
}

static int gemm_flags_setup(dyhip_device* dev) {
  dev->gemm_flags = reinterpret_cast<unsigned*>(static_cast<char*>(dev->gemm_ws) + dev->gemm_ws_bytes);
  dev->gemm_spin_limit = 1u << 22;  // polls about a microsecond apart: seconds
  dev->gemm_raise_flags = 1;
  return gemm_flags_clear(dev);
}

// One queue's give-up counter; the queue's stream has been synchronised.
static int gemm_giveups_of_queue(dyhip_device* q, unsigned* gave_up) {
  *gave_up = 0;
  if (!q->gemm_flags_used || q->gemm_flags == nullptr) return DYHIP_OK;
  q->gemm_flags_used = false;
  DYHIP_CHECK_HIP(hipMemcpyAsync(gave_up, q->gemm_flags + kGemmFlagWords - 1, sizeof(unsigned), hipMemcpyDeviceToHost,
                                 q->stream));
  DYHIP_CHECK_HIP(hipStreamSynchronize(q->stream));
  // a waiter that gave up cleared a flag that its late producer raised afterwards: start the next launch clean
  if (*gave_up != 0) DYHIP_CHECK_STATUS(gemm_flags_clear(q));
  return DYHIP_OK;
}

// Called by every entry point that has just synchronised dev's stream and hands results to the host: turns waits
// that gave up inside a 256 x 256-tile GEMM (on this queue, or on a queue forked from it: a graph launched here may
// hold products recorded there) into an error.
int dyhip::gemm_check_giveups(dyhip_device* dev) {
  unsigned total = 0, n = 0;
  DYHIP_CHECK_STATUS(gemm_giveups_of_queue(dev, &n));
  total += n;
  for (dyhip_device* f : dev->forks) {
    if (!f->gemm_flags_used) continue;
    DYHIP_CHECK_HIP(hipStreamSynchronize(f->stream));
    DYHIP_CHECK_STATUS(gemm_giveups_of_queue(f, &n));
    total += n;
  }
  if (total != 0)
    return fail(DYHIP_ERR_RUNTIME, "GEMM: %u blocks gave up waiting for a partial tile; the products since the last "
                                   "synchronisation are incomplete", total);
  return DYHIP_OK;
}

extern "C" {

const char* dyhip_last_error(void) { return g_last_error; }

// ---------------------------------------------------------------------------
// pools
// ---------------------------------------------------------------------------
int dyhip_pool_create_host(const char* name, size_t cap_bytes, size_t expanding_unit, dyhip_pool** out) {
  DYHIP_REQUIRE(out != nullptr, "null output pointer");
  return pool_new(name, cap_bytes, expanding_unit, new HostAllocator(), true, out);
}

int dyhip_pool_destroy(dyhip_pool* pool) {
  DYHIP_REQUIRE(pool != nullptr, "null pool handle");
  pool_delete(pool);
  return DYHIP_OK;
}

int dyhip_pool_allocate(dyhip_pool* pool, size_t nbytes, void** out) {
  DYHIP_REQUIRE(pool != nullptr && out != nullptr, "null pool handle or output pointer");
  const size_t rounded = pool->alloc->round_up_align(nbytes);
  dyhip_pool::Block* cur = &pool->blocks.back();
  if (rounded + cur->used > cur->capacity) {
    // grow by the smallest multiple of the expanding unit that holds the request
    const size_t unit = pool->expanding_unit;
    const size_t new_size = (nbytes + unit - 1) / unit * unit;
    DYHIP_CHECK_STATUS(pool_add_block(pool, new_size ? new_size : unit));
    pool->cap += new_size;
    cur = &pool->blocks.back();
    if (rounded + cur->used > cur->capacity)
      return fail(DYHIP_ERR_OUT_OF_MEMORY, "%s cannot hold %zu bytes", pool->name.c_str(), nbytes);
  }
  *out = cur->mem + cur->used;
  cur->used += rounded;
  return DYHIP_OK;
}

int dyhip_pool_free(dyhip_pool* pool) {
  DYHIP_REQUIRE(pool != nullptr, "null pool handle");
  if (pool->blocks.size() > 1) {
    // consolidate: one block of the total capacity, so that the next graph of
    // the same size fits without growing again
    // The consolidated block is allocated before the old ones are released: if that fails the pool
    // keeps its blocks (emptied) and stays usable.
    std::vector<dyhip_pool::Block> old;
    old.swap(pool->blocks);
    const int st = pool_add_block(pool, pool->cap);
    if (st != DYHIP_OK) {
      pool->blocks.swap(old);
      for (auto& b : pool->blocks) b.used = 0;
      // allocation continues from the newest block, as after growth
      return st;
    }
    for (auto& b : old) pool->alloc->free(b.mem);
  }
  pool->blocks[0].used = 0;
  return DYHIP_OK;
}

int dyhip_pool_zero_allocated(dyhip_pool* pool) {
  DYHIP_REQUIRE(pool != nullptr, "null pool handle");
  for (auto& b : pool->blocks)
    if (b.used > 0 && !pool->alloc->zero(b.mem, b.used))
      return fail(DYHIP_ERR_RUNTIME, "%s failed to zero its allocated prefix", pool->name.c_str());
  return DYHIP_OK;
}

int dyhip_pool_used(dyhip_pool* pool, size_t* used) {
  DYHIP_REQUIRE(pool != nullptr && used != nullptr, "null pool handle or output pointer");
  size_t u = 0;
  for (auto& b : pool->blocks) u += b.used;
  *used = u;
  return DYHIP_OK;
}

int dyhip_pool_set_used(dyhip_pool* pool, size_t used) {
  DYHIP_REQUIRE(pool != nullptr, "null pool handle");
  if (used != pool->blocks.back().used) {
    DYHIP_REQUIRE(pool->blocks.size() == 1,
                  "Dynet does not support both dynamic increasing of memory pool size, and automatic batching or "
                  "memory checkpointing. If you want to use automatic batching or checkpointing, please "
                  "pre-allocate enough memory using the --dynet-mem command line option.");
    DYHIP_REQUIRE(used <= pool->blocks[0].capacity, "set_used(%zu) beyond the pool capacity %zu", used,
                  pool->blocks[0].capacity);
    pool->blocks[0].used = used;
  }
  return DYHIP_OK;
}

int dyhip_pool_capacity(dyhip_pool* pool, size_t* cap) {
  DYHIP_REQUIRE(pool != nullptr && cap != nullptr, "null pool handle or output pointer");
  *cap = pool->cap;
  return DYHIP_OK;
}

int dyhip_pool_num_blocks(dyhip_pool* pool, int* n) {
  DYHIP_REQUIRE(pool != nullptr && n != nullptr, "null pool handle or output pointer");
  *n = static_cast<int>(pool->blocks.size());
  return DYHIP_OK;
}

// ---------------------------------------------------------------------------
// device
// ---------------------------------------------------------------------------
int dyhip_device_count(int* count) {
  DYHIP_REQUIRE(count != nullptr, "null output pointer");
  int n = 0;
  hipError_t e = hipGetDeviceCount(&n);
  if (e != hipSuccess) {
    (void)hipGetLastError();
    *count = 0;
    return fail(DYHIP_ERR_NO_DEVICE, "hipGetDeviceCount failed: %s", hipGetErrorString(e));
  }
  *count = n;
  return DYHIP_OK;
}

int dyhip_device_create(int ordinal, const size_t pool_mb[4], dyhip_device** out) {
  DYHIP_REQUIRE(out != nullptr && pool_mb != nullptr, "null output pointer or pool sizes");
  int n = 0;
  DYHIP_CHECK_STATUS(dyhip_device_count(&n));
  if (n == 0) return fail(DYHIP_ERR_NO_DEVICE, "no HIP device is visible");
  DYHIP_REQUIRE(ordinal >= 0 && ordinal < n, "device ordinal %d out of range [0, %d)", ordinal, n);
  for (int i = 0; i < 4; ++i)
    DYHIP_REQUIRE(pool_mb[i] > 0, "Attempt to allocate memory of size 0 in DeviceMempoolSizes");
  DYHIP_CHECK_HIP(hipSetDevice(ordinal));
  hipDeviceProp_t prop;
  DYHIP_CHECK_HIP(hipGetDeviceProperties(&prop, ordinal));
  dyhip_device* dev = new dyhip_device();
  dev->parent = nullptr;
  dev->sync_next = 0;
  dev->ordinal = ordinal;
  dev->num_cus = prop.multiProcessorCount;
  dev->max_lds_per_block = prop.sharedMemPerBlockOptin > 0 ? prop.sharedMemPerBlockOptin : prop.sharedMemPerBlock;
  for (auto& p : dev->pools) p = nullptr;
  dev->scalars = nullptr;
  dev->rng_state = nullptr;
  dev->rng_stream = 0;
  dev->forks_made = 0;
  dev->alloc = nullptr;
  dev->gemm_ws = nullptr;
  dev->gemm_ws_bytes = 0;
  dev->wide_gemm_ready = 0;
  dev->gemm_flags = nullptr;
  dev->gemm_flags_used = false;
  dev->ln_scratch = nullptr;
  dev->stream_threshold = size_t(8) << 20;
  hipError_t e = hipStreamCreateWithFlags(&dev->stream, hipStreamNonBlocking);
  if (e != hipSuccess) {
    delete dev;
    return fail(DYHIP_ERR_RUNTIME, "hipStreamCreateWithFlags failed: %s", hipGetErrorString(e));
  }
  (void)hipEventCreate(&dev->ev_start);
  (void)hipEventCreate(&dev->ev_stop);
  dev->alloc = new HipAllocator(ordinal, dev->stream);
  static const char* names[4] = {"GPU forward memory", "GPU backward memory", "GPU parameter memory",
                                 "GPU scratch memory"};
  int st = DYHIP_OK;
  for (int i = 0; i < 4 && st == DYHIP_OK; ++i)
    st = pool_new(names[i], pool_mb[i] << 20, size_t(1) << 24, dev->alloc, false, &dev->pools[i]);
  if (st == DYHIP_OK) {
    dev->scalars = static_cast<float*>(dev->alloc->malloc(256));
    if (dev->scalars == nullptr) st = fail(DYHIP_ERR_OUT_OF_MEMORY, "failed to allocate the device scalars");
  }
  if (st == DYHIP_OK) {
    const float vals[3] = {-1.f, 1.f, 0.f};
    if (hipMemcpy(dev->scalars, vals, sizeof(vals), hipMemcpyHostToDevice) != hipSuccess)
      st = fail(DYHIP_ERR_RUNTIME, "failed to initialise the device scalars");
  }
  if (st == DYHIP_OK) {
    dev->rng_state = static_cast<uint64_t*>(dev->alloc->malloc(256));
    if (dev->rng_state == nullptr) st = fail(DYHIP_ERR_OUT_OF_MEMORY, "failed to allocate the random generator state");
  }
  if (st == DYHIP_OK) st = dyhip_reset_rng(dev, 0);
  if (st == DYHIP_OK) st = ln_static_scratch_setup(dev);  // this device is current (hipSetDevice above)
  if (st == DYHIP_OK) {
    dev->gemm_ws_bytes = size_t(128) << 20;
    dev->gemm_ws = dev->alloc->malloc(dev->gemm_ws_bytes + kGemmFlagWords * sizeof(unsigned));
    if (dev->gemm_ws == nullptr) st = fail(DYHIP_ERR_OUT_OF_MEMORY, "failed to allocate the GEMM split-K workspace");
    else st = gemm_flags_setup(dev);
  }
  if (st != DYHIP_OK) {
    dyhip_device_destroy(dev);
    return st;
  }
  *out = dev;
  return DYHIP_OK;
}

int dyhip_device_fork(dyhip_device* parent, dyhip_device** out) {
  DYHIP_CHECK_DEV(parent);
  DYHIP_REQUIRE(out != nullptr, "null output pointer");
  DYHIP_REQUIRE(parent->parent == nullptr, "fork the device itself, not one of its forked queues");
  DYHIP_CHECK_HIP(hipSetDevice(parent->ordinal));
  dyhip_device* dev = new dyhip_device(*parent);  // shares pools, scalars, allocator, thresholds
  dev->parent = parent;
  dev->sync_events.clear();
  dev->forks.clear();
  dev->sync_next = 0;
  dev->gemm_ws = nullptr;
  dev->rng_state = nullptr;
  hipError_t e = hipStreamCreateWithFlags(&dev->stream, hipStreamNonBlocking);
  if (e != hipSuccess) {
    delete dev;
    return fail(DYHIP_ERR_RUNTIME, "hipStreamCreateWithFlags failed: %s", hipGetErrorString(e));
  }
  (void)hipEventCreate(&dev->ev_start);
  (void)hipEventCreate(&dev->ev_stop);
  dev->gemm_flags = nullptr;
  dev->gemm_flags_used = false;
  dev->gemm_ws = parent->alloc->malloc(dev->gemm_ws_bytes + kGemmFlagWords * sizeof(unsigned));
  dev->rng_state = static_cast<uint64_t*>(parent->alloc->malloc(256));
  dev->rng_stream = ++parent->forks_made;
  if (dev->gemm_ws == nullptr || dev->rng_state == nullptr) {
    dyhip_device_destroy(dev);
    return fail(DYHIP_ERR_OUT_OF_MEMORY, "failed to allocate the workspace of the forked queue");
  }
  if (gemm_flags_setup(dev) != DYHIP_OK) {
    dyhip_device_destroy(dev);
    return DYHIP_ERR_RUNTIME;
  }
  // the queue draws from its own stream of the parent's generator (same key, own counter)
  hipError_t ce = hipMemcpy(dev->rng_state, parent->rng_state, 8, hipMemcpyDeviceToDevice);
  if (ce == hipSuccess) ce = hipMemset(dev->rng_state + 1, 0, 8);
  if (ce != hipSuccess) {
    dyhip_device_destroy(dev);
    return fail(DYHIP_ERR_RUNTIME, "failed to initialise the random generator of the forked queue");
  }
  parent->forks.push_back(dev);
  *out = dev;
  return DYHIP_OK;
}

int dyhip_device_wait(dyhip_device* dev, dyhip_device* other) {
  DYHIP_CHECK_DEV(dev);
  DYHIP_CHECK_DEV(other);
  DYHIP_REQUIRE(dev->ordinal == other->ordinal, "both queues must belong to the same GPU");
  if (dev == other) return DYHIP_OK;
  // a wait refers to the event's latest record at the time of the call, so a small ring of
  // events per queue serves any number of waits (eager or captured)
  constexpr size_t kRing = 16;
  if (other->sync_events.size() < kRing) {
    hipEvent_t fresh;
    DYHIP_CHECK_HIP(hipEventCreateWithFlags(&fresh, hipEventDisableTiming));
    other->sync_events.push_back(fresh);
    other->sync_next = other->sync_events.size() - 1;
  } else {
    other->sync_next = (other->sync_next + 1) % kRing;
  }
  hipEvent_t ev = other->sync_events[other->sync_next];
  DYHIP_CHECK_HIP(hipEventRecord(ev, other->stream));
  DYHIP_CHECK_HIP(hipStreamWaitEvent(dev->stream, ev, 0));
  return DYHIP_OK;
}

int dyhip_device_destroy(dyhip_device* dev) {
  DYHIP_CHECK_DEV(dev);
  (void)hipSetDevice(dev->ordinal);
  (void)hipStreamSynchronize(dev->stream);
  for (hipEvent_t ev : dev->sync_events) (void)hipEventDestroy(ev);
  if (dev->parent != nullptr) {  // a forked queue owns its stream, events and split-K workspace only
    auto& fl = dev->parent->forks;
    for (size_t i = 0; i < fl.size(); ++i)
      if (fl[i] == dev) {
        fl.erase(fl.begin() + i);
        break;
      }
    if (dev->gemm_ws) dev->alloc->free(dev->gemm_ws);
    if (dev->rng_state) dev->alloc->free(dev->rng_state);
    (void)hipEventDestroy(dev->ev_start);
    (void)hipEventDestroy(dev->ev_stop);
    (void)hipStreamDestroy(dev->stream);
    delete dev;
    return DYHIP_OK;
  }
  while (!dev->forks.empty()) dyhip_device_destroy(dev->forks.back());
  for (auto& p : dev->pools)
    if (p) pool_delete(p);
  if (dev->scalars) dev->alloc->free(dev->scalars);
  if (dev->rng_state) dev->alloc->free(dev->rng_state);
  if (dev->gemm_ws) dev->alloc->free(dev->gemm_ws);
  delete dev->alloc;
  (void)hipEventDestroy(dev->ev_start);
  (void)hipEventDestroy(dev->ev_stop);
  (void)hipStreamDestroy(dev->stream);
  delete dev;
  return DYHIP_OK;
}

int dyhip_device_sync(dyhip_device* dev) {
  DYHIP_CHECK_DEV(dev);
  DYHIP_CHECK_HIP(hipStreamSynchronize(dev->stream));
  return gemm_check_giveups(dev);
}

int dyhip_device_set_gemm_handoff(dyhip_device* dev, unsigned spin_limit, int raise_flags) {
  DYHIP_CHECK_DEV(dev);
  dev->gemm_spin_limit = spin_limit;
  dev->gemm_raise_flags = raise_flags ? 1 : 0;
  return DYHIP_OK;
}

int dyhip_device_ordinal(const dyhip_device* dev, int* ordinal) {
  DYHIP_CHECK_DEV(dev);
  DYHIP_REQUIRE(ordinal != nullptr, "null output pointer");
  *ordinal = dev->ordinal;
  return DYHIP_OK;
}

int dyhip_device_stream(dyhip_device* dev, void** hip_stream) {
  DYHIP_CHECK_DEV(dev);
  DYHIP_REQUIRE(hip_stream != nullptr, "null output pointer");
  *hip_stream = static_cast<void*>(dev->stream);
  return DYHIP_OK;
}

int dyhip_device_pool(dyhip_device* dev, int which, dyhip_pool** pool) {
  DYHIP_CHECK_DEV(dev);
  DYHIP_REQUIRE(pool != nullptr && which >= 0 && which < 4, "pool index %d out of range", which);
  *pool = dev->pools[which];
  return DYHIP_OK;
}

int dyhip_device_scalar(dyhip_device* dev, int which, const float** ptr) {
  DYHIP_CHECK_DEV(dev);
  DYHIP_REQUIRE(ptr != nullptr && which >= 0 && which < 3, "scalar index %d out of range", which);
  *ptr = dev->scalars + which;
  return DYHIP_OK;
}

int dyhip_device_set_stream_threshold(dyhip_device* dev, size_t bytes) {
  DYHIP_CHECK_DEV(dev);
  dev->stream_threshold = bytes;
  return DYHIP_OK;
}

int dyhip_device_allocate(dyhip_device* dev, int which_pool, size_t nbytes, void** out) {
  DYHIP_CHECK_DEV(dev);
  DYHIP_REQUIRE(which_pool >= 0 && which_pool < 4, "pool index %d out of range", which_pool);
  return dyhip_pool_allocate(dev->pools[which_pool], nbytes, out);
}

// ---------------------------------------------------------------------------
// copies
// ---------------------------------------------------------------------------
int dyhip_memcpy_h2d(dyhip_device* dev, void* dst, const void* src_host, size_t nbytes) {
  DYHIP_CHECK_DEV(dev);
  if (nbytes == 0) return DYHIP_OK;
  DYHIP_REQUIRE(dst != nullptr && src_host != nullptr, "null pointer in h2d copy");
  DYHIP_CHECK_HIP(hipMemcpyAsync(dst, src_host, nbytes, hipMemcpyHostToDevice, dev->stream));
  return DYHIP_OK;
}

int dyhip_host_alloc(size_t nbytes, void** out) {
  DYHIP_REQUIRE(out != nullptr && nbytes > 0, "null output pointer or empty allocation");
  void* p = nullptr;
  const hipError_t e = hipHostMalloc(&p, nbytes, hipHostMallocDefault);
  if (e != hipSuccess) return fail(DYHIP_ERR_OUT_OF_MEMORY, "hipHostMalloc(%zu) failed: %s", nbytes, hipGetErrorString(e));
  *out = p;
  return DYHIP_OK;
}

int dyhip_host_free(void* p) {
  if (p == nullptr) return DYHIP_OK;
  DYHIP_CHECK_HIP(hipHostFree(p));
  return DYHIP_OK;
}

int dyhip_memcpy_d2h(dyhip_device* dev, void* dst_host, const void* src, size_t nbytes) {
  DYHIP_CHECK_DEV(dev);
  if (nbytes == 0) return DYHIP_OK;
  DYHIP_REQUIRE(dst_host != nullptr && src != nullptr, "null pointer in d2h copy");
  DYHIP_CHECK_HIP(hipMemcpyAsync(dst_host, src, nbytes, hipMemcpyDeviceToHost, dev->stream));
  DYHIP_CHECK_HIP(hipStreamSynchronize(dev->stream));
  return gemm_check_giveups(dev);  // the bytes may be the output of a product that is incomplete
}

int dyhip_memcpy_d2d(dyhip_device* dev, void* dst, const void* src, size_t nbytes) {
  DYHIP_CHECK_DEV(dev);
  if (nbytes == 0) return DYHIP_OK;
  DYHIP_REQUIRE(dst != nullptr && src != nullptr, "null pointer in d2d copy");
  DYHIP_CHECK_HIP(hipMemcpyAsync(dst, src, nbytes, hipMemcpyDeviceToDevice, dev->stream));
  return DYHIP_OK;
}

int dyhip_zero(dyhip_device* dev, void* dst, size_t nbytes) {
  DYHIP_CHECK_DEV(dev);
  if (nbytes == 0) return DYHIP_OK;
  DYHIP_REQUIRE(dst != nullptr, "null pointer in zero");
  DYHIP_CHECK_HIP(zero_fill(dst, nbytes, dev->stream));
  return DYHIP_OK;
}

// ---------------------------------------------------------------------------
// HIP graphs
// ---------------------------------------------------------------------------
int dyhip_graph_begin_capture(dyhip_device* dev) {
  DYHIP_CHECK_DEV(dev);
  DYHIP_CHECK_HIP(hipStreamBeginCapture(dev->stream, hipStreamCaptureModeThreadLocal));
  return DYHIP_OK;
}

int dyhip_graph_end_capture(dyhip_device* dev, dyhip_graph** out) {
  DYHIP_CHECK_DEV(dev);
  DYHIP_REQUIRE(out != nullptr, "null output pointer");
  hipGraph_t graph = nullptr;
  DYHIP_CHECK_HIP(hipStreamEndCapture(dev->stream, &graph));
  hipGraphExec_t exec = nullptr;
  hipError_t e = hipGraphInstantiate(&exec, graph, nullptr, nullptr, 0);
  if (e != hipSuccess) {
    (void)hipGraphDestroy(graph);
    return fail(DYHIP_ERR_RUNTIME, "hipGraphInstantiate failed: %s", hipGetErrorString(e));
  }
  dyhip_graph* g = new dyhip_graph();
  g->graph = graph;
  g->exec = exec;
  *out = g;
  return DYHIP_OK;
}

int dyhip_graph_launch(dyhip_device* dev, dyhip_graph* graph) {
  DYHIP_CHECK_DEV(dev);
  DYHIP_REQUIRE(graph != nullptr, "null graph handle");
  DYHIP_CHECK_HIP(hipGraphLaunch(graph->exec, dev->stream));
  // a recorded large GEMM runs again with every replay, on this queue or on one forked from it: the next
  // synchronisation looks at their give-up counters
  if (dev->wide_gemm_ready != 0) dev->gemm_flags_used = true;
  for (dyhip_device* f : dev->forks)
    if (f->wide_gemm_ready != 0) f->gemm_flags_used = true;
  return DYHIP_OK;
}

int dyhip_graph_destroy(dyhip_graph* graph) {
  DYHIP_REQUIRE(graph != nullptr, "null graph handle");
  (void)hipGraphExecDestroy(graph->exec);
  (void)hipGraphDestroy(graph->graph);
  delete graph;
  return DYHIP_OK;
}

// ---------------------------------------------------------------------------
// timing
// ---------------------------------------------------------------------------
int dyhip_timer_start(dyhip_device* dev) {
  DYHIP_CHECK_DEV(dev);
  DYHIP_CHECK_HIP(hipEventRecord(dev->ev_start, dev->stream));
  return DYHIP_OK;
}

int dyhip_timer_stop(dyhip_device* dev, float* elapsed_ms) {
  DYHIP_CHECK_DEV(dev);
  DYHIP_REQUIRE(elapsed_ms != nullptr, "null output pointer");
  DYHIP_CHECK_HIP(hipEventRecord(dev->ev_stop, dev->stream));
  DYHIP_CHECK_HIP(hipEventSynchronize(dev->ev_stop));
  DYHIP_CHECK_HIP(hipEventElapsedTime(elapsed_ms, dev->ev_start, dev->ev_stop));
  return DYHIP_OK;
}

}  // extern "C"
