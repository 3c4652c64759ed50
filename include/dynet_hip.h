/*
 * dynet_hip.h -- C-ABI of libdynet_hip.so, the MI355X (gfx950) implementation
 * of the device layer and fused-layer kernels that sit behind DyNet's
 * Node::forward_dev_impl / backward_dev_impl<Device_GPU>.
 *
 * Conventions
 *  - Every entry point returns an int status (DYHIP_OK == 0), mirroring
 *    DYNET_C_STATUS / DYNET_C_OK of contrib/c/dynet_c/define.h:42-46; no C++
 *    exception crosses this boundary.  dyhip_last_error() gives the message of
 *    the last failure on the calling thread.
 *  - All tensors are fp32, column-major, batch outermost (dynet/dim.h:34-304):
 *    element (i, j, b) of a rows x cols tensor is v[i + j*rows + b*rows*cols].
 *    Indices are 32-bit unsigned.  Pointers are DEVICE pointers unless the
 *    parameter name ends in _host.
 *  - forward entry points overwrite their output; backward entry points
 *    ACCUMULATE (+=) into the gradient buffer, exactly like every
 *    backward_dev_impl (dynet/exec.cc:207-208 zeroes the buffers once).
 *  - Kernels never allocate.  Scratch is passed in as (ws, ws_bytes); the size
 *    needed comes from the matching *_workspace() query.  A DyNet adapter
 *    takes it from pools[SCS] as the reference's nodes do
 *    (dynet/nodes-lstm.cc:125,234).
 *  - Launches are asynchronous on the device's single in-order stream
 *    (the reference runs everything on the null stream, dynet/devices.cc:113);
 *    dyhip_device_sync() or a D2H copy synchronises.
 */
#ifndef DYNET_HIP_H
#define DYNET_HIP_H

#include <stddef.h>

#ifdef __cplusplus
extern "C" {
#endif

/* ---- status ------------------------------------------------------------- */
enum {
  DYHIP_OK = 0,
  DYHIP_ERR_INVALID_ARG = 1, /* std::invalid_argument in the reference (dynet/except.h:41-46) */
  DYHIP_ERR_RUNTIME = 2,     /* dynet::cuda_exception / std::runtime_error (dynet/cuda.h:20-52) */
  DYHIP_ERR_OUT_OF_MEMORY = 3, /* dynet::out_of_memory (dynet/except.h:11-14) */
  DYHIP_ERR_NO_DEVICE = 4
};
const char* dyhip_last_error(void);

/* ---- device: replaces Device_GPU (dynet/devices.h:46-61, devices.cc:91-121)
 * and initialize_gpu's enumeration (dynet/cuda.cc:15-100) ------------------ */
typedef struct dyhip_device dyhip_device;
typedef struct dyhip_pool dyhip_pool;

/* DeviceMempool (dynet/device-structs.h:15) */
enum { DYHIP_POOL_FXS = 0, DYHIP_POOL_DEDFS = 1, DYHIP_POOL_PS = 2, DYHIP_POOL_SCS = 3 };
/* the three device-resident scalars (dynet/devices.h:35-37, devices.cc:101-110) */
enum { DYHIP_SCALAR_MINUSONE = 0, DYHIP_SCALAR_ONE = 1, DYHIP_SCALAR_ZERO = 2 };

int dyhip_device_count(int* count);
/* pool_mb[4] = FXS, DEDFS, PS, SCS sizes in MiB (DeviceMempoolSizes, devices.cc:17-57) */
int dyhip_device_create(int ordinal, const size_t pool_mb[4], dyhip_device** out);
int dyhip_device_destroy(dyhip_device* dev);
/* Waits for everything queued on the device.  Also a point where a failure inside an earlier asynchronous launch
 * surfaces: DYHIP_ERR_RUNTIME if blocks of a large GEMM gave up waiting for each other's partial tiles (their bounded
 * wait, seconds long, ran out), in which case the products since the last synchronisation are incomplete.  Every
 * entry point that synchronises and hands device results to the host reports it the same way (dyhip_memcpy_d2h,
 * dyhip_lookup_plan_invalid_ids), for the queue itself and for the queues forked from it. */
int dyhip_device_sync(dyhip_device* dev);
/* The bounded wait of that hand-off: spin_limit polls (about a microsecond apart; default 1 << 22) before a block gives
 * up; raise_flags = 0 makes the producing blocks store their partial tiles without raising their flags, so that with
 * spin_limit = 0 every consumer gives up at once while every kernel still runs to its end: the host-driven test of
 * the error path.  Applies to products issued afterwards on this queue.  No counterpart in the reference. */
int dyhip_device_set_gemm_handoff(dyhip_device* dev, unsigned spin_limit, int raise_flags);
int dyhip_device_ordinal(const dyhip_device* dev, int* ordinal);
int dyhip_device_stream(dyhip_device* dev, void** hip_stream);
int dyhip_device_pool(dyhip_device* dev, int which, dyhip_pool** pool);
int dyhip_device_scalar(dyhip_device* dev, int which, const float** ptr);
/* A second in-order queue on the same GPU: shares the pools, scalars and settings of
 * `parent`, has its own HIP stream (default priority) and split-K workspace.  Work issued
 * on the two handles may overlap on the GPU; dyhip_device_wait orders it: everything
 * issued on `dev` afterwards runs after everything issued on `other` before the call.
 * Both calls are legal inside a graph capture begun on the parent (the forked queue joins
 * the capture with its first wait and must be waited for before the capture ends).
 * Destroy forked queues before their parent.  No counterpart in the reference, which
 * issues everything on the null stream. */
int dyhip_device_fork(dyhip_device* parent, dyhip_device** out);
int dyhip_device_wait(dyhip_device* dev, dyhip_device* other);
/* Tensors of at least this many bytes are streamed with non-temporal accesses
 * (default 8 MiB, twice the per-XCD L2); 0 streams everything, SIZE_MAX nothing.
 * A tuning knob with no counterpart in the reference. */
int dyhip_device_set_stream_threshold(dyhip_device* dev, size_t bytes);
/* Device::allocate_tensor (dynet/devices.cc:82-88) */
int dyhip_device_allocate(dyhip_device* dev, int which_pool, size_t nbytes, void** out);

/* ---- pools: AlignedMemoryPool / InternalMemoryPool
 * (dynet/aligned-mem-pool.h:11-69, aligned-mem-pool.cc:8-91) over GPUAllocator
 * (hipMalloc, 256-byte alignment; dynet/mem.h:41-47, mem.cc:71-90) or
 * CPUAllocator (32-byte alignment; dynet/mem.h:26-31) --------------------- */
int dyhip_pool_create_host(const char* name, size_t cap_bytes, size_t expanding_unit, dyhip_pool** out);
int dyhip_pool_destroy(dyhip_pool* pool);
int dyhip_pool_allocate(dyhip_pool* pool, size_t nbytes, void** out);
int dyhip_pool_free(dyhip_pool* pool);
int dyhip_pool_zero_allocated(dyhip_pool* pool);
int dyhip_pool_used(dyhip_pool* pool, size_t* used);
int dyhip_pool_set_used(dyhip_pool* pool, size_t used);
int dyhip_pool_capacity(dyhip_pool* pool, size_t* cap);
int dyhip_pool_num_blocks(dyhip_pool* pool, int* n);

/* ---- copies: TensorTools::set_elements / as_vector / copy_elements / zero
 * (dynet/tensor.cc:66-93,106-229) ----------------------------------------- */
int dyhip_memcpy_h2d(dyhip_device* dev, void* dst, const void* src_host, size_t nbytes);
int dyhip_memcpy_d2h(dyhip_device* dev, void* dst_host, const void* src, size_t nbytes); /* blocking */
/* Page-locked host staging memory.  dyhip_memcpy_h2d from such a buffer is asynchronous: the buffer
 * must stay untouched until the copy has run (dyhip_device_sync or any later blocking call).  The
 * reference stages ids and pointer tables from pageable memory (dynet/param-nodes.cc:318,
 * dynet/exec.cc:351-355), which makes every such copy a synchronisation point. */
int dyhip_host_alloc(size_t nbytes, void** out);
int dyhip_host_free(void* p);
int dyhip_memcpy_d2d(dyhip_device* dev, void* dst, const void* src, size_t nbytes);
int dyhip_zero(dyhip_device* dev, void* dst, size_t nbytes);
int dyhip_constant(dyhip_device* dev, size_t n, float value, float* dst);       /* TensorTools::constant */
int dyhip_accumulate(dyhip_device* dev, size_t n, const float* src, float* dst); /* TensorTools::accumulate: dst += src */

/* Launch-bound inner loops: record the launches issued on the device stream
 * between begin and end into a HIP graph and replay it with one call.  The
 * reference has no counterpart (it launches node by node on the null stream);
 * entry points that copy from host memory or synchronise (those taking *_host
 * ids/labels) must stay outside a capture. */
typedef struct dyhip_graph dyhip_graph;
int dyhip_graph_begin_capture(dyhip_device* dev);
int dyhip_graph_end_capture(dyhip_device* dev, dyhip_graph** out);
int dyhip_graph_launch(dyhip_device* dev, dyhip_graph* graph);
int dyhip_graph_destroy(dyhip_graph* graph);

/* stream-ordered timing for benchmarks (hipEvent pair on the device stream) */
int dyhip_timer_start(dyhip_device* dev);
int dyhip_timer_stop(dyhip_device* dev, float* elapsed_ms); /* blocks until the stop event */

/* ---- elementwise nodes -------------------------------------------------- */
/* operator codes */
enum {
  DYHIP_OP_TANH = 0,     /* Tanh            dynet/nodes-trig.cc:312-326 */
  DYHIP_OP_LOGISTIC = 1, /* LogisticSigmoid dynet/nodes-activations.cc:65-78 */
  DYHIP_OP_RECTIFY = 2,  /* Rectify         dynet/nodes-activations.cc:31-44 */
  DYHIP_OP_NEGATE = 3,   /* Negate          dynet/nodes-arith-unary.cc:195-209 */
  DYHIP_OP_IDENTITY = 4
};
/* which form of scalar_logistic_sigmoid_op (dynet/simd-functors.h:74-126) */
enum {
  DYHIP_LOGISTIC_PACKET = 0, /* packetOp: clamp +-18 + rational polynomial (what the CPU path runs on full SIMD packets) */
  DYHIP_LOGISTIC_SCALAR = 1  /* operator(): 1/(1+exp(-x)) */
};
int dyhip_unary_forward(dyhip_device* dev, int op, int logistic_mode, size_t n, const float* x, float* y);
int dyhip_unary_backward(dyhip_device* dev, int op, size_t n, const float* fx, const float* dEdf, float* dEdx);

/* CwiseMultiply (dynet/nodes-arith-cwise.cc:196-307) and CwiseSum (:50-156) for
 * equal dims; n = elements per batch element, bd0/bd1 = batch counts (equal,
 * or one of them 1).  backward: i selects the argument. */
int dyhip_cmult_forward(dyhip_device* dev, size_t n, unsigned bd0, unsigned bd1, const float* a, const float* b, float* y);
int dyhip_cmult_backward(dyhip_device* dev, size_t n, unsigned bd0, unsigned bd1, const float* a, const float* b,
                         const float* dEdf, unsigned i, float* dEdxi, void* ws, size_t ws_bytes);
int dyhip_csum_forward(dyhip_device* dev, size_t n, unsigned bd0, unsigned bd1, const float* a, const float* b, float* y);
int dyhip_csum_backward(dyhip_device* dev, size_t n, unsigned bd0, unsigned bd1, const float* dEdf, unsigned i,
                        float* dEdxi, void* ws, size_t ws_bytes);

/* PickRange (dynet/nodes-select.cc:230-259): fx = x sliced to [start, end) along one dimension.
 * The tensor is described as inner x len x outer, column-major: inner = product of the dimensions
 * before the sliced one, len = its size, outer = product of the later ones times the batch size.
 * Forward copies (bit-exact); backward accumulates dEdf into the slice of dEdxi (:258). */
int dyhip_pick_range_forward(dyhip_device* dev, size_t inner, size_t len, size_t outer, size_t start, size_t end,
                             const float* x, float* fx);
int dyhip_pick_range_backward(dyhip_device* dev, size_t inner, size_t len, size_t outer, size_t start, size_t end,
                              const float* dEdf, float* dEdxi);

/* Sum node / esum (dynet/nodes-arith-sum.cc:65-129): fx = sum of k same-shaped arguments whose batch
 * size is bd or 1 (broadcast), added in the reference's association order (groups of four).  xs_host
 * and bds_host are HOST arrays.  Backward per argument is dyhip_csum_backward (dx_i += dEdf, summed
 * over the batch for a batch-1 argument, :115-128). */
int dyhip_sum_forward(dyhip_device* dev, unsigned k, size_t n, unsigned bd, const float* const* xs_host,
                      const unsigned* bds_host, float* fx);

/* ---- reductions --------------------------------------------------------- */
/* workspace for every batch reduction of an n x bd tensor (sum_batches fwd,
 * the broadcast-argument backward of cmult/csum) */
int dyhip_batch_reduce_workspace(size_t n, unsigned bd, size_t* ws_bytes);
/* ---- CwiseSum / CwiseMultiply / CwiseQuotient with broadcast over dimensions as well as the batch
 * (dynet/nodes-arith-cwise.cc:50-156, :196-307, :338-421, backward_helper included) and the constant
 * nodes of dynet/nodes-arith-const.cc:33-75.  A tensor is dims[5] = {d0, d1, d2, d3, bd}, column-major,
 * batch outermost, missing dimensions 1; on every axis the two arguments agree or one of them is 1
 * (CwiseQuotient: only the right one); the result takes the larger.  backward accumulates into dEdxi
 * (argument i's own shape), summing over the axes it was broadcast over:
 *   sum: dEdf    multiply: dEdf * other    quotient: i = 0: dEdf / b, i = 1: -(dEdf / (b*b) * a).
 * The batch-only cases are the streaming kernels of dyhip_csum_* / dyhip_cmult_*. ------------------- */
#define DYHIP_CWISE_SUM 0
#define DYHIP_CWISE_MULT 1
#define DYHIP_CWISE_QUOTIENT 2
int dyhip_cwise_forward(dyhip_device* dev, int op, const unsigned* dims_a, const unsigned* dims_b, const float* a,
                        const float* b, float* fx);
int dyhip_cwise_backward_workspace(const unsigned* dims_a, const unsigned* dims_b, unsigned i, size_t* ws_bytes);
int dyhip_cwise_backward(dyhip_device* dev, int op, const unsigned* dims_a, const unsigned* dims_b, const float* a,
                         const float* b, const float* dEdf, unsigned i, float* dEdxi, void* ws, size_t ws_bytes);
/* ConstantPlusX: fx = c + x, backward dEdx += dEdf (dyhip_accumulate); ConstantMinusX: fx = c - x, backward
 * dEdx -= dEdf (dyhip_unary_backward with DYHIP_OP_NEGATE). */
int dyhip_const_plus_x_forward(dyhip_device* dev, size_t n, float c, const float* x, float* fx);
int dyhip_const_minus_x_forward(dyhip_device* dev, size_t n, float c, const float* x, float* fx);

/* SumDimension({}, include_batch_dim) = sum_batches (dynet/nodes-arith-sum.cc:197-248, expr.cc:218) */
int dyhip_sum_batches_forward(dyhip_device* dev, size_t n, unsigned bd, const float* x, float* y, void* ws, size_t ws_bytes);
int dyhip_sum_batches_backward(dyhip_device* dev, size_t n, unsigned bd, const float* dEdf, float* dEdx);
/* mean_elems / std_elems (dynet/expr.cc:229-238; MomentDimension nodes-moments.cc:181-309,
 * StdDimension :434-555): one value per batch element over its n elements */
int dyhip_mean_elems_forward(dyhip_device* dev, size_t n, unsigned bd, const float* x, float* y);
int dyhip_mean_elems_backward(dyhip_device* dev, size_t n, unsigned bd, const float* dEdf, float* dEdx);
int dyhip_std_elems_forward(dyhip_device* dev, size_t n, unsigned bd, const float* x, float* y);
int dyhip_std_elems_backward(dyhip_device* dev, size_t n, unsigned bd, const float* x, const float* fx,
                             const float* dEdf, float* dEdx);

/* ---- fused LayerNorm: the 8-node composite of dynet/expr.cc:248-253 in one
 * kernel each way.  y = g * (x - mean) / (std + 1e-8f) + b per batch element.
 * backward accumulates dx[n*bd], dg[n], db[n]; any of them may be NULL. ---- */
int dyhip_layer_norm_forward(dyhip_device* dev, size_t n, unsigned bd, const float* x, const float* g,
                             const float* b, float* y);
int dyhip_layer_norm_backward_workspace(size_t n, unsigned bd, size_t* ws_bytes);
int dyhip_layer_norm_backward(dyhip_device* dev, size_t n, unsigned bd, const float* x, const float* g,
                              const float* dEdf, float* dx, float* dg, float* db, void* ws, size_t ws_bytes);
/* The same without a workspace argument, for callers that cannot allocate or carry one: code under HIP
 * graph capture, tight serving loops, harnesses that forbid hipMalloc.  It has no counterpart in the
 * reference (whose nodes take scratch from pools[SCS]).  The scratch is a static device array of
 * DYHIP_LN_STATIC_SCRATCH_BYTES that each GPU holds until the process ends; the call allocates nothing and
 * fails with DYHIP_ERR_INVALID_ARG when the scratch that this call's path needs exceeds that size: nothing when
 * dg and db are both NULL; rows of up to 2048 floats, a multiple of 4, 16-byte aligned: at most 256 partial
 * rows of dg and db, any bd; such rows of up to 16384 floats: the same, so n = 4096 fits up to 128 blocks of
 * rows; any other row: 8 bytes per row of the batch plus up to 64 partial rows of dg and db (never more than
 * dyhip_layer_norm_backward_workspace(n, bd)).  All calls on one GPU share the array:
 * calls that overlap on one GPU (two queues, two threads) race; calls on one queue are ordered. */
#define DYHIP_LN_STATIC_SCRATCH_BYTES (4u << 20)
int dyhip_layer_norm_backward_static(dyhip_device* dev, size_t n, unsigned bd, const float* x, const float* g,
                                     const float* dEdf, float* dx, float* dg, float* db);

/* ---- GEMM shim: dynet/matrix-multiply.h, fp32 in / fp32 accumulate on MFMA.
 * The device-pointer acc_scalar of the reference (kSCALAR_ONE / kSCALAR_ZERO)
 * becomes the by-value beta. ---------------------------------------------- */
/* MatrixMultiply (:16-37): y[MxN] = beta*y + l[MxK] * r[KxN] */
int dyhip_gemm_nn(dyhip_device* dev, size_t M, size_t N, size_t K, const float* l, const float* r, float beta, float* y);
/* MatrixTranspMultiplyAcc (:97-117): y[MxN] += l[KxM]^T * r[KxN] */
int dyhip_gemm_tn_acc(dyhip_device* dev, size_t M, size_t N, size_t K, const float* l, const float* r, float* y);
/* MatrixMultiplyTranspAcc (:162-180): y[MxN] += l[MxK] * r[NxK]^T */
int dyhip_gemm_nt_acc(dyhip_device* dev, size_t M, size_t N, size_t K, const float* l, const float* r, float* y);
/* Which kernel the three calls above take for a problem with packed leading dimensions and 16-byte aligned
 * operands: *wide_tiles = 1 when the 256 x 256-tile kernel takes the whole product (large outputs with enough
 * depth per CU), 2 when it takes the leading columns that form full rounds of one tile per CU and the rest runs
 * as a product of its own, 0 for the 128-wide kernel or the fragment-order product.  trans_l / trans_r as in
 * dyhip_gemm_strided_batched.  No counterpart in the reference (cuBLAS picks its kernels silently); for tests
 * and tuning. */
int dyhip_gemm_uses_wide_tiles(dyhip_device* dev, int trans_l, int trans_r, size_t M, size_t N, size_t K, int* wide_tiles);
/* How the 256 x 256-tile kernel deals an M x N x K product (K rounded down to a multiple of 32) to `segments`
 * blocks: starts[s], s = 0..segments, is the first k-tile of block segment s in the sequence of all k-tiles of all
 * tiles (tile by tile, k ascending; starts[segments] = their number), *k_tiles_per_tile the k-tiles of one tile, and
 * *finish_in_kernel whether a tile cut by a segment boundary is finished inside the kernel (by the block that holds its
 * first k-tiles, from the partial tiles of the blocks that hold the rest) or by a second kernel.  Needs no device.
 * No counterpart in the reference; for tests of the hand-off's invariants. */
int dyhip_gemm_wide_segments(size_t M, size_t N, size_t K, unsigned segments, unsigned* starts,
                             unsigned* k_tiles_per_tile, int* finish_in_kernel);
/* The cublasSgemmStridedBatched branches of the three shims (dynet/matrix-multiply.h:27-34, 110-117,
 * 175-182), taken when the left operand is batched: for b in [0, batch)
 *   y_b[MxN] = beta*y_b + op(l_b) * op(r_b),   x_b = x + b*stride_x (strides in floats),
 * with op = transpose where trans_l / trans_r is non-zero (not both) and the operand shapes of the
 * three calls above.  A stride of 0 shares an operand between the items, as the reference passes for
 * an operand whose batch size is 1; stride_y must be at least M*N.  One launch for all items. */
int dyhip_gemm_strided_batched(dyhip_device* dev, int trans_l, int trans_r, size_t M, size_t N, size_t K,
                               const float* l, size_t stride_l, const float* r, size_t stride_r, float beta, float* y,
                               size_t stride_y, unsigned batch);
/* the two transposed forms with an explicit beta (beta = 0 overwrites y, which saves zeroing a
 * gradient buffer that has a single producer); the cublasSgemm calls behind
 * dynet/matrix-multiply.h:104-113,169-178 take the same scalar */
int dyhip_gemm_tn(dyhip_device* dev, size_t M, size_t N, size_t K, const float* l, const float* r, float beta, float* y);
int dyhip_gemm_nt(dyhip_device* dev, size_t M, size_t N, size_t K, const float* l, const float* r, float beta, float* y);

/* AffineTransform with one (W, x) pair (dynet/nodes-affinetransform.cc:77-113):
 * fx[MxN] = bias[M] broadcast over the N columns + W[MxK] * x[KxN], the bias folded into
 * the GEMM epilogue.  Its backward (:115-156) is dyhip_sum_batches_forward-style reduction
 * for the bias (dyhip_csum_backward), dyhip_gemm_nt_acc for W and dyhip_gemm_tn_acc for x. */
int dyhip_affine_forward(dyhip_device* dev, size_t M, size_t N, size_t K, const float* bias, const float* W,
                         const float* x, float* fx);

/* ---- fused LSTM nodes (dynet/nodes-lstm.cc) ------------------------------ */
/* VanillaLSTMGates::forward_dev_impl (:101-235).  xs[k] (HOST array of DEVICE
 * pointers) has x_dims[k] rows and B columns; mask_x/mask_h NULL = no dropout,
 * else their batch counts are B or 1.  Gate order i, f, o, g; +1 forget bias
 * is applied inside.  Workspace is only needed for num_inputs > 1 or dropout. */
int dyhip_lstm_gates_workspace(unsigned num_inputs, unsigned I, unsigned H, unsigned B, int dropout, size_t* ws_bytes);
int dyhip_lstm_gates_forward(dyhip_device* dev, unsigned num_inputs, const float* const* xs_host,
                             const unsigned* x_dims_host, unsigned H, unsigned B, const float* h_tm1,
                             const float* Wx, const float* Wh, const float* b, const float* mask_x,
                             unsigned mask_x_bd, const float* mask_h, unsigned mask_h_bd, int logistic_mode,
                             float* fx, void* ws, size_t ws_bytes);
/* dpre = [dEdf*fx*(1-fx) rows 0..3H ; dEdf*(1-fx^2) rows 3H..4H] (:358-361), computed once */
int dyhip_lstm_gates_dpre(dyhip_device* dev, unsigned H, unsigned B, const float* fx, const float* dEdf, float* dpre);
/* VanillaLSTMGates::backward_dev_impl (:237-527) for argument i (inputs, then
 * h, Wx, Wh, b).  dpre may be NULL: it is then recomputed into the workspace,
 * as the reference does on each of its five calls. */
int dyhip_lstm_gates_backward_workspace(unsigned num_inputs, unsigned I, unsigned H, unsigned B, int dropout, size_t* ws_bytes);
int dyhip_lstm_gates_backward(dyhip_device* dev, unsigned num_inputs, const float* const* xs_host,
                              const unsigned* x_dims_host, unsigned H, unsigned B, const float* h_tm1,
                              const float* Wx, const float* Wh, const float* mask_x, unsigned mask_x_bd,
                              const float* mask_h, unsigned mask_h_bd, const float* fx, const float* dEdf,
                              const float* dpre, unsigned i, float* dEdxi, void* ws, size_t ws_bytes);
/* VanillaLSTMC (:562-615) and VanillaLSTMH (:650-703) */
int dyhip_lstm_c_forward(dyhip_device* dev, unsigned H, unsigned B, const float* c_tm1, const float* gates, float* c);
int dyhip_lstm_c_backward(dyhip_device* dev, unsigned H, unsigned B, const float* c_tm1, const float* gates,
                          const float* dEdf, unsigned i, float* dEdxi);
int dyhip_lstm_h_forward(dyhip_device* dev, unsigned H, unsigned B, const float* c, const float* gates, float* h);
int dyhip_lstm_h_backward(dyhip_device* dev, unsigned H, unsigned B, const float* c, const float* gates,
                          const float* dEdf, unsigned i, float* dEdxi);

/* ---- fused cell step: VanillaLSTMGates + VanillaLSTMC + VanillaLSTMH of one timestep
 * (dynet/nodes-lstm.cc:101-235,562-615,650-703 forward; :237-527,591-615,670-703 backward)
 * around one recurrent GEMM.  The input projection xproj = Wx * x is formed for all
 * timesteps at once (dyhip_gemm_nn over T*B columns); a timestep is then
 *   dyhip_lstm_recurrent_forward : Wh * h_tm1 as unreduced split-K slices in ws
 *   dyhip_lstm_cell_forward      : gates = act(b + [f: +1] + xproj + sum of slices),
 *                                  c = i*g + f*c_tm1, h = o*tanh(c)
 * and backwards, newest timestep first,
 *   dyhip_lstm_cell_backward     : dh_t = dh + sum of the slices left by the t+1 call below;
 *                                  writes dpre_t (4H x B, gradient of the pre-activations)
 *                                  and dc_tm1
 *   dyhip_lstm_recurrent_backward: Wh^T * dpre_t as slices for the t-1 call.
 * Weight gradients are then GEMMs over all timesteps (dyhip_gemm_nt with K = T*B), dx is
 * dyhip_gemm_tn(Wx, dpre) and db a batch reduction of dpre.  These two-call entry points take
 * no dropout masks (a caller applies the builder's masks around them: h_tm1 (.) mask_h before
 * dyhip_lstm_recurrent_forward, the product of dyhip_gemm_tn(Wh, dpre) times mask_h into dh;
 * the one-launch timesteps further down take the recurrent mask as an argument).  gates may alias xproj (each element is read before it is written).  rec/splits
 * = NULL/0 and c_tm1 = NULL stand for the zero initial state (dynet/lstm.cc:1060-1061);
 * dc = NULL for the last timestep, dc_tm1 = NULL for the first. */
int dyhip_lstm_cell_workspace(dyhip_device* dev, unsigned H, unsigned B, size_t* fwd_bytes, size_t* bwd_bytes);
int dyhip_lstm_recurrent_forward(dyhip_device* dev, unsigned H, unsigned B, const float* Wh, const float* h_tm1,
                                 void* ws, size_t ws_bytes, unsigned* splits);
int dyhip_lstm_cell_forward(dyhip_device* dev, unsigned H, unsigned B, const float* xproj, const float* b,
                            const float* rec, unsigned splits, const float* c_tm1, int logistic_mode, float* gates,
                            float* c, float* h);
int dyhip_lstm_recurrent_backward(dyhip_device* dev, unsigned H, unsigned B, const float* Wh, const float* dpre,
                                  void* ws, size_t ws_bytes, unsigned* splits);
int dyhip_lstm_cell_backward(dyhip_device* dev, unsigned H, unsigned B, const float* gates, const float* c,
                             const float* c_tm1, const float* dh, const float* rec, unsigned splits, const float* dc,
                             float* dpre, float* dc_tm1);

/* Single-launch form of a forward timestep: the recurrent product Wh * h_tm1 and the cell update of
 * dyhip_lstm_cell_forward in one kernel, the product staying on chip.  A block owns 16 hidden units,
 * i.e. the gate rows j, H+j, 2H+j, 3H+j of the slicing in dynet/nodes-lstm.cc:213-223, and reads both
 * operands in matrix-core fragment order: the weights from a packed copy of Wh (4*H*H floats; refresh
 * it with dyhip_lstm_pack_recurrent whenever Wh changes), the state from a packed copy of h_tm1
 * (dyhip_lstm_packed_state_floats(H, B) floats).  Supported when H is a multiple of 128
 * (dyhip_lstm_step_supported reports it; the two-call form above covers every other size).  Same
 * results as the two-call form up to fp32 summation order.  gates may alias xproj.
 *   dyhip_lstm_step_forward         h_tm1 plain (H x B): for single timesteps
 *   dyhip_lstm_step_forward_packed  h_tm1 packed; also writes h_packed (may be null), the packed copy of
 *                                   the new h, so a chain of timesteps never repacks; packed_Wh =
 *                                   h_tm1_packed = c_tm1 = NULL stand for the zero initial state
 *   dyhip_lstm_pack_state           packs a rows x B state that did not come from a step (a non-zero h_0) */
int dyhip_lstm_step_supported(dyhip_device* dev, unsigned H, unsigned B, int* supported);
int dyhip_lstm_pack_recurrent(dyhip_device* dev, unsigned H, const float* Wh, float* packed);
int dyhip_lstm_packed_state_floats(unsigned rows, unsigned B, size_t* floats);
int dyhip_lstm_pack_state(dyhip_device* dev, unsigned rows, unsigned B, const float* v, float* packed);
int dyhip_lstm_step_forward(dyhip_device* dev, unsigned H, unsigned B, const float* packed_Wh, const float* h_tm1,
                            const float* xproj, const float* b, const float* c_tm1, int logistic_mode, float* gates,
                            float* c, float* h);
int dyhip_lstm_step_forward_packed(dyhip_device* dev, unsigned H, unsigned B, const float* packed_Wh,
                                   const float* h_tm1_packed, const float* xproj, const float* b, const float* c_tm1,
                                   int logistic_mode, float* gates, float* c, float* h, float* h_packed);
/* The backward timestep over the same packed operands: dyhip_lstm_recurrent_backward_packed forms the
 * slices of Wh^T * dpre (what dyhip_lstm_recurrent_backward does) from a packed copy of Wh^T
 * (dyhip_lstm_pack_recurrent_transposed, 4*H*H floats) and the packed dpre of the timestep above
 * (dyhip_lstm_packed_state_floats(4*H, B) floats), which dyhip_lstm_cell_backward_packed writes next to
 * the plain dpre.  ws holds the slices (the bwd_bytes of dyhip_lstm_cell_workspace suffice). */
int dyhip_lstm_pack_recurrent_transposed(dyhip_device* dev, unsigned H, const float* Wh, float* packed);
int dyhip_lstm_recurrent_backward_packed(dyhip_device* dev, unsigned H, unsigned B, const float* packed_WhT,
                                         const float* dpre_packed, void* ws, size_t ws_bytes, unsigned* splits);
int dyhip_lstm_cell_backward_packed(dyhip_device* dev, unsigned H, unsigned B, const float* gates, const float* c,
                                    const float* c_tm1, const float* dh, const float* rec, unsigned splits,
                                    const float* dc, float* dpre, float* dc_tm1, float* dpre_packed);
/* The backward timestep in ONE launch (the mirror of dyhip_lstm_step_forward_packed; no counterpart in the
 * reference, whose backward is the three nodes' backward_dev_impl, dynet/nodes-lstm.cc:238-372,605-614,684-701):
 *   dh_t  = dh + Wh^T * dpre_{t+1}                       (the product over its whole depth 4H, inside the kernel)
 *   dpre_t, dc_tm1 = cell backward(gates_t, c_t, c_tm1, dh_t, dc)   (the formulas of dyhip_lstm_cell_backward)
 * Wh^T and dpre_{t+1} are read in the fragment order of the 16x16x4 matrix-core instruction:
 * dyhip_lstm_pack_recurrent_transposed16 packs Wh (4*H*H floats, once per weight update); the kernel itself writes
 * dpre_t in that order to dpre_packed16 (dyhip_lstm_packed_state16_floats(4*H, B) floats) for the launch of
 * timestep t-1, next to the plain dpre (4H x B) that the weight-gradient products over all timesteps read.
 * dpre_next_packed16 null: the last timestep, no recurrent term; c_tm1, dc, dc_tm1, dpre_packed16 may be null
 * as in dyhip_lstm_cell_backward.  dyhip_lstm_pack_state16 packs a 4H x B dpre that did not come from a launch of
 * this kernel.  Sizes as dyhip_lstm_step_supported says. */
int dyhip_lstm_pack_recurrent_transposed16(dyhip_device* dev, unsigned H, const float* Wh, float* packed);
int dyhip_lstm_packed_state16_floats(unsigned rows, unsigned B, size_t* floats);
int dyhip_lstm_pack_state16(dyhip_device* dev, unsigned rows, unsigned B, const float* v, float* packed);
int dyhip_lstm_step_backward_packed(dyhip_device* dev, unsigned H, unsigned B, const float* packed_WhT16,
                                    const float* dpre_next_packed16, const float* gates, const float* c,
                                    const float* c_tm1, const float* dh, const float* dc, float* dpre, float* dc_tm1,
                                    float* dpre_packed16);
/* The two single-launch timesteps with the recurrent dropout mask of CompactVanillaLSTMBuilder (dynet/lstm.cc:964-982:
 * one mask per layer and sequence, H x B, already scaled by 1 / retention; the node applies it as h_tm1 (.) mask_h,
 * dynet/nodes-lstm.cc:178-198, and hands the gradient back through it, :448-470).  Forward: h is written plain,
 * h_packed = h (.) mask_h, which is what the next timestep multiplies Wh by.  Backward: dh_t = dh + (Wh^T * dpre_{t+1})
 * (.) mask_h.  mask_h = NULL: the calls above.  The input mask is applied by the caller to x before the product over
 * all timesteps (dyhip_cmult_forward with the mask as the batch-1 argument) and to dx after it. */
int dyhip_lstm_step_forward_packed_dropout(dyhip_device* dev, unsigned H, unsigned B, const float* packed_Wh,
                                           const float* h_tm1_packed, const float* xproj, const float* b,
                                           const float* c_tm1, const float* mask_h, int logistic_mode, float* gates,
                                           float* c, float* h, float* h_packed);
int dyhip_lstm_step_backward_packed_dropout(dyhip_device* dev, unsigned H, unsigned B, const float* packed_WhT16,
                                            const float* dpre_next_packed16, const float* gates, const float* c,
                                            const float* c_tm1, const float* dh, const float* dc, const float* mask_h,
                                            float* dpre, float* dc_tm1, float* dpre_packed16);
/* The whole forward of a timestep in one launch, input product included: gates = act(b + [f: +1] +
 * Wx * x + Wh * h_tm1) from packed copies of both weight matrices (dyhip_lstm_pack_input: Wx is
 * 4H x I, I a multiple of 128), then c and h; x and h_tm1 are plain.  For callers
 * that see one timestep at a time (decoding, the single-step configuration).  packed_Wh / h_tm1 /
 * c_tm1 = NULL stand for the zero initial state. */
int dyhip_lstm_pack_input(dyhip_device* dev, unsigned I, unsigned H, const float* Wx, float* packed);
int dyhip_lstm_step_forward_x(dyhip_device* dev, unsigned I, unsigned H, unsigned B, const float* packed_Wx,
                              const float* x, const float* packed_Wh, const float* h_tm1, const float* b,
                              const float* c_tm1, int logistic_mode, float* gates, float* c, float* h);

/* ---- random tensors: TensorTools::randomize_{uniform,normal,bernoulli}
 * (dynet/tensor.cc:261-303), Device_GPU::reset_rng (dynet/devices.cc:130-135), the Dropout
 * node (dynet/nodes-dropout.cc:32-47); RandomUniform/Normal/Bernoulli nodes
 * (dynet/nodes-random.cc:68-137) and the LSTM builders' dropout masks
 * (dynet/lstm.cc:964-982) are single calls of the randomize functions. ----------------
 * Generator: Philox4x32-10 (the generator the reference asks cuRAND for), key = seed + 1.
 * Element k of a call is word k % 4 of Philox(counter {lo, hi, queue, 0}, key {key, 0})
 * with block number hi:lo = position + k / 4; afterwards position += ceil(n / 4).  Key and
 * position live in device memory (a captured graph draws fresh numbers on every replay);
 * every forked queue has its own position and queue number, so queues never share numbers.
 * u = word * 2^-32 + 2^-33 in (0, 1]; uniform = u * (right - left) + left; bernoulli =
 * floor(u + p) * scale; normal = Box-Muller on word pairs (sin, cos) * stddev + mean.
 * The order in which cuRAND hands out its Philox words is not reproduced. */
int dyhip_reset_rng(dyhip_device* dev, unsigned seed);
int dyhip_rng_state(dyhip_device* dev, unsigned long long* key, unsigned long long* position, unsigned* queue);
int dyhip_rng_set_position(dyhip_device* dev, unsigned long long position);
int dyhip_randomize_uniform(dyhip_device* dev, size_t n, float left, float right, float* out);
int dyhip_randomize_bernoulli(dyhip_device* dev, size_t n, float p, float scale, float* out);
int dyhip_randomize_normal(dyhip_device* dev, size_t n, float mean, float stddev, float* out);
/* fx = x (.) m with m = bernoulli(1 - p) / (1 - p) written to mask (the node's aux_mem,
 * n floats); backward: dEdxi += dEdf (.) mask. */
int dyhip_dropout_forward(dyhip_device* dev, size_t n, float p, const float* x, float* mask, float* fx);
int dyhip_dropout_backward(dyhip_device* dev, size_t n, const float* mask, const float* dEdf, float* dEdxi);

/* ---- LookupNode (dynet/param-nodes.cc:304-329) and
 * LookupParameterStorage::accumulate_grads (dynet/model.cc:728-743) -------- */
/* fx[:, b] = table[:, ids[b]] * mult; bit-exact gather when mult == 1.0f.
 * ids_host (may be NULL) is bounds-checked against vocab like the CPU path
 * (:323) and copied to ids_dev (the node's aux_mem, :318). */
int dyhip_lookup_forward(dyhip_device* dev, unsigned n_ids, const unsigned* ids_host, unsigned* ids_dev,
                         size_t dim, unsigned vocab, const float* table, float mult, float* fx);
/* all_grads[:, ids[b]] += g[:, b] without float atomics: the ids are grouped by value (the "plan") and one
 * kernel sums each run of equal ids.  Deterministic; a row that fewer than 15 ids name is summed in
 * ascending b starting from its old value, i.e. bit-identical to the CPU path (:735-741); a row named
 * more often is summed by several thread groups (entries interleaved over a fixed number of slots, slots
 * added in ascending order).  ids >= vocab are skipped (the reference throws on the host,
 * dynet/param-nodes.cc:323, and does not check device-resident ids); dyhip_lookup_plan_invalid_ids
 * tells how many there were. */
int dyhip_lookup_accumulate_grads_workspace(unsigned n_ids, size_t dim, unsigned vocab, size_t* ws_bytes);
/* The same in two phases.  The plan depends only on the ids, so an executor can build it right after the
 * forward gather (the ids sit in the node's aux_mem from then on) and the backward pass is left with the
 * reduction kernel.  Up to 65535 ids the plan is built by one kernel; beyond that by a radix sort over
 * all blocks (three launches per 8 bits of the vocabulary size) and one kernel for the run ends.  The plan is opaque; vocab must be below 2^31 - 1.  dyhip_lookup_accumulate_grads_planned takes no
 * workspace any more (its size query returns 0; ws may be NULL). */
int dyhip_lookup_plan_bytes(unsigned n_ids, size_t* plan_bytes);
int dyhip_lookup_plan_workspace(unsigned n_ids, unsigned vocab, size_t* ws_bytes);
int dyhip_lookup_build_plan(dyhip_device* dev, unsigned n_ids, const unsigned* ids_dev, unsigned vocab, void* plan,
                            size_t plan_bytes, void* ws, size_t ws_bytes);
int dyhip_lookup_plan_invalid_ids(dyhip_device* dev, unsigned n_ids, const void* plan, unsigned* count);
int dyhip_lookup_accumulate_grads_planned_workspace(unsigned n_ids, size_t dim, size_t* ws_bytes);
int dyhip_lookup_accumulate_grads_planned(dyhip_device* dev, unsigned n_ids, const void* plan, size_t dim,
                                          unsigned vocab, const float* g, float* all_grads, void* ws, size_t ws_bytes);
int dyhip_lookup_accumulate_grads(dyhip_device* dev, unsigned n_ids, const unsigned* ids_dev, size_t dim,
                                  unsigned vocab, const float* g, float* all_grads, void* ws, size_t ws_bytes);

/* ---- logsumexp / PickNegLogSoftmax / LogSumExp / argmax ------------------ */
/* TensorTools::logsumexp_dev (dynet/tensor.cc:468-507), vector per batch element */
int dyhip_logsumexp_cols(dyhip_device* dev, size_t rows, unsigned bd, const float* x, float* m, float* z);
/* PickNegLogSoftmax (dynet/nodes-pickneglogsoftmax.cc:72-145).  aux (device,
 * 3*bd*4 bytes, :72-74) = [z | m | ids] with ids[b] = b*rows + label_b;
 * labels_host are bounds-checked (:100). */
int dyhip_pnls_forward(dyhip_device* dev, size_t rows, unsigned bd, const float* x, const unsigned* labels_host,
                       void* aux, float* fx);
/* same, for callers that have already written ids (b*rows + label_b, validated) into
 * the third part of aux on the device: no host copy, no synchronisation, capturable */
int dyhip_pnls_forward_staged(dyhip_device* dev, size_t rows, unsigned bd, const float* x, void* aux, float* fx);
int dyhip_pnls_backward(dyhip_device* dev, size_t rows, unsigned bd, const float* x, const void* aux,
                        const float* dEdf, float* dEdx);
/* The same with dEdx overwritten instead of accumulated into: for an executor that knows this
 * node is the first consumer to contribute to dEdx, it saves zero-filling the buffer
 * (dynet/exec.cc:207-208) and reading it back, two passes over a rows x bd tensor. */
int dyhip_pnls_backward_assign(dyhip_device* dev, size_t rows, unsigned bd, const float* x, const void* aux,
                               const float* dEdf, float* dEdx);
/* Softmax over dim 0 (dynet/nodes-softmaxes.cc:40-87 forward, :89-125 backward): x is rows x cols
 * with cols = columns x batch.  Forward needs 2*cols floats of scratch (the reference's z and m from
 * pools[SCS], :45-48), backward cols floats (:97-98). */
int dyhip_softmax_forward(dyhip_device* dev, size_t rows, unsigned cols, const float* x, float* fx, void* ws,
                          size_t ws_bytes);
int dyhip_softmax_backward(dyhip_device* dev, size_t rows, unsigned cols, const float* fx, const float* dEdf,
                           float* dEdx, void* ws, size_t ws_bytes);
/* Softmax over dim 1 (dynet/nodes-softmaxes.cc:74-85 forward, :114-122 backward): x is rows x cols per batch
 * element, each row is normalised over its columns.  One kernel each, no scratch (the reference takes z and
 * m, rows x bd floats each, from pools[SCS]). */
int dyhip_softmax_rows_forward(dyhip_device* dev, size_t rows, size_t cols, unsigned bd, const float* x, float* fx);
int dyhip_softmax_rows_backward(dyhip_device* dev, size_t rows, size_t cols, unsigned bd, const float* fx,
                                const float* dEdf, float* dEdx);
/* LogSumExpDimension (dynet/nodes-logsumexp.cc:126-145) through TensorTools::logsumexp_dev's GPU branch
 * (dynet/tensor.cc:487-496): x is rows x cols per batch element, dim in {0, 1} is the reduced dimension;
 * m (the reference's scratch tensor ms) and fx hold cols x bd values for dim 0, rows x bd for dim 1.
 * backward: dEdx[i,j,b] += exp(x[i,j,b] - fx[o,b]) * dEdf[o,b], o = j for dim 0, i for dim 1. */
int dyhip_logsumexp_dim_forward(dyhip_device* dev, size_t rows, size_t cols, unsigned bd, const float* x, unsigned dim,
                                float* m, float* fx);
int dyhip_logsumexp_dim_backward(dyhip_device* dev, size_t rows, size_t cols, unsigned bd, const float* x,
                                 const float* fx, const float* dEdf, unsigned dim, float* dEdx);
/* LogSoftmax (dynet/nodes-softmaxes.cc:141-185 forward, :187-213 backward).  aux = the node's aux_mem,
 * 2*cols floats [z | m] (:136-138); backward overwrites z with the column sums of dEdf, as the reference does. */
int dyhip_log_softmax_forward(dyhip_device* dev, size_t rows, unsigned cols, const float* x, void* aux, float* fx);
int dyhip_log_softmax_backward(dyhip_device* dev, size_t rows, unsigned cols, const float* fx, const float* dEdf,
                               void* aux, float* dEdx);
/* LogSumExp node over any number k >= 1 of arguments (dynet/nodes-logsumexp.cc:38-97; up to 32 in one launch, more
 * chained through fx).  An entry whose arguments are all -inf is NaN, as in the reference. */
int dyhip_logsumexp_node_forward(dyhip_device* dev, unsigned k, size_t n, unsigned bd, const float* const* xs_host,
                                 const unsigned* bds_host, float* fx);
int dyhip_logsumexp_node_backward(dyhip_device* dev, unsigned k, size_t n, unsigned bd, const float* const* xs_host,
                                  const unsigned* bds_host, const float* fx, const float* dEdf, unsigned i,
                                  float* dEdxi, void* ws, size_t ws_bytes);
/* TensorTools::argmax_dev along dim 0 (dynet/tensor.cc:527-538): first maximum, 64-bit indices */
int dyhip_argmax_cols(dyhip_device* dev, size_t rows, unsigned bd, const float* x, long long* idx);
/* Argmax::forward_dev_impl over a vector per batch element (dynet/nodes-argmax.cc:44-55): idx (the node's aux_mem,
 * bd 64-bit indices, :37-39) = argmax along dim 0, fx = 1 at each batch element's argmax and 0 elsewhere.  Nothing is
 * copied to the host (the reference reads the indices back and sets the ones element by element).  backward
 * (:57-68) is dyhip_accumulate(dEdf -> dEdxi) for the straight-through estimator and nothing otherwise. */
int dyhip_argmax_onehot_forward(dyhip_device* dev, size_t rows, unsigned bd, const float* x, long long* idx, float* fx);

/* ---- dynet::gpu::* helpers (dynet/gpu-ops.h:9-15), same argument lists ---- */
int dyhip_dense_to_sparse_assign(dyhip_device* dev, int n, const unsigned* ids, const float* src, float* trg);
int dyhip_sparse_to_dense_assign(dyhip_device* dev, int n, const unsigned* ids, const float* src, float* trg);
int dyhip_dense_to_sparse_subtract(dyhip_device* dev, int n, const unsigned* ids, const float* src, float* trg);
int dyhip_sparse_to_dense_block_assign_and_multiply(dyhip_device* dev, int n, const unsigned* idx, int bsize,
                                                    float mult, const float* src, float* trg);
int dyhip_dense_to_sparse_block_add(dyhip_device* dev, int n, const unsigned* ids, int bsize, const float* src, float* trg);
int dyhip_parallel_memcpy(dyhip_device* dev, int num_seqs, int max_len, float** src, float** trg, size_t* len);
int dyhip_parallel_accumulate(dyhip_device* dev, int num_seqs, int max_len, float** src, float** trg, size_t* len);

/* n_seg equal-length tensors copied one behind the other: dst[s * len, (s + 1) * len) = src_host[s][0, len).  What
 * combine_tensors (dynet/exec.cc:298-364) does for the arguments of a batched node, for the case that matters to the
 * accumulation of one parameter gradient over the timesteps of an unrolled RNN: the executor adds T products of depth
 * B into the same dEdf of a ParameterNode (dynet/exec.cc:247-280, dynet/nodes-lstm.cc:472-500), which is ONE product
 * of depth T*B over the gathered operands (dyhip_gemm_nt_acc) -- 0.6 ms instead of 2.3 ms for the two-layer LSTM-LM.
 * src_host is a HOST array of DEVICE pointers; they travel as kernel arguments, so the call copies nothing from the
 * host, does not synchronise, and may be recorded into a graph. */
int dyhip_gather_segments(dyhip_device* dev, unsigned n_seg, size_t len, const float* const* src_host, float* dst);

/* ---- parameter nodes / trainer ------------------------------------------- */
/* ParameterNode::forward_dev_impl (dynet/param-nodes.cc:201-215): dst = src * mult */
int dyhip_scale_copy(dyhip_device* dev, size_t n, const float* src, float mult, float* dst);
/* SimpleSGDTrainer::update_rule_dev (dynet/training.cc:619-622): p -= g * (lr*gscale/wd) */
int dyhip_sgd_update(dyhip_device* dev, size_t n, float* p, const float* g, float lr, float gscale, float wd);
/* Trainer::clip_gradients (dynet/training.cc:173-187) without the per-parameter blocking
 * device-to-host copy of dynet/model.cc:830-842: *gscale (device) = min(1, threshold /
 * sqrt(sum of the n squared norms)); threshold <= 0 disables clipping (gscale = 1). */
int dyhip_clip_scale(dyhip_device* dev, unsigned n, const float* sqnorms, float threshold, float* gscale);
/* The same, also storing the gradient norm in *norm (device, may be null).  Where the reference throws
 * "Magnitude of gradient is bad" for a NaN or infinite norm (dynet/training.cc:176-180: only with clipping
 * enabled, threshold > 0), both forms set *gscale = 0, and dyhip_sgd_update_scaled / dyhip_sgd_update_rows
 * given a scale of 0 leave the parameters untouched (gradients are still cleared): the diverged step is dropped
 * on the device.  Nothing else reports it: a caller that wants the reference's error must read the norm slot
 * (this form) and raise it when the value is not finite.  With threshold <= 0 the scale is 1 whatever the norm,
 * as in the reference (dynet/training.cc:174). */
int dyhip_clip_scale_norm(dyhip_device* dev, unsigned n, const float* sqnorms, float threshold, float* gscale,
                          float* norm);
/* the SGD rule with gscale read on the device; clear_grad != 0 also zeroes g (ParameterStorage::clear) */
int dyhip_sgd_update_scaled(dyhip_device* dev, size_t n, float* p, float* g, float lr, const float* gscale,
                            float wd, int clear_grad);
/* Sparse lookup update (dynet/training.cc:215-226,630-637) over the distinct ids of a lookup plan:
 * values[:, id] -= grads[:, id] * (lr*gscale/wd); grads[:, id] = 0 (LookupParameterStorage::clear
 * restricted to the touched rows, dynet/model.cc:175-186) */
int dyhip_sgd_update_rows(dyhip_device* dev, unsigned n_ids, const void* plan, size_t dim, unsigned vocab,
                          float* values, float* grads, float lr, const float* gscale, float wd);
/* LookupParameterStorage::g_squared_l2norm_dev over non_zero_grads (dynet/model.cc:664-675): the sum of
 * squares of the gradient rows named by the plan, each distinct id once */
int dyhip_squared_l2norm_rows_workspace(unsigned n_ids, size_t* ws_bytes);
int dyhip_squared_l2norm_rows(dyhip_device* dev, unsigned n_ids, const void* plan, size_t dim, unsigned vocab,
                              const float* grads, float* out, void* ws, size_t ws_bytes);
/* ParameterStorage::g_squared_l2norm_dev (dynet/model.cc): *out(device) = sum g^2 */
int dyhip_squared_l2norm_workspace(size_t n, size_t* ws_bytes);
int dyhip_squared_l2norm(dyhip_device* dev, size_t n, const float* g, float* out, void* ws, size_t ws_bytes);

#ifdef __cplusplus
}
#endif
#endif
