/*
 * dynet_cpu_oracle.h -- TEST INFRASTRUCTURE ONLY.
 *
 * A plain-C restatement of DyNet's CPU (Device_CPU / Eigen::DefaultDevice)
 * path for the fused-layer operators.  It exists so that the HIP kernels can
 * be checked against "what the reference's CPU path computes" on machines
 * where the reference itself cannot be built (its arithmetic lives in Eigen,
 * an un-vendored dependency pinned to snapshot b2e267dc99d4 that is absent
 * here).  Nothing in the shipped library links, loads or calls this file:
 * only tests, the smoke check and the benchmark's cpu_baseline leg may.
 *
 * Conventions (dynet/dim.h:34-304, dynet/tensor-eigen.h:21-63): all tensors
 * are fp32, column-major, batch outermost; element (i, j, b) of a tensor with
 * `rows` rows and `cols` columns lives at v[i + j*rows + b*rows*cols].
 * Forward functions overwrite their output; backward functions ACCUMULATE
 * (+=) into the gradient buffer exactly like every backward_dev_impl does.
 *
 * Parity status per function (what pins the restatement) is listed in the
 * header comment of each function in dynet_cpu_oracle.c.  Functions whose
 * arithmetic crosses the Eigen boundary (tanh/exp/log packet approximations,
 * summation trees, packet-vs-scalar logistic selection) say
 * "parity unpinned at the Eigen boundary" there: libm and sequential fp32
 * sums are used instead, which agree with Eigen to a few ulp.
 *
 * Every function returns 0 on success and a negative value on an argument
 * error (the cases where the reference raises std::invalid_argument).
 */
#ifndef DYNET_CPU_ORACLE_H
#define DYNET_CPU_ORACLE_H

#include <stddef.h>

#ifdef __cplusplus
extern "C" {
#endif

/* unary operator codes (shared with the HIP library's DYHIP_OP_* values) */
enum {
  ORC_OP_TANH = 0,
  ORC_OP_LOGISTIC = 1,
  ORC_OP_RECTIFY = 2,
  ORC_OP_NEGATE = 3,
  ORC_OP_IDENTITY = 4
};

/* which form of scalar_logistic_sigmoid_op is evaluated */
enum {
  ORC_LOGISTIC_PACKET = 0, /* packetOp: clamp +-18, rational polynomial */
  ORC_LOGISTIC_SCALAR = 1  /* operator(): 1/(1+exp(-x)) */
};

/* ---- scalar functors ---------------------------------------------------- */
float orc_logistic_packet(float x);
float orc_logistic_scalar(float x);

/* ---- elementwise nodes -------------------------------------------------- */
int orc_unary_forward(int op, int logistic_mode, size_t n, const float* x, float* y);
int orc_unary_backward(int op, size_t n, const float* fx, const float* dEdf, float* dEdx);

/* n = elements per batch element; bd0/bd1 = batch counts of the two args
 * (equal, or one of them 1). */
int orc_cmult_forward(size_t n, unsigned bd0, unsigned bd1, const float* a, const float* b, float* y);
int orc_cmult_backward(size_t n, unsigned bd0, unsigned bd1, const float* a, const float* b,
                       const float* dEdf, unsigned i, float* dEdxi);
int orc_csum_forward(size_t n, unsigned bd0, unsigned bd1, const float* a, const float* b, float* y);
int orc_csum_backward(size_t n, unsigned bd0, unsigned bd1, const float* dEdf, unsigned i, float* dEdxi);

/* the same three operators with broadcast over any of {d0, d1, d2, d3, bd}: dims arrays of 5;
 * op 0 = sum, 1 = multiply, 2 = quotient (only the right argument may be broadcast) */
int orc_cwise_forward(int op, const unsigned* dims_a, const unsigned* dims_b, const float* a, const float* b, float* fx);
int orc_cwise_backward(int op, const unsigned* dims_a, const unsigned* dims_b, const float* a, const float* b,
                       const float* dEdf, unsigned i, float* dEdxi);
int orc_const_plus_x_forward(size_t n, float c, const float* x, float* fx);
int orc_const_minus_x_forward(size_t n, float c, const float* x, float* fx);

/* ---- reductions --------------------------------------------------------- */
int orc_sum_batches_forward(size_t n, unsigned bd, const float* x, float* y);
int orc_sum_batches_backward(size_t n, unsigned bd, const float* dEdf, float* dEdx);
/* mean_elems / std_elems: one scalar per batch element over its n elements */
int orc_mean_elems_forward(size_t n, unsigned bd, const float* x, float* y);
int orc_mean_elems_backward(size_t n, unsigned bd, const float* dEdf, float* dEdx);
int orc_std_elems_forward(size_t n, unsigned bd, const float* x, float* y);
int orc_std_elems_backward(size_t n, unsigned bd, const float* x, const float* fx,
                           const float* dEdf, float* dEdx);

/* ---- layer_norm composite ---------------------------------------------- */
int orc_layer_norm_forward(size_t n, unsigned bd, const float* x, const float* g,
                           const float* b, float* y);
/* dx[n*bd], dg[n], db[n] are accumulated into; any of them may be NULL */
int orc_layer_norm_backward(size_t n, unsigned bd, const float* x, const float* g,
                            const float* dEdf, float* dx, float* dg, float* db);

/* ---- GEMM shim ---------------------------------------------------------- */
/* y[M x N] = beta*y + l[M x K] * r[K x N] */
int orc_gemm_nn(size_t M, size_t N, size_t K, const float* l, const float* r, float beta, float* y);
/* y[M x N] += l[K x M]^T * r[K x N] */
int orc_gemm_tn_acc(size_t M, size_t N, size_t K, const float* l, const float* r, float* y);
/* y[M x N] += l[M x K] * r[N x K]^T */
int orc_gemm_nt_acc(size_t M, size_t N, size_t K, const float* l, const float* r, float* y);

/* ---- fused LSTM nodes --------------------------------------------------- */
/* xs[k] has x_dims[k] rows and B columns.  mask_x / mask_h may be NULL (no
 * dropout); otherwise their batch counts are B or 1. */
int orc_lstm_gates_forward(unsigned num_inputs, const float* const* xs, const unsigned* x_dims,
                           unsigned H, unsigned B, const float* h_tm1, const float* Wx,
                           const float* Wh, const float* b, const float* mask_x,
                           unsigned mask_x_bd, const float* mask_h, unsigned mask_h_bd,
                           int logistic_mode, float* fx);
/* argument index i follows the node: [0,num_inputs) inputs, then h, Wx, Wh, b */
int orc_lstm_gates_backward(unsigned num_inputs, const float* const* xs, const unsigned* x_dims,
                            unsigned H, unsigned B, const float* h_tm1, const float* Wx,
                            const float* Wh, const float* mask_x, unsigned mask_x_bd,
                            const float* mask_h, unsigned mask_h_bd, const float* fx,
                            const float* dEdf, unsigned i, float* dEdxi);
int orc_lstm_c_forward(unsigned H, unsigned B, const float* c_tm1, const float* gates, float* c);
int orc_lstm_c_backward(unsigned H, unsigned B, const float* c_tm1, const float* gates,
                        const float* dEdf, unsigned i, float* dEdxi);
int orc_lstm_h_forward(unsigned H, unsigned B, const float* c, const float* gates, float* h);
int orc_lstm_h_backward(unsigned H, unsigned B, const float* c, const float* gates,
                        const float* dEdf, unsigned i, float* dEdxi);

/* ---- lookup ------------------------------------------------------------- */
int orc_lookup_forward(unsigned n_ids, const unsigned* ids, size_t dim, unsigned vocab,
                       const float* table, float mult, float* fx);
int orc_lookup_accumulate_grads(unsigned n_ids, const unsigned* ids, size_t dim, unsigned vocab,
                                const float* g, float* all_grads);

/* ---- logsumexp / pickneglogsoftmax -------------------------------------- */
/* per batch column: m[b] = max, z[b] = log sum exp(x - m) + m */
int orc_logsumexp_cols(size_t rows, unsigned bd, const float* x, float* m, float* z);
/* aux = [z(B) | m(B) | ids(B as u32 = b*rows + label)] */
int orc_sum_forward(unsigned k, size_t n, unsigned bd, const float* const* xs, const unsigned* bds, float* fx);
int orc_softmax_forward(size_t rows, unsigned cols, const float* x, float* fx);
int orc_softmax_backward(size_t rows, unsigned cols, const float* fx, const float* dEdf, float* dEdx);
int orc_softmax_rows_forward(size_t rows, size_t cols, unsigned bd, const float* x, float* fx);
int orc_softmax_rows_backward(size_t rows, size_t cols, unsigned bd, const float* fx, const float* dEdf, float* dEdx);
int orc_logsumexp_dim_forward(size_t rows, size_t cols, unsigned bd, const float* x, unsigned dim, float* m, float* z);
int orc_logsumexp_dim_backward(size_t rows, size_t cols, unsigned bd, const float* x, const float* fx,
                               const float* dEdf, unsigned dim, float* dEdx);
int orc_log_softmax_forward(size_t rows, unsigned cols, const float* x, float* aux, float* fx);
int orc_log_softmax_backward(size_t rows, unsigned cols, const float* fx, const float* dEdf, float* dEdx);
int orc_pnls_forward(size_t rows, unsigned bd, const float* x, const unsigned* labels,
                     void* aux, float* fx);
int orc_pnls_backward(size_t rows, unsigned bd, const float* x, const void* aux,
                      const float* dEdf, float* dEdx);
/* LogSumExp node over k args, each n x bds[k] (bds[k] == bd or 1) */
int orc_logsumexp_node_forward(unsigned k, size_t n, unsigned bd, const float* const* xs,
                               const unsigned* bds, float* fx);
int orc_logsumexp_node_backward(unsigned k, size_t n, unsigned bd, const float* const* xs,
                                const unsigned* bds, const float* fx, const float* dEdf,
                                unsigned i, float* dEdxi);
int orc_argmax_cols(size_t rows, unsigned bd, const float* x, long long* idx);
int orc_argmax_onehot_forward(size_t rows, unsigned bd, const float* x, long long* idx, float* fx);

/* ---- scatter/gather helpers (dynet::gpu::*) ------------------------------ */
int orc_dense_to_sparse_assign(int n, const unsigned* idx, const float* src, float* trg);
int orc_sparse_to_dense_assign(int n, const unsigned* idx, const float* src, float* trg);
int orc_dense_to_sparse_subtract(int n, const unsigned* idx, const float* src, float* trg);
int orc_sparse_to_dense_block_assign_and_multiply(int n, const unsigned* idx, int bsize, float mult,
                                                  const float* src, float* trg);
int orc_dense_to_sparse_block_add(int n, const unsigned* idx, int bsize, const float* src, float* trg);
int orc_parallel_memcpy(int num_seqs, int max_len, float* const* src, float* const* trg,
                        const size_t* len);
int orc_parallel_accumulate(int num_seqs, int max_len, float* const* src, float* const* trg,
                            const size_t* len);

/* ---- parameter nodes / trainer ------------------------------------------ */
int orc_scale_copy(size_t n, const float* src, float mult, float* dst);
int orc_sgd_update(size_t n, float* p, const float* g, float lr, float gscale, float wd);
int orc_squared_l2norm(size_t n, const float* g, float* out);

/* ---- PickRange ---------------------------------------------------------- */
int orc_pick_range_forward(size_t inner, size_t len, size_t outer, size_t start, size_t end, const float* x,
                           float* fx);
int orc_pick_range_backward(size_t inner, size_t len, size_t outer, size_t start, size_t end, const float* dEdf,
                            float* dEdxi);

/* ---- random tensors (Philox4x32-10; key = seed + 1) ----------------------- */
void orc_philox4x32_10(const unsigned ctr[4], const unsigned key[2], unsigned out[4]);
int orc_random_words(unsigned long long key, unsigned long long position, unsigned queue, size_t n,
                     unsigned* words);
int orc_randomize_uniform(unsigned long long key, unsigned long long position, unsigned queue, size_t n,
                          float left, float right, float* out);
int orc_randomize_bernoulli(unsigned long long key, unsigned long long position, unsigned queue, size_t n,
                            float p, float scale, float* out);
int orc_randomize_normal(unsigned long long key, unsigned long long position, unsigned queue, size_t n,
                         float mean, float stddev, float* out);
int orc_dropout_forward(unsigned long long key, unsigned long long position, unsigned queue, size_t n, float p,
                        const float* x, float* mask, float* fx);
int orc_dropout_backward(size_t n, const float* mask, const float* dEdf, float* dEdxi);

#ifdef __cplusplus
}
#endif
#endif
