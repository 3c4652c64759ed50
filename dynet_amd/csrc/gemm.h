// Internal interface of the fp32 MFMA GEMM (gemm.hip), shared with the fused
// LSTM launchers.
#pragma once

#include "common.h"

namespace dyhip {

// One K-segment of a GEMM: C += op(A) * op(B) over this segment's K.
//   a_kmajor == false : A(i,k) = A[i + k*lda]   (contiguous along the output row index)
//   a_kmajor == true  : A(i,k) = A[k + i*lda]   (contiguous along K, i.e. a transposed operand)
//   b_kmajor == true  : B(k,j) = B[k + j*ldb]
//   b_kmajor == false : B(k,j) = B[j + k*ldb]
struct GemmSeg {
  const float* A;
  size_t lda;
  const float* B;
  size_t ldb;
  size_t K;
};

constexpr int kGemmMaxSeg = 2;

enum GemmEpilogue {
  kEpiAxpby = 0,      // C = beta*C + sum
  kEpiLstmGates = 1,  // C = act(bias[i] + (H <= i < 2H ? 1 : 0) + sum), logistic rows [0,3H), tanh rows [3H,4H)
  kEpiBias = 2,       // C = bias[i] + sum   (AffineTransform: bias broadcast over the columns)
  kEpiPartials = 3    // no epilogue: the split-K slices stay in the caller's buffer, summed by the consumer
};

struct GemmEpiParams {
  int kind;
  float beta;
  const float* bias;  // kEpiLstmGates, kEpiBias
  unsigned H;         // kEpiLstmGates
  int logistic_mode;  // kEpiLstmGates
  // kEpiPartials: slices of M*N floats each are written here; *splits_out receives their number
  float* partials;
  size_t partials_bytes;
  unsigned* splits_out;
};

// `count` independent products in one launch: item b uses A + b*stride_a, B + b*stride_b, C + b*stride_c
// (strides in floats; 0 shares an operand between the items).  One K segment, axpby epilogue, no split-K.
struct GemmBatch {
  unsigned count;
  size_t stride_a, stride_b, stride_c;
};

// C is M x N column-major (ldc = M).  Segments share the operand layouts.
int gemm_run(dyhip_device* dev, bool a_kmajor, bool b_kmajor, size_t M, size_t N, int nseg, const GemmSeg* segs,
             float* C, const GemmEpiParams& epi, const GemmBatch* batch = nullptr);

// reduce.hip: out[j] (+)= sum over `splits` partial rows of n floats, in ascending order
int combine_partial_rows(dyhip_device* dev, size_t n, unsigned splits, const float* partial, float* out, bool accumulate);

// gemm_small.hip: one-launch products for operands of a few hundred KB, any layout, single or strided-batched, with
// the axpby or the bias epilogue.
bool gemm_small_eligible(const dyhip_device* dev, size_t M, size_t N, size_t K, const GemmEpiParams& epi, unsigned batch,
                         bool tile_kernel_vectorizes);
int gemm_small_run(dyhip_device* dev, bool a_kmajor, bool b_kmajor, size_t M, size_t N, const GemmSeg& s, float* C,
                   const GemmEpiParams& epi, const GemmBatch* batch);

// gemm_wide.hip: the 256 x 256-tile kernel for large outputs.  gemm_wide_eligible tells whether a one-segment,
// unbatched product qualifies; gemm_wide_run computes C = beta*C + sum (or bias[i] + sum when bias is set) over the
// first K32 (a multiple of 32) of the depth.
bool gemm_wide_eligible(const dyhip_device* dev, bool a_kmajor, bool b_kmajor, size_t M, size_t N, size_t K,
                        const float* A, size_t lda, const float* B, size_t ldb, const float* C);
// For a product that does not qualify as a whole: the number of leading columns that form full rounds of one tile per
// CU and qualify on their own (0 if none); the caller hands the remaining columns to whatever kernel suits them.
size_t gemm_wide_whole_rounds_columns(const dyhip_device* dev, bool a_kmajor, bool b_kmajor, size_t M, size_t N, size_t K,
                                      const float* A, size_t lda, const float* B, size_t ldb, const float* C);
int gemm_wide_run(dyhip_device* dev, bool a_kmajor, bool b_kmajor, size_t M, size_t N, size_t K32, const float* A,
                  size_t lda, const float* B, size_t ldb, float* C, float beta, const float* bias);

void gemm_wide_describe(size_t M, size_t N, size_t K, unsigned segments, unsigned* starts, unsigned* k_tiles_per_tile,
                        int* finish_in_kernel);

// gemm_wide.hip: C[M x N] = beta*C + A[M x K] * B[N x K]^T for a depth of at most 128 (both operands contiguous
// along the output index): operand tiles fetched whole, one latency per block.
bool gemm_shallow_nt_eligible(const dyhip_device* dev, size_t M, size_t N, size_t K, const float* A, size_t lda,
                              const float* B, size_t ldb, const float* C);
int gemm_shallow_nt_run(dyhip_device* dev, size_t M, size_t N, size_t K, const float* A, size_t lda, const float* B,
                        size_t ldb, float* C, float beta);

// lstm.hip: C = beta * C + A^T B by the fragment-order product for small outputs with deep sums (A is K x M, B is
// K x N, k contiguous); *taken tells whether it ran or the shape should go to gemm_run.
int skinny_tn_gemm(dyhip_device* dev, size_t M, size_t N, size_t K, const float* A, size_t lda, const float* B,
                   size_t ldb, float beta, float* C, bool* taken);
// lstm.hip: the streaming l^T * r kernel (at most four columns of r) over the items of a strided batch
int thin_tn_batched(dyhip_device* dev, size_t M, size_t N, size_t K, const float* A, size_t lda, const float* B, size_t ldb,
                    float beta, float* C, const GemmBatch* batch, bool* taken);

// lstm.hip: C = epilogue(A0 B0 [+ A1 B1]) in one launch for a right operand of a few 32-column tiles (A: M x K with rows
// contiguous, B: K x N with k contiguous; two segments only with the gates epilogue); *taken tells whether it ran.
int skinny_nn_gemm(dyhip_device* dev, size_t M, size_t N, int nseg, const GemmSeg* segs, float* C, const GemmEpiParams& epi,
                   bool* taken);

}  // namespace dyhip
