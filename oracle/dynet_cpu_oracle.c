/*
 * dynet_cpu_oracle.c -- TEST INFRASTRUCTURE ONLY (see dynet_cpu_oracle.h).
 *
 * Plain-C restatement of the CPU (Device_CPU) bodies of DyNet's fused-layer
 * nodes.  Each function cites the reference file:line it follows (paths are
 * relative to the DyNet source tree) and says what pins it.
 *
 * Build: gcc -O2 -ffp-contract=off -fPIC -shared (see oracle/Makefile).
 * -ffp-contract=off keeps every multiply-add as two rounded operations, so
 * the only fused multiply-adds are the explicit fmaf() calls that stand for
 * Eigen's pmadd in the logistic polynomial.
 *
 * Arithmetic that lives inside Eigen (tanh/exp/log packet approximations,
 * the shape of summation trees, GEMM blocking) cannot be restated from the
 * reference tree; this file uses libm (tanhf/expf/logf/sqrtf) and sequential
 * fp32 sums in index order.  Those spots are marked
 * "parity unpinned at the Eigen boundary".
 */
#include "dynet_cpu_oracle.h"

#include <math.h>
#include <stdlib.h>
#include <string.h>

/* ======================================================================== */
/* scalar functors                                                           */
/* ======================================================================== */

/* dynet/simd-functors.h:81-125 (scalar_logistic_sigmoid_op::packetOp): clamp
 * to [-18, 18], odd numerator / even denominator rational polynomial in
 * Horner form, each pmadd(a,b,c) = a*b+c restated as fmaf, then +0.5 and a
 * clamp to [0,1].  Coefficients are the doubles of the source rounded to
 * float by pset1<Packet4f/8f>.  Pinned by: sigma(-x)+sigma(x)=1 to 1 ulp,
 * |poly - 1/(1+e^-x)| < 2e-7 absolute on [-18,18] (tests), and the LSTM gate
 * known-answer vectors of tests/test-rnn.cc:301-339. */
/* pmin / pmax as the SSE and AVX packets implement them (minps / maxps of (a, b)): the second
 * operand comes back when either one is NaN.  A NaN input therefore clamps to 18 and gives 1.0f.
 * Which operand order the pinned Eigen snapshot passes is not visible from the reference:
 * parity unpinned at the Eigen boundary for NaN inputs. */
static float packet_min(float a, float b) { return a < b ? a : b; }
static float packet_max(float a, float b) { return a > b ? a : b; }

float orc_logistic_packet(float _x) {
  float x = packet_max(packet_min(_x, 18.0f), -18.0f);
  const float alpha_1 = (float)2.48287947061529e-01;
  const float alpha_3 = (float)8.51377133304701e-03;
  const float alpha_5 = (float)6.08574864600143e-05;
  const float alpha_7 = (float)1.15627324459942e-07;
  const float alpha_9 = (float)4.37031012579801e-11;
  const float beta_0 = (float)9.93151921023180e-01;
  const float beta_2 = (float)1.16817656904453e-01;
  const float beta_4 = (float)1.70198817374094e-03;
  const float beta_6 = (float)6.29106785017040e-06;
  const float beta_8 = (float)5.76102136993427e-09;
  const float beta_10 = (float)6.10247389755681e-13;
  float x2 = x * x;
  float p = fmaf(x2, alpha_9, alpha_7);
  p = fmaf(x2, p, alpha_5);
  p = fmaf(x2, p, alpha_3);
  p = fmaf(x2, p, alpha_1);
  p = x * p;
  float q = fmaf(x2, beta_10, beta_8);
  q = fmaf(x2, q, beta_6);
  q = fmaf(x2, q, beta_4);
  q = fmaf(x2, q, beta_2);
  q = fmaf(x2, q, beta_0);
  return packet_max(packet_min(p / q + 0.5f, 1.0f), 0.0f);
}

/* dynet/simd-functors.h:76-79 (scalar operator()).  Uses libm expf: parity
 * unpinned at the Eigen boundary only through numext::exp == std::exp. */
float orc_logistic_scalar(float x) { return 1.0f / (1.0f + expf(-x)); }

static float logistic(int mode, float x) {
  return mode == ORC_LOGISTIC_SCALAR ? orc_logistic_scalar(x) : orc_logistic_packet(x);
}

/* ======================================================================== */
/* elementwise nodes                                                         */
/* ======================================================================== */

/* Tanh      dynet/nodes-trig.cc:312-315   y = tanh(x)   (Eigen .tanh():
 *           parity unpinned at the Eigen boundary; libm tanhf here)
 * Logistic  dynet/nodes-activations.cc:65-68
 * Rectify   dynet/nodes-activations.cc:31-34   y = max(x, 0)
 * Negate    dynet/nodes-arith-unary.cc:195-198
 * Pinned by: fp64 closed forms in tests, grad-check inputs of
 * tests/test-nodes.cc:854-860,944-960,1408-1484. */
int orc_unary_forward(int op, int logistic_mode, size_t n, const float* x, float* y) {
  size_t i;
  switch (op) {
    case ORC_OP_TANH: for (i = 0; i < n; ++i) y[i] = tanhf(x[i]); break;
    case ORC_OP_LOGISTIC: for (i = 0; i < n; ++i) y[i] = logistic(logistic_mode, x[i]); break;
    case ORC_OP_RECTIFY: for (i = 0; i < n; ++i) y[i] = x[i] > 0.f ? x[i] : 0.f; break;
    case ORC_OP_NEGATE: for (i = 0; i < n; ++i) y[i] = -x[i]; break;
    case ORC_OP_IDENTITY: for (i = 0; i < n; ++i) y[i] = x[i]; break;
    default: return -1;
  }
  return 0;
}

/* Tanh bwd      nodes-trig.cc:317-325 + simd-functors.h:535-544: dx += (1 - t*t) * d
 * Logistic bwd  nodes-activations.cc:70-77 + simd-functors.h:509-521: dx += (1 - t) * t * d
 *               (scalar form; the packet form multiplies (1-t)*(t*d): same to 1 ulp)
 * Rectify bwd   nodes-activations.cc:36-43: dx += cast<bool>(fx) * d  => ReLU'(0) = 0
 * Negate bwd    nodes-arith-unary.cc:200-208: dx -= d
 * All take the node OUTPUT fx, not the input. */
int orc_unary_backward(int op, size_t n, const float* fx, const float* dEdf, float* dEdx) {
  size_t i;
  switch (op) {
    case ORC_OP_TANH:
      for (i = 0; i < n; ++i) dEdx[i] += (1.f - fx[i] * fx[i]) * dEdf[i];
      break;
    case ORC_OP_LOGISTIC:
      for (i = 0; i < n; ++i) dEdx[i] += (1.f - fx[i]) * fx[i] * dEdf[i];
      break;
    case ORC_OP_RECTIFY:
      for (i = 0; i < n; ++i) dEdx[i] += (fx[i] != 0.f ? 1.f : 0.f) * dEdf[i];
      break;
    case ORC_OP_NEGATE:
      for (i = 0; i < n; ++i) dEdx[i] -= dEdf[i];
      break;
    case ORC_OP_IDENTITY:
      for (i = 0; i < n; ++i) dEdx[i] += dEdf[i];
      break;
    default: return -1;
  }
  return 0;
}

static int bd_ok(unsigned bd0, unsigned bd1) {
  return bd0 >= 1 && bd1 >= 1 && (bd0 == bd1 || bd0 == 1 || bd1 == 1);
}

/* CwiseMultiply fwd, same dims, batch sizes equal or one side 1:
 * dynet/nodes-arith-cwise.cc:196-212 (CPU: per-batch chip loop). */
int orc_cmult_forward(size_t n, unsigned bd0, unsigned bd1, const float* a, const float* b, float* y) {
  if (!bd_ok(bd0, bd1)) return -1;
  unsigned bd = bd0 > bd1 ? bd0 : bd1;
  for (unsigned k = 0; k < bd; ++k) {
    const float* pa = a + (bd0 > 1 ? (size_t)k * n : 0);
    const float* pb = b + (bd1 > 1 ? (size_t)k * n : 0);
    for (size_t i = 0; i < n; ++i) y[(size_t)k * n + i] = pa[i] * pb[i];
  }
  return 0;
}

/* CwiseMultiply bwd: dynet/nodes-arith-cwise.cc:245-273.  Same batch size:
 * dxi += dy * other; other has bd 1: broadcast; xi has bd 1: sum over the
 * batch of dy * other (sequential in b here: Eigen's reduction order is
 * parity unpinned at the Eigen boundary). */
int orc_cmult_backward(size_t n, unsigned bd0, unsigned bd1, const float* a, const float* b,
                       const float* dEdf, unsigned i, float* dEdxi) {
  if (!bd_ok(bd0, bd1) || i > 1) return -1;
  unsigned bd = bd0 > bd1 ? bd0 : bd1;
  const float* other = i == 0 ? b : a;
  unsigned bd_other = i == 0 ? bd1 : bd0;
  unsigned bd_self = i == 0 ? bd0 : bd1;
  if (bd_self == bd) {
    for (unsigned k = 0; k < bd; ++k) {
      const float* po = other + (bd_other > 1 ? (size_t)k * n : 0);
      for (size_t j = 0; j < n; ++j) dEdxi[(size_t)k * n + j] += dEdf[(size_t)k * n + j] * po[j];
    }
  } else { /* self is broadcast: reduce over the batch first, then accumulate */
    for (size_t j = 0; j < n; ++j) {
      float s = 0.f;
      for (unsigned k = 0; k < bd; ++k) s += dEdf[(size_t)k * n + j] * other[(size_t)k * n + j];
      dEdxi[j] += s;
    }
  }
  return 0;
}

/* CwiseSum fwd: dynet/nodes-arith-cwise.cc:50-67. */
int orc_csum_forward(size_t n, unsigned bd0, unsigned bd1, const float* a, const float* b, float* y) {
  if (!bd_ok(bd0, bd1)) return -1;
  unsigned bd = bd0 > bd1 ? bd0 : bd1;
  for (unsigned k = 0; k < bd; ++k) {
    const float* pa = a + (bd0 > 1 ? (size_t)k * n : 0);
    const float* pb = b + (bd1 > 1 ? (size_t)k * n : 0);
    for (size_t i = 0; i < n; ++i) y[(size_t)k * n + i] = pa[i] + pb[i];
  }
  return 0;
}

/* CwiseSum bwd: dynet/nodes-arith-cwise.cc:99-122.  CPU path for the
 * batch-broadcast argument: for b in order: dxi += dy[:,b]. */
int orc_csum_backward(size_t n, unsigned bd0, unsigned bd1, const float* dEdf, unsigned i, float* dEdxi) {
  if (!bd_ok(bd0, bd1) || i > 1) return -1;
  unsigned bd = bd0 > bd1 ? bd0 : bd1;
  unsigned bd_self = i == 0 ? bd0 : bd1;
  if (bd_self == bd) {
    for (size_t j = 0; j < n * (size_t)bd; ++j) dEdxi[j] += dEdf[j];
  } else {
    for (unsigned k = 0; k < bd; ++k)
      for (size_t j = 0; j < n; ++j) dEdxi[j] += dEdf[(size_t)k * n + j];
  }
  return 0;
}

/* ---- CwiseSum / CwiseMultiply / CwiseQuotient with broadcast over dimensions and batch --------------
 * dynet/nodes-arith-cwise.cc: forward :50-97 (sum), :196-243 (multiply), :338-351 (quotient); backward
 * :99-156, :245-307, :353-421.  A tensor is given by dims[5] = {d0, d1, d2, d3, bd} (column-major, batch
 * outermost; missing dimensions are 1).  For every axis the two arguments agree or one of them is 1
 * (CwiseQuotient: only the right one may be 1, :320-325); the output takes the larger.
 * Forward: fx[e] = a[bcast e] op b[bcast e].
 * Backward of argument i: dEdxi[o] (+/-)= sum over the axes where argument i is 1 and the output is not of
 *   sum:       dEdf                                  (:141-156, Eigen .sum(red_axis))
 *   multiply:  dEdf * other                          (:284-307)
 *   quotient:  i = 0: dEdf / b                       (:363-374, no axis is ever reduced)
 *              i = 1: -(dEdf / (b*b) * a)            (:376-421; b squared first, as the reference does)
 * summed here sequentially in the order of the output's linear index (parity unpinned at the Eigen boundary
 * for the order of a reduction).  Pinned in tests/test_oracle.py by numpy broadcasting in fp64, by central
 * differences, and by the batch-only cases agreeing with orc_csum_* / orc_cmult_*. */
static int cw_dims_ok(const unsigned* da, const unsigned* db, int quotient) {
  for (int j = 0; j < 5; ++j) {
    if (da[j] == 0 || db[j] == 0) return 0;
    if (da[j] != db[j] && da[j] != 1 && db[j] != 1) return 0;
    if (quotient && da[j] != db[j] && db[j] != 1) return 0;
  }
  return 1;
}

static size_t cw_offset(const unsigned* idx, const unsigned* dims) {
  size_t off = 0, stride = 1;
  for (int j = 0; j < 5; ++j) {
    off += (dims[j] == 1 ? 0 : idx[j]) * stride;
    stride *= dims[j];
  }
  return off;
}

int orc_cwise_forward(int op, const unsigned* da, const unsigned* db, const float* a, const float* b, float* fx) {
  if (op < 0 || op > 2 || !cw_dims_ok(da, db, op == 2)) return -1;
  unsigned df[5], idx[5];
  for (int j = 0; j < 5; ++j) df[j] = da[j] > db[j] ? da[j] : db[j];
  size_t e = 0;
  for (idx[4] = 0; idx[4] < df[4]; ++idx[4])
    for (idx[3] = 0; idx[3] < df[3]; ++idx[3])
      for (idx[2] = 0; idx[2] < df[2]; ++idx[2])
        for (idx[1] = 0; idx[1] < df[1]; ++idx[1])
          for (idx[0] = 0; idx[0] < df[0]; ++idx[0], ++e) {
            const float x = a[cw_offset(idx, da)], y = b[cw_offset(idx, db)];
            fx[e] = op == 0 ? x + y : op == 1 ? x * y : x / y;
          }
  return 0;
}

int orc_cwise_backward(int op, const unsigned* da, const unsigned* db, const float* a, const float* b,
                       const float* dEdf, unsigned i, float* dEdxi) {
  if (op < 0 || op > 2 || i > 1 || !cw_dims_ok(da, db, op == 2)) return -1;
  unsigned df[5], idx[5];
  for (int j = 0; j < 5; ++j) df[j] = da[j] > db[j] ? da[j] : db[j];
  const unsigned* di = i == 0 ? da : db;
  /* the reference forms the reduced tensor first (`.sum(red_axis)`) and then adds it to dEdxi; without a
   * reduction the terms go straight into dEdxi */
  int reduces = 0;
  size_t n_self = 1;
  for (int j = 0; j < 5; ++j) {
    reduces |= di[j] == 1 && df[j] > 1;
    n_self *= di[j];
  }
  float* acc = dEdxi;
  if (reduces) {
    acc = (float*)calloc(n_self, sizeof(float));
    if (!acc) return -1;
  }
  size_t e = 0;
  for (idx[4] = 0; idx[4] < df[4]; ++idx[4])
    for (idx[3] = 0; idx[3] < df[3]; ++idx[3])
      for (idx[2] = 0; idx[2] < df[2]; ++idx[2])
        for (idx[1] = 0; idx[1] < df[1]; ++idx[1])
          for (idx[0] = 0; idx[0] < df[0]; ++idx[0], ++e) {
            const float x = a[cw_offset(idx, da)], y = b[cw_offset(idx, db)], d = dEdf[e];
            float* out = acc + cw_offset(idx, di);
            if (op == 0) *out += d;
            else if (op == 1) *out += d * (i == 0 ? y : x);
            else if (i == 0) *out += d / y;
            else if (reduces) *out += d / (y * y) * x;
            else *out -= d / (y * y) * x;
          }
  if (reduces) {
    for (size_t j = 0; j < n_self; ++j) {
      if (op == 2) dEdxi[j] -= acc[j];
      else dEdxi[j] += acc[j];
    }
    free(acc);
  }
  return 0;
}

/* ConstantPlusX / ConstantMinusX, dynet/nodes-arith-const.cc:33-75: fx = c + x (c - x); backward
 * dEdx += dEdf (-= dEdf). */
int orc_const_plus_x_forward(size_t n, float c, const float* x, float* fx) {
  for (size_t j = 0; j < n; ++j) fx[j] = c + x[j];
  return 0;
}
int orc_const_minus_x_forward(size_t n, float c, const float* x, float* fx) {
  for (size_t j = 0; j < n; ++j) fx[j] = c - x[j];
  return 0;
}

/* ======================================================================== */
/* reductions                                                                */
/* ======================================================================== */

/* SumDimension with dims={} and include_batch_dim (sum_batches):
 * dynet/nodes-arith-sum.cc:197-203, ctor dynet/expr.cc:218.
 * y[j] = sum_b x[j,b]; sequential in b (parity unpinned at the Eigen
 * boundary for the order).  Pinned by tests/test-nodes.cc:206-213 (-6.5). */
int orc_sum_batches_forward(size_t n, unsigned bd, const float* x, float* y) {
  for (size_t j = 0; j < n; ++j) {
    float s = 0.f;
    for (unsigned k = 0; k < bd; ++k) s += x[(size_t)k * n + j];
    y[j] = s;
  }
  return 0;
}

/* dynet/nodes-arith-sum.cc:219-230: dx[:,b] += dy. */
int orc_sum_batches_backward(size_t n, unsigned bd, const float* dEdf, float* dEdx) {
  for (unsigned k = 0; k < bd; ++k)
    for (size_t j = 0; j < n; ++j) dEdx[(size_t)k * n + j] += dEdf[j];
  return 0;
}

/* mean_elems = MomentDimension(order 1, all dims, no batch):
 * dynet/expr.cc:229-233, dynet/nodes-moments.cc:181-209: sum / n with n a
 * float.  Sequential sum. */
int orc_mean_elems_forward(size_t n, unsigned bd, const float* x, float* y) {
  float fn = (float)n;
  for (unsigned k = 0; k < bd; ++k) {
    float s = 0.f;
    for (size_t j = 0; j < n; ++j) s += x[(size_t)k * n + j];
    y[k] = s / fn;
  }
  return 0;
}

/* dynet/nodes-moments.cc:264-274 (order 1): dx += broadcast(dy) / n. */
int orc_mean_elems_backward(size_t n, unsigned bd, const float* dEdf, float* dEdx) {
  float fn = (float)n;
  for (unsigned k = 0; k < bd; ++k)
    for (size_t j = 0; j < n; ++j) dEdx[(size_t)k * n + j] += dEdf[k] / fn;
  return 0;
}

/* std_elems = StdDimension(all dims, no batch): dynet/expr.cc:234-238,
 * dynet/nodes-moments.cc:434-463: two-pass population std,
 * sqrt(sum((x-mean)^2)/n).  Pinned by tests/test-nodes.cc:2383-2390
 * (0.128319368) through the same formula on param_cube1. */
int orc_std_elems_forward(size_t n, unsigned bd, const float* x, float* y) {
  float fn = (float)n;
  for (unsigned k = 0; k < bd; ++k) {
    const float* px = x + (size_t)k * n;
    float s = 0.f;
    for (size_t j = 0; j < n; ++j) s += px[j];
    float mean = s / fn;
    float v = 0.f;
    for (size_t j = 0; j < n; ++j) {
      float d = px[j] - mean;
      v += d * d;
    }
    y[k] = sqrtf(v / fn);
  }
  return 0;
}

/* dynet/nodes-moments.cc:497-527 + simd-functors.h:213-225:
 * dx += (2/n) * (x - mean) * (dy / (2*fx)). */
int orc_std_elems_backward(size_t n, unsigned bd, const float* x, const float* fx,
                           const float* dEdf, float* dEdx) {
  float fn = (float)n;
  for (unsigned k = 0; k < bd; ++k) {
    const float* px = x + (size_t)k * n;
    float s = 0.f;
    for (size_t j = 0; j < n; ++j) s += px[j];
    float mean = s / fn;
    float sb = dEdf[k] / (2.f * fx[k]);
    float c = 2.f / fn;
    for (size_t j = 0; j < n; ++j) dEdx[(size_t)k * n + j] += c * (px[j] - mean) * sb;
  }
  return 0;
}

/* ======================================================================== */
/* layer_norm composite                                                      */
/* ======================================================================== */

/* dynet/expr.cc:248-253:
 *   mu = mean_elems(x); xc = x + (-mu); sigma = std_elems(x);
 *   y = cmult(g, cdiv(xc, sigma + 1e-8)) + b
 * i.e. eight nodes: MomentDimension, Negate, CwiseSum (dim broadcast),
 * StdDimension, ConstantPlusX(1e-8f), CwiseQuotient (dim broadcast),
 * CwiseMultiply (g has batch 1), CwiseSum (b has batch 1).  The epsilon is
 * added to sigma, not to the variance.  Pinned by tests/test-nodes.cc:2415-2426
 * (g=1,b=0 => |mean(y)|<1e-6, rms(y)=1) and tests/python/test.py:506-519
 * (numpy closed form g/std*(x-mean)+b). */
int orc_layer_norm_forward(size_t n, unsigned bd, const float* x, const float* g,
                           const float* b, float* y) {
  float* mu = (float*)malloc(sizeof(float) * bd);
  float* sigma = (float*)malloc(sizeof(float) * bd);
  if (!mu || !sigma) { free(mu); free(sigma); return -2; }
  orc_mean_elems_forward(n, bd, x, mu);
  orc_std_elems_forward(n, bd, x, sigma);
  for (unsigned k = 0; k < bd; ++k) {
    float neg = -mu[k];
    float s = 1e-8f + sigma[k];
    for (size_t j = 0; j < n; ++j) {
      float xc = x[(size_t)k * n + j] + neg;
      float q = xc / s;
      y[(size_t)k * n + j] = g[j] * q + b[j];
    }
  }
  free(mu); free(sigma);
  return 0;
}

/* Backward of the composite, node by node in the executor's reverse order
 * (dynet/exec.cc:166-284), each node's rule from:
 *   CwiseSum      nodes-arith-cwise.cc:99-156   (db = sum_b dy; dgq = dy)
 *   CwiseMultiply nodes-arith-cwise.cc:245-273  (dg = sum_b dgq*q; dq = dgq*g)
 *   CwiseQuotient nodes-arith-cwise.cc:353-421  (dxc = dq/s; ds = -sum_i dq/s^2*xc)
 *   ConstantPlusX nodes-arith-const.cc:67-74    (dsigma = ds)
 *   StdDimension  nodes-moments.cc:497-527      (dx += (2/n)(x-mean) * dsigma/(2 sigma))
 *   CwiseSum      (dx += dxc; dneg = sum_i dxc)
 *   Negate        nodes-arith-unary.cc:200-208  (dmu = -dneg)
 *   MomentDim     nodes-moments.cc:264-274      (dx += dmu / n)
 * dx, dg, db are accumulated into (each may be NULL).  Pinned by the central
 * difference check of tests/test-nodes.cc:2404-2412 and by an fp64 analytic
 * LayerNorm gradient in tests. */
int orc_layer_norm_backward(size_t n, unsigned bd, const float* x, const float* g,
                            const float* dEdf, float* dx, float* dg, float* db) {
  float fn = (float)n;
  float* dg_tmp = dg ? (float*)calloc(n, sizeof(float)) : NULL;
  float* db_tmp = db ? (float*)calloc(n, sizeof(float)) : NULL;
  float* dxc = (float*)malloc(sizeof(float) * n);
  if ((dg && !dg_tmp) || (db && !db_tmp) || !dxc) { free(dg_tmp); free(db_tmp); free(dxc); return -2; }
  for (unsigned k = 0; k < bd; ++k) {
    const float* px = x + (size_t)k * n;
    const float* pdy = dEdf + (size_t)k * n;
    float s0 = 0.f;
    for (size_t j = 0; j < n; ++j) s0 += px[j];
    float mean = s0 / fn;
    float v = 0.f;
    for (size_t j = 0; j < n; ++j) { float d = px[j] - mean; v += d * d; }
    float sigma = sqrtf(v / fn);
    float s = 1e-8f + sigma;
    float neg = -mean;
    float s2 = s * s;
    float ds = 0.f, dneg = 0.f;
    for (size_t j = 0; j < n; ++j) {
      float xc = px[j] + neg;
      float q = xc / s;
      float dgq = pdy[j];
      if (db_tmp) db_tmp[j] += dgq;
      if (dg_tmp) dg_tmp[j] += dgq * q;
      float dq = dgq * g[j];
      dxc[j] = dq / s;
      ds -= dq / s2 * xc;
      dneg += dxc[j];
    }
    if (dx) {
      float dsigma = ds;
      float sb = dsigma / (2.f * sigma);
      float c = 2.f / fn;
      float dmu = -dneg;
      for (size_t j = 0; j < n; ++j) {
        float acc = dx[(size_t)k * n + j];
        acc += c * (px[j] - mean) * sb; /* StdDimension */
        acc += dxc[j];                  /* CwiseSum arg 0 */
        acc += dmu / fn;                /* MomentDimension */
        dx[(size_t)k * n + j] = acc;
      }
    }
  }
  if (dg) for (size_t j = 0; j < n; ++j) dg[j] += dg_tmp[j];
  if (db) for (size_t j = 0; j < n; ++j) db[j] += db_tmp[j];
  free(dg_tmp); free(db_tmp); free(dxc);
  return 0;
}

/* ======================================================================== */
/* GEMM shim                                                                 */
/* ======================================================================== */

/* MatrixMultiply, CPU: dynet/matrix-multiply.h:45-55: y = acc*y, then
 * colbatch(y) += l * colbatch(r) with l unbatched (the batch of r folds into
 * columns).  Naive sequential-k fp32 dot products: Eigen's GEMM blocking and
 * summation order are parity unpinned at the Eigen boundary. */
int orc_gemm_nn(size_t M, size_t N, size_t K, const float* l, const float* r, float beta, float* y) {
  /* y = beta*y first (matrix-multiply.h:47), then accumulate rank-1 updates in
   * ascending k, so every y[i,j] sums its K products in index order. */
  for (size_t e = 0; e < M * N; ++e) y[e] = beta * y[e];
  for (size_t j = 0; j < N; ++j)
    for (size_t k = 0; k < K; ++k) {
      const float rkj = r[k + j * K];
      const float* lk = l + k * M;
      float* yj = y + j * M;
      for (size_t i = 0; i < M; ++i) yj[i] += lk[i] * rkj;
    }
  return 0;
}

/* MatrixTranspMultiplyAcc, CPU: dynet/matrix-multiply.h:120-125:
 * colbatch(y) += l^T * colbatch(r); l is K x M. */
int orc_gemm_tn_acc(size_t M, size_t N, size_t K, const float* l, const float* r, float* y) {
  for (size_t j = 0; j < N; ++j)
    for (size_t i = 0; i < M; ++i) {
      float acc = 0.f;
      for (size_t k = 0; k < K; ++k) acc += l[k + i * K] * r[k + j * K];
      y[i + j * M] += acc;
    }
  return 0;
}

/* MatrixMultiplyTranspAcc, CPU: dynet/matrix-multiply.h:183-187:
 * y += colbatch(l) * colbatch(r)^T; l is M x K, r is N x K (K folds the
 * batch, which is how the weight gradients sum over the batch). */
int orc_gemm_nt_acc(size_t M, size_t N, size_t K, const float* l, const float* r, float* y) {
  for (size_t k = 0; k < K; ++k)
    for (size_t j = 0; j < N; ++j) {
      const float rjk = r[j + k * N];
      const float* lk = l + k * M;
      float* yj = y + j * M;
      for (size_t i = 0; i < M; ++i) yj[i] += lk[i] * rjk;
    }
  return 0;
}

/* ======================================================================== */
/* fused LSTM nodes                                                          */
/* ======================================================================== */

/* concatenate the inputs along rows: dynet/nodes-lstm.cc:127-141 */
static float* concat_inputs(unsigned num_inputs, const float* const* xs, const unsigned* x_dims,
                            unsigned I, unsigned B) {
  float* x_t = (float*)malloc(sizeof(float) * (size_t)I * B);
  if (!x_t) return NULL;
  unsigned off = 0;
  for (unsigned k = 0; k < num_inputs; ++k) {
    for (unsigned bb = 0; bb < B; ++bb)
      memcpy(x_t + (size_t)bb * I + off, xs[k] + (size_t)bb * x_dims[k], sizeof(float) * x_dims[k]);
    off += x_dims[k];
  }
  return x_t;
}

/* broadcast a mask with batch 1 to B columns: nodes-lstm.cc:158-172,179-193 */
static float* expand_mask(const float* mask, unsigned dim, unsigned mask_bd, unsigned B) {
  float* m = (float*)malloc(sizeof(float) * (size_t)dim * B);
  if (!m) return NULL;
  for (unsigned bb = 0; bb < B; ++bb)
    memcpy(m + (size_t)bb * dim, mask + (mask_bd > 1 ? (size_t)bb * dim : 0), sizeof(float) * dim);
  return m;
}

static float* masked(const float* v, const float* mask, size_t n) {
  float* o = (float*)malloc(sizeof(float) * n);
  if (!o) return NULL;
  for (size_t i = 0; i < n; ++i) o[i] = v[i] * mask[i];
  return o;
}

/* VanillaLSTMGates::forward_dev_impl, dynet/nodes-lstm.cc:101-235 (dim checks
 * :24-59).  fx[4H x B] <- b broadcast (:144-153); rows [H,2H) += 1.0 forget
 * bias (:154, constant nodes-lstm.h:11); optional dropout x*mask_x, h*mask_h
 * (:156-198); fx += Wx*x; fx += Wh*h (:217-218); rows [0,3H) <- logistic,
 * rows [3H,4H) <- tanh (:222-232).  Gate order i, f, o, g.  Weight noise is
 * not restated (the reference skips the GEMMs when it is on, :200-215).
 * Pinned by the 16+16 known-answer values of tests/test-rnn.cc:301-339 and
 * :359-400, and by multi-input == single concatenated input (:462-497). */
int orc_lstm_gates_forward(unsigned num_inputs, const float* const* xs, const unsigned* x_dims,
                           unsigned H, unsigned B, const float* h_tm1, const float* Wx,
                           const float* Wh, const float* b, const float* mask_x,
                           unsigned mask_x_bd, const float* mask_h, unsigned mask_h_bd,
                           int logistic_mode, float* fx) {
  if (num_inputs < 1) return -1;
  unsigned I = 0;
  for (unsigned k = 0; k < num_inputs; ++k) I += x_dims[k];
  int dropout = mask_x != NULL && mask_h != NULL;
  if ((mask_x != NULL) != (mask_h != NULL)) return -1;
  if (dropout && !((mask_x_bd == B || mask_x_bd == 1) && (mask_h_bd == B || mask_h_bd == 1))) return -1;
  size_t G = (size_t)4 * H;
  float* x_t = concat_inputs(num_inputs, xs, x_dims, I, B);
  float *mx = NULL, *mh = NULL, *xd = NULL, *hd = NULL;
  const float* xin = x_t;
  const float* hin = h_tm1;
  if (dropout) {
    mx = expand_mask(mask_x, I, mask_x_bd, B);
    mh = expand_mask(mask_h, H, mask_h_bd, B);
    xd = masked(x_t, mx, (size_t)I * B);
    hd = masked(h_tm1, mh, (size_t)H * B);
    xin = xd; hin = hd;
  }
  for (unsigned bb = 0; bb < B; ++bb) memcpy(fx + bb * G, b, sizeof(float) * G);
  for (unsigned bb = 0; bb < B; ++bb)
    for (unsigned r = H; r < 2 * H; ++r) fx[bb * G + r] += 1.0f;
  orc_gemm_nn(G, B, I, Wx, xin, 1.0f, fx);
  orc_gemm_nn(G, B, H, Wh, hin, 1.0f, fx);
  for (unsigned bb = 0; bb < B; ++bb) {
    for (unsigned r = 0; r < 3 * H; ++r) fx[bb * G + r] = logistic(logistic_mode, fx[bb * G + r]);
    for (unsigned r = 3 * H; r < 4 * H; ++r) fx[bb * G + r] = tanhf(fx[bb * G + r]);
  }
  free(x_t); free(mx); free(mh); free(xd); free(hd);
  return 0;
}

/* dpre = [dEdf_ifo * fx_ifo * (1 - fx_ifo) ; dEdf_g * (1 - fx_g^2)], recomputed
 * in each backward call by the reference (nodes-lstm.cc:358-361,403-406,
 * 454-457,487-490,515-519).  Uses the node OUTPUT fx. */
static float* lstm_dpre(unsigned H, unsigned B, const float* fx, const float* dEdf) {
  size_t G = (size_t)4 * H;
  float* d = (float*)malloc(sizeof(float) * G * B);
  if (!d) return NULL;
  for (unsigned bb = 0; bb < B; ++bb) {
    for (unsigned r = 0; r < 3 * H; ++r) {
      size_t k = bb * G + r;
      d[k] = dEdf[k] * fx[k] * (1.f - fx[k]);
    }
    for (unsigned r = 3 * H; r < 4 * H; ++r) {
      size_t k = bb * G + r;
      d[k] = dEdf[k] * (1.f - fx[k] * fx[k]);
    }
  }
  return d;
}

/* VanillaLSTMGates::backward_dev_impl, dynet/nodes-lstm.cc:237-527.
 *   i < num_inputs : dx_i += Wx[:, slice_i]^T dpre  (:326-383; under dropout
 *                    the product goes to a zeroed temp and dx += temp * mask slice)
 *   i = num_inputs : dh += Wh^T dpre                 (:384-417)
 *   i = +1         : dWx += dpre * x_t^T (x_t masked under dropout, :419-467)
 *   i = +2         : dWh += dpre * h^T               (:469-500)
 *   i = +3         : db += sum_b dpre                (:502-520)
 * Masks get no gradient (:522).  Pinned by central differences on the inputs
 * of tests/test-rnn.cc:341-357,402-460,499-529,601-630 and by the adjoint
 * identity <dy, J v> = <J^T dy, v> in fp64. */
int orc_lstm_gates_backward(unsigned num_inputs, const float* const* xs, const unsigned* x_dims,
                            unsigned H, unsigned B, const float* h_tm1, const float* Wx,
                            const float* Wh, const float* mask_x, unsigned mask_x_bd,
                            const float* mask_h, unsigned mask_h_bd, const float* fx,
                            const float* dEdf, unsigned i, float* dEdxi) {
  if (num_inputs < 1 || i > num_inputs + 3) return -1;
  unsigned I = 0;
  for (unsigned k = 0; k < num_inputs; ++k) I += x_dims[k];
  int dropout = mask_x != NULL && mask_h != NULL;
  size_t G = (size_t)4 * H;
  float* dpre = lstm_dpre(H, B, fx, dEdf);
  if (!dpre) return -2;
  float *mx = NULL, *mh = NULL;
  if (dropout) {
    mx = expand_mask(mask_x, I, mask_x_bd, B);
    mh = expand_mask(mask_h, H, mask_h_bd, B);
  }
  if (i < num_inputs) {
    unsigned off = 0;
    for (unsigned j = 0; j < i; ++j) off += x_dims[j];
    unsigned di = x_dims[i];
    const float* Wx_slice = Wx + (size_t)off * G; /* columns [off, off+di) */
    if (dropout) {
      float* tmp = (float*)calloc((size_t)di * B, sizeof(float));
      orc_gemm_tn_acc(di, B, G, Wx_slice, dpre, tmp);
      for (unsigned bb = 0; bb < B; ++bb)
        for (unsigned r = 0; r < di; ++r)
          dEdxi[(size_t)bb * di + r] += tmp[(size_t)bb * di + r] * mx[(size_t)bb * I + off + r];
      free(tmp);
    } else {
      orc_gemm_tn_acc(di, B, G, Wx_slice, dpre, dEdxi);
    }
  } else if (i == num_inputs) {
    if (dropout) {
      float* tmp = (float*)calloc((size_t)H * B, sizeof(float));
      orc_gemm_tn_acc(H, B, G, Wh, dpre, tmp);
      for (size_t k = 0; k < (size_t)H * B; ++k) dEdxi[k] += tmp[k] * mh[k];
      free(tmp);
    } else {
      orc_gemm_tn_acc(H, B, G, Wh, dpre, dEdxi);
    }
  } else if (i == num_inputs + 1) {
    float* x_t = concat_inputs(num_inputs, xs, x_dims, I, B);
    if (dropout) {
      float* xd = masked(x_t, mx, (size_t)I * B);
      free(x_t); x_t = xd;
    }
    orc_gemm_nt_acc(G, I, B, dpre, x_t, dEdxi);
    free(x_t);
  } else if (i == num_inputs + 2) {
    if (dropout) {
      float* hd = masked(h_tm1, mh, (size_t)H * B);
      orc_gemm_nt_acc(G, H, B, dpre, hd, dEdxi);
      free(hd);
    } else {
      orc_gemm_nt_acc(G, H, B, dpre, h_tm1, dEdxi);
    }
  } else {
    for (size_t r = 0; r < G; ++r) {
      float s = 0.f;
      for (unsigned bb = 0; bb < B; ++bb) s += dpre[bb * G + r];
      dEdxi[r] += s;
    }
  }
  free(dpre); free(mx); free(mh);
  return 0;
}

/* VanillaLSTMC::forward_dev_impl, dynet/nodes-lstm.cc:562-589:
 * c = i*g + f*c_prev.  Pinned by tests/test-rnn.cc:285-300. */
int orc_lstm_c_forward(unsigned H, unsigned B, const float* c_tm1, const float* gates, float* c) {
  for (unsigned bb = 0; bb < B; ++bb) {
    const float* gt = gates + (size_t)bb * 4 * H;
    for (unsigned r = 0; r < H; ++r)
      c[(size_t)bb * H + r] = gt[r] * gt[3 * H + r] + gt[H + r] * c_tm1[(size_t)bb * H + r];
  }
  return 0;
}

/* VanillaLSTMC::backward_dev_impl, dynet/nodes-lstm.cc:591-615.
 * i=0: dc_prev += dc*f.  i=1: di += dc*g; df += dc*c_prev; dg += dc*i (the o
 * rows are untouched). */
int orc_lstm_c_backward(unsigned H, unsigned B, const float* c_tm1, const float* gates,
                        const float* dEdf, unsigned i, float* dEdxi) {
  if (i > 1) return -1;
  for (unsigned bb = 0; bb < B; ++bb) {
    const float* gt = gates + (size_t)bb * 4 * H;
    const float* dc = dEdf + (size_t)bb * H;
    if (i == 0) {
      for (unsigned r = 0; r < H; ++r) dEdxi[(size_t)bb * H + r] += dc[r] * gt[H + r];
    } else {
      float* dg = dEdxi + (size_t)bb * 4 * H;
      for (unsigned r = 0; r < H; ++r) {
        dg[r] += dc[r] * gt[3 * H + r];
        dg[H + r] += dc[r] * c_tm1[(size_t)bb * H + r];
        dg[3 * H + r] += dc[r] * gt[r];
      }
    }
  }
  return 0;
}

/* VanillaLSTMH::forward_dev_impl, dynet/nodes-lstm.cc:650-668: h = o*tanh(c).
 * Pinned by tests/test-rnn.cc:245-259. */
int orc_lstm_h_forward(unsigned H, unsigned B, const float* c, const float* gates, float* h) {
  for (unsigned bb = 0; bb < B; ++bb) {
    const float* gt = gates + (size_t)bb * 4 * H;
    for (unsigned r = 0; r < H; ++r) h[(size_t)bb * H + r] = gt[2 * H + r] * tanhf(c[(size_t)bb * H + r]);
  }
  return 0;
}

/* VanillaLSTMH::backward_dev_impl, dynet/nodes-lstm.cc:670-703.
 * i=0: dc += dh*o*(1 - tanh(c)^2) (tanh recomputed, :692-694);
 * i=1: do += dh*tanh(c) into rows [2H,3H). */
int orc_lstm_h_backward(unsigned H, unsigned B, const float* c, const float* gates,
                        const float* dEdf, unsigned i, float* dEdxi) {
  if (i > 1) return -1;
  for (unsigned bb = 0; bb < B; ++bb) {
    const float* gt = gates + (size_t)bb * 4 * H;
    for (unsigned r = 0; r < H; ++r) {
      float t = tanhf(c[(size_t)bb * H + r]);
      float dh = dEdf[(size_t)bb * H + r];
      if (i == 0) dEdxi[(size_t)bb * H + r] += dh * gt[2 * H + r] * (1.f - t * t);
      else dEdxi[(size_t)bb * 4 * H + 2 * H + r] += dh * t;
    }
  }
  return 0;
}

/* ======================================================================== */
/* lookup                                                                    */
/* ======================================================================== */

/* LookupNode::forward_dev_impl, dynet/param-nodes.cc:304-329 (CPU branch
 * :321-327): fx[:,b] = table[:, ids[b]] * current_weight_decay(); every id is
 * bounds-checked (:323).  Row r of the table is contiguous at r*dim
 * (dynet/model.cc:146-159).  With mult == 1.0f the result is a bit-exact
 * gather.  Pinned by memcmp against table[ids] in tests. */
int orc_lookup_forward(unsigned n_ids, const unsigned* ids, size_t dim, unsigned vocab,
                       const float* table, float mult, float* fx) {
  for (unsigned b = 0; b < n_ids; ++b) {
    if (ids[b] >= vocab) return -1;
    const float* row = table + (size_t)ids[b] * dim;
    for (size_t j = 0; j < dim; ++j) fx[(size_t)b * dim + j] = row[j] * mult;
  }
  return 0;
}

/* LookupParameterStorage::accumulate_grads_dev, CPU branch,
 * dynet/model.cc:728-743: for b in order: grads[ids[b]] += g[:, b].
 * Sequential and deterministic.  Pinned by brute force on duplicate-heavy
 * tiny tables and by sum(all_grads) == sum(g) in fp64. */
int orc_lookup_accumulate_grads(unsigned n_ids, const unsigned* ids, size_t dim, unsigned vocab,
                                const float* g, float* all_grads) {
  for (unsigned b = 0; b < n_ids; ++b) {
    if (ids[b] >= vocab) return -1;
    float* row = all_grads + (size_t)ids[b] * dim;
    for (size_t j = 0; j < dim; ++j) row[j] += g[(size_t)b * dim + j];
  }
  return 0;
}

/* ======================================================================== */
/* logsumexp / pickneglogsoftmax                                             */
/* ======================================================================== */

/* TensorTools::logsumexp_dev, CPU branch, dynet/tensor.cc:468-507 for a
 * vector per batch element (axis 0): m = max; z = log(sum exp(x - m)) + m.
 * expf/logf and the sequential sum are parity unpinned at the Eigen
 * boundary.  Pinned by fp64 scipy logsumexp and lse(x+c) = lse(x)+c. */
int orc_logsumexp_cols(size_t rows, unsigned bd, const float* x, float* m, float* z) {
  if (rows == 0) return -1;
  for (unsigned b = 0; b < bd; ++b) {
    const float* px = x + (size_t)b * rows;
    float mx = px[0];
    for (size_t i = 1; i < rows; ++i) mx = px[i] > mx ? px[i] : mx;
    float s = 0.f;
    for (size_t i = 0; i < rows; ++i) s += expf(px[i] - mx);
    m[b] = mx;
    z[b] = logf(s) + mx;
  }
  return 0;
}

/* Sum::forward_dev_impl (dynet/nodes-arith-sum.cc:65-113).  Equal batch sizes: the first
 * (up to) four arguments are added left to right, then the remainder (num_args - 4) % 4,
 * then groups of four, each group added left to right before it is added to fx (:67-89).
 * Mixed batch sizes: fx = 0, then fx += x_i in order, batch-1 arguments broadcast (:91-111).
 * Pinned by fp64 sums and, for the association order, by a case where it changes the bits. */
int orc_sum_forward(unsigned k, size_t n, unsigned bd, const float* const* xs, const unsigned* bds, float* fx) {
  if (k == 0) return -1;
  size_t tot = n * (size_t)bd;
  int same = 1;
  for (unsigned i = 0; i < k; ++i) {
    if (bds[i] != bd && bds[i] != 1) return -1;
    if (bds[i] != bds[0]) same = 0;
  }
  if (same && bds[0] != bd) return -1;
  if (same) {
    unsigned first = k < 4 ? k : 4;
    for (size_t e = 0; e < tot; ++e) {
      float v = xs[0][e];
      for (unsigned i = 1; i < first; ++i) v = v + xs[i][e];
      fx[e] = v;
    }
    if (k <= 4) return 0;
    unsigned rem = (k - 4) % 4, at = 4;
    if (rem) {
      for (size_t e = 0; e < tot; ++e) {
        float v = xs[at][e];
        for (unsigned i = 1; i < rem; ++i) v = v + xs[at + i][e];
        fx[e] += v;
      }
      at += rem;
    }
    for (; at < k; at += 4)
      for (size_t e = 0; e < tot; ++e) fx[e] += ((xs[at][e] + xs[at + 1][e]) + xs[at + 2][e]) + xs[at + 3][e];
    return 0;
  }
  for (size_t e = 0; e < tot; ++e) fx[e] = 0.f;
  for (unsigned i = 0; i < k; ++i)
    for (unsigned b = 0; b < bd; ++b)
      for (size_t j = 0; j < n; ++j) fx[(size_t)b * n + j] += xs[i][(bds[i] == bd ? (size_t)b * n : 0) + j];
  return 0;
}

/* Softmax::forward_dev_impl, dimension 0, CPU branch (dynet/nodes-softmaxes.cc:58-74):
 * per column m = max, fx = exp(x - m), z = sum fx, fx = fx / z.
 * Pinned by fp64 scipy softmax, columns summing to 1 and shift invariance. */
int orc_softmax_forward(size_t rows, unsigned cols, const float* x, float* fx) {
  if (rows == 0) return -1;
  for (unsigned c = 0; c < cols; ++c) {
    const float* px = x + (size_t)c * rows;
    float* pf = fx + (size_t)c * rows;
    float m = px[0];
    for (size_t i = 1; i < rows; ++i) m = px[i] > m ? px[i] : m;
    for (size_t i = 0; i < rows; ++i) pf[i] = expf(px[i] - m);
    float z = 0.f;
    for (size_t i = 0; i < rows; ++i) z += pf[i];
    for (size_t i = 0; i < rows; ++i) pf[i] = pf[i] / z;
  }
  return 0;
}

/* Softmax::backward_dev_impl, dimension 0, CPU branch (dynet/nodes-softmaxes.cc:89-113):
 * z[col] = sum fx*dEdf; dx += (dEdf - z[col]) * fx.  Pinned by central differences. */
int orc_softmax_backward(size_t rows, unsigned cols, const float* fx, const float* dEdf, float* dEdx) {
  for (unsigned c = 0; c < cols; ++c) {
    const float* pf = fx + (size_t)c * rows;
    const float* pd = dEdf + (size_t)c * rows;
    float* po = dEdx + (size_t)c * rows;
    float z = 0.f;
    for (size_t i = 0; i < rows; ++i) z += pf[i] * pd[i];
    for (size_t i = 0; i < rows; ++i) po[i] += (pd[i] - z) * pf[i];
  }
  return 0;
}

/* Softmax::forward_dev_impl, dimension 1 (dynet/nodes-softmaxes.cc:74-85): x is rows x cols per batch
 * element; per (row, batch) m = max over the columns, fx = exp(x - m), z = sum over the columns, fx /= z.
 * Pinned by scipy.special.softmax and by equality with the dimension-0 routine on the transposed matrix. */
int orc_softmax_rows_forward(size_t rows, size_t cols, unsigned bd, const float* x, float* fx) {
  if (rows == 0 || cols == 0) return -1;
  for (unsigned b = 0; b < bd; ++b)
    for (size_t i = 0; i < rows; ++i) {
      const float* px = x + (size_t)b * rows * cols + i;
      float* pf = fx + (size_t)b * rows * cols + i;
      float m = px[0];
      for (size_t j = 1; j < cols; ++j) m = px[j * rows] > m ? px[j * rows] : m;
      for (size_t j = 0; j < cols; ++j) pf[j * rows] = expf(px[j * rows] - m);
      float z = 0.f;
      for (size_t j = 0; j < cols; ++j) z += pf[j * rows];
      for (size_t j = 0; j < cols; ++j) pf[j * rows] = pf[j * rows] / z;
    }
  return 0;
}

/* Softmax::backward_dev_impl, dimension 1 (dynet/nodes-softmaxes.cc:114-122): per (row, batch)
 * z = sum_j fx*dEdf; dx += (dEdf - z) * fx.  Pinned by central differences. */
int orc_softmax_rows_backward(size_t rows, size_t cols, unsigned bd, const float* fx, const float* dEdf, float* dEdx) {
  for (unsigned b = 0; b < bd; ++b)
    for (size_t i = 0; i < rows; ++i) {
      const size_t o = (size_t)b * rows * cols + i;
      float z = 0.f;
      for (size_t j = 0; j < cols; ++j) z += fx[o + j * rows] * dEdf[o + j * rows];
      for (size_t j = 0; j < cols; ++j) dEdx[o + j * rows] += (dEdf[o + j * rows] - z) * fx[o + j * rows];
    }
  return 0;
}

/* LogSumExpDimension::forward_dev_impl (dynet/nodes-logsumexp.cc:126-132) through TensorTools::logsumexp_dev,
 * GPU branch (dynet/tensor.cc:487-496): m = max along `dim`, z = log(sum exp(x - m)) + m.  The result has
 * cols x bd entries for dim 0 and rows x bd for dim 1.  (The reference's CPU branch, :498-504, walks x.d[1]
 * entries whatever the axis and is only right for square matrices; the GPU branch is the one restated.)
 * Pinned by scipy.special.logsumexp. */
int orc_logsumexp_dim_forward(size_t rows, size_t cols, unsigned bd, const float* x, unsigned dim, float* m, float* z) {
  if (rows == 0 || cols == 0 || dim > 1) return -1;
  const size_t len = dim == 0 ? rows : cols, others = dim == 0 ? cols : rows;
  const size_t step = dim == 0 ? 1 : rows, ostep = dim == 0 ? rows : 1;
  for (unsigned b = 0; b < bd; ++b)
    for (size_t o = 0; o < others; ++o) {
      const float* px = x + (size_t)b * rows * cols + o * ostep;
      float mx = px[0];
      for (size_t k = 1; k < len; ++k) mx = px[k * step] > mx ? px[k * step] : mx;
      float s = 0.f;
      for (size_t k = 0; k < len; ++k) s += expf(px[k * step] - mx);
      m[(size_t)b * others + o] = mx;
      z[(size_t)b * others + o] = logf(s) + mx;
    }
  return 0;
}

/* LogSumExpDimension::backward_dev_impl (dynet/nodes-logsumexp.cc:134-145):
 * dx[i,j,b] += exp(x[i,j,b] - fx[o,b]) * dEdf[o,b] with o = j for dim 0 and o = i for dim 1.
 * Pinned by central differences. */
int orc_logsumexp_dim_backward(size_t rows, size_t cols, unsigned bd, const float* x, const float* fx,
                               const float* dEdf, unsigned dim, float* dEdx) {
  if (dim > 1) return -1;
  const size_t others = dim == 0 ? cols : rows;
  for (unsigned b = 0; b < bd; ++b)
    for (size_t j = 0; j < cols; ++j)
      for (size_t i = 0; i < rows; ++i) {
        const size_t e = ((size_t)b * cols + j) * rows + i, o = (size_t)b * others + (dim == 0 ? j : i);
        dEdx[e] += expf(x[e] - fx[o]) * dEdf[o];
      }
  return 0;
}

/* LogSoftmax::forward_dev_impl, CPU branch (dynet/nodes-softmaxes.cc:141-185): aux = [z | m]
 * (2*cols floats, :136-138) from TensorTools::logsumexp; fx = x - z[col]. */
int orc_log_softmax_forward(size_t rows, unsigned cols, const float* x, float* aux, float* fx) {
  float* z = aux;
  float* m = aux + cols;
  if (orc_logsumexp_cols(rows, cols, x, m, z)) return -1;
  for (unsigned c = 0; c < cols; ++c)
    for (size_t i = 0; i < rows; ++i) fx[(size_t)c * rows + i] = x[(size_t)c * rows + i] - z[c];
  return 0;
}

/* LogSoftmax::backward_dev_impl, CPU branch (dynet/nodes-softmaxes.cc:187-213):
 * z[col] = sum dEdf; dx += exp(fx) * -z[col] + dEdf. */
int orc_log_softmax_backward(size_t rows, unsigned cols, const float* fx, const float* dEdf, float* dEdx) {
  for (unsigned c = 0; c < cols; ++c) {
    const float* pf = fx + (size_t)c * rows;
    const float* pd = dEdf + (size_t)c * rows;
    float* po = dEdx + (size_t)c * rows;
    float z = 0.f;
    for (size_t i = 0; i < rows; ++i) z += pd[i];
    for (size_t i = 0; i < rows; ++i) po[i] += (expf(pf[i]) * -z) + pd[i];
  }
  return 0;
}

/* PickNegLogSoftmax::forward_dev_impl, dynet/nodes-pickneglogsoftmax.cc:79-119:
 * aux = [z | m | ids] with ids[b] = b*rows + label_b (:102), labels
 * bounds-checked (:100); fx[b] = z[b] - x[ids[b]] (:113,:115). */
int orc_pnls_forward(size_t rows, unsigned bd, const float* x, const unsigned* labels,
                     void* aux, float* fx) {
  float* z = (float*)aux;
  float* m = z + bd;
  unsigned* ids = (unsigned*)(m + bd);
  for (unsigned b = 0; b < bd; ++b) {
    if (labels[b] >= rows) return -1;
    ids[b] = (unsigned)(rows * b + labels[b]);
  }
  orc_logsumexp_cols(rows, bd, x, m, z);
  for (unsigned b = 0; b < bd; ++b) fx[b] = x[ids[b]];
  for (unsigned b = 0; b < bd; ++b) fx[b] = z[b] - fx[b];
  return 0;
}

/* PickNegLogSoftmax::backward_dev_impl, CPU branch,
 * dynet/nodes-pickneglogsoftmax.cc:122-145: per batch element
 * dx[:,b] += exp(x[:,b] - z[b]) * dy[b]; dx[ids[b]] -= dy[b]. */
int orc_pnls_backward(size_t rows, unsigned bd, const float* x, const void* aux,
                      const float* dEdf, float* dEdx) {
  const float* z = (const float*)aux;
  const unsigned* ids = (const unsigned*)(z + 2 * (size_t)bd);
  for (unsigned b = 0; b < bd; ++b) {
    for (size_t i = 0; i < rows; ++i)
      dEdx[(size_t)b * rows + i] += expf(x[(size_t)b * rows + i] - z[b]) * dEdf[b];
    dEdx[ids[b]] -= dEdf[b];
  }
  return 0;
}

/* LogSumExp node, dynet/nodes-logsumexp.cc:38-74: running max over the k
 * arguments, sum of exp(x_i - max), log + max; arguments with batch 1 are
 * broadcast. */
int orc_logsumexp_node_forward(unsigned k, size_t n, unsigned bd, const float* const* xs,
                               const unsigned* bds, float* fx) {
  if (k == 0) return -1;
  size_t tot = n * (size_t)bd;
  if (k == 1) { memcpy(fx, xs[0], sizeof(float) * tot); return 0; }
  float* ms = (float*)malloc(sizeof(float) * tot);
  if (!ms) return -2;
  for (size_t e = 0; e < tot; ++e) ms[e] = xs[0][bds[0] > 1 ? e : e % n];
  for (unsigned a = 1; a < k; ++a)
    for (size_t e = 0; e < tot; ++e) {
      float v = xs[a][bds[a] > 1 ? e : e % n];
      ms[e] = v > ms[e] ? v : ms[e];
    }
  for (size_t e = 0; e < tot; ++e) fx[e] = expf(xs[0][bds[0] > 1 ? e : e % n] - ms[e]);
  for (unsigned a = 1; a < k; ++a)
    for (size_t e = 0; e < tot; ++e) fx[e] += expf(xs[a][bds[a] > 1 ? e : e % n] - ms[e]);
  for (size_t e = 0; e < tot; ++e) fx[e] = logf(fx[e]) + ms[e];
  free(ms);
  return 0;
}

/* dynet/nodes-logsumexp.cc:77-97: dx_i += exp(x_i - fx) * dy; a batch-1
 * argument receives the sum over the batch. */
int orc_logsumexp_node_backward(unsigned k, size_t n, unsigned bd, const float* const* xs,
                                const unsigned* bds, const float* fx, const float* dEdf,
                                unsigned i, float* dEdxi) {
  if (i >= k) return -1;
  size_t tot = n * (size_t)bd;
  if (k == 1) { for (size_t e = 0; e < tot; ++e) dEdxi[e] += dEdf[e]; return 0; }
  if (bds[i] == bd) {
    for (size_t e = 0; e < tot; ++e) dEdxi[e] += expf(xs[i][e] - fx[e]) * dEdf[e];
  } else {
    for (size_t j = 0; j < n; ++j) {
      float s = 0.f;
      for (unsigned b = 0; b < bd; ++b) s += expf(xs[i][j] - fx[(size_t)b * n + j]) * dEdf[(size_t)b * n + j];
      dEdxi[j] += s;
    }
  }
  return 0;
}

/* TensorTools::argmax_dev, dynet/tensor.cc:527-538 (Eigen argmax along dim 0,
 * 64-bit indices).  Ties resolve to the FIRST maximum here; Eigen's tie rule
 * is parity unpinned at the Eigen boundary.  Pinned by
 * tests/test-tensor.cc:53-61 ({1,2,1;4,5,6} -> {1,2}). */
int orc_argmax_cols(size_t rows, unsigned bd, const float* x, long long* idx) {
  if (rows == 0) return -1;
  for (unsigned b = 0; b < bd; ++b) {
    const float* px = x + (size_t)b * rows;
    size_t best = 0;
    for (size_t i = 1; i < rows; ++i) if (px[i] > px[best]) best = i;
    idx[b] = (long long)best;
  }
  return 0;
}

/* Argmax::forward_dev_impl, dynet/nodes-argmax.cc:44-55: the indices, then fx = 0 with a 1 at
 * idx[b] + b * rows.  Pinned by tests/test-nodes.cc:1277-1288 ({1.1,2.6,3.3 | 4.0,5.1,6.6} -> 0,0,1,0,0,1). */
int orc_argmax_onehot_forward(size_t rows, unsigned bd, const float* x, long long* idx, float* fx) {
  if (orc_argmax_cols(rows, bd, x, idx) != 0) return -1;
  for (size_t e = 0; e < rows * (size_t)bd; ++e) fx[e] = 0.0f;
  for (unsigned b = 0; b < bd; ++b) fx[(size_t)idx[b] + (size_t)b * rows] = 1.0f;
  return 0;
}

/* ======================================================================== */
/* scatter/gather helpers: what dynet/gpu-ops.cu:12-166 computes, restated  */
/* sequentially (the atomics there make the result order-dependent; the     */
/* sequential order is the CPU path's).                                      */
/* ======================================================================== */

int orc_dense_to_sparse_assign(int n, const unsigned* idx, const float* src, float* trg) {
  for (int i = 0; i < n; ++i) trg[idx[i]] = src[i]; /* gpu-ops.cu:12-29 */
  return 0;
}
int orc_sparse_to_dense_assign(int n, const unsigned* idx, const float* src, float* trg) {
  for (int i = 0; i < n; ++i) trg[i] = src[idx[i]]; /* gpu-ops.cu:32-49 */
  return 0;
}
int orc_dense_to_sparse_subtract(int n, const unsigned* idx, const float* src, float* trg) {
  for (int i = 0; i < n; ++i) trg[idx[i]] -= src[i]; /* gpu-ops.cu:52-69 */
  return 0;
}
int orc_sparse_to_dense_block_assign_and_multiply(int n, const unsigned* idx, int bsize, float mult,
                                                  const float* src, float* trg) {
  for (int i = 0; i < n; ++i) /* gpu-ops.cu:72-90 */
    for (int j = 0; j < bsize; ++j) trg[(size_t)i * bsize + j] = src[(size_t)idx[i] * bsize + j] * mult;
  return 0;
}
int orc_dense_to_sparse_block_add(int n, const unsigned* idx, int bsize, const float* src, float* trg) {
  for (int i = 0; i < n; ++i) /* gpu-ops.cu:148-166 */
    for (int j = 0; j < bsize; ++j) trg[(size_t)idx[i] * bsize + j] += src[(size_t)i * bsize + j];
  return 0;
}
/* gpu-ops.cu:93-118 and callers dynet/exec.cc:298-361 */
int orc_parallel_memcpy(int num_seqs, int max_len, float* const* src, float* const* trg,
                        const size_t* len) {
  (void)max_len;
  for (int s = 0; s < num_seqs; ++s) memcpy(trg[s], src[s], sizeof(float) * len[s]);
  return 0;
}
/* gpu-ops.cu:121-145 and callers dynet/exec.cc:363-411 */
int orc_parallel_accumulate(int num_seqs, int max_len, float* const* src, float* const* trg,
                            const size_t* len) {
  (void)max_len;
  for (int s = 0; s < num_seqs; ++s)
    for (size_t i = 0; i < len[s]; ++i) trg[s][i] += src[s][i];
  return 0;
}

/* ======================================================================== */
/* parameter nodes / trainer                                                 */
/* ======================================================================== */

/* ParameterNode::forward_dev_impl, dynet/param-nodes.cc:201-215:
 * fx = values * current_weight_decay(). */
int orc_scale_copy(size_t n, const float* src, float mult, float* dst) {
  for (size_t i = 0; i < n; ++i) dst[i] = src[i] * mult;
  return 0;
}

/* SimpleSGDTrainer::update_rule_dev, dynet/training.cc:619-622:
 * p -= g * (lr * gscale / current_weight_decay). */
int orc_sgd_update(size_t n, float* p, const float* g, float lr, float gscale, float wd) {
  float s = lr * gscale / wd;
  for (size_t i = 0; i < n; ++i) p[i] -= g[i] * s;
  return 0;
}

/* ParameterStorage::g_squared_l2norm_dev, dynet/model.cc (tvec(g).square().sum());
 * sequential fp32 sum: parity unpinned at the Eigen boundary for the order. */
int orc_squared_l2norm(size_t n, const float* g, float* out) {
  float s = 0.f;
  for (size_t i = 0; i < n; ++i) s += g[i] * g[i];
  *out = s;
  return 0;
}

/* ======================================================================== */
/* random tensors                                                            */
/* ======================================================================== */

/* The reference's GPU device draws from cuRAND's Philox4x32-10 keyed with seed + 1
 * (dynet/devices.cc:130-135); its CPU device from std::mt19937.  Neither stream is
 * reproduced: what is restated here is the generator itself (Salmon et al.,
 * "Parallel random numbers: as easy as 1, 2, 3", SC'11: ten rounds of two 32x32->64
 * multiplies with the Weyl-bumped key) and the reference's conversions
 * (dynet/tensor.cc:261-303,446-448).  Pinned by the Random123 known-answer vectors
 * for philox4x32-10; the assignment of counters to tensor elements is this
 * build's own (stated in orc_random_words), parity unpinned against cuRAND's. */
void orc_philox4x32_10(const unsigned ctr[4], const unsigned key[2], unsigned out[4]) {
  unsigned c[4] = {ctr[0], ctr[1], ctr[2], ctr[3]};
  unsigned k[2] = {key[0], key[1]};
  for (int round = 0; round < 10; ++round) {
    if (round > 0) {
      k[0] += 0x9E3779B9u; /* golden ratio */
      k[1] += 0xBB67AE85u; /* sqrt(3) - 1 */
    }
    unsigned long long a = 0xD2511F53ull * c[0];
    unsigned long long b = 0xCD9E8D57ull * c[2];
    unsigned hi_a = (unsigned)(a >> 32), lo_a = (unsigned)a;
    unsigned hi_b = (unsigned)(b >> 32), lo_b = (unsigned)b;
    unsigned n0 = hi_b ^ c[1] ^ k[0];
    unsigned n2 = hi_a ^ c[3] ^ k[1];
    c[0] = n0;
    c[1] = lo_b;
    c[2] = n2;
    c[3] = lo_a;
  }
  for (int i = 0; i < 4; ++i) out[i] = c[i];
}

/* words[k] = word k % 4 of Philox(counter {lo, hi, queue, 0}, key {key_lo, key_hi})
 * where hi:lo = position + k / 4. */
int orc_random_words(unsigned long long key, unsigned long long position, unsigned queue, size_t n,
                     unsigned* words) {
  unsigned kk[2] = {(unsigned)key, (unsigned)(key >> 32)};
  for (size_t k0 = 0; k0 < n; k0 += 4) {
    unsigned long long blk = position + k0 / 4;
    unsigned ctr[4] = {(unsigned)blk, (unsigned)(blk >> 32), queue, 0u}, out[4];
    orc_philox4x32_10(ctr, kk, out);
    for (size_t e = 0; e < 4 && k0 + e < n; ++e) words[k0 + e] = out[e];
  }
  return 0;
}

/* cuRAND's uniform conversion: (0, 1] */
static float unit_interval(unsigned x) {
  float f = (float)x;
  f = f * 2.3283064365386963e-10f; /* 2^-32 */
  return f + 1.1641532182693481e-10f; /* 2^-33 */
}

/* TensorTools::randomize_uniform, GPU branch, dynet/tensor.cc:290-303: uniform in
 * (0, 1], then scale_dev(val, right - left, left) unless the range is (0, 1). */
int orc_randomize_uniform(unsigned long long key, unsigned long long position, unsigned queue, size_t n,
                          float left, float right, float* out) {
  unsigned w[4];
  for (size_t k = 0; k < n; ++k) {
    if (k % 4 == 0) orc_random_words(key, position + k / 4, queue, 4, w);
    float u = unit_interval(w[k % 4]);
    if (left != 0.f || right != 1.f) {
      float a = right - left;
      u = u * a;
      u = u + left;
    }
    out[k] = u;
  }
  return 0;
}

/* TensorTools::randomize_bernoulli, GPU branch, dynet/tensor.cc:261-275:
 * floor(u + p) (uniform_to_bernoulli_dev, :446-448) then * scale. */
int orc_randomize_bernoulli(unsigned long long key, unsigned long long position, unsigned queue, size_t n,
                            float p, float scale, float* out) {
  if (!(p >= 0.f && p <= 1.f)) return -1;
  unsigned w[4];
  for (size_t k = 0; k < n; ++k) {
    if (k % 4 == 0) orc_random_words(key, position + k / 4, queue, 4, w);
    float u = unit_interval(w[k % 4]);
    float s = u + p;
    out[k] = floorf(s) * scale;
  }
  return 0;
}

/* TensorTools::randomize_normal, dynet/tensor.cc:277-288 (curandGenerateNormal):
 * Box-Muller on consecutive word pairs, sine first, as cuRAND does. */
int orc_randomize_normal(unsigned long long key, unsigned long long position, unsigned queue, size_t n,
                         float mean, float stddev, float* out) {
  unsigned w[4];
  for (size_t k = 0; k < n; k += 2) {
    if (k % 4 == 0) orc_random_words(key, position + k / 4, queue, 4, w);
    float u = unit_interval(w[k % 4]);
    float ang = (float)w[k % 4 + 1] * 1.4629180792671596e-9f; /* 2 pi 2^-32 */
    ang = ang + 7.3145903963357980e-10f;                      /* 2 pi 2^-33 */
    float s = sqrtf(-2.0f * logf(u));
    float z0 = s * sinf(ang), z1 = s * cosf(ang);
    z0 = z0 * stddev;
    z1 = z1 * stddev;
    out[k] = z0 + mean;
    if (k + 1 < n) out[k + 1] = z1 + mean;
  }
  return 0;
}

/* Dropout::forward_dev_impl / backward_dev_impl, dynet/nodes-dropout.cc:32-47:
 * m = bernoulli(1 - p) * 1/(1 - p); fx = x (.) m; dEdxi += dEdf (.) m. */
int orc_dropout_forward(unsigned long long key, unsigned long long position, unsigned queue, size_t n, float p,
                        const float* x, float* mask, float* fx) {
  if (!(p >= 0.f && p < 1.f)) return -1;
  float keep = 1.f - p;
  float scale = 1.f / keep;
  int st = orc_randomize_bernoulli(key, position, queue, n, keep, scale, mask);
  if (st) return st;
  for (size_t k = 0; k < n; ++k) fx[k] = x[k] * mask[k];
  return 0;
}

int orc_dropout_backward(size_t n, const float* mask, const float* dEdf, float* dEdxi) {
  for (size_t k = 0; k < n; ++k) dEdxi[k] += dEdf[k] * mask[k];
  return 0;
}

/* ======================================================================== */
/* PickRange                                                                 */
/* ======================================================================== */

/* PickRange::forward_dev_impl / backward_dev_impl, dynet/nodes-select.cc:230-259:
 * fx = x.slice(start along dim, end - start); dEdxi.slice(...) += dEdf.  The tensor
 * is given as inner x len x outer (column-major), the sliced dimension being len. */
int orc_pick_range_forward(size_t inner, size_t len, size_t outer, size_t start, size_t end, const float* x,
                           float* fx) {
  if (!(start < end && end <= len)) return -1;
  size_t w = end - start;
  for (size_t o = 0; o < outer; ++o)
    for (size_t k = 0; k < w; ++k)
      for (size_t i = 0; i < inner; ++i) fx[i + inner * (k + w * o)] = x[i + inner * (start + k + len * o)];
  return 0;
}

int orc_pick_range_backward(size_t inner, size_t len, size_t outer, size_t start, size_t end, const float* dEdf,
                            float* dEdxi) {
  if (!(start < end && end <= len)) return -1;
  size_t w = end - start;
  for (size_t o = 0; o < outer; ++o)
    for (size_t k = 0; k < w; ++k)
      for (size_t i = 0; i < inner; ++i) dEdxi[i + inner * (start + k + len * o)] += dEdf[i + inner * (k + w * o)];
  return 0;
}
