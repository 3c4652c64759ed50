"""ctypes/numpy front end of the CPU oracle (TEST INFRASTRUCTURE ONLY).

Loads ``oracle/libdynet_cpu_oracle.so`` (built by ``oracle/Makefile``) and
wraps every ``orc_*`` function so that tests can call it with numpy arrays.
Only tests, the smoke check and the benchmark's cpu_baseline leg import this
module; the shipped package never does.

All arrays are fp32, laid out as DyNet lays tensors out: column-major with the
batch outermost.  In numpy terms a DyNet tensor of Dim({r, c}, bd) is a
C-contiguous array of shape (bd, c, r); a vector batch Dim({n}, bd) is
(bd, n).  The wrappers only look at the flat buffer, so any C-contiguous
array with the right number of elements works.
"""
import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libdynet_cpu_oracle.so")

OP_TANH, OP_LOGISTIC, OP_RECTIFY, OP_NEGATE, OP_IDENTITY = range(5)
LOGISTIC_PACKET, LOGISTIC_SCALAR = 0, 1


def build(force=False):
    """Compile the oracle with gcc (building the checker is not using it)."""
    args = ["make", "-C", _HERE]
    if force:
        args.append("-B")
    subprocess.run(args, check=True, stdout=subprocess.DEVNULL)


def _load():
    if not os.path.exists(_LIB_PATH):
        build()
    return C.CDLL(_LIB_PATH)


_lib = _load()
_lib.orc_logistic_packet.restype = C.c_float
_lib.orc_logistic_packet.argtypes = [C.c_float]
_lib.orc_logistic_scalar.restype = C.c_float
_lib.orc_logistic_scalar.argtypes = [C.c_float]

_f = C.POINTER(C.c_float)
_u = C.POINTER(C.c_uint)


def _fp(a):
    if a is None:
        return None
    assert a.dtype == np.float32 and a.flags["C_CONTIGUOUS"], (a.dtype, a.flags)
    return a.ctypes.data_as(_f)


def _up(a):
    assert a.dtype == np.uint32 and a.flags["C_CONTIGUOUS"]
    return a.ctypes.data_as(_u)


def _f32(a):
    return np.ascontiguousarray(a, dtype=np.float32)


def _u32(a):
    return np.ascontiguousarray(a, dtype=np.uint32)


def _check(rc, what):
    if rc != 0:
        raise ValueError("%s: oracle returned %d (argument error)" % (what, rc))


def _ptr_array(arrs):
    arr = (_f * len(arrs))(*[_fp(a) for a in arrs])
    return arr


# ---- scalar functors -------------------------------------------------------
def logistic_packet(x):
    return np.array([_lib.orc_logistic_packet(float(v)) for v in np.ravel(x)], np.float32).reshape(np.shape(x))


def logistic_scalar(x):
    return np.array([_lib.orc_logistic_scalar(float(v)) for v in np.ravel(x)], np.float32).reshape(np.shape(x))


# ---- elementwise -----------------------------------------------------------
def unary_forward(op, x, logistic_mode=LOGISTIC_PACKET):
    x = _f32(x)
    y = np.empty_like(x)
    _check(_lib.orc_unary_forward(op, logistic_mode, C.c_size_t(x.size), _fp(x), _fp(y)), "unary_forward")
    return y


def unary_backward(op, fx, dEdf, dEdx):
    """Accumulates into dEdx in place and returns it."""
    fx, dEdf = _f32(fx), _f32(dEdf)
    _check(_lib.orc_unary_backward(op, C.c_size_t(fx.size), _fp(fx), _fp(dEdf), _fp(dEdx)), "unary_backward")
    return dEdx


def _binary_fwd(fn, n, bd0, bd1, a, b):
    a, b = _f32(a), _f32(b)
    y = np.empty((max(bd0, bd1), n), np.float32)
    _check(fn(C.c_size_t(n), bd0, bd1, _fp(a), _fp(b), _fp(y)), fn.__name__)
    return y


def cmult_forward(n, bd0, bd1, a, b):
    return _binary_fwd(_lib.orc_cmult_forward, n, bd0, bd1, a, b)


def csum_forward(n, bd0, bd1, a, b):
    return _binary_fwd(_lib.orc_csum_forward, n, bd0, bd1, a, b)


def cmult_backward(n, bd0, bd1, a, b, dEdf, i, dEdxi):
    _check(_lib.orc_cmult_backward(C.c_size_t(n), bd0, bd1, _fp(_f32(a)), _fp(_f32(b)), _fp(_f32(dEdf)), i,
                                   _fp(dEdxi)), "cmult_backward")
    return dEdxi


def csum_backward(n, bd0, bd1, dEdf, i, dEdxi):
    _check(_lib.orc_csum_backward(C.c_size_t(n), bd0, bd1, _fp(_f32(dEdf)), i, _fp(dEdxi)), "csum_backward")
    return dEdxi


CWISE_SUM, CWISE_MULT, CWISE_QUOTIENT = range(3)


def _dims5(d):
    d = list(d) + [1] * (5 - len(d))
    return (C.c_uint * 5)(*d)


def cwise_forward(op, dims_a, dims_b, a, b):
    """dims: (d0, d1, d2, d3, bd), column-major with the batch outermost; numpy shape = reversed dims."""
    a, b = _f32(a), _f32(b)
    full = [max(x, y) for x, y in zip(dims_a, dims_b)]
    fx = np.empty(tuple(reversed(full)), np.float32)
    _check(_lib.orc_cwise_forward(op, _dims5(dims_a), _dims5(dims_b), _fp(a), _fp(b), _fp(fx)), "cwise_forward")
    return fx


def cwise_backward(op, dims_a, dims_b, a, b, dEdf, i, dEdxi):
    _check(_lib.orc_cwise_backward(op, _dims5(dims_a), _dims5(dims_b), _fp(_f32(a)), _fp(_f32(b)), _fp(_f32(dEdf)), i,
                                   _fp(dEdxi)), "cwise_backward")
    return dEdxi


def const_plus_x_forward(c, x):
    x = _f32(x)
    y = np.empty_like(x)
    _check(_lib.orc_const_plus_x_forward(C.c_size_t(x.size), C.c_float(c), _fp(x), _fp(y)), "const_plus_x")
    return y


def const_minus_x_forward(c, x):
    x = _f32(x)
    y = np.empty_like(x)
    _check(_lib.orc_const_minus_x_forward(C.c_size_t(x.size), C.c_float(c), _fp(x), _fp(y)), "const_minus_x")
    return y


# ---- reductions ------------------------------------------------------------
def sum_batches_forward(n, bd, x):
    x = _f32(x)
    y = np.empty(n, np.float32)
    _check(_lib.orc_sum_batches_forward(C.c_size_t(n), bd, _fp(x), _fp(y)), "sum_batches_forward")
    return y


def sum_batches_backward(n, bd, dEdf, dEdx):
    _check(_lib.orc_sum_batches_backward(C.c_size_t(n), bd, _fp(_f32(dEdf)), _fp(dEdx)), "sum_batches_backward")
    return dEdx


def mean_elems_forward(n, bd, x):
    y = np.empty(bd, np.float32)
    _check(_lib.orc_mean_elems_forward(C.c_size_t(n), bd, _fp(_f32(x)), _fp(y)), "mean_elems_forward")
    return y


def mean_elems_backward(n, bd, dEdf, dEdx):
    _check(_lib.orc_mean_elems_backward(C.c_size_t(n), bd, _fp(_f32(dEdf)), _fp(dEdx)), "mean_elems_backward")
    return dEdx


def std_elems_forward(n, bd, x):
    y = np.empty(bd, np.float32)
    _check(_lib.orc_std_elems_forward(C.c_size_t(n), bd, _fp(_f32(x)), _fp(y)), "std_elems_forward")
    return y


def std_elems_backward(n, bd, x, fx, dEdf, dEdx):
    _check(_lib.orc_std_elems_backward(C.c_size_t(n), bd, _fp(_f32(x)), _fp(_f32(fx)), _fp(_f32(dEdf)),
                                       _fp(dEdx)), "std_elems_backward")
    return dEdx


# ---- layer norm ------------------------------------------------------------
def layer_norm_forward(n, bd, x, g, b):
    y = np.empty((bd, n), np.float32)
    _check(_lib.orc_layer_norm_forward(C.c_size_t(n), bd, _fp(_f32(x)), _fp(_f32(g)), _fp(_f32(b)), _fp(y)),
           "layer_norm_forward")
    return y


def layer_norm_backward(n, bd, x, g, dEdf, dx=None, dg=None, db=None):
    _check(_lib.orc_layer_norm_backward(C.c_size_t(n), bd, _fp(_f32(x)), _fp(_f32(g)), _fp(_f32(dEdf)),
                                        _fp(dx), _fp(dg), _fp(db)), "layer_norm_backward")
    return dx, dg, db


# ---- GEMM ------------------------------------------------------------------
def gemm_nn(M, N, K, l, r, beta, y):
    _check(_lib.orc_gemm_nn(C.c_size_t(M), C.c_size_t(N), C.c_size_t(K), _fp(_f32(l)), _fp(_f32(r)),
                            C.c_float(beta), _fp(y)), "gemm_nn")
    return y


def gemm_tn_acc(M, N, K, l, r, y):
    _check(_lib.orc_gemm_tn_acc(C.c_size_t(M), C.c_size_t(N), C.c_size_t(K), _fp(_f32(l)), _fp(_f32(r)), _fp(y)),
           "gemm_tn_acc")
    return y


def gemm_nt_acc(M, N, K, l, r, y):
    _check(_lib.orc_gemm_nt_acc(C.c_size_t(M), C.c_size_t(N), C.c_size_t(K), _fp(_f32(l)), _fp(_f32(r)), _fp(y)),
           "gemm_nt_acc")
    return y


# ---- LSTM ------------------------------------------------------------------
def _lstm_common(xs, x_dims):
    xs = [_f32(x) for x in xs]
    dims = (C.c_uint * len(xs))(*[int(d) for d in x_dims])
    return xs, _ptr_array(xs), dims


def lstm_gates_forward(xs, x_dims, H, B, h_tm1, Wx, Wh, b, mask_x=None, mask_x_bd=0, mask_h=None, mask_h_bd=0,
                       logistic_mode=LOGISTIC_PACKET):
    xs, xp, dims = _lstm_common(xs, x_dims)
    fx = np.empty((B, 4 * H), np.float32)
    mx = None if mask_x is None else _f32(mask_x)
    mh = None if mask_h is None else _f32(mask_h)
    _check(_lib.orc_lstm_gates_forward(len(xs), xp, dims, H, B, _fp(_f32(h_tm1)), _fp(_f32(Wx)), _fp(_f32(Wh)),
                                       _fp(_f32(b)), _fp(mx), mask_x_bd, _fp(mh), mask_h_bd, logistic_mode,
                                       _fp(fx)), "lstm_gates_forward")
    return fx


def lstm_gates_backward(xs, x_dims, H, B, h_tm1, Wx, Wh, fx, dEdf, i, dEdxi, mask_x=None, mask_x_bd=0,
                        mask_h=None, mask_h_bd=0):
    xs, xp, dims = _lstm_common(xs, x_dims)
    mx = None if mask_x is None else _f32(mask_x)
    mh = None if mask_h is None else _f32(mask_h)
    _check(_lib.orc_lstm_gates_backward(len(xs), xp, dims, H, B, _fp(_f32(h_tm1)), _fp(_f32(Wx)), _fp(_f32(Wh)),
                                        _fp(mx), mask_x_bd, _fp(mh), mask_h_bd, _fp(_f32(fx)), _fp(_f32(dEdf)),
                                        i, _fp(dEdxi)), "lstm_gates_backward")
    return dEdxi


def lstm_c_forward(H, B, c_tm1, gates):
    c = np.empty((B, H), np.float32)
    _check(_lib.orc_lstm_c_forward(H, B, _fp(_f32(c_tm1)), _fp(_f32(gates)), _fp(c)), "lstm_c_forward")
    return c


def lstm_c_backward(H, B, c_tm1, gates, dEdf, i, dEdxi):
    _check(_lib.orc_lstm_c_backward(H, B, _fp(_f32(c_tm1)), _fp(_f32(gates)), _fp(_f32(dEdf)), i, _fp(dEdxi)),
           "lstm_c_backward")
    return dEdxi


def lstm_h_forward(H, B, c, gates):
    h = np.empty((B, H), np.float32)
    _check(_lib.orc_lstm_h_forward(H, B, _fp(_f32(c)), _fp(_f32(gates)), _fp(h)), "lstm_h_forward")
    return h


def lstm_h_backward(H, B, c, gates, dEdf, i, dEdxi):
    _check(_lib.orc_lstm_h_backward(H, B, _fp(_f32(c)), _fp(_f32(gates)), _fp(_f32(dEdf)), i, _fp(dEdxi)),
           "lstm_h_backward")
    return dEdxi


# ---- lookup ----------------------------------------------------------------
def lookup_forward(ids, dim, vocab, table, mult=1.0):
    ids = _u32(ids)
    fx = np.empty((ids.size, dim), np.float32)
    _check(_lib.orc_lookup_forward(ids.size, _up(ids), C.c_size_t(dim), vocab, _fp(_f32(table)), C.c_float(mult),
                                   _fp(fx)), "lookup_forward")
    return fx


def lookup_accumulate_grads(ids, dim, vocab, g, all_grads):
    ids = _u32(ids)
    _check(_lib.orc_lookup_accumulate_grads(ids.size, _up(ids), C.c_size_t(dim), vocab, _fp(_f32(g)),
                                            _fp(all_grads)), "lookup_accumulate_grads")
    return all_grads


# ---- logsumexp / pnls ------------------------------------------------------
def logsumexp_cols(rows, bd, x):
    m = np.empty(bd, np.float32)
    z = np.empty(bd, np.float32)
    _check(_lib.orc_logsumexp_cols(C.c_size_t(rows), bd, _fp(_f32(x)), _fp(m), _fp(z)), "logsumexp_cols")
    return m, z


def sum_forward(n, bd, xs, bds):
    """Sum node; its backward per argument is csum_backward (dx_i += dEdf, batch-summed for batch-1 arguments)."""
    xs = [_f32(x) for x in xs]
    fx = np.empty((bd, n), np.float32)
    bds_c = (C.c_uint * len(xs))(*bds)
    _check(_lib.orc_sum_forward(len(xs), C.c_size_t(n), bd, _ptr_array(xs), bds_c, _fp(fx)), "sum_forward")
    return fx


def softmax_forward(rows, cols, x):
    fx = np.empty((cols, rows), np.float32)
    _check(_lib.orc_softmax_forward(C.c_size_t(rows), cols, _fp(_f32(x)), _fp(fx)), "softmax_forward")
    return fx


def softmax_backward(rows, cols, fx, dEdf, dEdx):
    _check(_lib.orc_softmax_backward(C.c_size_t(rows), cols, _fp(_f32(fx)), _fp(_f32(dEdf)), _fp(dEdx)),
           "softmax_backward")
    return dEdx


def softmax_rows_forward(rows, cols, bd, x):
    """Softmax along dim 1; x and the result are (bd, cols, rows) arrays (column-major matrices per batch element)."""
    fx = np.empty((bd, cols, rows), np.float32)
    _check(_lib.orc_softmax_rows_forward(C.c_size_t(rows), C.c_size_t(cols), bd, _fp(_f32(x)), _fp(fx)),
           "softmax_rows_forward")
    return fx


def softmax_rows_backward(rows, cols, bd, fx, dEdf, dEdx):
    _check(_lib.orc_softmax_rows_backward(C.c_size_t(rows), C.c_size_t(cols), bd, _fp(_f32(fx)), _fp(_f32(dEdf)),
                                          _fp(dEdx)), "softmax_rows_backward")
    return dEdx


def logsumexp_dim_forward(rows, cols, bd, x, dim):
    """Returns (m, z), each (bd, cols) for dim 0 and (bd, rows) for dim 1."""
    others = cols if dim == 0 else rows
    m, z = np.empty((bd, others), np.float32), np.empty((bd, others), np.float32)
    _check(_lib.orc_logsumexp_dim_forward(C.c_size_t(rows), C.c_size_t(cols), bd, _fp(_f32(x)), dim, _fp(m), _fp(z)),
           "logsumexp_dim_forward")
    return m, z


def logsumexp_dim_backward(rows, cols, bd, x, fx, dEdf, dim, dEdx):
    _check(_lib.orc_logsumexp_dim_backward(C.c_size_t(rows), C.c_size_t(cols), bd, _fp(_f32(x)), _fp(_f32(fx)),
                                           _fp(_f32(dEdf)), dim, _fp(dEdx)), "logsumexp_dim_backward")
    return dEdx


def log_softmax_forward(rows, cols, x):
    """Returns (fx, aux) with aux = [z | m]."""
    fx = np.empty((cols, rows), np.float32)
    aux = np.empty(2 * cols, np.float32)
    _check(_lib.orc_log_softmax_forward(C.c_size_t(rows), cols, _fp(_f32(x)), _fp(aux), _fp(fx)),
           "log_softmax_forward")
    return fx, aux


def log_softmax_backward(rows, cols, fx, dEdf, dEdx):
    _check(_lib.orc_log_softmax_backward(C.c_size_t(rows), cols, _fp(_f32(fx)), _fp(_f32(dEdf)), _fp(dEdx)),
           "log_softmax_backward")
    return dEdx


def pnls_forward(rows, bd, x, labels):
    """Returns (fx[bd], aux) with aux the raw 3*bd*4-byte buffer [z|m|ids]."""
    labels = _u32(labels)
    aux = np.empty(3 * bd, np.float32)
    fx = np.empty(bd, np.float32)
    _check(_lib.orc_pnls_forward(C.c_size_t(rows), bd, _fp(_f32(x)), _up(labels), aux.ctypes.data_as(C.c_void_p),
                                 _fp(fx)), "pnls_forward")
    return fx, aux


def pnls_backward(rows, bd, x, aux, dEdf, dEdx):
    _check(_lib.orc_pnls_backward(C.c_size_t(rows), bd, _fp(_f32(x)), aux.ctypes.data_as(C.c_void_p),
                                  _fp(_f32(dEdf)), _fp(dEdx)), "pnls_backward")
    return dEdx


def logsumexp_node_forward(n, bd, xs, bds):
    xs = [_f32(x) for x in xs]
    fx = np.empty((bd, n), np.float32)
    bds_c = (C.c_uint * len(xs))(*bds)
    _check(_lib.orc_logsumexp_node_forward(len(xs), C.c_size_t(n), bd, _ptr_array(xs), bds_c, _fp(fx)),
           "logsumexp_node_forward")
    return fx


def logsumexp_node_backward(n, bd, xs, bds, fx, dEdf, i, dEdxi):
    xs = [_f32(x) for x in xs]
    bds_c = (C.c_uint * len(xs))(*bds)
    _check(_lib.orc_logsumexp_node_backward(len(xs), C.c_size_t(n), bd, _ptr_array(xs), bds_c, _fp(_f32(fx)),
                                            _fp(_f32(dEdf)), i, _fp(dEdxi)), "logsumexp_node_backward")
    return dEdxi


def argmax_cols(rows, bd, x):
    idx = np.empty(bd, np.int64)
    _check(_lib.orc_argmax_cols(C.c_size_t(rows), bd, _fp(_f32(x)), idx.ctypes.data_as(C.POINTER(C.c_longlong))),
           "argmax_cols")
    return idx


def argmax_onehot_forward(rows, bd, x):
    """Argmax node: (indices, one-hot output)."""
    idx = np.empty(bd, np.int64)
    fx = np.empty((bd, rows), np.float32)
    _check(_lib.orc_argmax_onehot_forward(C.c_size_t(rows), bd, _fp(_f32(x)), idx.ctypes.data_as(C.POINTER(C.c_longlong)),
                                          _fp(fx)), "argmax_onehot_forward")
    return idx, fx


# ---- scatter / gather helpers ---------------------------------------------
def dense_to_sparse_assign(idx, src, trg):
    idx = _u32(idx)
    _lib.orc_dense_to_sparse_assign(idx.size, _up(idx), _fp(_f32(src)), _fp(trg))
    return trg


def sparse_to_dense_assign(idx, src):
    idx = _u32(idx)
    trg = np.empty(idx.size, np.float32)
    _lib.orc_sparse_to_dense_assign(idx.size, _up(idx), _fp(_f32(src)), _fp(trg))
    return trg


def dense_to_sparse_subtract(idx, src, trg):
    idx = _u32(idx)
    _lib.orc_dense_to_sparse_subtract(idx.size, _up(idx), _fp(_f32(src)), _fp(trg))
    return trg


def sparse_to_dense_block_assign_and_multiply(idx, bsize, mult, src):
    idx = _u32(idx)
    trg = np.empty((idx.size, bsize), np.float32)
    _lib.orc_sparse_to_dense_block_assign_and_multiply(idx.size, _up(idx), bsize, C.c_float(mult), _fp(_f32(src)),
                                                       _fp(trg))
    return trg


def dense_to_sparse_block_add(idx, bsize, src, trg):
    idx = _u32(idx)
    _lib.orc_dense_to_sparse_block_add(idx.size, _up(idx), bsize, _fp(_f32(src)), _fp(trg))
    return trg


# ---- parameter nodes / trainer --------------------------------------------
def scale_copy(src, mult):
    src = _f32(src)
    dst = np.empty_like(src)
    _lib.orc_scale_copy(C.c_size_t(src.size), _fp(src), C.c_float(mult), _fp(dst))
    return dst


def sgd_update(p, g, lr, gscale=1.0, wd=1.0):
    _lib.orc_sgd_update(C.c_size_t(p.size), _fp(p), _fp(_f32(g)), C.c_float(lr), C.c_float(gscale), C.c_float(wd))
    return p


def squared_l2norm(g):
    g = _f32(g)
    out = C.c_float(0)
    _lib.orc_squared_l2norm(C.c_size_t(g.size), _fp(g), C.byref(out))
    return np.float32(out.value)


# ---- random tensors --------------------------------------------------------
def philox4x32_10(ctr, key):
    c = (C.c_uint * 4)(*[int(v) & 0xFFFFFFFF for v in ctr])
    k = (C.c_uint * 2)(*[int(v) & 0xFFFFFFFF for v in key])
    out = (C.c_uint * 4)()
    _lib.orc_philox4x32_10(c, k, out)
    return [int(v) for v in out]


def random_words(key, position, queue, n):
    out = np.empty(n, np.uint32)
    _lib.orc_random_words(C.c_ulonglong(key), C.c_ulonglong(position), C.c_uint(queue), C.c_size_t(n),
                          out.ctypes.data_as(C.POINTER(C.c_uint)))
    return out


def _rng_args(key, position, queue, n):
    return C.c_ulonglong(key), C.c_ulonglong(position), C.c_uint(queue), C.c_size_t(n)


def randomize_uniform(key, position, queue, n, left=0.0, right=1.0):
    out = np.empty(n, np.float32)
    _check(_lib.orc_randomize_uniform(*_rng_args(key, position, queue, n), C.c_float(left), C.c_float(right),
                                     _fp(out)), "randomize_uniform")
    return out


def randomize_bernoulli(key, position, queue, n, p, scale=1.0):
    out = np.empty(n, np.float32)
    _check(_lib.orc_randomize_bernoulli(*_rng_args(key, position, queue, n), C.c_float(p), C.c_float(scale),
                                       _fp(out)), "randomize_bernoulli")
    return out


def randomize_normal(key, position, queue, n, mean=0.0, stddev=1.0):
    out = np.empty(n, np.float32)
    _check(_lib.orc_randomize_normal(*_rng_args(key, position, queue, n), C.c_float(mean), C.c_float(stddev),
                                    _fp(out)), "randomize_normal")
    return out


def dropout_forward(key, position, queue, p, x):
    x = _f32(x)
    mask, fx = np.empty_like(x), np.empty_like(x)
    _check(_lib.orc_dropout_forward(*_rng_args(key, position, queue, x.size), C.c_float(p), _fp(x), _fp(mask),
                                   _fp(fx)), "dropout_forward")
    return mask, fx


def dropout_backward(mask, dEdf, dEdxi):
    _check(_lib.orc_dropout_backward(C.c_size_t(mask.size), _fp(_f32(mask)), _fp(_f32(dEdf)), _fp(dEdxi)),
           "dropout_backward")
    return dEdxi


# ---- PickRange -------------------------------------------------------------
def pick_range_forward(inner, length, outer, start, end, x):
    x = _f32(x)
    fx = np.empty(inner * max(end - start, 0) * outer, np.float32)
    _check(_lib.orc_pick_range_forward(C.c_size_t(inner), C.c_size_t(length), C.c_size_t(outer), C.c_size_t(start),
                                       C.c_size_t(end), _fp(x), _fp(fx)), "pick_range_forward")
    return fx


def pick_range_backward(inner, length, outer, start, end, dEdf, dEdxi):
    _check(_lib.orc_pick_range_backward(C.c_size_t(inner), C.c_size_t(length), C.c_size_t(outer), C.c_size_t(start),
                                        C.c_size_t(end), _fp(_f32(dEdf)), _fp(dEdxi)), "pick_range_backward")
    return dEdxi
