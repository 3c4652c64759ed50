"""Host-side mirror of DyNet's Device / pools / Tensor plumbing over the C-ABI.

``Device`` owns a ``dyhip_device`` (one HIP stream, four bump pools FXS / DEDFS /
PS / SCS, the three device scalars).  ``DevTensor`` is DyNet's ``Tensor`` reduced
to what the kernels need: a device pointer plus a shape.  Every method is a
direct call into ``libdynet_hip.so``; a non-zero status raises ``DyhipError``
with the library's message (the adapter-side equivalent of rethrowing
``dynet::cuda_exception`` / ``std::invalid_argument``).
"""
import ctypes as C

import numpy as np

from . import lib
from .lib import cdll

_vp = C.c_void_p
_sz = C.c_size_t
_u = C.c_uint
_f = C.c_float
_i = C.c_int


class DyhipError(RuntimeError):
    def __init__(self, status, message):
        super().__init__("dyhip status %d: %s" % (status, message))
        self.status = status


def _check(status):
    if status != lib.OK:
        raise DyhipError(status, lib.last_error())


def device_count():
    n = _i(0)
    status = cdll.dyhip_device_count(C.byref(n))
    if status == lib.ERR_NO_DEVICE:
        return 0
    _check(status)
    return n.value


class DevTensor:
    """A device buffer with a shape (numpy order: batch outermost, DyNet's column-major inside)."""

    __slots__ = ("dev", "ptr", "shape", "dtype")

    def __init__(self, dev, ptr, shape, dtype=np.float32):
        self.dev = dev
        self.ptr = int(ptr)
        self.shape = tuple(int(s) for s in shape)
        self.dtype = np.dtype(dtype)

    @property
    def size(self):
        return int(np.prod(self.shape)) if self.shape else 1

    @property
    def nbytes(self):
        return self.size * self.dtype.itemsize

    def numpy(self):
        out = np.empty(self.shape, self.dtype)
        if out.nbytes:
            _check(cdll.dyhip_memcpy_d2h(self.dev.handle, _vp(out.ctypes.data), _vp(self.ptr), _sz(out.nbytes)))
        return out

    def set(self, array):
        a = np.ascontiguousarray(array, dtype=self.dtype)
        assert a.size == self.size, (a.shape, self.shape)
        if a.nbytes:
            _check(cdll.dyhip_memcpy_h2d(self.dev.handle, _vp(self.ptr), _vp(a.ctypes.data), _sz(a.nbytes)))
            self.dev.sync()  # the source array may be a temporary
        return self

    def offset(self, elems, shape):
        return DevTensor(self.dev, self.ptr + elems * self.dtype.itemsize, shape, self.dtype)


def _p(t):
    if t is None:
        return _vp(None)
    if isinstance(t, DevTensor):
        return _vp(t.ptr)
    return _vp(int(t))


class PinnedArray:
    """A page-locked host array (numpy view over dyhip_host_alloc memory) for asynchronous host->device copies."""

    def __init__(self, shape, dtype=np.float32):
        self.shape, self.dtype = tuple(int(s) for s in shape), np.dtype(dtype)
        self.nbytes = int(np.prod(self.shape)) * self.dtype.itemsize
        p = _vp(None)
        _check(cdll.dyhip_host_alloc(_sz(max(self.nbytes, 1)), C.byref(p)))
        self.ptr = p.value
        self.array = np.frombuffer((C.c_char * self.nbytes).from_address(self.ptr), dtype=self.dtype).reshape(self.shape)

    def close(self):
        if self.ptr:
            self.array = None
            cdll.dyhip_host_free(_vp(self.ptr))
            self.ptr = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


class Device:
    """One GPU: stream, pools, scalars.  ``mem_mb`` = MiB for (FXS, DEDFS, PS, SCS)."""

    def __init__(self, ordinal=0, mem_mb=(128, 128, 128, 128)):
        self.handle = None
        sizes = (_sz * 4)(*[int(m) for m in mem_mb])
        h = _vp(None)
        _check(cdll.dyhip_device_create(_i(ordinal), sizes, C.byref(h)))
        self.handle = h
        self.ordinal = ordinal

    def fork(self):
        """A second in-order queue on the same GPU (own stream and split-K workspace, shared pools)."""
        h = _vp(None)
        _check(cdll.dyhip_device_fork(self.handle, C.byref(h)))
        q = Device.__new__(Device)
        q.handle, q.ordinal, q._parent = h, self.ordinal, self
        self._forks = getattr(self, "_forks", [])
        self._forks.append(q)
        return q

    def wait(self, other):
        """Work issued on this queue from now on runs after what has been issued on ``other`` so far."""
        _check(cdll.dyhip_device_wait(self.handle, other.handle))

    def close(self):
        if self.handle is not None:
            for q in getattr(self, "_forks", []):
                q.handle = None  # the library destroys live forked queues with their device
            cdll.dyhip_device_destroy(self.handle)
            self.handle = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    # ---- plumbing ---------------------------------------------------------
    def sync(self):
        _check(cdll.dyhip_device_sync(self.handle))

    def set_gemm_handoff(self, spin_limit=1 << 22, raise_flags=True):
        """Bounded wait of the large GEMM's hand-off between blocks (a test hook for its error path)."""
        _check(cdll.dyhip_device_set_gemm_handoff(self.handle, _u(int(spin_limit)), _i(1 if raise_flags else 0)))

    def set_stream_threshold(self, nbytes):
        _check(cdll.dyhip_device_set_stream_threshold(self.handle, _sz(int(nbytes))))

    def pool(self, which):
        p = _vp(None)
        _check(cdll.dyhip_device_pool(self.handle, _i(which), C.byref(p)))
        return Pool(p, owned=False)

    def scalar_ptr(self, which):
        p = _vp(None)
        _check(cdll.dyhip_device_scalar(self.handle, _i(which), C.byref(p)))
        return p.value

    def alloc(self, nbytes, pool=lib.POOL_FXS):
        p = _vp(None)
        _check(cdll.dyhip_device_allocate(self.handle, _i(pool), _sz(int(nbytes)), C.byref(p)))
        return p.value

    def empty(self, shape, dtype=np.float32, pool=lib.POOL_FXS):
        shape = (shape,) if np.isscalar(shape) else tuple(shape)
        n = int(np.prod(shape)) if shape else 1
        t = DevTensor(self, self.alloc(max(n, 1) * np.dtype(dtype).itemsize, pool), shape, dtype)
        if getattr(self, "poison_empty", False) and n > 0 and np.dtype(dtype) == np.float32:
            # debugging aid for tests: an element a kernel forgets to write shows up as NaN instead of
            # whatever the pool held before (fresh pools are zero-filled, which hides such gaps)
            _check(cdll.dyhip_constant(self.handle, _sz(n), _f(float("nan")), _vp(t.ptr)))
        return t

    def tensor(self, array, dtype=np.float32, pool=lib.POOL_FXS):
        a = np.ascontiguousarray(array, dtype=dtype)
        return self.empty(a.shape, dtype, pool).set(a)

    def zeros(self, shape, dtype=np.float32, pool=lib.POOL_FXS):
        t = self.empty(shape, dtype, pool)
        _check(cdll.dyhip_zero(self.handle, _vp(t.ptr), _sz(t.nbytes)))
        return t

    def workspace(self, nbytes):
        """Scratch from the SCS pool (what a DyNet node takes from pools[SCS])."""
        nbytes = int(nbytes)
        if nbytes == 0:
            return None, 0
        return self.alloc(nbytes, lib.POOL_SCS), nbytes

    def free_pool(self, which):
        self.pool(which).free()

    def graph_begin(self):
        _check(cdll.dyhip_graph_begin_capture(self.handle))

    def graph_end(self):
        g = _vp(None)
        _check(cdll.dyhip_graph_end_capture(self.handle, C.byref(g)))
        return Graph(self, g)

    def timer_start(self):
        _check(cdll.dyhip_timer_start(self.handle))

    def timer_stop(self):
        ms = _f(0)
        _check(cdll.dyhip_timer_stop(self.handle, C.byref(ms)))
        return ms.value

    def copy_h2d_async(self, dst, pinned):
        """Queue a copy from a PinnedArray; the array must not change until the copy has run."""
        _check(cdll.dyhip_memcpy_h2d(self.handle, _p(dst), _vp(pinned.ptr), _sz(pinned.nbytes)))

    def copy_d2d(self, dst, src, nbytes):
        _check(cdll.dyhip_memcpy_d2d(self.handle, _p(dst), _p(src), _sz(int(nbytes))))

    def zero(self, t):
        _check(cdll.dyhip_zero(self.handle, _p(t), _sz(t.nbytes)))

    def zero_bytes(self, ptr, nbytes):
        """dyhip_zero on a raw device address (any alignment)."""
        _check(cdll.dyhip_zero(self.handle, _vp(ptr), _sz(nbytes)))

    def constant(self, t, value):
        _check(cdll.dyhip_constant(self.handle, _sz(t.size), _f(value), _p(t)))

    def accumulate(self, src, dst):
        _check(cdll.dyhip_accumulate(self.handle, _sz(src.size), _p(src), _p(dst)))

    # ---- elementwise ------------------------------------------------------
    def unary_forward(self, op, x, y, logistic_mode=lib.LOGISTIC_PACKET, n=None):
        _check(cdll.dyhip_unary_forward(self.handle, _i(op), _i(logistic_mode), _sz(x.size if n is None else n), _p(x),
                                        _p(y)))

    def unary_backward(self, op, fx, dEdf, dEdx, n=None):
        _check(cdll.dyhip_unary_backward(self.handle, _i(op), _sz(fx.size if n is None else n), _p(fx), _p(dEdf),
                                         _p(dEdx)))

    def cmult_forward(self, n, bd0, bd1, a, b, y):
        _check(cdll.dyhip_cmult_forward(self.handle, _sz(n), _u(bd0), _u(bd1), _p(a), _p(b), _p(y)))

    def csum_forward(self, n, bd0, bd1, a, b, y):
        _check(cdll.dyhip_csum_forward(self.handle, _sz(n), _u(bd0), _u(bd1), _p(a), _p(b), _p(y)))

    def sum_forward(self, n, bd, xs, bds, fx):
        ptrs = (_vp * len(xs))(*[x.ptr for x in xs])
        bds_c = (_u * len(xs))(*[int(b) for b in bds])
        _check(cdll.dyhip_sum_forward(self.handle, _u(len(xs)), _sz(n), _u(bd), ptrs, bds_c, _p(fx)))

    def batch_reduce_workspace(self, n, bd):
        b = _sz(0)
        _check(cdll.dyhip_batch_reduce_workspace(_sz(n), _u(bd), C.byref(b)))
        return b.value

    def cmult_backward(self, n, bd0, bd1, a, b, dEdf, i, dEdxi):
        ws, nb = self.workspace(self.batch_reduce_workspace(n, max(bd0, bd1)))
        _check(cdll.dyhip_cmult_backward(self.handle, _sz(n), _u(bd0), _u(bd1), _p(a), _p(b), _p(dEdf), _u(i),
                                         _p(dEdxi), _vp(ws), _sz(nb)))

    def csum_backward(self, n, bd0, bd1, dEdf, i, dEdxi):
        ws, nb = self.workspace(self.batch_reduce_workspace(n, max(bd0, bd1)))
        _check(cdll.dyhip_csum_backward(self.handle, _sz(n), _u(bd0), _u(bd1), _p(dEdf), _u(i), _p(dEdxi), _vp(ws),
                                        _sz(nb)))

    # ---- reductions -------------------------------------------------------
    def sum_batches_forward(self, n, bd, x, y, ws=None, ws_bytes=None):
        if ws is None:
            ws, ws_bytes = self.workspace(self.batch_reduce_workspace(n, bd))
        _check(cdll.dyhip_sum_batches_forward(self.handle, _sz(n), _u(bd), _p(x), _p(y), _vp(ws), _sz(ws_bytes)))

    def sum_batches_backward(self, n, bd, dEdf, dEdx):
        _check(cdll.dyhip_sum_batches_backward(self.handle, _sz(n), _u(bd), _p(dEdf), _p(dEdx)))

    def mean_elems_forward(self, n, bd, x, y):
        _check(cdll.dyhip_mean_elems_forward(self.handle, _sz(n), _u(bd), _p(x), _p(y)))

    def mean_elems_backward(self, n, bd, dEdf, dEdx):
        _check(cdll.dyhip_mean_elems_backward(self.handle, _sz(n), _u(bd), _p(dEdf), _p(dEdx)))

    def std_elems_forward(self, n, bd, x, y):
        _check(cdll.dyhip_std_elems_forward(self.handle, _sz(n), _u(bd), _p(x), _p(y)))

    def std_elems_backward(self, n, bd, x, fx, dEdf, dEdx):
        _check(cdll.dyhip_std_elems_backward(self.handle, _sz(n), _u(bd), _p(x), _p(fx), _p(dEdf), _p(dEdx)))

    # ---- layer norm -------------------------------------------------------
    def layer_norm_forward(self, n, bd, x, g, b, y):
        _check(cdll.dyhip_layer_norm_forward(self.handle, _sz(n), _u(bd), _p(x), _p(g), _p(b), _p(y)))

    def layer_norm_backward_workspace(self, n, bd):
        b = _sz(0)
        _check(cdll.dyhip_layer_norm_backward_workspace(_sz(n), _u(bd), C.byref(b)))
        return b.value

    def layer_norm_backward(self, n, bd, x, g, dEdf, dx=None, dg=None, db=None, ws=None, ws_bytes=None):
        if ws is None:
            ws, ws_bytes = self.workspace(self.layer_norm_backward_workspace(n, bd))
        _check(cdll.dyhip_layer_norm_backward(self.handle, _sz(n), _u(bd), _p(x), _p(g), _p(dEdf), _p(dx), _p(dg),
                                              _p(db), _vp(ws), _sz(ws_bytes)))

    # ---- cwise ops with dimension broadcast ---------------------------------------
    @staticmethod
    def _dims5(d):
        d = list(d) + [1] * (5 - len(d))
        return (C.c_uint * 5)(*d)

    def cwise_forward(self, op, dims_a, dims_b, a, b, fx):
        """dims: (d0, d1, d2, d3, bd), column-major with the batch outermost (numpy shape = reversed dims)."""
        _check(cdll.dyhip_cwise_forward(self.handle, _i(op), self._dims5(dims_a), self._dims5(dims_b), _p(a), _p(b), _p(fx)))

    def cwise_backward_workspace(self, dims_a, dims_b, i):
        nb = _sz(0)
        _check(cdll.dyhip_cwise_backward_workspace(self._dims5(dims_a), self._dims5(dims_b), _u(i), C.byref(nb)))
        return nb.value

    def cwise_backward(self, op, dims_a, dims_b, a, b, dEdf, i, dEdxi, ws=None, nbytes=None):
        da, db = self._dims5(dims_a), self._dims5(dims_b)
        if ws is None:
            ws, nbytes = self.workspace(self.cwise_backward_workspace(dims_a, dims_b, i))
        _check(cdll.dyhip_cwise_backward(self.handle, _i(op), da, db, _p(a), _p(b), _p(dEdf), _u(i), _p(dEdxi), _vp(ws),
                                         _sz(nbytes)))

    def const_plus_x_forward(self, c, x, fx):
        _check(cdll.dyhip_const_plus_x_forward(self.handle, _sz(x.size), C.c_float(c), _p(x), _p(fx)))

    def const_minus_x_forward(self, c, x, fx):
        _check(cdll.dyhip_const_minus_x_forward(self.handle, _sz(x.size), C.c_float(c), _p(x), _p(fx)))

    def layer_norm_backward_static(self, n, bd, x, g, dEdf, dx=None, dg=None, db=None):
        """No workspace argument and no allocation: the scratch is a static device array of the library."""
        _check(cdll.dyhip_layer_norm_backward_static(self.handle, _sz(n), _u(bd), _p(x), _p(g), _p(dEdf), _p(dx),
                                                     _p(dg), _p(db)))

    # ---- GEMM -------------------------------------------------------------
    def gemm_nn(self, M, N, K, l, r, beta, y):
        _check(cdll.dyhip_gemm_nn(self.handle, _sz(M), _sz(N), _sz(K), _p(l), _p(r), _f(beta), _p(y)))

    def affine_forward(self, M, N, K, bias, W, x, fx):
        _check(cdll.dyhip_affine_forward(self.handle, _sz(M), _sz(N), _sz(K), _p(bias), _p(W), _p(x), _p(fx)))

    def gemm_tn(self, M, N, K, l, r, beta, y):
        _check(cdll.dyhip_gemm_tn(self.handle, _sz(M), _sz(N), _sz(K), _p(l), _p(r), _f(beta), _p(y)))

    def gemm_nt(self, M, N, K, l, r, beta, y):
        _check(cdll.dyhip_gemm_nt(self.handle, _sz(M), _sz(N), _sz(K), _p(l), _p(r), _f(beta), _p(y)))

    def gemm_strided_batched(self, trans_l, trans_r, M, N, K, l, stride_l, r, stride_r, beta, y, stride_y, batch):
        _check(cdll.dyhip_gemm_strided_batched(self.handle, _i(trans_l), _i(trans_r), _sz(M), _sz(N), _sz(K), _p(l),
                                               _sz(stride_l), _p(r), _sz(stride_r), _f(beta), _p(y), _sz(stride_y),
                                               _u(batch)))

    def gemm_uses_wide_tiles(self, trans_l, trans_r, M, N, K):
        out = C.c_int(0)
        _check(cdll.dyhip_gemm_uses_wide_tiles(self.handle, _i(trans_l), _i(trans_r), _sz(M), _sz(N), _sz(K),
                                               C.byref(out)))
        return int(out.value)  # 0: no, 1: the whole product, 2: its leading full-round columns

    @staticmethod
    def gemm_wide_segments(M, N, K, segments):
        """(starts, k_tiles_per_tile, finish_in_kernel) of the 256 x 256-tile GEMM's work distribution; needs no GPU."""
        starts = (C.c_uint * (segments + 1))()
        nt, fin = C.c_uint(0), C.c_int(0)
        _check(cdll.dyhip_gemm_wide_segments(_sz(M), _sz(N), _sz(K), _u(segments), starts, C.byref(nt), C.byref(fin)))
        return list(starts), int(nt.value), bool(fin.value)

    def gemm_tn_acc(self, M, N, K, l, r, y):
        _check(cdll.dyhip_gemm_tn_acc(self.handle, _sz(M), _sz(N), _sz(K), _p(l), _p(r), _p(y)))

    def gemm_nt_acc(self, M, N, K, l, r, y):
        _check(cdll.dyhip_gemm_nt_acc(self.handle, _sz(M), _sz(N), _sz(K), _p(l), _p(r), _p(y)))

    # ---- LSTM -------------------------------------------------------------
    @staticmethod
    def _xs(xs, x_dims):
        ptrs = (_vp * len(xs))(*[(x.ptr if isinstance(x, DevTensor) else int(x)) for x in xs])
        dims = (_u * len(xs))(*[int(d) for d in x_dims])
        return ptrs, dims

    def lstm_gates_forward(self, xs, x_dims, H, B, h_tm1, Wx, Wh, b, fx, mask_x=None, mask_x_bd=0, mask_h=None,
                           mask_h_bd=0, logistic_mode=lib.LOGISTIC_PACKET):
        ptrs, dims = self._xs(xs, x_dims)
        need = _sz(0)
        _check(cdll.dyhip_lstm_gates_workspace(_u(len(xs)), _u(sum(x_dims)), _u(H), _u(B),
                                               _i(1 if mask_x is not None else 0), C.byref(need)))
        ws, nb = self.workspace(need.value)
        _check(cdll.dyhip_lstm_gates_forward(self.handle, _u(len(xs)), ptrs, dims, _u(H), _u(B), _p(h_tm1), _p(Wx),
                                             _p(Wh), _p(b), _p(mask_x), _u(mask_x_bd), _p(mask_h), _u(mask_h_bd),
                                             _i(logistic_mode), _p(fx), _vp(ws), _sz(nb)))

    def lstm_gates_dpre(self, H, B, fx, dEdf, dpre):
        _check(cdll.dyhip_lstm_gates_dpre(self.handle, _u(H), _u(B), _p(fx), _p(dEdf), _p(dpre)))

    def lstm_gates_backward(self, xs, x_dims, H, B, h_tm1, Wx, Wh, fx, dEdf, i, dEdxi, dpre=None, mask_x=None,
                            mask_x_bd=0, mask_h=None, mask_h_bd=0):
        ptrs, dims = self._xs(xs, x_dims)
        need = _sz(0)
        _check(cdll.dyhip_lstm_gates_backward_workspace(_u(len(xs)), _u(sum(x_dims)), _u(H), _u(B),
                                                        _i(1 if mask_x is not None else 0), C.byref(need)))
        ws, nb = self.workspace(need.value)
        _check(cdll.dyhip_lstm_gates_backward(self.handle, _u(len(xs)), ptrs, dims, _u(H), _u(B), _p(h_tm1), _p(Wx),
                                              _p(Wh), _p(mask_x), _u(mask_x_bd), _p(mask_h), _u(mask_h_bd), _p(fx),
                                              _p(dEdf), _p(dpre), _u(i), _p(dEdxi), _vp(ws), _sz(nb)))

    def lstm_c_forward(self, H, B, c_tm1, gates, c):
        _check(cdll.dyhip_lstm_c_forward(self.handle, _u(H), _u(B), _p(c_tm1), _p(gates), _p(c)))

    def lstm_c_backward(self, H, B, c_tm1, gates, dEdf, i, dEdxi):
        _check(cdll.dyhip_lstm_c_backward(self.handle, _u(H), _u(B), _p(c_tm1), _p(gates), _p(dEdf), _u(i),
                                          _p(dEdxi)))

    def lstm_h_forward(self, H, B, c, gates, h):
        _check(cdll.dyhip_lstm_h_forward(self.handle, _u(H), _u(B), _p(c), _p(gates), _p(h)))

    def lstm_h_backward(self, H, B, c, gates, dEdf, i, dEdxi):
        _check(cdll.dyhip_lstm_h_backward(self.handle, _u(H), _u(B), _p(c), _p(gates), _p(dEdf), _u(i), _p(dEdxi)))

    # ---- fused cell path --------------------------------------------------
    def lstm_cell_workspace(self, H, B):
        f, b = _sz(0), _sz(0)
        _check(cdll.dyhip_lstm_cell_workspace(self.handle, _u(H), _u(B), C.byref(f), C.byref(b)))
        return f.value, b.value

    def lstm_recurrent_forward(self, H, B, Wh, h_tm1, ws, ws_bytes):
        n = _u(0)
        _check(cdll.dyhip_lstm_recurrent_forward(self.handle, _u(H), _u(B), _p(Wh), _p(h_tm1), _vp(ws), _sz(ws_bytes),
                                                 C.byref(n)))
        return n.value

    def lstm_recurrent_backward(self, H, B, Wh, dpre, ws, ws_bytes):
        n = _u(0)
        _check(cdll.dyhip_lstm_recurrent_backward(self.handle, _u(H), _u(B), _p(Wh), _p(dpre), _vp(ws), _sz(ws_bytes),
                                                  C.byref(n)))
        return n.value

    def lstm_cell_forward(self, H, B, xproj, b, rec, splits, c_tm1, gates, c, h, logistic_mode=lib.LOGISTIC_PACKET):
        _check(cdll.dyhip_lstm_cell_forward(self.handle, _u(H), _u(B), _p(xproj), _p(b), _vp(rec), _u(splits),
                                            _p(c_tm1), _i(logistic_mode), _p(gates), _p(c), _p(h)))

    def lstm_step_supported(self, H, B):
        ok = C.c_int(0)
        _check(cdll.dyhip_lstm_step_supported(self.handle, _u(H), _u(B), C.byref(ok)))
        return bool(ok.value)

    def lstm_pack_recurrent(self, H, Wh, packed):
        _check(cdll.dyhip_lstm_pack_recurrent(self.handle, _u(H), _p(Wh), _p(packed)))

    def lstm_step_forward(self, H, B, packed_Wh, h_tm1, xproj, b, c_tm1, gates, c, h,
                          logistic_mode=lib.LOGISTIC_PACKET):
        _check(cdll.dyhip_lstm_step_forward(self.handle, _u(H), _u(B), _p(packed_Wh), _p(h_tm1), _p(xproj), _p(b),
                                            _p(c_tm1), _i(logistic_mode), _p(gates), _p(c), _p(h)))

    def lstm_packed_state_floats(self, rows, B):
        n = C.c_size_t(0)
        _check(cdll.dyhip_lstm_packed_state_floats(_u(rows), _u(B), C.byref(n)))
        return n.value

    def lstm_pack_state(self, rows, B, v, packed):
        _check(cdll.dyhip_lstm_pack_state(self.handle, _u(rows), _u(B), _p(v), _p(packed)))

    def lstm_step_forward_packed(self, H, B, packed_Wh, h_tm1_packed, xproj, b, c_tm1, gates, c, h, h_packed,
                                 logistic_mode=lib.LOGISTIC_PACKET, mask_h=None):
        if mask_h is not None:  # recurrent dropout: h_packed = h (.) mask_h
            _check(cdll.dyhip_lstm_step_forward_packed_dropout(self.handle, _u(H), _u(B), _p(packed_Wh), _p(h_tm1_packed),
                                                               _p(xproj), _p(b), _p(c_tm1), _p(mask_h), _i(logistic_mode),
                                                               _p(gates), _p(c), _p(h), _p(h_packed)))
            return
        _check(cdll.dyhip_lstm_step_forward_packed(self.handle, _u(H), _u(B), _p(packed_Wh), _p(h_tm1_packed), _p(xproj),
                                                   _p(b), _p(c_tm1), _i(logistic_mode), _p(gates), _p(c), _p(h),
                                                   _p(h_packed)))

    def lstm_pack_recurrent_transposed(self, H, Wh, packed):
        _check(cdll.dyhip_lstm_pack_recurrent_transposed(self.handle, _u(H), _p(Wh), _p(packed)))

    def lstm_recurrent_backward_packed(self, H, B, packed_WhT, dpre_packed, ws, ws_bytes):
        n = _u(0)
        _check(cdll.dyhip_lstm_recurrent_backward_packed(self.handle, _u(H), _u(B), _p(packed_WhT), _p(dpre_packed),
                                                         _vp(ws), _sz(ws_bytes), C.byref(n)))
        return n.value

    def lstm_cell_backward_packed(self, H, B, gates, c, c_tm1, dh, rec, splits, dc, dpre, dc_tm1, dpre_packed):
        _check(cdll.dyhip_lstm_cell_backward_packed(self.handle, _u(H), _u(B), _p(gates), _p(c), _p(c_tm1), _p(dh),
                                                    _vp(rec), _u(splits), _p(dc), _p(dpre), _p(dc_tm1), _p(dpre_packed)))

    def lstm_pack_recurrent_transposed16(self, H, Wh, packed):
        _check(cdll.dyhip_lstm_pack_recurrent_transposed16(self.handle, _u(H), _p(Wh), _p(packed)))

    @staticmethod
    def lstm_packed_state16_floats(rows, B):
        n = C.c_size_t(0)
        _check(cdll.dyhip_lstm_packed_state16_floats(_u(rows), _u(B), C.byref(n)))
        return n.value

    def lstm_pack_state16(self, rows, B, v, packed):
        _check(cdll.dyhip_lstm_pack_state16(self.handle, _u(rows), _u(B), _p(v), _p(packed)))

    def lstm_step_backward_packed(self, H, B, packed_WhT16, dpre_next_packed16, gates, c, c_tm1, dh, dc, dpre, dc_tm1,
                                  dpre_packed16, mask_h=None):
        """One launch per backward timestep: Wh^T * dpre_{t+1} over its whole depth and the cell backward of step t."""
        if mask_h is not None:  # recurrent dropout: the product reaches dh through the mask
            _check(cdll.dyhip_lstm_step_backward_packed_dropout(self.handle, _u(H), _u(B), _p(packed_WhT16),
                                                                _p(dpre_next_packed16), _p(gates), _p(c), _p(c_tm1),
                                                                _p(dh), _p(dc), _p(mask_h), _p(dpre), _p(dc_tm1),
                                                                _p(dpre_packed16)))
            return
        _check(cdll.dyhip_lstm_step_backward_packed(self.handle, _u(H), _u(B), _p(packed_WhT16),
                                                    _p(dpre_next_packed16), _p(gates), _p(c), _p(c_tm1), _p(dh), _p(dc),
                                                    _p(dpre), _p(dc_tm1), _p(dpre_packed16)))

    def gather_segments(self, segments, length, dst):
        """dst = the equal-length tensors `segments` one behind the other (pointers travel as kernel arguments)."""
        ptrs = (C.c_void_p * len(segments))(*[t.ptr if isinstance(t, DevTensor) else int(t) for t in segments])
        _check(cdll.dyhip_gather_segments(self.handle, _u(len(segments)), _sz(int(length)), ptrs, _p(dst)))

    def lstm_pack_input(self, I, H, Wx, packed):
        _check(cdll.dyhip_lstm_pack_input(self.handle, _u(I), _u(H), _p(Wx), _p(packed)))

    def lstm_step_forward_x(self, I, H, B, packed_Wx, x, packed_Wh, h_tm1, b, c_tm1, gates, c, h,
                            logistic_mode=lib.LOGISTIC_PACKET):
        _check(cdll.dyhip_lstm_step_forward_x(self.handle, _u(I), _u(H), _u(B), _p(packed_Wx), _p(x), _p(packed_Wh),
                                              _p(h_tm1), _p(b), _p(c_tm1), _i(logistic_mode), _p(gates), _p(c), _p(h)))

    def lstm_cell_backward(self, H, B, gates, c, c_tm1, dh, rec, splits, dc, dpre, dc_tm1):
        _check(cdll.dyhip_lstm_cell_backward(self.handle, _u(H), _u(B), _p(gates), _p(c), _p(c_tm1), _p(dh), _vp(rec),
                                             _u(splits), _p(dc), _p(dpre), _p(dc_tm1)))

    def pick_range_forward(self, inner, length, outer, start, end, x, fx):
        _check(cdll.dyhip_pick_range_forward(self.handle, _sz(inner), _sz(length), _sz(outer), _sz(start), _sz(end),
                                             _p(x), _p(fx)))

    def pick_range_backward(self, inner, length, outer, start, end, dEdf, dEdxi):
        _check(cdll.dyhip_pick_range_backward(self.handle, _sz(inner), _sz(length), _sz(outer), _sz(start), _sz(end),
                                              _p(dEdf), _p(dEdxi)))

    # ---- random tensors ---------------------------------------------------
    def reset_rng(self, seed):
        _check(cdll.dyhip_reset_rng(self.handle, _u(seed)))

    def rng_state(self):
        """(key, position, queue) of this queue's Philox stream; synchronises."""
        k, pos, q = C.c_ulonglong(0), C.c_ulonglong(0), _u(0)
        _check(cdll.dyhip_rng_state(self.handle, C.byref(k), C.byref(pos), C.byref(q)))
        return k.value, pos.value, q.value

    def rng_set_position(self, position):
        _check(cdll.dyhip_rng_set_position(self.handle, C.c_ulonglong(position)))

    def randomize_uniform(self, out, left=0.0, right=1.0):
        _check(cdll.dyhip_randomize_uniform(self.handle, _sz(out.size), _f(left), _f(right), _p(out)))

    def randomize_bernoulli(self, out, p, scale=1.0):
        _check(cdll.dyhip_randomize_bernoulli(self.handle, _sz(out.size), _f(p), _f(scale), _p(out)))

    def randomize_normal(self, out, mean=0.0, stddev=1.0):
        _check(cdll.dyhip_randomize_normal(self.handle, _sz(out.size), _f(mean), _f(stddev), _p(out)))

    def dropout_forward(self, p, x, mask, fx):
        _check(cdll.dyhip_dropout_forward(self.handle, _sz(x.size), _f(p), _p(x), _p(mask), _p(fx)))

    def dropout_backward(self, mask, dEdf, dEdxi):
        _check(cdll.dyhip_dropout_backward(self.handle, _sz(mask.size), _p(mask), _p(dEdf), _p(dEdxi)))

    # ---- lookup -----------------------------------------------------------
    def lookup_forward(self, ids_host, ids_dev, dim, vocab, table, fx, mult=1.0):
        n = ids_dev.size
        hp = _vp(None)
        if ids_host is not None:
            ids_host = np.ascontiguousarray(ids_host, dtype=np.uint32)
            assert ids_host.size == n
            hp = _vp(ids_host.ctypes.data)
        _check(cdll.dyhip_lookup_forward(self.handle, _u(n), hp, _p(ids_dev), _sz(dim), _u(vocab), _p(table),
                                         _f(mult), _p(fx)))

    def lookup_accumulate_grads_workspace(self, n_ids, dim, vocab):
        b = _sz(0)
        _check(cdll.dyhip_lookup_accumulate_grads_workspace(_u(n_ids), _sz(dim), _u(vocab), C.byref(b)))
        return b.value

    def lookup_accumulate_grads(self, ids_dev, dim, vocab, g, all_grads, ws=None, ws_bytes=None):
        n = ids_dev.size
        if ws is None:
            ws, ws_bytes = self.workspace(self.lookup_accumulate_grads_workspace(n, dim, vocab))
        _check(cdll.dyhip_lookup_accumulate_grads(self.handle, _u(n), _p(ids_dev), _sz(dim), _u(vocab), _p(g),
                                                  _p(all_grads), _vp(ws), _sz(ws_bytes)))

    @staticmethod
    def lookup_plan_parts(plan_words, n):
        """Splits a plan read back as uint32 words into (gid, gpos, roff, rrem): ids grouped by value,
        their positions, entries of the run before / from each entry.  The plan starts with one 16-byte
        record (id, position, before, from) per grouped entry."""
        rec = np.asarray(plan_words[:4 * n]).reshape(n, 4)
        return tuple(np.ascontiguousarray(rec[:, q]) for q in range(4))

    def lookup_plan_invalid_ids(self, n_ids, plan):
        """How many ids of the plan were >= vocab (the reduction skips them); synchronises."""
        c = C.c_uint(0)
        _check(cdll.dyhip_lookup_plan_invalid_ids(self.handle, _u(n_ids), _p(plan), C.byref(c)))
        return c.value

    def lookup_build_plan(self, ids_dev, vocab):
        """Plan of a lookup's ids (ids grouped by value with run offsets); returns the plan buffer (FXS pool)."""
        n = ids_dev.size
        pb, wb = _sz(0), _sz(0)
        _check(cdll.dyhip_lookup_plan_bytes(_u(n), C.byref(pb)))
        _check(cdll.dyhip_lookup_plan_workspace(_u(n), _u(vocab), C.byref(wb)))
        plan = DevTensor(self, self.alloc(max(pb.value, 1)), (pb.value // 4,), np.uint32)
        ws, nb = self.workspace(wb.value)
        _check(cdll.dyhip_lookup_build_plan(self.handle, _u(n), _p(ids_dev), _u(vocab), _p(plan), _sz(pb.value),
                                            _vp(ws), _sz(nb)))
        return plan

    def lookup_plan_buffers(self, n_ids, vocab):
        """(plan, workspace, workspace bytes) for repeated lookup_build_plan_into calls."""
        pb, wb = _sz(0), _sz(0)
        _check(cdll.dyhip_lookup_plan_bytes(_u(n_ids), C.byref(pb)))
        _check(cdll.dyhip_lookup_plan_workspace(_u(n_ids), _u(vocab), C.byref(wb)))
        plan = DevTensor(self, self.alloc(max(pb.value, 1)), (pb.value // 4,), np.uint32)
        ws, nb = self.workspace(wb.value)
        return plan, ws, nb

    def lookup_build_plan_into(self, ids_dev, vocab, plan, ws, ws_bytes):
        _check(cdll.dyhip_lookup_build_plan(self.handle, _u(ids_dev.size), _p(ids_dev), _u(vocab), _p(plan),
                                            _sz(plan.nbytes), _vp(ws), _sz(ws_bytes)))

    def lookup_accumulate_grads_planned_workspace(self, n_ids, dim):
        b = _sz(0)
        _check(cdll.dyhip_lookup_accumulate_grads_planned_workspace(_u(n_ids), _sz(dim), C.byref(b)))
        return b.value

    def lookup_accumulate_grads_planned(self, n_ids, plan, dim, vocab, g, all_grads, ws=None, ws_bytes=None):
        if ws is None:
            ws, ws_bytes = self.workspace(self.lookup_accumulate_grads_planned_workspace(n_ids, dim))
        _check(cdll.dyhip_lookup_accumulate_grads_planned(self.handle, _u(n_ids), _p(plan), _sz(dim), _u(vocab), _p(g),
                                                          _p(all_grads), _vp(ws), _sz(ws_bytes)))

    # ---- logsumexp / pnls -------------------------------------------------
    def logsumexp_cols(self, rows, bd, x, m, z):
        _check(cdll.dyhip_logsumexp_cols(self.handle, _sz(rows), _u(bd), _p(x), _p(m), _p(z)))

    def pnls_forward(self, rows, bd, x, labels_host, aux, fx):
        labels_host = np.ascontiguousarray(labels_host, dtype=np.uint32)
        assert labels_host.size == bd
        _check(cdll.dyhip_pnls_forward(self.handle, _sz(rows), _u(bd), _p(x), _vp(labels_host.ctypes.data), _p(aux),
                                       _p(fx)))

    def pnls_forward_staged(self, rows, bd, x, aux, fx):
        _check(cdll.dyhip_pnls_forward_staged(self.handle, _sz(rows), _u(bd), _p(x), _p(aux), _p(fx)))

    def pnls_backward(self, rows, bd, x, aux, dEdf, dEdx, assign=False):
        fn = cdll.dyhip_pnls_backward_assign if assign else cdll.dyhip_pnls_backward
        _check(fn(self.handle, _sz(rows), _u(bd), _p(x), _p(aux), _p(dEdf), _p(dEdx)))

    def softmax_forward(self, rows, cols, x, fx):
        ws, nb = self.workspace(8 * cols)
        _check(cdll.dyhip_softmax_forward(self.handle, _sz(rows), _u(cols), _p(x), _p(fx), _vp(ws), _sz(nb)))

    def softmax_backward(self, rows, cols, fx, dEdf, dEdx):
        ws, nb = self.workspace(4 * cols)
        _check(cdll.dyhip_softmax_backward(self.handle, _sz(rows), _u(cols), _p(fx), _p(dEdf), _p(dEdx), _vp(ws),
                                           _sz(nb)))

    def softmax_rows_forward(self, rows, cols, bd, x, fx):
        _check(cdll.dyhip_softmax_rows_forward(self.handle, _sz(rows), _sz(cols), _u(bd), _p(x), _p(fx)))

    def softmax_rows_backward(self, rows, cols, bd, fx, dEdf, dEdx):
        _check(cdll.dyhip_softmax_rows_backward(self.handle, _sz(rows), _sz(cols), _u(bd), _p(fx), _p(dEdf), _p(dEdx)))

    def logsumexp_dim_forward(self, rows, cols, bd, x, dim, m, fx):
        _check(cdll.dyhip_logsumexp_dim_forward(self.handle, _sz(rows), _sz(cols), _u(bd), _p(x), _u(dim), _p(m), _p(fx)))

    def logsumexp_dim_backward(self, rows, cols, bd, x, fx, dEdf, dim, dEdx):
        _check(cdll.dyhip_logsumexp_dim_backward(self.handle, _sz(rows), _sz(cols), _u(bd), _p(x), _p(fx), _p(dEdf),
                                                 _u(dim), _p(dEdx)))

    def log_softmax_forward(self, rows, cols, x, aux, fx):
        _check(cdll.dyhip_log_softmax_forward(self.handle, _sz(rows), _u(cols), _p(x), _p(aux), _p(fx)))

    def log_softmax_backward(self, rows, cols, fx, dEdf, aux, dEdx):
        _check(cdll.dyhip_log_softmax_backward(self.handle, _sz(rows), _u(cols), _p(fx), _p(dEdf), _p(aux), _p(dEdx)))

    def logsumexp_node_forward(self, n, bd, xs, bds, fx):
        ptrs, b = self._xs(xs, bds)
        _check(cdll.dyhip_logsumexp_node_forward(self.handle, _u(len(xs)), _sz(n), _u(bd), ptrs, b, _p(fx)))

    def logsumexp_node_backward(self, n, bd, xs, bds, fx, dEdf, i, dEdxi):
        ptrs, b = self._xs(xs, bds)
        ws, nb = self.workspace(n * bd * 4 + 256 + self.batch_reduce_workspace(n, bd))
        _check(cdll.dyhip_logsumexp_node_backward(self.handle, _u(len(xs)), _sz(n), _u(bd), ptrs, b, _p(fx), _p(dEdf),
                                                  _u(i), _p(dEdxi), _vp(ws), _sz(nb)))

    def argmax_cols(self, rows, bd, x, idx):
        _check(cdll.dyhip_argmax_cols(self.handle, _sz(rows), _u(bd), _p(x), _p(idx)))

    def argmax_onehot_forward(self, rows, bd, x, idx, fx):
        _check(cdll.dyhip_argmax_onehot_forward(self.handle, _sz(rows), _u(bd), _p(x), _p(idx), _p(fx)))

    # ---- dynet::gpu helpers -----------------------------------------------
    def dense_to_sparse_assign(self, n, ids, src, trg):
        _check(cdll.dyhip_dense_to_sparse_assign(self.handle, _i(n), _p(ids), _p(src), _p(trg)))

    def sparse_to_dense_assign(self, n, ids, src, trg):
        _check(cdll.dyhip_sparse_to_dense_assign(self.handle, _i(n), _p(ids), _p(src), _p(trg)))

    def dense_to_sparse_subtract(self, n, ids, src, trg):
        _check(cdll.dyhip_dense_to_sparse_subtract(self.handle, _i(n), _p(ids), _p(src), _p(trg)))

    def sparse_to_dense_block_assign_and_multiply(self, n, idx, bsize, mult, src, trg):
        _check(cdll.dyhip_sparse_to_dense_block_assign_and_multiply(self.handle, _i(n), _p(idx), _i(bsize), _f(mult),
                                                                    _p(src), _p(trg)))

    def dense_to_sparse_block_add(self, n, ids, bsize, src, trg):
        _check(cdll.dyhip_dense_to_sparse_block_add(self.handle, _i(n), _p(ids), _i(bsize), _p(src), _p(trg)))

    def parallel_memcpy(self, num_seqs, max_len, src, trg, lens):
        _check(cdll.dyhip_parallel_memcpy(self.handle, _i(num_seqs), _i(max_len), _p(src), _p(trg), _p(lens)))

    def parallel_accumulate(self, num_seqs, max_len, src, trg, lens):
        _check(cdll.dyhip_parallel_accumulate(self.handle, _i(num_seqs), _i(max_len), _p(src), _p(trg), _p(lens)))

    # ---- parameter nodes / trainer ----------------------------------------
    def scale_copy(self, n, src, mult, dst):
        _check(cdll.dyhip_scale_copy(self.handle, _sz(n), _p(src), _f(mult), _p(dst)))

    def sgd_update(self, n, p, g, lr, gscale=1.0, wd=1.0):
        _check(cdll.dyhip_sgd_update(self.handle, _sz(n), _p(p), _p(g), _f(lr), _f(gscale), _f(wd)))

    def clip_scale(self, n, sqnorms, threshold, gscale, norm=None):
        _check(cdll.dyhip_clip_scale_norm(self.handle, _u(n), _p(sqnorms), _f(threshold), _p(gscale), _p(norm)))

    def sgd_update_scaled(self, n, p, g, lr, gscale_dev, wd=1.0, clear_grad=True):
        _check(cdll.dyhip_sgd_update_scaled(self.handle, _sz(n), _p(p), _p(g), _f(lr), _p(gscale_dev), _f(wd),
                                            _i(1 if clear_grad else 0)))

    def sgd_update_rows(self, n_ids, plan, dim, vocab, values, grads, lr, gscale_dev, wd=1.0):
        _check(cdll.dyhip_sgd_update_rows(self.handle, _u(n_ids), _p(plan), _sz(dim), _u(vocab), _p(values),
                                          _p(grads), _f(lr), _p(gscale_dev), _f(wd)))

    def squared_l2norm_rows(self, n_ids, plan, dim, vocab, grads, out):
        need = _sz(0)
        _check(cdll.dyhip_squared_l2norm_rows_workspace(_u(n_ids), C.byref(need)))
        ws, nb = self.workspace(need.value)
        _check(cdll.dyhip_squared_l2norm_rows(self.handle, _u(n_ids), _p(plan), _sz(dim), _u(vocab), _p(grads),
                                              _p(out), _vp(ws), _sz(nb)))

    def squared_l2norm(self, n, g, out):
        need = _sz(0)
        _check(cdll.dyhip_squared_l2norm_workspace(_sz(n), C.byref(need)))
        ws, nb = self.workspace(need.value)
        _check(cdll.dyhip_squared_l2norm(self.handle, _sz(n), _p(g), _p(out), _vp(ws), _sz(nb)))


class Graph:
    """A captured launch sequence (HIP graph) bound to its device's stream."""

    def __init__(self, dev, handle):
        self.dev = dev
        self.handle = handle

    def launch(self):
        _check(cdll.dyhip_graph_launch(self.dev.handle, self.handle))

    def destroy(self):
        if self.handle is not None:
            cdll.dyhip_graph_destroy(self.handle)
            self.handle = None


class Pool:
    """AlignedMemoryPool handle (device pools are borrowed from the Device; host pools are owned)."""

    def __init__(self, handle, owned):
        self.handle = handle
        self.owned = owned

    @classmethod
    def create_host(cls, name, cap_bytes, expanding_unit=1 << 24):
        h = _vp(None)
        _check(cdll.dyhip_pool_create_host(name.encode(), _sz(cap_bytes), _sz(expanding_unit), C.byref(h)))
        return cls(h, owned=True)

    def destroy(self):
        if self.owned and self.handle is not None:
            cdll.dyhip_pool_destroy(self.handle)
            self.handle = None

    def allocate(self, nbytes):
        p = _vp(None)
        _check(cdll.dyhip_pool_allocate(self.handle, _sz(nbytes), C.byref(p)))
        return p.value

    def free(self):
        _check(cdll.dyhip_pool_free(self.handle))

    def zero_allocated(self):
        _check(cdll.dyhip_pool_zero_allocated(self.handle))

    def used(self):
        v = _sz(0)
        _check(cdll.dyhip_pool_used(self.handle, C.byref(v)))
        return v.value

    def set_used(self, n):
        _check(cdll.dyhip_pool_set_used(self.handle, _sz(n)))

    def capacity(self):
        v = _sz(0)
        _check(cdll.dyhip_pool_capacity(self.handle, C.byref(v)))
        return v.value

    def num_blocks(self):
        v = _i(0)
        _check(cdll.dyhip_pool_num_blocks(self.handle, C.byref(v)))
        return v.value
