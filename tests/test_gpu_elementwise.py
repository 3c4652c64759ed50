"""GPU parity: elementwise nodes, reductions and the fused LayerNorm against the
CPU oracle on identical seeded inputs, through the C-ABI.

Sizes: the configuration named by the baseline (a 4096 x 1024 fp32 tensor;
sum_batches as Dim({64,1024}, bd 64); layer_norm as Dim({1024}, bd 4096) with
g ~ U(0.5,1.5), b ~ N(0,0.1)) plus ragged / misaligned / tiny edge cases.
"""
import numpy as np
import pytest

from dynet_amd import lib
from oracle import cpu_oracle as orc
from util import assert_shadow, F32, FWD_RTOL, GRAD_RTOL, assert_close, f32, rms

pytestmark = pytest.mark.gpu

N_BIG = 4096 * 1024
OPS = [(lib.OP_TANH, "tanh"), (lib.OP_LOGISTIC, "logistic"), (lib.OP_RECTIFY, "rectify"), (lib.OP_NEGATE, "negate")]


def _inputs(n, seed):
    rng = np.random.default_rng(seed)
    x = f32(rng.standard_normal(n))
    if n >= 8:
        x[:8] = [0.0, -0.0, 1e-4, -1e-4, 20.0, -20.0, 9.0, -7.5]  # tails and the zero of ReLU
    return x, f32(rng.standard_normal(n)), f32(rng.standard_normal(n))


@pytest.mark.parametrize("op,name", OPS)
@pytest.mark.parametrize("n", [N_BIG, 1027, 3, 1, 5, 6, N_BIG + 2])  # 1027, 5, 6, N_BIG + 2: 128-bit groups and a tail of 3, 1, 2, 2
def test_unary_forward_backward(dev, op, name, n):
    x, dy, dx0 = _inputs(n, 100 + op)
    dx_t = dev.tensor(x)
    y_t = dev.empty(n)
    dev.unary_forward(op, dx_t, y_t)
    y = y_t.numpy()
    ref = orc.unary_forward(op, x)
    if op in (lib.OP_RECTIFY, lib.OP_NEGATE):
        assert y.tobytes() == ref.tobytes()
    else:
        assert_close(y, ref, FWD_RTOL, name + " fwd")
    # backward accumulates into a non-zero gradient buffer, from the oracle's fx
    g_t = dev.tensor(dx0)
    dev.unary_backward(op, dev.tensor(ref), dev.tensor(dy), g_t)
    want = orc.unary_backward(op, ref, dy, dx0.copy())
    assert_close(g_t.numpy(), want, GRAD_RTOL, name + " bwd", floor=1e-6)


def test_logistic_packet_form_is_bit_exact_and_scalar_form_is_accurate(dev):
    x, _, _ = _inputs(1 << 20, 7)
    x[8:4096] = np.linspace(-30, 30, 4088)
    xt, yt = dev.tensor(x), dev.empty(x.size)
    dev.unary_forward(lib.OP_LOGISTIC, xt, yt, lib.LOGISTIC_PACKET)
    assert yt.numpy().tobytes() == orc.unary_forward(orc.OP_LOGISTIC, x, orc.LOGISTIC_PACKET).tobytes()
    dev.unary_forward(lib.OP_LOGISTIC, xt, yt, lib.LOGISTIC_SCALAR)
    assert_close(yt.numpy(), orc.unary_forward(orc.OP_LOGISTIC, x, orc.LOGISTIC_SCALAR), FWD_RTOL, "logistic scalar")


def test_logistic_packet_form_is_bit_exact_on_a_dense_sweep(dev):
    """Every float in [-19, 19] at a stride of 64 bit patterns, every 4096-th float elsewhere (infinities, NaN
    patterns and denormals included): the same bits as the oracle's IEEE division."""
    pos = np.arange(0, 0x80000000, 4096, dtype=np.uint64)
    lo, hi = f32(2.0 ** -40).view(np.uint32), f32(19.0).view(np.uint32)
    dense = np.arange(int(lo.item()), int(hi.item()), 64, dtype=np.uint64)
    bits = np.concatenate([pos, dense]).astype(np.uint32)
    bits = np.concatenate([bits, bits | np.uint32(0x80000000)])
    x = bits.view(np.float32)
    yt = dev.empty(x.size)
    dev.unary_forward(lib.OP_LOGISTIC, dev.tensor(x), yt, lib.LOGISTIC_PACKET)
    got, want = yt.numpy(), orc.unary_forward(orc.OP_LOGISTIC, x, orc.LOGISTIC_PACKET)
    same = (got.view(np.uint32) == want.view(np.uint32)) | (np.isnan(got) & np.isnan(want))
    assert same.all(), (x[~same][:5], got[~same][:5], want[~same][:5])


def test_tanh_is_relatively_accurate_everywhere(dev):
    x = f32(np.concatenate([np.linspace(-12, 12, 200001), np.logspace(-30, 1, 4000), -np.logspace(-30, 1, 4000)]))
    yt = dev.empty(x.size)
    dev.unary_forward(lib.OP_TANH, dev.tensor(x), yt)
    ref = np.tanh(x.astype(np.float64))
    err = np.abs(yt.numpy() - ref)
    assert np.max(err / np.maximum(np.abs(ref), 1e-37)) < 1e-6


def test_tanh_special_values(dev):
    """NaN goes through (tanhf(NaN) = NaN, as on the reference's CPU and GPU paths), infinities saturate."""
    x = f32([np.nan, -np.nan, np.inf, -np.inf, 0.0, -0.0, 1e-40, 100.0] * 65)
    yt = dev.empty(x.size)
    dev.unary_forward(lib.OP_TANH, dev.tensor(x), yt)
    got, want = yt.numpy(), orc.unary_forward(orc.OP_TANH, x)
    assert np.array_equal(np.isnan(got), np.isnan(want)) and np.isnan(got[:2]).all()
    ok = ~np.isnan(want)
    assert np.max(np.abs(got[ok] - want[ok])) <= 1e-6
    assert abs(got[2] - 1.0) < 1e-7 and abs(got[3] + 1.0) < 1e-7 and got[4] == 0.0  # saturates within one ulp


def test_unary_on_a_misaligned_buffer(dev):
    x, dy, dx0 = _inputs(4099, 11)
    base = dev.tensor(np.concatenate([[0.0], x]))  # view starting 4 bytes into the allocation
    xt = base.offset(1, (4099,))
    ybase = dev.zeros(4100)
    dev.unary_forward(lib.OP_TANH, xt, ybase.offset(1, (4099,)))
    out = ybase.numpy()
    assert out[0] == 0.0
    assert_close(out[1:], orc.unary_forward(orc.OP_TANH, x), FWD_RTOL, "misaligned tanh")


def test_unary_rejects_unknown_operator(dev):
    from dynet_amd import DyhipError

    t = dev.zeros(4)
    with pytest.raises(DyhipError) as e:
        dev.unary_forward(99, t, t)
    assert e.value.status == lib.ERR_INVALID_ARG


@pytest.mark.parametrize("n,bd0,bd1", [(N_BIG // 64, 64, 64), (1024, 4096, 1), (1024, 1, 4096), (7, 5, 1), (5, 1, 1),
                                       (7, 20000, 1), (1, 1, 70000), (24, 1, 3000)])
def test_cmult_and_csum(dev, n, bd0, bd1):
    rng = np.random.default_rng(21)
    bd = max(bd0, bd1)
    a, b = f32(rng.standard_normal((bd0, n))), f32(rng.standard_normal((bd1, n)))
    dy = f32(rng.standard_normal((bd, n)))
    at, bt, dyt = dev.tensor(a), dev.tensor(b), dev.tensor(dy)
    yt = dev.empty((bd, n))
    dev.cmult_forward(n, bd0, bd1, at, bt, yt)
    assert yt.numpy().tobytes() == orc.cmult_forward(n, bd0, bd1, a, b).tobytes()
    dev.csum_forward(n, bd0, bd1, at, bt, yt)
    assert yt.numpy().tobytes() == orc.csum_forward(n, bd0, bd1, a, b).tobytes()
    for i, (bdi, other) in enumerate(((bd0, b), (bd1, a))):
        g0 = f32(rng.standard_normal((bdi, n)))
        gt = dev.tensor(g0)
        dev.cmult_backward(n, bd0, bd1, at, bt, dyt, i, gt)
        want = orc.cmult_backward(n, bd0, bd1, a, b, dy, i, g0.copy())
        floor = rms(dy) * rms(other) * np.sqrt(bd if bdi != bd else 1)
        assert_close(gt.numpy(), want, GRAD_RTOL, "cmult bwd %d" % i, floor=floor)
        gt = dev.tensor(g0)
        dev.csum_backward(n, bd0, bd1, dyt, i, gt)
        want = orc.csum_backward(n, bd0, bd1, dy, i, g0.copy())
        assert_close(gt.numpy(), want, GRAD_RTOL, "csum bwd %d" % i, floor=rms(dy) * np.sqrt(bd if bdi != bd else 1))


@pytest.mark.parametrize("n,bd", [(64 * 1024, 64), (1024, 4096), (1027, 33), (3, 2), (5, 1), (4096, 7), (1, 100000), (2, 777),
                                  (255, 1000),
                                  # batch elements of at most 32 floats, many of them: the flat walk (and its limits)
                                  (1, 32768), (1, 32767), (3, 100000), (7, 50001), (20, 5000), (31, 4000), (32, 3000),
                                  (33, 3000), (1, 3000000)])
def test_sum_batches(dev, n, bd):
    rng = np.random.default_rng(31)
    x = f32(rng.standard_normal((bd, n)))
    yt = dev.empty(n)
    dev.sum_batches_forward(n, bd, dev.tensor(x), yt)
    ref = orc.sum_batches_forward(n, bd, x)
    # the batch order does not matter beyond rounding: compare with fp64
    assert_close(yt.numpy(), x.astype(np.float64).sum(0), FWD_RTOL, "sum_batches vs fp64", floor=np.sqrt(bd))
    # ... and with the oracle's sequential fp32 sum, which has itself drifted by a few 1e-5 of sqrt(bd) x |partial sums|
    # once the batch has tens of thousands of elements (-314.1896 against -314.1811 in fp64 at 3 x 100 000)
    assert_close(yt.numpy(), ref, FWD_RTOL * (1 if bd < 30000 else 8), "sum_batches fwd", floor=np.sqrt(bd))
    dy, g0 = f32(rng.standard_normal(n)), f32(rng.standard_normal((bd, n)))
    gt = dev.tensor(g0)
    dev.sum_batches_backward(n, bd, dev.tensor(dy), gt)
    assert gt.numpy().tobytes() == orc.sum_batches_backward(n, bd, dy, g0.copy()).tobytes()


def test_sum_batches_golden_cadd_broadcast2_neg_val(dev, golden):
    g = golden["node_values"]
    x1 = dev.tensor(f32(g["fixture_params"]["param1"]).reshape(1, 3))
    x2 = dev.tensor(f32(g["fixture_params"]["param4"]).reshape(2, 3))
    neg, y, z = dev.empty((2, 3)), dev.empty((2, 3)), dev.empty(3)
    dev.unary_forward(lib.OP_NEGATE, x2, neg)
    dev.csum_forward(3, 1, 2, x1, neg, y)
    dev.sum_batches_forward(3, 2, y, z)
    exp = g["cadd_broadcast2_neg_val"]
    assert abs(float(z.numpy().astype(np.float64).sum()) - exp["expected"]) <= exp["rel_tol"] * abs(exp["expected"])


@pytest.mark.parametrize("n,bd", [(1024, 4096), (9, 3), (1000, 17), (1, 4), (50, 3000), (100, 7), (200, 9), (400, 5), (1500, 3),
                                  (3000, 3), (5000, 2), (10000, 2), (16384, 2), (16385, 2), (70000, 2), (24577, 5), (30000, 64), (7, 1000), (3, 70001),
                                  (17, 999), (32, 513), (5, 1), (2, 300), (12, 257)])
def test_mean_std_elems(dev, n, bd):
    rng = np.random.default_rng(41)
    x = f32(rng.standard_normal((bd, n)) + 0.5)
    xt = dev.tensor(x)
    mt, st = dev.empty(bd), dev.empty(bd)
    dev.mean_elems_forward(n, bd, xt, mt)
    dev.std_elems_forward(n, bd, xt, st)
    assert_close(mt.numpy(), orc.mean_elems_forward(n, bd, x), FWD_RTOL, "mean_elems", floor=1.0 / np.sqrt(n))
    sd_ref = orc.std_elems_forward(n, bd, x)
    assert_close(st.numpy(), sd_ref, FWD_RTOL, "std_elems", floor=1e-6)
    if n > 1:
        dy, g0 = f32(rng.standard_normal(bd)), f32(rng.standard_normal((bd, n)))
        gt = dev.tensor(g0)
        dev.mean_elems_backward(n, bd, dev.tensor(dy), gt)
        assert_close(gt.numpy(), orc.mean_elems_backward(n, bd, dy, g0.copy()), GRAD_RTOL, "mean bwd", floor=1e-6)
        gt = dev.tensor(g0)
        dev.std_elems_backward(n, bd, xt, dev.tensor(sd_ref), dev.tensor(dy), gt)
        assert_close(gt.numpy(), orc.std_elems_backward(n, bd, x, sd_ref, dy, g0.copy()), GRAD_RTOL, "std bwd",
                     floor=1e-3)


@pytest.mark.parametrize("n,bd", [(300001, 3), (1048576, 4), (2000003, 1)])
def test_mean_std_long_elements(dev, n, bd):
    """Elements of 10^5..10^6 floats: the sequential fp32 sums of the CPU restatement have themselves drifted by
    several 1e-5 at this length, so the check is against the same formulas (dynet/nodes-moments.cc:264-274, 497-527)
    in fp64."""
    rng = np.random.default_rng(43)
    x = f32(rng.standard_normal((bd, n)) * 1.5 + 0.5)
    xt = dev.tensor(x)
    mt, st = dev.empty(bd), dev.empty(bd)
    dev.mean_elems_forward(n, bd, xt, mt)
    dev.std_elems_forward(n, bd, xt, st)
    x64 = x.astype(np.float64)
    mean, sd = x64.mean(axis=1), x64.std(axis=1)
    assert_close(mt.numpy(), mean, FWD_RTOL, "mean_elems", floor=1e-3)
    assert_close(st.numpy(), sd, FWD_RTOL, "std_elems", floor=1e-6)
    dy, g0 = f32(rng.standard_normal(bd)), f32(rng.standard_normal((bd, n)))
    gt = dev.tensor(g0)
    dev.std_elems_backward(n, bd, xt, dev.tensor(f32(sd)), dev.tensor(dy), gt)
    ref = g0 + (2.0 / n) * (x64 - mean[:, None]) * (dy.astype(np.float64) / (2.0 * f32(sd)))[:, None]
    assert_close(gt.numpy(), ref, GRAD_RTOL, "std bwd", floor=1e-3)
    gt = dev.tensor(g0)
    dev.mean_elems_backward(n, bd, dev.tensor(dy), gt)
    assert_close(gt.numpy(), g0 + dy.astype(np.float64)[:, None] / n, GRAD_RTOL, "mean bwd", floor=1e-3)


def test_std_golden_std_dim_value(dev, golden):
    g = golden["node_values"]
    x = f32(g["fixture_params"]["param_cube1"]).reshape(3, 3, 3)
    cols = np.ascontiguousarray(np.stack([x[:, j, :].reshape(-1) for j in range(3)]))
    y, z = dev.empty(3), dev.empty(1)
    dev.std_elems_forward(9, 3, dev.tensor(cols), y)
    dev.mean_elems_forward(3, 1, y, z)
    exp = g["std_dim_value"]
    assert abs(float(z.numpy()[0]) - exp["expected"]) <= exp["rel_tol"] * exp["expected"]


# ---------------------------------------------------------------------------
# fused LayerNorm
# ---------------------------------------------------------------------------
def _ln_case(n, bd, seed):
    rng = np.random.default_rng(seed)
    x = f32(rng.standard_normal((bd, n)))
    g = f32(rng.uniform(0.5, 1.5, n))
    b = f32(rng.standard_normal(n) * 0.1)
    dy = f32(rng.standard_normal((bd, n)))
    return rng, x, g, b, dy


def _ln_fp64(x, g, b, dy):
    """y = g (x - mean) / (std + 1e-8) + b per row in fp64 and its analytic gradients: with s = std + eps, q = xc / s,
    dq = dy g:  dx = dq / s - mean(dq) / s - xc * sum(dq xc) / (n s^2 std);  dg = sum_b dy q;  db = sum_b dy."""
    x, g, b, dy = (np.asarray(a, np.float64) for a in (x, g, b, dy))
    n = x.shape[1]
    xc = x - x.mean(axis=1, keepdims=True)
    std = np.sqrt((xc * xc).mean(axis=1, keepdims=True))
    s = std + np.float64(np.float32(1e-8))
    q = xc / s
    dq = dy * g
    dxc = dq / s - xc * (dq * xc).sum(axis=1, keepdims=True) / (n * s * s * std)
    dx = dxc - dxc.mean(axis=1, keepdims=True)
    return g * q + b, dx, (dy * q).sum(axis=0), dy.sum(axis=0)


@pytest.mark.parametrize("n,bd", [(1024, 4096), (2048, 64), (512, 33), (256, 5), (64, 1), (12, 7), (1027, 9),
                                  (4096, 6), (3, 1), (4096, 1024), (4100, 300), (37, 1000), (70, 2051),
                                  (8192, 70), (16384, 33), (2052, 19), (12288, 5), (16388, 9),
                                  # rows that are not a multiple of four floats: one float per lane and step up to
                                  # 1024 (backward) / 2048 (forward) floats, the block-per-row kernels beyond
                                  (650, 3000), (1001, 20), (250, 100), (50, 9), (65, 130), (1022, 5), (1026, 3),
                                  (2046, 3), (2050, 2),
                                  # rows of up to 256 floats: 4, 8 or 16 lanes a row, several rows a wavefront; row
                                  # counts that leave groups of the last wavefront without a row, and enough rows
                                  # for several sweeps of every wavefront
                                  (4, 3), (8, 40000), (16, 100001), (20, 77), (32, 65537), (64, 70001), (100, 4099),
                                  (128, 33000), (132, 129), (192, 3001), (256, 20000),
                                  # the same with rows that cannot take 128-bit accesses
                                  (3, 1000), (5, 100003), (7, 1000), (10, 50001), (30, 20001), (50, 30000), (70, 10001),
                                  (150, 3000), (250, 5001)])
def test_layer_norm_forward_backward(dev, n, bd):
    rng, x, g, b, dy = _ln_case(n, bd, 51)
    xt, gt, bt, dyt = dev.tensor(x), dev.tensor(g), dev.tensor(b), dev.tensor(dy)
    yt = dev.empty((bd, n))
    dev.layer_norm_forward(n, bd, xt, gt, bt, yt)
    ref = orc.layer_norm_forward(n, bd, x, g, b)
    # y = g*q + b with |g*q| ~ 1: relative to the size of the terms
    assert_close(yt.numpy(), ref, FWD_RTOL, "layer_norm fwd", floor=1.0)
    dx0, dg0, db0 = f32(rng.standard_normal((bd, n))), f32(rng.standard_normal(n)), f32(rng.standard_normal(n))
    dxt, dgt, dbt = dev.tensor(dx0), dev.tensor(dg0), dev.tensor(db0)
    dev.layer_norm_backward(n, bd, xt, gt, dyt, dxt, dgt, dbt)
    wx, wg, wb = orc.layer_norm_backward(n, bd, x, g, dy, dx0.copy(), dg0.copy(), db0.copy())
    assert_close(dxt.numpy(), wx, GRAD_RTOL, "layer_norm dx", floor=1.0)
    assert_close(dgt.numpy(), wg, GRAD_RTOL, "layer_norm dg", floor=np.sqrt(bd))
    assert_close(dbt.numpy(), wb, GRAD_RTOL, "layer_norm db", floor=np.sqrt(bd))
    # and per element against the fp64 value of the same fp32 inputs: the device result must be as close to it as
    # the CPU path is (within a small factor), so that no kernel hides behind the floor of the relative bars above
    y64, dx64, dg64, db64 = _ln_fp64(x, g, b, dy)
    assert_shadow(yt.numpy(), ref, y64, "layer_norm fwd vs fp64", rel_min=1e-3)
    assert_shadow(dxt.numpy(), wx, dx0.astype(np.float64) + dx64, "layer_norm dx vs fp64", rel_min=1e-2)
    assert_shadow(dgt.numpy(), wg, dg0.astype(np.float64) + dg64, "layer_norm dg vs fp64", k=6.0, rel_min=1.0)
    assert_shadow(dbt.numpy(), wb, db0.astype(np.float64) + db64, "layer_norm db vs fp64", k=6.0, rel_min=1.0)
    # one argument at a time, as Node::backward is called
    dxt2 = dev.tensor(dx0)
    dev.layer_norm_backward(n, bd, xt, gt, dyt, dx=dxt2)
    assert dxt2.numpy().tobytes() == dxt.numpy().tobytes()
    dgt2 = dev.tensor(dg0)
    dev.layer_norm_backward(n, bd, xt, gt, dyt, dg=dgt2)
    assert dgt2.numpy().tobytes() == dgt.numpy().tobytes()


def test_layer_norm_random_short_rows(dev):
    """Seeded random row widths of 4..400 floats and row counts of 1..6000, half of them on tensors that start 4 bytes
    past a 16-byte boundary: every several-rows-a-wavefront kernel (4, 8, 16, 32 lanes a row, with and without 128-bit
    accesses) and the one-wavefront-per-row kernels above them, against the oracle."""
    rng0 = np.random.default_rng(404)
    for it in range(36):
        n = int(rng0.choice([int(rng0.integers(4, 70)), 4 * int(rng0.integers(1, 70)), int(rng0.integers(70, 400))]))
        bd = int(rng0.choice([int(rng0.integers(1, 40)), int(rng0.integers(40, 6000))]))
        shift = int(rng0.integers(0, 2))
        rng, x, g, b, dy = _ln_case(n, bd, 1000 + it)
        def put(a):
            base = dev.empty(a.size + shift)
            t = base.offset(shift, a.shape)
            t.set(a)
            return t
        what = "n=%d bd=%d shift=%d" % (n, bd, shift)
        xo, go, bo, dyo = put(x), put(g), put(b), put(dy)
        yo = put(np.zeros((bd, n), np.float32))
        dev.layer_norm_forward(n, bd, xo, go, bo, yo)
        assert_close(yo.numpy(), orc.layer_norm_forward(n, bd, x, g, b), FWD_RTOL, "layer_norm fwd " + what, floor=1.0)
        dx0, dg0, db0 = f32(rng.standard_normal((bd, n))), f32(rng.standard_normal(n)), f32(rng.standard_normal(n))
        dxo, dgo, dbo = put(dx0), put(dg0), put(db0)
        dev.layer_norm_backward(n, bd, xo, go, dyo, dxo, dgo, dbo)
        wx, wg, wb = orc.layer_norm_backward(n, bd, x, g, dy, dx0.copy(), dg0.copy(), db0.copy())
        assert_close(dxo.numpy(), wx, GRAD_RTOL, "layer_norm dx " + what, floor=1.0)
        assert_close(dgo.numpy(), wg, GRAD_RTOL, "layer_norm dg " + what, floor=np.sqrt(bd))
        assert_close(dbo.numpy(), wb, GRAD_RTOL, "layer_norm db " + what, floor=np.sqrt(bd))
        for w in (lib.POOL_FXS, lib.POOL_DEDFS, lib.POOL_SCS):
            dev.sync()
            dev.free_pool(w)


def test_layer_norm_on_pointers_off_a_16_byte_boundary(dev):
    """Rows of a multiple of four floats whose tensors start 4 bytes past a 16-byte boundary: no 128-bit accesses, the
    one-float-per-lane kernels (a lane then owns other elements of a row, so the row sums round differently: the
    results are held to the oracle's bars, not to the aligned call's bits)."""
    n, bd = 512, 300
    rng, x, g, b, dy = _ln_case(n, bd, 77)
    def off(a):
        base = dev.empty(a.size + 1)
        t = base.offset(1, a.shape)
        t.set(a)
        return t
    xo, go, bo, dyo = off(x), off(g), off(b), off(dy)
    yo = off(np.zeros((bd, n), np.float32))
    dev.layer_norm_forward(n, bd, xo, go, bo, yo)
    assert_close(yo.numpy(), orc.layer_norm_forward(n, bd, x, g, b), FWD_RTOL, "layer_norm fwd (offset pointers)", floor=1.0)
    dx0, dg0, db0 = f32(rng.standard_normal((bd, n))), f32(rng.standard_normal(n)), f32(rng.standard_normal(n))
    dxo, dgo, dbo = off(dx0), off(dg0), off(db0)
    dev.layer_norm_backward(n, bd, xo, go, dyo, dxo, dgo, dbo)
    wx, wg, wb = orc.layer_norm_backward(n, bd, x, g, dy, dx0.copy(), dg0.copy(), db0.copy())
    assert_close(dxo.numpy(), wx, GRAD_RTOL, "layer_norm dx (offset pointers)", floor=1.0)
    assert_close(dgo.numpy(), wg, GRAD_RTOL, "layer_norm dg (offset pointers)", floor=np.sqrt(bd))
    assert_close(dbo.numpy(), wb, GRAD_RTOL, "layer_norm db (offset pointers)", floor=np.sqrt(bd))



CWISE_SHAPES = [
    # dims_a, dims_b as (d0, d1, d2, d3, bd)
    ((1024, 1, 1, 1, 4096), (1, 1, 1, 1, 4096)),  # x - mean and x / sigma of the layer_norm composite, baseline shape
    ((1024, 1, 1, 1, 33), (1, 1, 1, 1, 33)),
    ((5, 3, 1, 1, 4), (5, 1, 1, 1, 1)),
    ((5, 3, 1, 1, 4), (1, 3, 1, 1, 4)),
    ((4, 3, 2, 1, 3), (4, 1, 2, 1, 1)),
    ((2, 3, 4, 5, 2), (1, 3, 1, 5, 1)),
    ((128, 70, 1, 1, 9), (128, 1, 1, 1, 1)),      # kept axes are a prefix: the coalesced batch reduction
    ((64, 100, 1, 1, 3), (1, 100, 1, 1, 3)),      # 64 terms per output: one wavefront each
    ((7, 1, 1, 1, 3), (7, 1, 1, 1, 3)),           # nothing broadcast
    ((6, 2, 1, 1, 5), (6, 2, 1, 1, 1)),           # batch only: the streaming kernels
    ((1023, 3, 1, 1, 2), (1, 3, 1, 1, 1)),        # d0 not a multiple of 4
    # three axes left after merging: a column vector per batch element against a matrix (broadcast over the middle
    # axis; its gradient sums over that axis with lanes along the rows), short inner axes (a block folds over rows)
    ((256, 64, 1, 1, 40), (256, 1, 1, 1, 40)),
    ((64, 70, 1, 1, 150), (64, 1, 1, 1, 150)),
    ((20, 7, 1, 1, 300), (20, 1, 1, 1, 300)),
    ((12, 5, 3, 1, 4), (12, 1, 3, 1, 4)),
    ((130, 9, 1, 1, 70000), (130, 1, 1, 1, 70000)),  # more than 65535 entries along the outer axis
    ((8, 3, 1, 1, 5), (8, 3, 1, 1, 1)),
    # gradients of the broadcast argument: a short reduced middle axis (lanes along the rows), a short contiguous
    # reduced axis (a wavefront per output), few outputs with a long reduced axis (pieces through scratch, strided,
    # 128-bit and ragged), reduced axes with a kept axis between them (two stages through scratch)
    ((1024, 35, 1, 1, 16), (1024, 1, 1, 1, 16)),
    ((50, 1, 1, 1, 500), (1, 1, 1, 1, 500)),
    ((9, 4, 1, 1, 300), (1, 4, 1, 1, 300)),
    ((3, 20000, 1, 1, 1), (3, 1, 1, 1, 1)),
    ((20000, 3, 1, 1, 1), (1, 3, 1, 1, 1)),
    ((10001, 3, 1, 1, 2), (1, 3, 1, 1, 2)),
    ((7, 9, 11, 1, 20), (7, 1, 11, 1, 1)),
    ((128, 96, 1, 1, 8), (1, 96, 1, 1, 1)),
    ((2, 2, 2, 2, 500), (2, 1, 2, 1, 500)),
    ((6, 40, 3, 5, 4), (6, 1, 3, 1, 4)),
]


@pytest.mark.parametrize("op", [lib.CWISE_SUM, lib.CWISE_MULT, lib.CWISE_QUOTIENT])
@pytest.mark.parametrize("da,db", CWISE_SHAPES)
def test_cwise_with_dimension_broadcast(dev, op, da, db):
    """CwiseSum / CwiseMultiply / CwiseQuotient with broadcast over dimensions (dynet/nodes-arith-cwise.cc incl. the
    backward_helper reductions), both argument orders, against the oracle."""
    from dynet_amd import DyhipError

    rng = np.random.default_rng(sum(da) + 3 * sum(db) + op)
    for swap in (False, True):
        d0, d1 = (db, da) if swap else (da, db)
        if op == lib.CWISE_QUOTIENT and any(x != y and y != 1 for x, y in zip(d0, d1)):
            t = dev.zeros(4)
            with pytest.raises(DyhipError) as e:
                dev.cwise_forward(op, d0, d1, t, t, t)
            assert e.value.status == lib.ERR_INVALID_ARG and "CwiseQuotient" in str(e.value)
            continue
        a = f32(rng.standard_normal(d0[::-1]))
        b = f32(rng.standard_normal(d1[::-1]))
        if op == lib.CWISE_QUOTIENT:
            b = f32(np.sign(b) * (np.abs(b) + 0.5))  # keep the divisor away from zero
        at, bt = dev.tensor(a), dev.tensor(b)
        want = orc.cwise_forward(op, d0, d1, a, b)
        fx = dev.empty(want.shape)
        dev.cwise_forward(op, d0, d1, at, bt, fx)
        if op == lib.CWISE_QUOTIENT:
            assert_close(fx.numpy(), want, FWD_RTOL, "cwise fwd")  # one correctly rounded division each
        else:
            assert fx.numpy().tobytes() == want.tobytes()
        dy = f32(rng.standard_normal(want.shape))
        dyt = dev.tensor(dy)
        for i, x in enumerate((a, b)):
            g0 = f32(rng.standard_normal(x.shape))
            gt = dev.tensor(g0)
            dev.cwise_backward(op, d0, d1, at, bt, dyt, i, gt)
            ref = orc.cwise_backward(op, d0, d1, a, b, dy, i, g0.copy())
            terms = want.size / x.size  # terms summed into one output element
            other = np.abs(b if i == 0 else a).max() if op != lib.CWISE_SUM else 1.0
            if op == lib.CWISE_QUOTIENT:
                other = (1.0 / np.abs(b).min()) * (1.0 if i == 0 else np.abs(a).max() / np.abs(b).min())
            assert_close(gt.numpy(), ref, GRAD_RTOL, "cwise bwd op %d arg %d" % (op, i),
                         floor=np.maximum(np.abs(g0), rms(dy) * other * np.sqrt(terms)))


def test_cwise_random_broadcast_shapes(dev):
    """Forty random shapes of up to five axes with random broadcast patterns (one long axis now and then, so that every
    reduction form is reached: thread, wavefront, lanes along rows, pieces through scratch, two stages): forward and
    both gradients of CwiseMultiply and CwiseQuotient against the oracle (dynet/nodes-arith-cwise.cc:196-307, 338-421)."""
    rng = np.random.default_rng(2024)
    for case in range(40):
        full = [int(rng.integers(1, 9)) for _ in range(5)]
        if case % 3 == 0:
            full[int(rng.integers(0, 5))] = int(rng.choice([70, 300, 1100, 9000]))
        if case % 7 == 0:
            full[0] = 4 * int(rng.integers(1, 40))
        keep = [bool(rng.integers(0, 2)) for _ in range(5)]
        da = tuple(full)
        db = tuple(f if k else 1 for f, k in zip(full, keep))
        for op in (lib.CWISE_MULT, lib.CWISE_QUOTIENT):
            a = f32(rng.standard_normal(da[::-1]))
            b = f32(rng.standard_normal(db[::-1]))
            if op == lib.CWISE_QUOTIENT:
                b = f32(np.sign(b) * (np.abs(b) + 0.5))
            at, bt = dev.tensor(a), dev.tensor(b)
            want = orc.cwise_forward(op, da, db, a, b)
            fx = dev.empty(want.shape)
            dev.cwise_forward(op, da, db, at, bt, fx)
            assert_close(fx.numpy(), want, FWD_RTOL, "cwise fwd %s x %s" % (da, db))
            dy = f32(rng.standard_normal(want.shape))
            dyt = dev.tensor(dy)
            for i, x in enumerate((a, b)):
                g0 = f32(rng.standard_normal(x.shape))
                gt = dev.tensor(g0)
                dev.cwise_backward(op, da, db, at, bt, dyt, i, gt)
                ref = orc.cwise_backward(op, da, db, a, b, dy, i, g0.copy())
                terms = want.size / x.size
                other = np.abs(b if i == 0 else a).max()
                if op == lib.CWISE_QUOTIENT:
                    other = (1.0 / np.abs(b).min()) * (1.0 if i == 0 else np.abs(a).max() / np.abs(b).min())
                assert_close(gt.numpy(), ref, GRAD_RTOL, "cwise bwd op %d arg %d %s x %s" % (op, i, da, db),
                             floor=np.maximum(np.abs(g0), rms(dy) * other * np.sqrt(terms)))
        for w in (lib.POOL_FXS, lib.POOL_DEDFS, lib.POOL_SCS):
            dev.sync()
            dev.free_pool(w)


def test_layer_norm_composite_of_eight_nodes_on_the_device(dev):
    """dynet/expr.cc:248-253 issued node by node through the C-ABI (mean_elems, Negate, CwiseSum, std_elems,
    ConstantPlusX, CwiseQuotient, CwiseMultiply, CwiseSum; forward and backward) at the baseline's shape, against
    the fused kernels and against the oracle's layer_norm."""
    n, bd = 1024, 4096
    rng, x, g, b, dy = _ln_case(n, bd, 77)
    X, S, G = (n, 1, 1, 1, bd), (1, 1, 1, 1, bd), (n, 1, 1, 1, 1)
    xt, gt, bt, dyt = dev.tensor(x), dev.tensor(g), dev.tensor(b), dev.tensor(dy)
    e = lambda *s: dev.empty(s)
    z = lambda *s: dev.zeros(s, pool=lib.POOL_DEDFS)
    mu, neg, xc, sigma, se, q, gq, y = e(bd), e(bd), e(bd, n), e(bd), e(bd), e(bd, n), e(bd, n), e(bd, n)
    dev.mean_elems_forward(n, bd, xt, mu)
    dev.unary_forward(lib.OP_NEGATE, mu, neg)
    dev.cwise_forward(lib.CWISE_SUM, X, S, xt, neg, xc)
    dev.std_elems_forward(n, bd, xt, sigma)
    dev.const_plus_x_forward(1e-8, sigma, se)
    dev.cwise_forward(lib.CWISE_QUOTIENT, X, S, xc, se, q)
    dev.cwise_forward(lib.CWISE_MULT, G, X, gt, q, gq)
    dev.cwise_forward(lib.CWISE_SUM, X, G, gq, bt, y)
    fused = e(bd, n)
    dev.layer_norm_forward(n, bd, xt, gt, bt, fused)
    ref = orc.layer_norm_forward(n, bd, x, g, b).reshape(bd, n)
    assert_close(y.numpy(), ref, FWD_RTOL, "composite fwd vs oracle", floor=1.0)
    assert_close(y.numpy(), fused.numpy(), FWD_RTOL, "composite fwd vs fused", floor=1.0)
    # backward, in reverse topological order; every node accumulates into its arguments' gradients
    d_gq, d_b, d_g, d_q, d_xc, d_se, d_x, d_neg, d_mu = z(bd, n), z(n), z(n), z(bd, n), z(bd, n), z(bd), z(bd, n), z(bd), z(bd)
    dev.cwise_backward(lib.CWISE_SUM, X, G, gq, bt, dyt, 0, d_gq)
    dev.cwise_backward(lib.CWISE_SUM, X, G, gq, bt, dyt, 1, d_b)
    dev.cwise_backward(lib.CWISE_MULT, G, X, gt, q, d_gq, 0, d_g)
    dev.cwise_backward(lib.CWISE_MULT, G, X, gt, q, d_gq, 1, d_q)
    dev.cwise_backward(lib.CWISE_QUOTIENT, X, S, xc, se, d_q, 0, d_xc)
    dev.cwise_backward(lib.CWISE_QUOTIENT, X, S, xc, se, d_q, 1, d_se)
    dev.std_elems_backward(n, bd, xt, sigma, d_se, d_x)            # ConstantPlusX: d_sigma += d_se, same buffer
    dev.cwise_backward(lib.CWISE_SUM, X, S, xt, neg, d_xc, 0, d_x)
    dev.cwise_backward(lib.CWISE_SUM, X, S, xt, neg, d_xc, 1, d_neg)
    dev.unary_backward(lib.OP_NEGATE, neg, d_neg, d_mu)
    dev.mean_elems_backward(n, bd, d_mu, d_x)
    fx_, fg_, fb_ = z(bd, n), z(n), z(n)
    dev.layer_norm_backward(n, bd, xt, gt, dyt, fx_, fg_, fb_)
    wx, wg, wb = orc.layer_norm_backward(n, bd, x, g, dy, np.zeros((bd, n), F32), np.zeros(n, F32), np.zeros(n, F32))
    for got, fusedv, want, fl, what in ((d_x, fx_, wx, 1.0, "dx"), (d_g, fg_, wg, np.sqrt(bd), "dg"), (d_b, fb_, wb, np.sqrt(bd), "db")):
        assert_close(got.numpy(), want.reshape(got.shape), GRAD_RTOL, "composite %s vs oracle" % what, floor=fl)
        assert_close(got.numpy(), fusedv.numpy(), GRAD_RTOL, "composite %s vs fused" % what, floor=fl)


def test_layer_norm_golden_vectors(dev, golden):
    g = golden["node_values"]
    x = f32(g["fixture_params"]["param1"]).reshape(1, 3)
    yt = dev.empty((1, 3))
    dev.layer_norm_forward(3, 1, dev.tensor(x), dev.tensor(np.ones(3, F32)), dev.tensor(np.zeros(3, F32)), yt)
    y = yt.numpy().astype(np.float64)
    exp = g["layer_norm_forward"]
    assert abs(y.sum() / 3.0) < exp["mean_abs_max"]
    assert abs(np.sqrt((y ** 2).sum() / 3.0) - exp["rms"]) <= exp["rms_rel_tol"]
    exp = g["layer_norm_python"]
    v = np.arange(exp["n"]).astype(np.float64)
    vt = dev.tensor(f32(v))
    yt = dev.empty((1, exp["n"]))
    dev.layer_norm_forward(exp["n"], 1, vt, vt, vt, yt)
    assert np.allclose(yt.numpy().reshape(-1), v / v.std() * (v - v.mean()) + v, rtol=exp["rtol"], atol=exp["atol"])


def test_layer_norm_invariances_at_full_size(dev):
    n, bd = 1024, 4096
    _, x, g, b, _ = _ln_case(n, bd, 52)
    gt, bt = dev.tensor(g), dev.tensor(b)
    y0, y1 = dev.empty((bd, n)), dev.empty((bd, n))
    dev.layer_norm_forward(n, bd, dev.tensor(x), gt, bt, y0)
    dev.layer_norm_forward(n, bd, dev.tensor(x * F32(4.0)), gt, bt, y1)  # exact power-of-two scaling
    assert_close(y1.numpy(), y0.numpy(), FWD_RTOL, "LN(4x) == LN(x)", floor=1.0)
    dev.layer_norm_forward(n, bd, dev.tensor(x + F32(2.0)), gt, bt, y1)
    assert_close(y1.numpy(), y0.numpy(), 5e-5, "LN(x+2) == LN(x)", floor=1.0)


@pytest.mark.parametrize("k,n,bd", [(k, 1031, 6) for k in (1, 2, 4, 5, 7, 8, 11, 32, 33, 35, 36, 37, 128)] + [(35, 1, 128), (70, 1, 1)])
def test_sum_node_bit_exact(dev, k, n, bd):
    """Argument counts across one launch's capacity (eight groups, 32 arguments) and the group of `(k - 4) % 4`."""
    rng = np.random.default_rng(k)
    xs = [f32(rng.standard_normal((bd, n)) * 10.0 ** rng.integers(-2, 3)) for _ in range(k)]
    fx = dev.empty((bd, n))
    dev.sum_forward(n, bd, [dev.tensor(x) for x in xs], [bd] * k, fx)
    assert fx.numpy().tobytes() == orc.sum_forward(n, bd, xs, [bd] * k).tobytes()


@pytest.mark.parametrize("bds", [[5, 1, 5], [1, 5, 5, 1, 1, 5, 1, 5, 5, 1, 5], [5] + [1] * 40])
def test_sum_node_broadcast_and_backward(dev, bds):
    rng = np.random.default_rng(3)
    n, bd = 300, 5
    xs = [f32(rng.standard_normal((b, n))) for b in bds]
    fx = dev.empty((bd, n))
    dev.sum_forward(n, bd, [dev.tensor(x) for x in xs], bds, fx)
    assert fx.numpy().tobytes() == orc.sum_forward(n, bd, xs, bds).tobytes()
    dy = f32(rng.standard_normal((bd, n)))
    for i, b in enumerate(bds):
        g0 = f32(rng.standard_normal((b, n)))
        dx = dev.tensor(g0)
        dev.csum_backward(n, b, bd, dev.tensor(dy), 0, dx)
        want = orc.csum_backward(n, b, bd, dy, 0, g0.copy())
        assert_close(dx.numpy(), want, GRAD_RTOL, f"sum bwd arg {i}", floor=np.sqrt(bd))
