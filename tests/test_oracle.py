"""Pins the CPU oracle (oracle/) before anything is compared against it.

Each oracle function is checked against (i) the known-answer vectors the
reference's own tests hold (tests/golden/*.json, transcribed from
tests/test-rnn.cc, tests/test-nodes.cc, tests/test-tensor.cc,
tests/python/test.py of the DyNet tree), and (ii) what the mathematics fixes:
independent fp64 numpy formulas, central differences, invariances and brute
force on tiny inputs -- chosen so that a dropped term, a wrong sign or a
transposed operand fails.  No GPU needed.
"""
import numpy as np
import pytest
from scipy.special import logsumexp as sp_logsumexp

from oracle import cpu_oracle as orc
from util import assert_close

F32 = np.float32


def f32(a):
    return np.asarray(a, dtype=F32)


def sigmoid64(x):
    return 1.0 / (1.0 + np.exp(-np.asarray(x, np.float64)))


def assert_rel(a, b, rel, what=""):
    a = np.asarray(a, np.float64)
    b = np.asarray(b, np.float64)
    err = np.abs(a - b)
    tol = rel * np.abs(b)
    assert np.all(err <= tol), "%s: max rel err %g" % (what, np.max(err / np.maximum(np.abs(b), 1e-300)))


# ---------------------------------------------------------------------------
# logistic functor
# ---------------------------------------------------------------------------
def test_logistic_packet_matches_exact_sigmoid_absolutely():
    xs = np.concatenate([np.linspace(-25, 25, 20001), [0.0, -18.0, 18.0, -1e-8, 1e-8]]).astype(F32)
    y = orc.logistic_packet(xs)
    assert np.max(np.abs(y.astype(np.float64) - sigmoid64(xs))) < 2e-7
    assert y.min() >= 0.0 and y.max() <= 1.0
    # clamp: everything beyond +-18 equals the value at +-18
    assert np.all(orc.logistic_packet(f32([19, 100, 1e30])) == orc.logistic_packet(f32([18])))
    assert np.all(orc.logistic_packet(f32([-19, -100, -1e30])) == orc.logistic_packet(f32([-18])))


def test_logistic_packet_symmetry_and_midpoint():
    xs = np.linspace(0, 18, 1801).astype(F32)
    s = orc.logistic_packet(xs).astype(np.float64) + orc.logistic_packet(-xs).astype(np.float64)
    assert np.max(np.abs(s - 1.0)) <= 1.2e-7
    assert orc.logistic_packet(f32([0.0]))[0] == F32(0.5)


def test_logistic_packet_is_not_relatively_accurate_in_the_left_tail():
    # documents WHY the kernel mirrors the polynomial: against the exact form the
    # packet form is off by far more than 1e-5 relative once sigma(x) is small
    x = f32([-12.0])
    rel = abs(float(orc.logistic_packet(x)[0]) - sigmoid64(-12.0)) / sigmoid64(-12.0)
    assert rel > 1e-4


def test_logistic_scalar_is_exact_form():
    xs = np.linspace(-30, 30, 2001).astype(F32)
    assert_rel(orc.logistic_scalar(xs), sigmoid64(xs), 3e-7, "logistic_scalar")


# ---------------------------------------------------------------------------
# elementwise
# ---------------------------------------------------------------------------
def test_unary_forward_against_fp64(golden):
    rng = np.random.default_rng(1)
    x = np.concatenate([rng.standard_normal(4096) * 3, golden["node_values"]["fixture_params"]["param1"], [0.0, -0.0]])
    x = f32(x)
    assert_rel(orc.unary_forward(orc.OP_TANH, x), np.tanh(x.astype(np.float64)), 3e-7, "tanh")
    assert np.array_equal(orc.unary_forward(orc.OP_RECTIFY, x), np.maximum(x, 0))
    assert np.array_equal(orc.unary_forward(orc.OP_NEGATE, x), -x)
    assert np.max(np.abs(orc.unary_forward(orc.OP_LOGISTIC, x).astype(np.float64) - sigmoid64(x))) < 2e-7
    assert_rel(orc.unary_forward(orc.OP_LOGISTIC, x, orc.LOGISTIC_SCALAR), sigmoid64(x), 3e-7, "logistic scalar")


@pytest.mark.parametrize("op", [orc.OP_TANH, orc.OP_LOGISTIC, orc.OP_RECTIFY, orc.OP_NEGATE])
def test_unary_backward_accumulates_the_derivative(op):
    rng = np.random.default_rng(2)
    x = f32(rng.standard_normal(513))
    x[:3] = [0.0, -1.0, 2.0]
    dy = f32(rng.standard_normal(513))
    fx = orc.unary_forward(op, x, orc.LOGISTIC_SCALAR)
    base = f32(rng.standard_normal(513))
    dx = orc.unary_backward(op, fx, dy, base.copy())
    x64 = x.astype(np.float64)
    deriv = {orc.OP_TANH: 1 - np.tanh(x64) ** 2, orc.OP_LOGISTIC: sigmoid64(x64) * (1 - sigmoid64(x64)),
             orc.OP_RECTIFY: (x64 > 0).astype(np.float64), orc.OP_NEGATE: -np.ones_like(x64)}[op]
    want = base.astype(np.float64) + deriv * dy
    assert np.max(np.abs(dx - want)) < 1e-6 * max(1.0, np.max(np.abs(want)))
    if op == orc.OP_RECTIFY:  # ReLU'(0) = 0 because the mask is cast<bool>(fx)
        assert dx[0] == base[0]


def test_cmult_and_csum_broadcast_forward_backward():
    rng = np.random.default_rng(3)
    n, bd = 7, 5
    a, b1, dy = f32(rng.standard_normal((bd, n))), f32(rng.standard_normal((1, n))), f32(rng.standard_normal((bd, n)))
    assert np.allclose(orc.cmult_forward(n, bd, 1, a, b1), a * b1, rtol=0, atol=0)
    assert np.allclose(orc.cmult_forward(n, 1, bd, b1, a), a * b1, rtol=0, atol=0)
    assert np.allclose(orc.csum_forward(n, bd, 1, a, b1), a + b1, rtol=0, atol=0)
    # backward to the full-batch argument and to the broadcast argument
    da = orc.cmult_backward(n, bd, 1, a, b1, dy, 0, np.ones((bd, n), F32))
    assert np.allclose(da, 1 + dy * b1, rtol=1e-6)
    db = orc.cmult_backward(n, bd, 1, a, b1, dy, 1, np.ones((1, n), F32))
    assert np.allclose(db, 1 + (dy.astype(np.float64) * a).sum(0), rtol=1e-5)
    db = orc.csum_backward(n, bd, 1, dy, 1, np.ones((1, n), F32))
    assert np.allclose(db, 1 + dy.astype(np.float64).sum(0), rtol=1e-5)
    da = orc.csum_backward(n, bd, 1, dy, 0, np.ones((bd, n), F32))
    assert np.allclose(da, 1 + dy)


# ---------------------------------------------------------------------------
# reductions (golden: cadd_broadcast2_neg_val, std_dim_value)
# ---------------------------------------------------------------------------
CWISE_SHAPES = [
    # dims_a, dims_b as (d0, d1, d2, d3, bd)
    ((1024, 1, 1, 1, 6), (1, 1, 1, 1, 6)),      # x - mean, x / sigma of the layer_norm composite
    ((5, 3, 1, 1, 4), (5, 1, 1, 1, 1)),         # a column vector against a matrix batch
    ((5, 3, 1, 1, 4), (1, 3, 1, 1, 4)),
    ((4, 3, 2, 1, 3), (4, 1, 2, 1, 1)),         # kept axes on both sides of a broadcast one
    ((2, 3, 4, 5, 2), (1, 3, 1, 5, 1)),
    ((7, 1, 1, 1, 3), (7, 1, 1, 1, 3)),         # nothing broadcast
    ((6, 2, 1, 1, 5), (6, 2, 1, 1, 1)),         # batch only
]


@pytest.mark.parametrize("op", [orc.CWISE_SUM, orc.CWISE_MULT, orc.CWISE_QUOTIENT])
@pytest.mark.parametrize("da,db", CWISE_SHAPES)
def test_cwise_broadcast_against_numpy_broadcasting(op, da, db):
    """orc_cwise_*: numpy's own broadcasting in fp64 is the yardstick (shape = reversed dims), both argument
    orders; the backward is the broadcast-reduced product rule, summed with np.sum over the broadcast axes."""
    rng = np.random.default_rng(sum(da) + 7 * sum(db) + op)
    for swap in (False, True):
        d0, d1 = (db, da) if swap else (da, db)
        if op == orc.CWISE_QUOTIENT and any(x != y and y != 1 for x, y in zip(d0, d1)):
            with pytest.raises(ValueError):
                orc.cwise_forward(op, d0, d1, np.zeros(d0[::-1], F32), np.ones(d1[::-1], F32))
            continue
        a = f32(rng.standard_normal(d0[::-1]))
        b = f32(rng.standard_normal(d1[::-1]) + (3.0 if op == orc.CWISE_QUOTIENT else 0.0))
        a64, b64 = a.astype(np.float64), b.astype(np.float64)
        want = a64 + b64 if op == orc.CWISE_SUM else a64 * b64 if op == orc.CWISE_MULT else a64 / b64
        fx = orc.cwise_forward(op, d0, d1, a, b)
        assert fx.shape == want.shape
        assert_close(fx, want, 1e-6, "cwise fwd", floor=1e-3)
        dy = f32(rng.standard_normal(want.shape))
        for i, (x, dims) in enumerate(((a, d0), (b, d1))):
            if op == orc.CWISE_SUM:
                term = dy.astype(np.float64) * np.ones_like(want)
            elif op == orc.CWISE_MULT:
                term = dy * (b64 if i == 0 else a64) * np.ones_like(want)
            else:
                term = dy / b64 if i == 0 else -(dy * a64 / (b64 * b64))
            axes = tuple(k for k, (n_x, n_f) in enumerate(zip(x.shape, want.shape)) if n_x == 1 and n_f > 1)
            red = term.sum(axis=axes, keepdims=True) if axes else term
            g0 = f32(rng.standard_normal(x.shape))
            got = orc.cwise_backward(op, d0, d1, a, b, dy, i, g0.copy())
            assert_close(got, g0 + red, 1e-5, "cwise bwd %d" % i, floor=np.sqrt(want.size / x.size))


def test_cwise_broadcast_reduces_to_the_batch_only_operators():
    rng = np.random.default_rng(3)
    n, bd = 12, 5
    a, b, dy = f32(rng.standard_normal((bd, n))), f32(rng.standard_normal((1, n))), f32(rng.standard_normal((bd, n)))
    da, db = (n, 1, 1, 1, bd), (n, 1, 1, 1, 1)
    assert orc.cwise_forward(orc.CWISE_SUM, da, db, a, b).reshape(bd, n).tobytes() == orc.csum_forward(n, bd, 1, a, b).tobytes()
    assert orc.cwise_forward(orc.CWISE_MULT, da, db, a, b).reshape(bd, n).tobytes() == orc.cmult_forward(n, bd, 1, a, b).tobytes()
    for i, shape in ((0, (bd, n)), (1, (1, n))):
        g0 = f32(rng.standard_normal(shape))
        # bitwise without a reduction; with one the general form sums first and then adds (backward_helper's
        # `+= (...).sum(red_axis)`), the batch-only CPU branch adds term by term
        same = (lambda u, v: u.tobytes() == v.tobytes()) if i == 0 else (lambda u, v: np.allclose(u, v, rtol=1e-6, atol=1e-6))
        assert same(orc.cwise_backward(orc.CWISE_MULT, da, db, a, b, dy, i, g0.copy()),
                    orc.cmult_backward(n, bd, 1, a, b, dy, i, g0.copy()))
        assert same(orc.cwise_backward(orc.CWISE_SUM, da, db, a, b, dy, i, g0.copy()),
                    orc.csum_backward(n, bd, 1, dy, i, g0.copy()))


def test_layer_norm_composite_of_eight_nodes_equals_the_layer_norm_oracle():
    """dynet/expr.cc:248-253 node by node through the oracle's own node functions - mean_elems, Negate + CwiseSum,
    std_elems, ConstantPlusX, CwiseQuotient, CwiseMultiply, CwiseSum - forward and backward, against
    orc_layer_norm_* (which restates the same graph in one function)."""
    rng = np.random.default_rng(12)
    n, bd = 24, 5
    x, g, b = f32(rng.standard_normal((bd, n))), f32(rng.uniform(0.5, 1.5, n)), f32(rng.standard_normal(n) * 0.1)
    dy = f32(rng.standard_normal((bd, n)))
    X, S, G = (n, 1, 1, 1, bd), (1, 1, 1, 1, bd), (n, 1, 1, 1, 1)
    mu = orc.mean_elems_forward(n, bd, x)
    neg = orc.unary_forward(orc.OP_NEGATE, mu)
    xc = orc.cwise_forward(orc.CWISE_SUM, X, S, x, neg)
    sigma = orc.std_elems_forward(n, bd, x)
    se = orc.const_plus_x_forward(1e-8, sigma)
    q = orc.cwise_forward(orc.CWISE_QUOTIENT, X, S, xc, se)
    gq = orc.cwise_forward(orc.CWISE_MULT, G, X, g, q)
    y = orc.cwise_forward(orc.CWISE_SUM, X, G, gq, b)
    assert_close(y.reshape(bd, n), orc.layer_norm_forward(n, bd, x, g, b).reshape(bd, n), 1e-6, "composite fwd", floor=1.0)
    z = lambda *s: np.zeros(s, F32)
    d_gq, d_b = orc.cwise_backward(orc.CWISE_SUM, X, G, gq, b, dy, 0, z(bd, n)), orc.cwise_backward(orc.CWISE_SUM, X, G, gq, b, dy, 1, z(n))
    d_g, d_q = orc.cwise_backward(orc.CWISE_MULT, G, X, g, q, d_gq, 0, z(n)), orc.cwise_backward(orc.CWISE_MULT, G, X, g, q, d_gq, 1, z(bd, n))
    d_xc = orc.cwise_backward(orc.CWISE_QUOTIENT, X, S, xc, se, d_q, 0, z(bd, n))
    d_se = orc.cwise_backward(orc.CWISE_QUOTIENT, X, S, xc, se, d_q, 1, z(bd))
    d_x = orc.std_elems_backward(n, bd, x, sigma, d_se, z(bd, n))            # ConstantPlusX passes d_se through
    d_x = orc.cwise_backward(orc.CWISE_SUM, X, S, x, neg, d_xc, 0, d_x)
    d_neg = orc.cwise_backward(orc.CWISE_SUM, X, S, x, neg, d_xc, 1, z(bd))
    d_mu = orc.unary_backward(orc.OP_NEGATE, neg, d_neg, z(bd))
    d_x = orc.mean_elems_backward(n, bd, d_mu, d_x)
    wx, wg, wb = orc.layer_norm_backward(n, bd, x, g, dy, z(bd, n), z(n), z(n))
    assert_close(d_x, wx, 1e-5, "composite dx", floor=1.0)
    assert_close(d_g, wg, 1e-5, "composite dg", floor=np.sqrt(bd))
    assert_close(d_b, wb, 1e-5, "composite db", floor=np.sqrt(bd))


def test_sum_batches_golden_cadd_broadcast2_neg_val(golden):
    g = golden["node_values"]
    x1 = f32(g["fixture_params"]["param1"]).reshape(1, 3)
    x2 = f32(g["fixture_params"]["param4"]).reshape(2, 3)
    neg = orc.unary_forward(orc.OP_NEGATE, x2)
    y = orc.csum_forward(3, 1, 2, x1, neg)  # x1 - x2 == x1 + (-x2), dynet/expr.cc:70
    z = orc.sum_batches_forward(3, 2, y).astype(np.float64).sum()
    exp = g["cadd_broadcast2_neg_val"]
    assert abs(z - exp["expected"]) <= exp["rel_tol"] * abs(exp["expected"])


def test_sum_batches_backward_broadcasts():
    dy = f32([1, 2, 3])
    dx = orc.sum_batches_backward(3, 4, dy, np.full((4, 3), 10, F32))
    assert np.array_equal(dx, np.tile(dy, (4, 1)) + 10)


def test_std_golden_std_dim_value(golden):
    g = golden["node_values"]
    # x is Dim({3,3},3): element (i,j,b) at i + 3j + 9b.  std over rows AND batch per
    # column j == std_elems of the 9 gathered values
    x = f32(g["fixture_params"]["param_cube1"]).reshape(3, 3, 3)  # [b][j][i]
    cols = np.ascontiguousarray(np.stack([x[:, j, :].reshape(-1) for j in range(3)]))
    y = orc.std_elems_forward(9, 3, cols)
    z = float(orc.mean_elems_forward(3, 1, y)[0])
    exp = g["std_dim_value"]
    assert abs(z - exp["expected"]) <= exp["rel_tol"] * exp["expected"]
    assert np.allclose(y, cols.astype(np.float64).std(axis=1), rtol=1e-6)


def test_mean_std_backward_against_fp64_central_differences():
    rng = np.random.default_rng(4)
    n, bd = 6, 3
    x = f32(rng.standard_normal((bd, n)))
    dy = f32(rng.standard_normal(bd))
    sd = orc.std_elems_forward(n, bd, x)
    dx = orc.std_elems_backward(n, bd, x, sd, dy, np.zeros((bd, n), F32))
    dm = orc.mean_elems_backward(n, bd, dy, np.zeros((bd, n), F32))
    x64 = x.astype(np.float64)
    eps = 1e-6
    for b in range(bd):
        for j in range(n):
            xp, xm = x64.copy(), x64.copy()
            xp[b, j] += eps
            xm[b, j] -= eps
            num = (xp.std(1) - xm.std(1)) @ dy / (2 * eps)
            assert abs(dx[b, j] - num) < 1e-5
            assert abs(dm[b, j] - dy[b] / n) < 1e-7


# ---------------------------------------------------------------------------
# layer norm
# ---------------------------------------------------------------------------
def ln64(x, g, b):
    x = np.asarray(x, np.float64)
    mu = x.mean(-1, keepdims=True)
    sd = x.std(-1, keepdims=True)
    return g * (x - mu) / (sd + 1e-8) + b


def test_layer_norm_forward_golden_properties(golden):
    g = golden["node_values"]
    x = f32(g["fixture_params"]["param1"]).reshape(1, 3)
    y = orc.layer_norm_forward(3, 1, x, np.ones(3, F32), np.zeros(3, F32)).astype(np.float64)
    exp = g["layer_norm_forward"]
    assert abs(y.sum() / 3.0) < exp["mean_abs_max"]
    assert abs(np.sqrt((y ** 2).sum() / 3.0) - exp["rms"]) <= exp["rms_rel_tol"]


def test_layer_norm_forward_golden_python_closed_form(golden):
    exp = golden["node_values"]["layer_norm_python"]
    v = np.arange(exp["n"]).astype(np.float64)
    y = orc.layer_norm_forward(exp["n"], 1, f32(v), f32(v), f32(v))
    want = v / v.std() * (v - v.mean()) + v
    assert np.allclose(y.reshape(-1), want, rtol=exp["rtol"], atol=exp["atol"])


def test_layer_norm_forward_fp64_and_invariances():
    rng = np.random.default_rng(5)
    n, bd = 64, 9
    x = f32(rng.standard_normal((bd, n)) * 2 + 0.3)
    g = f32(rng.uniform(0.5, 1.5, n))
    b = f32(rng.standard_normal(n) * 0.1)
    y = orc.layer_norm_forward(n, bd, x, g, b)
    assert np.max(np.abs(y - ln64(x, g, b))) < 2e-6
    y_shift = orc.layer_norm_forward(n, bd, x + F32(4.0), g, b)
    assert np.max(np.abs(y_shift - y)) < 2e-5  # LN(x + c) == LN(x)
    y_scale = orc.layer_norm_forward(n, bd, x * F32(8.0), g, b)
    assert np.max(np.abs(y_scale - y)) < 2e-6  # LN(a x) == LN(x), a > 0 (power of two: exact scaling)
    # epsilon sits on sigma, not on the variance: a constant row gives exactly b
    yc = orc.layer_norm_forward(4, 1, np.full((1, 4), 3.0, F32), np.ones(4, F32), f32([1, 2, 3, 4]))
    assert np.array_equal(yc.reshape(-1), f32([1, 2, 3, 4]))


def ln_backward64(x, g, dy):
    """Analytic LayerNorm gradient (epsilon ignored), independent of the composite."""
    x, g, dy = (np.asarray(a, np.float64) for a in (x, g, dy))
    n = x.shape[-1]
    mu = x.mean(-1, keepdims=True)
    sd = x.std(-1, keepdims=True)
    xh = (x - mu) / sd
    dxh = dy * g
    dx = (dxh - dxh.mean(-1, keepdims=True) - xh * (dxh * xh).mean(-1, keepdims=True)) / sd
    return dx, (dy * xh).sum(0), dy.sum(0)


def test_layer_norm_backward_matches_analytic_fp64_and_accumulates():
    rng = np.random.default_rng(6)
    n, bd = 48, 7
    x = f32(rng.standard_normal((bd, n)))
    g = f32(rng.uniform(0.5, 1.5, n))
    dy = f32(rng.standard_normal((bd, n)))
    dx0, dg0, db0 = f32(rng.standard_normal((bd, n))), f32(rng.standard_normal(n)), f32(rng.standard_normal(n))
    dx, dg, db = orc.layer_norm_backward(n, bd, x, g, dy, dx0.copy(), dg0.copy(), db0.copy())
    wx, wg, wb = ln_backward64(x, g, dy)
    assert np.max(np.abs(dx - (dx0 + wx))) < 5e-6
    assert np.max(np.abs(dg - (dg0 + wg))) < 5e-6
    assert np.max(np.abs(db - (db0 + wb))) < 5e-6
    # NULL outputs are skipped
    dx_only, _, _ = orc.layer_norm_backward(n, bd, x, g, dy, dx0.copy(), None, None)
    assert np.array_equal(dx_only, dx)


def test_layer_norm_backward_golden_grad_check_recipe(golden):
    """tests/test-nodes.cc:2404-2412 with dynet/grad-check.cc's alpha and tolerances."""
    gp = golden["node_values"]["fixture_params"]
    rec = golden["node_values"]["grad_check"]
    x, g, b = f32(gp["param1"]), f32(gp["param2"]), f32(gp["param3"])

    def loss(x, g, b):  # to_scalar(y) = sqrt(sum(y^2)), tests/test-nodes.cc:102-107
        y = orc.layer_norm_forward(3, 1, f32(x).reshape(1, 3), f32(g), f32(b)).astype(np.float64)
        return np.sqrt((y ** 2).sum())

    y = orc.layer_norm_forward(3, 1, x.reshape(1, 3), g, b).astype(np.float64)
    dy = f32(y / np.sqrt((y ** 2).sum()))
    dx, dg, db = orc.layer_norm_backward(3, 1, x.reshape(1, 3), g, dy, np.zeros((1, 3), F32), np.zeros(3, F32),
                                         np.zeros(3, F32))
    a = rec["alpha"]
    for which, grad in (("x", dx.reshape(-1)), ("g", dg), ("b", db)):
        for i in range(3):
            args = {"x": x.copy(), "g": g.copy(), "b": b.copy()}
            args[which][i] += a
            right = loss(**args)
            args[which][i] -= 2 * a
            left = loss(**args)
            num = (right - left) / (2 * a)
            f = abs(num - grad[i])
            m = max(abs(num), abs(grad[i]))
            if f > rec["abs_tol"] and m > 0:
                f /= m
            assert f <= rec["rel_tol"], (which, i, num, grad[i])


# ---------------------------------------------------------------------------
# GEMM shim
# ---------------------------------------------------------------------------
def test_gemm_three_forms_against_fp64():
    rng = np.random.default_rng(7)
    M, N, K = 5, 4, 6
    # column-major [rows x cols] == numpy (cols, rows) C-order
    l = f32(rng.standard_normal((K, M)))  # M x K
    r = f32(rng.standard_normal((N, K)))  # K x N
    y0 = f32(rng.standard_normal((N, M)))
    y = orc.gemm_nn(M, N, K, l, r, 1.0, y0.copy())
    want = y0.T.astype(np.float64) + l.T.astype(np.float64) @ r.T.astype(np.float64)
    assert np.allclose(y.T, want, rtol=1e-5, atol=1e-6)
    y = orc.gemm_nn(M, N, K, l, r, 0.0, y0.copy())
    assert np.allclose(y.T, l.T.astype(np.float64) @ r.T, rtol=1e-5, atol=1e-6)
    lt = f32(rng.standard_normal((M, K)))  # K x M, used transposed
    y = orc.gemm_tn_acc(M, N, K, lt, r, y0.copy())
    assert np.allclose(y.T, y0.T + lt.astype(np.float64) @ r.T, rtol=1e-5, atol=1e-6)
    rt = f32(rng.standard_normal((K, N)))  # N x K, used transposed
    y = orc.gemm_nt_acc(M, N, K, l, rt, y0.copy())
    assert np.allclose(y.T, y0.T + l.T.astype(np.float64) @ rt, rtol=1e-5, atol=1e-6)


# ---------------------------------------------------------------------------
# fused LSTM nodes: golden vectors of tests/test-rnn.cc
# ---------------------------------------------------------------------------
def test_lstm_h_golden(golden):
    t = golden["lstm_nodes"]["lstm_node_h_fwd"]
    h = orc.lstm_h_forward(t["hidden_dim"], t["batch_size"], f32(t["c_t"]), f32(t["gates_t"])).reshape(-1)
    assert abs(h[0]) < t["small_abs"]
    assert_rel(h[1:], t["h_t"][1:], golden["lstm_nodes"]["rel_tol"], "lstm_h")


def test_lstm_c_golden(golden):
    t = golden["lstm_nodes"]["lstm_node_c_fwd"]
    c = orc.lstm_c_forward(t["hidden_dim"], t["batch_size"], f32(t["c_tm1"]), f32(t["gates_t"])).reshape(-1)
    assert np.all(np.abs(c[:3]) < t["small_abs"])
    assert_rel(c[3:], t["c_t"][3:], golden["lstm_nodes"]["rel_tol"], "lstm_c")


@pytest.mark.parametrize("mode", [orc.LOGISTIC_PACKET, orc.LOGISTIC_SCALAR])
def test_lstm_gates_golden(golden, mode):
    t = golden["lstm_nodes"]["lstm_node_gates_fwd"]
    g = orc.lstm_gates_forward([f32(t["x_t"])], [t["input_dim"]], t["hidden_dim"], t["batch_size"], f32(t["h_tm1"]),
                               f32(t["Wx"]), f32(t["Wh"]), f32(t["b"]), logistic_mode=mode)
    assert_rel(g.reshape(-1), t["gates"], golden["lstm_nodes"]["rel_tol"], "lstm_gates")


@pytest.mark.parametrize("mode", [orc.LOGISTIC_PACKET, orc.LOGISTIC_SCALAR])
def test_lstm_gates_dropout_golden(golden, mode):
    t = golden["lstm_nodes"]["lstm_node_gates_dropout_fwd"]
    B = t["batch_size"]
    g = orc.lstm_gates_forward([f32(t["x_t"])], [t["input_dim"]], t["hidden_dim"], B, f32(t["h_tm1"]),
                               f32(t["Wx"]), f32(t["Wh"]), f32(t["b"]), f32(t["mask_x"]), B, f32(t["mask_h"]), B,
                               logistic_mode=mode)
    assert_rel(g.reshape(-1), t["gates"], golden["lstm_nodes"]["rel_tol"], "lstm_gates_dropout")


# independent fp64 model of the three nodes ---------------------------------
def gates64(x, h, Wx, Wh, b, H, mask_x=None, mask_h=None):
    """x: (B, I), h: (B, H), Wx: (4H, I), Wh: (4H, H); returns (B, 4H)."""
    x, h = np.asarray(x, np.float64), np.asarray(h, np.float64)
    if mask_x is not None:
        x = x * mask_x
        h = h * mask_h
    pre = x @ np.asarray(Wx, np.float64).T + h @ np.asarray(Wh, np.float64).T + np.asarray(b, np.float64)
    pre[:, H:2 * H] += 1.0
    out = np.empty_like(pre)
    out[:, :3 * H] = sigmoid64(pre[:, :3 * H])
    out[:, 3 * H:] = np.tanh(pre[:, 3 * H:])
    return out


def cm(a, rows, cols):
    """column-major flat buffer of a (rows x cols) matrix -> numpy (rows, cols)."""
    return np.asarray(a).reshape(cols, rows).T


def lstm_case(rng, I, H, B):
    x = f32(rng.standard_normal((B, I)))
    h = f32(rng.standard_normal((B, H)))
    Wx = f32(rng.uniform(-0.4, 0.4, (I, 4 * H)))  # column-major 4H x I
    Wh = f32(rng.uniform(-0.4, 0.4, (H, 4 * H)))
    b = f32(rng.standard_normal(4 * H) * 0.1)
    return x, h, Wx, Wh, b


def test_lstm_gates_forward_fp64_and_multi_input_equivalence():
    rng = np.random.default_rng(8)
    I, H, B = 4, 5, 3
    x, h, Wx, Wh, b = lstm_case(rng, I, H, B)
    got = orc.lstm_gates_forward([x], [I], H, B, h, Wx, Wh, b, logistic_mode=orc.LOGISTIC_SCALAR)
    want = gates64(x, h, cm(Wx, 4 * H, I), cm(Wh, 4 * H, H), b, H)
    assert np.max(np.abs(got - want)) < 1e-6
    # multi-input == single concatenated input (tests/test-rnn.cc:462-497)
    x1, x3 = np.ascontiguousarray(x[:, :1]), np.ascontiguousarray(x[:, 1:])
    got2 = orc.lstm_gates_forward([x1, x3], [1, 3], H, B, h, Wx, Wh, b, logistic_mode=orc.LOGISTIC_SCALAR)
    assert np.array_equal(got, got2)
    # batch-broadcast masks == masks tiled over the batch
    mx, mh = f32(rng.integers(0, 2, (1, I)) * 0.9), f32(rng.integers(0, 2, (1, H)) * 0.8)
    ga = orc.lstm_gates_forward([x], [I], H, B, h, Wx, Wh, b, mx, 1, mh, 1)
    gb = orc.lstm_gates_forward([x], [I], H, B, h, Wx, Wh, b, np.tile(mx, (B, 1)), B, np.tile(mh, (B, 1)), B)
    assert np.array_equal(ga, gb)
    want = gates64(x, h, cm(Wx, 4 * H, I), cm(Wh, 4 * H, H), b, H, mx, mh)
    assert np.max(np.abs(ga - want)) < 1e-6


def test_fused_nodes_equal_unfused_builder_path():
    """tests/test-rnn.cc:155-184,214-243: three steps of gates/C/H equal the
    VanillaLSTMBuilder recurrence (dynet/lstm.cc:519-545: affine, pick_range,
    logistic(+1 on f), tanh, cmult) to 1e-5."""
    rng = np.random.default_rng(9)
    I, H, B = 3, 5, 2
    x, h, Wx, Wh, b = lstm_case(rng, I, H, B)
    c = f32(rng.standard_normal((B, H)))
    W64x, W64h = cm(Wx, 4 * H, I).astype(np.float64), cm(Wh, 4 * H, H).astype(np.float64)
    h64, c64 = h.astype(np.float64), c.astype(np.float64)
    for _ in range(3):
        gates = orc.lstm_gates_forward([x], [I], H, B, h, Wx, Wh, b, logistic_mode=orc.LOGISTIC_SCALAR)
        c = orc.lstm_c_forward(H, B, c, gates)
        h = orc.lstm_h_forward(H, B, c, gates)
        tmp = x.astype(np.float64) @ W64x.T + h64 @ W64h.T + b
        i_t, f_t = sigmoid64(tmp[:, :H]), sigmoid64(tmp[:, H:2 * H] + 1.0)
        o_t, g_t = sigmoid64(tmp[:, 2 * H:3 * H]), np.tanh(tmp[:, 3 * H:])
        c64 = f_t * c64 + i_t * g_t
        h64 = o_t * np.tanh(c64)
        assert_rel(h, h64, 1e-5, "fused vs unfused h")


@pytest.mark.parametrize("dropout,mask_bd_full,multi", [(False, True, False), (True, True, False),
                                                        (True, False, False), (False, True, True),
                                                        (True, True, True)])
def test_lstm_gates_backward_all_args_fp64(dropout, mask_bd_full, multi):
    """Gradients of every argument against central differences of the
    independent fp64 model, on the shapes of tests/test-rnn.cc:341-357,
    402-460,499-529,601-630 (I=5 or 4, H=3 or 5, B=2)."""
    rng = np.random.default_rng(10)
    I, H, B = (4, 5, 2) if multi else (5, 3, 2)
    x, h, Wx, Wh, b = lstm_case(rng, I, H, B)
    dims = [1, 3] if multi else [I]
    offs = np.cumsum([0] + dims)
    xs = [np.ascontiguousarray(x[:, offs[k]:offs[k + 1]]) for k in range(len(dims))]
    mx = mh = None
    mbd = 0
    if dropout:
        mbd = B if mask_bd_full else 1
        mx = f32(rng.integers(0, 2, (mbd, I)) * 0.9)
        mh = f32(rng.integers(0, 2, (mbd, H)) * 0.8)
    dy = f32(rng.standard_normal((B, 4 * H)))
    fx = orc.lstm_gates_forward(xs, dims, H, B, h, Wx, Wh, b, mx, mbd, mh, mbd, logistic_mode=orc.LOGISTIC_SCALAR)

    def loss(x_, h_, Wx_, Wh_, b_):
        return (gates64(x_, h_, cm(Wx_, 4 * H, I), cm(Wh_, 4 * H, H), b_, H, mx, mh) * dy).sum()

    base = [x.astype(np.float64), h.astype(np.float64), Wx.astype(np.float64), Wh.astype(np.float64),
            b.astype(np.float64)]

    def numgrad(k):
        g = np.zeros_like(base[k])
        it = np.nditer(base[k], flags=["multi_index"])
        eps = 1e-6
        for _ in it:
            idx = it.multi_index
            args = [a.copy() for a in base]
            args[k][idx] += eps
            up = loss(*args)
            args[k][idx] -= 2 * eps
            g[idx] = (up - loss(*args)) / (2 * eps)
        return g

    k_in = len(dims)
    # inputs
    gx = numgrad(0)
    for k in range(k_in):
        acc0 = f32(rng.standard_normal((B, dims[k])))
        got = orc.lstm_gates_backward(xs, dims, H, B, h, Wx, Wh, fx, dy, k, acc0.copy(), mx, mbd, mh, mbd)
        assert np.max(np.abs(got - (acc0 + gx[:, offs[k]:offs[k + 1]]))) < 2e-5, "dx%d" % k
    for j, (arg_i, shape) in enumerate([(k_in, (B, H)), (k_in + 1, (I, 4 * H)), (k_in + 2, (H, 4 * H)),
                                        (k_in + 3, (4 * H,))]):
        acc0 = f32(rng.standard_normal(shape))
        got = orc.lstm_gates_backward(xs, dims, H, B, h, Wx, Wh, fx, dy, arg_i, acc0.copy(), mx, mbd, mh, mbd)
        assert np.max(np.abs(got - (acc0 + numgrad(j + 1)))) < 2e-5, "arg %d" % arg_i


def test_lstm_c_h_backward_fp64():
    rng = np.random.default_rng(11)
    H, B = 3, 2
    c_prev = f32(rng.standard_normal((B, H)))
    gates = f32(rng.uniform(0.05, 0.95, (B, 4 * H)))
    dc = f32(rng.standard_normal((B, H)))
    g64 = gates.astype(np.float64)
    i_, f_, o_, g_ = (g64[:, k * H:(k + 1) * H] for k in range(4))
    got = orc.lstm_c_backward(H, B, c_prev, gates, dc, 0, np.ones((B, H), F32))
    assert np.allclose(got, 1 + dc * f_, rtol=1e-6)
    got = orc.lstm_c_backward(H, B, c_prev, gates, dc, 1, np.ones((B, 4 * H), F32))
    want = np.ones((B, 4 * H))
    want[:, :H] += dc * g_
    want[:, H:2 * H] += dc * c_prev
    want[:, 3 * H:] += dc * i_
    assert np.allclose(got, want, rtol=1e-6)  # the o rows stay untouched
    c = orc.lstm_c_forward(H, B, c_prev, gates)
    t = np.tanh(c.astype(np.float64))
    got = orc.lstm_h_backward(H, B, c, gates, dc, 0, np.ones((B, H), F32))
    assert np.allclose(got, 1 + dc * o_ * (1 - t * t), rtol=1e-5)
    got = orc.lstm_h_backward(H, B, c, gates, dc, 1, np.ones((B, 4 * H), F32))
    want = np.ones((B, 4 * H))
    want[:, 2 * H:3 * H] += dc * t
    assert np.allclose(got, want, rtol=1e-5)


# ---------------------------------------------------------------------------
# lookup
# ---------------------------------------------------------------------------
def test_lookup_forward_is_a_bit_exact_gather_and_checks_bounds(golden):
    table = f32(golden["node_values"]["fixture_params"]["param_square1"]).reshape(3, 3)  # lookup1: 3 rows of dim 3
    ids = [0, 2, 2, 1, 0]
    out = orc.lookup_forward(ids, 3, 3, table)
    assert out.tobytes() == table[ids].tobytes()
    assert np.array_equal(orc.lookup_forward(ids, 3, 3, table, 0.5), table[ids] * F32(0.5))
    with pytest.raises(ValueError):
        orc.lookup_forward([0, 3], 3, 3, table)


def test_lookup_accumulate_grads_brute_force_with_duplicates():
    rng = np.random.default_rng(12)
    V, D, n = 5, 4, 64
    ids = rng.integers(0, 3, n).astype(np.uint32)  # heavy duplication, rows 3..4 untouched
    g = f32(rng.standard_normal((n, D)))
    grads0 = f32(rng.standard_normal((V, D)))
    got = orc.lookup_accumulate_grads(ids, D, V, g, grads0.copy())
    want = grads0.copy()
    for b in range(n):  # sequential fp32, the CPU path's order
        want[ids[b]] = want[ids[b]] + g[b]
    assert got.tobytes() == want.tobytes()
    assert np.array_equal(got[3:], grads0[3:])
    assert abs(got.astype(np.float64).sum() - grads0.astype(np.float64).sum() - g.astype(np.float64).sum()) < 1e-4
    with pytest.raises(ValueError):
        orc.lookup_accumulate_grads([7], D, V, g[:1], grads0.copy())


# ---------------------------------------------------------------------------
# logsumexp / pickneglogsoftmax / argmax
# ---------------------------------------------------------------------------
def test_logsumexp_cols_against_scipy_and_shift_invariance():
    rng = np.random.default_rng(13)
    rows, bd = 301, 6
    x = f32(rng.standard_normal((bd, rows)) * 2)
    m, z = orc.logsumexp_cols(rows, bd, x)
    assert np.array_equal(m, x.max(1))
    assert_rel(z, sp_logsumexp(x.astype(np.float64), axis=1), 2e-6, "lse")
    _, z2 = orc.logsumexp_cols(rows, bd, x + F32(16.0))
    assert np.max(np.abs(z2 - z - 16.0)) < 1e-5
    _, zbig = orc.logsumexp_cols(3, 1, f32([[1000.0, 1000.0, -1000.0]]))
    assert abs(zbig[0] - (1000.0 + np.log(2.0))) < 1e-4  # no overflow


def test_pnls_forward_backward_fp64(golden):
    rng = np.random.default_rng(14)
    rows, bd = 37, 5
    x = f32(rng.standard_normal((bd, rows)) * 2)
    labels = rng.integers(0, rows, bd).astype(np.uint32)
    fx, aux = orc.pnls_forward(rows, bd, x, labels)
    ids = aux.view(np.uint32)[2 * bd:]
    assert np.array_equal(ids, np.arange(bd) * rows + labels)  # picks are index lookups: bit exact
    lse = sp_logsumexp(x.astype(np.float64), axis=1)
    want = lse - x[np.arange(bd), labels]
    assert_rel(fx, want, 1e-5, "pnls fwd")
    dy = f32(rng.standard_normal(bd))
    dx0 = f32(rng.standard_normal((bd, rows)))
    dx = orc.pnls_backward(rows, bd, x, aux, dy, dx0.copy())
    soft = np.exp(x.astype(np.float64) - lse[:, None])
    onehot = np.zeros((bd, rows))
    onehot[np.arange(bd), labels] = 1
    assert np.max(np.abs(dx - (dx0 + (soft - onehot) * dy[:, None]))) < 2e-6
    # sum_v (softmax - onehot) == 0 per row
    assert np.max(np.abs((dx - dx0).astype(np.float64).sum(1))) < 2e-6
    with pytest.raises(ValueError):
        orc.pnls_forward(rows, bd, x, np.full(bd, rows, np.uint32))
    # tests/test-nodes.cc:2088-2094: x1 = param1, idx = 1
    x1 = f32(golden["node_values"]["fixture_params"]["param1"]).reshape(1, 3)
    fx1, _ = orc.pnls_forward(3, 1, x1, [1])
    assert abs(fx1[0] - (sp_logsumexp(x1.astype(np.float64)) - x1[0, 1])) < 1e-6


def test_logsumexp_node_forward_backward():
    rng = np.random.default_rng(15)
    n, bd = 6, 4
    a, b, c1 = f32(rng.standard_normal((bd, n))), f32(rng.standard_normal((bd, n))), f32(rng.standard_normal((1, n)))
    fx = orc.logsumexp_node_forward(n, bd, [a, b, c1], [bd, bd, 1])
    want = np.log(np.exp(a.astype(np.float64)) + np.exp(b) + np.exp(c1))
    assert_rel(fx, want, 2e-6, "logsumexp node")
    dy = f32(rng.standard_normal((bd, n)))
    da = orc.logsumexp_node_backward(n, bd, [a, b, c1], [bd, bd, 1], fx, dy, 0, np.zeros((bd, n), F32))
    assert np.max(np.abs(da - np.exp(a - want) * dy)) < 2e-6
    dc = orc.logsumexp_node_backward(n, bd, [a, b, c1], [bd, bd, 1], fx, dy, 2, np.zeros((1, n), F32))
    assert np.max(np.abs(dc - (np.exp(c1 - want) * dy).sum(0))) < 2e-6
    one = orc.logsumexp_node_forward(n, bd, [a], [bd])
    assert np.array_equal(one, a)


def test_argmax_golden(golden):
    t = golden["node_values"]["argmax"]
    assert list(orc.argmax_cols(t["rows"], t["bd"], f32(t["x"]))) == t["expected"]
    assert list(orc.argmax_cols(4, 1, f32([3, 7, 7, 1]))) == [1]  # first maximum on ties


def test_argmax_node_golden(golden):
    t = golden["node_values"]["argmax_node"]
    idx, fx = orc.argmax_onehot_forward(t["rows"], t["bd"], f32(t["x"]))
    assert list(fx.ravel()) == t["expected"] and list(idx) == [2, 2]
    rng = np.random.default_rng(12)
    x = f32(rng.standard_normal((7, 13)))
    idx, fx = orc.argmax_onehot_forward(13, 7, x)
    assert np.array_equal(idx, np.argmax(x, axis=1)) and np.array_equal(fx, np.eye(13, dtype=np.float32)[idx])


# ---------------------------------------------------------------------------
# scatter/gather helpers, parameter copy, trainer
# ---------------------------------------------------------------------------
def test_gpu_ops_helpers_against_numpy():
    rng = np.random.default_rng(16)
    src = f32(rng.standard_normal(10))
    idx = np.array([3, 0, 7], np.uint32)
    assert np.array_equal(orc.sparse_to_dense_assign(idx, src), src[idx])
    trg = np.zeros(10, F32)
    orc.dense_to_sparse_assign(idx, src[:3], trg)
    assert np.array_equal(trg[idx], src[:3]) and trg.sum() == src[:3].sum()
    trg = np.ones(10, F32)
    orc.dense_to_sparse_subtract(np.array([2, 2, 5], np.uint32), f32([1, 2, 3]), trg)
    assert trg[2] == -2 and trg[5] == -2
    table = f32(rng.standard_normal((6, 4)))
    out = orc.sparse_to_dense_block_assign_and_multiply(np.array([5, 5, 1], np.uint32), 4, 2.0, table)
    assert np.array_equal(out, table[[5, 5, 1]] * 2)
    acc = np.zeros((6, 4), F32)
    orc.dense_to_sparse_block_add(np.array([5, 5, 1], np.uint32), 4, out, acc)
    assert np.allclose(acc[5], out[0] + out[1]) and np.array_equal(acc[1], out[2])


def test_scale_copy_sgd_and_norm():
    rng = np.random.default_rng(17)
    p, g = f32(rng.standard_normal(33)), f32(rng.standard_normal(33))
    assert np.array_equal(orc.scale_copy(p, 1.0), p)
    # p -= g * (lr * gscale / wd), dynet/training.cc:621
    want = p - g * F32(F32(0.1) * F32(0.5) / F32(1.0))
    assert np.array_equal(orc.sgd_update(p.copy(), g, 0.1, 0.5, 1.0), want)
    assert abs(orc.squared_l2norm(g) - (g.astype(np.float64) ** 2).sum()) < 1e-4


# ---- LM step composition -------------------------------------------------------
def test_lm_step_gradient_check():
    """Directional central difference of the LM loss against <grad, direction>: a dropped term, a wrong
    transpose or a mis-indexed timestep in the backward composition breaks it."""
    from oracle import lm_oracle
    from dynet_amd.lm import LstmLM
    V, E, H, L, B, T = 23, 6, 8, 2, 3, 4
    rng = np.random.default_rng(0)
    p = LstmLM.init_params(V, E, H, L, seed=4)
    for l in range(L):
        p[f"b{l}"] = rng.normal(0, 0.1, 4 * H).astype(np.float32)
    tokens = rng.integers(0, V, (T + 1, B)).astype(np.uint32)
    loss, cache = lm_oracle.forward(p, tokens, L)
    g = lm_oracle.backward(p, tokens, L, cache)
    for name in p:
        d = rng.normal(0, 1, p[name].shape).astype(np.float32)
        eps = 2e-2
        plus = {n: (a + eps * d if n == name else a).astype(np.float32) for n, a in p.items()}
        minus = {n: (a - eps * d if n == name else a).astype(np.float32) for n, a in p.items()}
        lp, _ = lm_oracle.forward(plus, tokens, L)
        lmn, _ = lm_oracle.forward(minus, tokens, L)
        fd = (float(lp) - float(lmn)) / (2 * eps)
        an = float(np.sum(g[name].astype(np.float64) * d))
        assert abs(fd - an) <= 2e-2 * max(abs(an), 0.5), (name, fd, an)


def test_lm_update_clips_and_touches_only_used_rows():
    from oracle import lm_oracle
    from dynet_amd.lm import LstmLM
    V, E, H, L, B, T = 23, 6, 8, 1, 3, 4
    rng = np.random.default_rng(1)
    p = LstmLM.init_params(V, E, H, L, seed=4)
    before = {n: a.copy() for n, a in p.items()}
    tokens = rng.integers(0, 5, (T + 1, B)).astype(np.uint32)
    loss, g, gscale = lm_oracle.step(p, tokens, L, lr=0.1, clip=0.25)
    norm = np.sqrt(sum(float(np.sum(a.astype(np.float64) ** 2)) for a in g.values()))
    assert norm > 0.25 and abs(gscale - 0.25 / norm) < 1e-5 * gscale
    assert np.array_equal(p["C"][5:], before["C"][5:])
    np.testing.assert_allclose(p["R"], before["R"] - 0.1 * gscale * g["R"], rtol=1e-6, atol=1e-7)


# ---- Softmax / LogSoftmax (the reference holds gradient checks only: tests/test-nodes.cc:1083-1160) ----
def test_softmax_and_log_softmax_closed_forms():
    from scipy.special import softmax, log_softmax
    rng = np.random.default_rng(21)
    for rows, cols in ((3, 1), (37, 5), (1000, 4)):
        x = (rng.standard_normal((cols, rows)) * 3).astype(np.float32)
        sm = orc.softmax_forward(rows, cols, x)
        want = softmax(x.astype(np.float64), axis=1)
        assert np.max(np.abs(sm - want) / np.maximum(want, 1e-30)) < 2e-6
        np.testing.assert_allclose(sm.sum(axis=1), 1.0, rtol=0, atol=3e-6)
        shifted = orc.softmax_forward(rows, cols, x + np.float32(11.5))
        np.testing.assert_allclose(shifted, sm, rtol=3e-6, atol=0)
        ls, aux = orc.log_softmax_forward(rows, cols, x)
        np.testing.assert_allclose(ls, log_softmax(x.astype(np.float64), axis=1), rtol=0, atol=4e-6)
        m, z = orc.logsumexp_cols(rows, cols, x)
        assert aux[:cols].tobytes() == z.tobytes() and aux[cols:].tobytes() == m.tobytes()
    # the values of the reference's gradient-check input {1.1, -2.2, 3.3} (tests/test-nodes.cc:47)
    x = np.array([[1.1, -2.2, 3.3]], np.float32)
    e = np.exp(np.array([1.1, -2.2, 3.3]) - 3.3)
    np.testing.assert_allclose(orc.softmax_forward(3, 1, x)[0], e / e.sum(), rtol=1e-6)


def test_softmax_and_log_softmax_backward_central_differences():
    from scipy.special import softmax, log_softmax
    rng = np.random.default_rng(22)
    rows, cols = 7, 3
    x = rng.standard_normal((cols, rows))
    dy = rng.standard_normal((cols, rows))
    for fwd64, fwd, bwd in ((lambda a: softmax(a, axis=1), orc.softmax_forward, orc.softmax_backward),
                            (lambda a: log_softmax(a, axis=1), lambda r, c, a: orc.log_softmax_forward(r, c, a)[0],
                             orc.log_softmax_backward)):
        fx = fwd(rows, cols, x.astype(np.float32))
        g0 = rng.standard_normal((cols, rows)).astype(np.float32)
        got = bwd(rows, cols, fx, dy.astype(np.float32), g0.copy())
        num = np.zeros_like(x)
        eps = 1e-6
        for idx in np.ndindex(*x.shape):
            xp, xm = x.copy(), x.copy()
            xp[idx] += eps
            xm[idx] -= eps
            num[idx] = ((fwd64(xp) - fwd64(xm)) * dy).sum() / (2 * eps)
        np.testing.assert_allclose(got - g0, num, rtol=2e-4, atol=2e-5)  # backward accumulates onto g0


def test_sum_node_association_order_and_broadcast():
    rng = np.random.default_rng(23)
    n, bd = 5, 3
    for k in (1, 2, 3, 4, 5, 6, 7, 8, 9, 13):
        xs = [(rng.standard_normal((bd, n)) * 10.0 ** rng.integers(-3, 4)).astype(np.float32) for _ in range(k)]
        got = orc.sum_forward(n, bd, xs, [bd] * k)
        np.testing.assert_allclose(got, np.sum([x.astype(np.float64) for x in xs], axis=0), rtol=0,
                                   atol=1e-6 * max(float(np.abs(x).max()) for x in xs) * k)
        # groups of four, each summed left to right before it joins fx (dynet/nodes-arith-sum.cc:67-89)
        want = xs[0].copy()
        for x in xs[1:4]:
            want = want + x
        rem = (k - 4) % 4 if k > 4 else 0
        at = 4
        if rem:
            g = xs[at].copy()
            for x in xs[at + 1:at + rem]:
                g = g + x
            want = want + g
            at += rem
        while at < k:
            want = want + (((xs[at] + xs[at + 1]) + xs[at + 2]) + xs[at + 3])
            at += 4
        assert got.tobytes() == want.astype(np.float32).tobytes(), k
    # a case where the grouping changes the bits: 1e8 + (-1e8 + 1 ...) vs left-to-right
    xs = [np.full((1, 1), v, np.float32) for v in (1.0, 1e8, -1e8, 1.0, 1.0, 1e8, -1e8, 1.0)]
    assert orc.sum_forward(1, 1, xs, [1] * 8)[0, 0] == np.float32(np.float32(np.float32(np.float32(1.0) + np.float32(1e8)) + np.float32(-1e8)) + np.float32(1.0)) + np.float32(np.float32(np.float32(np.float32(1.0) + np.float32(1e8)) + np.float32(-1e8)) + np.float32(1.0))
    # mixed batch sizes: broadcast of batch-1 arguments
    a, b, c = (rng.standard_normal((bd, n)).astype(np.float32), rng.standard_normal((1, n)).astype(np.float32),
               rng.standard_normal((bd, n)).astype(np.float32))
    got = orc.sum_forward(n, bd, [a, b, c], [bd, 1, bd])
    assert got.tobytes() == (((np.zeros_like(a) + a) + b) + c).tobytes()


# ---- random tensors ---------------------------------------------------------------------------
# Known-answer vectors of philox4x32-10 published with the generator (Random123 kat_vectors):
# counter words, key words -> output words.
PHILOX_KAT = [
    ([0, 0, 0, 0], [0, 0], [0x6627E8D5, 0xE169C58D, 0xBC57AC4C, 0x9B00DBD8]),
    ([0xFFFFFFFF] * 4, [0xFFFFFFFF] * 2, [0x408F276D, 0x41C83B0E, 0xA20BC7C6, 0x6D5451FD]),
    ([0x243F6A88, 0x85A308D3, 0x13198A2E, 0x03707344], [0xA4093822, 0x299F31D0],
     [0xD16CFE09, 0x94FDCCEB, 0x5001E420, 0x24126EA1]),
]


def _philox_python(ctr, key):
    """The published algorithm written a second time, straight from its definition (bijection of rounds:
    L' = mullo(R, M), R' = mulhi(R, M) ^ k ^ L on the two counter halves, then the word permutation)."""
    M = (0xD2511F53, 0xCD9E8D57)
    W = (0x9E3779B9, 0xBB67AE85)
    c, k = list(ctr), list(key)
    for r in range(10):
        hi0, lo0 = divmod(M[0] * c[0], 1 << 32)
        hi1, lo1 = divmod(M[1] * c[2], 1 << 32)
        c = [hi1 ^ c[1] ^ k[0], lo1, hi0 ^ c[3] ^ k[1], lo0]
        k = [(k[0] + W[0]) & 0xFFFFFFFF, (k[1] + W[1]) & 0xFFFFFFFF]
    return c


@pytest.mark.parametrize("ctr,key,want", PHILOX_KAT)
def test_philox_known_answers(ctr, key, want):
    assert orc.philox4x32_10(ctr, key) == want
    assert _philox_python(ctr, key) == want


def test_philox_words_follow_the_stated_counter_layout():
    rng = np.random.default_rng(0)
    for _ in range(20):
        key = int(rng.integers(0, 1 << 63)) * 2 + int(rng.integers(0, 2))
        pos = int(rng.integers(0, 1 << 40)) + (1 << 32) - 3  # crosses the 32-bit carry of the block number
        queue, n = int(rng.integers(0, 5)), int(rng.integers(1, 40))
        words = orc.random_words(key, pos, queue, n)
        for k in range(n):
            blk = pos + k // 4
            ref = _philox_python([blk & 0xFFFFFFFF, blk >> 32, queue, 0], [key & 0xFFFFFFFF, key >> 32])
            assert int(words[k]) == ref[k % 4]


def test_uniform_conversion_and_range():
    # u = w * 2^-32 + 2^-33 evaluated in fp32, in (0, 1]; the extreme words map to 2^-33 and 1
    words = orc.random_words(1, 0, 0, 4096)
    u = orc.randomize_uniform(1, 0, 0, 4096)
    want = (words.astype(np.float32) * np.float32(2.0 ** -32) + np.float32(2.0 ** -33)).astype(np.float32)
    assert np.array_equal(u, want)
    assert u.min() > 0 and u.max() <= 1
    v = orc.randomize_uniform(1, 0, 0, 4096, -3.0, 5.0)
    assert np.array_equal(v, (u * np.float32(8.0) + np.float32(-3.0)).astype(np.float32))


def test_random_distributions():
    from scipy import stats

    n = 400000
    u = orc.randomize_uniform(123, 77, 0, n).astype(np.float64)
    assert stats.kstest(u, "uniform").pvalue > 1e-3
    # successive words are uncorrelated
    assert abs(np.corrcoef(u[:-1], u[1:])[0, 1]) < 5e-3
    z = orc.randomize_normal(123, 77, 0, n, 2.0, 0.5).astype(np.float64)
    assert stats.kstest((z - 2.0) / 0.5, "norm").pvalue > 1e-3
    assert abs(np.corrcoef(z[0::2], z[1::2])[0, 1]) < 5e-3  # the two outputs of one Box-Muller pair
    for p in (0.0, 0.1, 0.5, 0.9, 1.0):
        b = orc.randomize_bernoulli(123, 77, 0, n, p, 3.0)
        assert set(np.unique(b)) <= {np.float32(0), np.float32(3)}
        rate = (b != 0).mean()
        assert abs(rate - p) < 4 * np.sqrt(max(p * (1 - p), 1e-12) / n) + 1e-6, (p, rate)
    # floor(u + p) is 1 exactly when u >= 1 - p (up to the rounding of the fp32 sum)
    u32 = orc.randomize_uniform(123, 77, 0, 1000)
    b = orc.randomize_bernoulli(123, 77, 0, 1000, 0.3)
    assert np.array_equal(b, np.floor(u32 + np.float32(0.3)).astype(np.float32))


def test_dropout_oracle():
    rng = np.random.default_rng(4)
    x, dy = f32(rng.standard_normal(1001)), f32(rng.standard_normal(1001))
    mask, fx = orc.dropout_forward(9, 0, 0, 0.2, x)
    keep_scale = np.float32(1.0) / np.float32(0.8)
    assert np.array_equal(mask, orc.randomize_bernoulli(9, 0, 0, 1001, 0.8, float(keep_scale)))
    assert np.array_equal(fx, x * mask)
    dx = orc.dropout_backward(mask, dy, np.ones(1001, np.float32))
    assert np.array_equal(dx, (np.float32(1) + dy * mask).astype(np.float32))
    with pytest.raises(ValueError):
        orc.dropout_forward(9, 0, 0, 1.0, x)


# ---- PickRange ----------------------------------------------------------------------------------
@pytest.mark.parametrize("dim", [0, 1, 2])
def test_pick_range_is_a_numpy_slice(dim):
    rng = np.random.default_rng(dim)
    d = (4, 5, 3)
    bd = 2
    # batch outermost, column-major: numpy shape (bd, d2, d1, d0)
    x = f32(rng.standard_normal((bd, d[2], d[1], d[0])))
    start, end = 1, 3
    inner = int(np.prod(d[:dim]))
    outer = int(np.prod(d[dim + 1:])) * bd
    got = orc.pick_range_forward(inner, d[dim], outer, start, end, x)
    sl = [slice(None)] * 4
    sl[3 - dim] = slice(start, end)
    assert np.array_equal(got, x[tuple(sl)].ravel())
    # backward is the adjoint: accumulates into the slice and nothing else
    dy = f32(rng.standard_normal(got.size))
    dx = np.ones(x.size, np.float32)
    orc.pick_range_backward(inner, d[dim], outer, start, end, dy, dx)
    want = np.ones_like(x)
    want[tuple(sl)] += dy.reshape(want[tuple(sl)].shape)
    assert np.array_equal(dx, want.ravel())
    with pytest.raises(ValueError):
        orc.pick_range_forward(inner, d[dim], outer, 3, 3, x)
    with pytest.raises(ValueError):
        orc.pick_range_forward(inner, d[dim], outer, 0, d[dim] + 1, x)


def test_softmax_along_dim_1_and_logsumexp_dim_against_scipy():
    """Pins: scipy.special.softmax / logsumexp in fp64; the dimension-1 softmax equals the dimension-0 routine
    on the transposed matrices; backward by central differences in fp64."""
    from scipy.special import logsumexp, softmax

    rng = np.random.default_rng(77)
    rows, cols, bd = 7, 5, 3
    x = (rng.standard_normal((bd, cols, rows)) * 3).astype(np.float32)  # [b][j][i]: column-major matrices
    fx = orc.softmax_rows_forward(rows, cols, bd, x)
    np.testing.assert_allclose(fx, softmax(x.astype(np.float64), axis=1), rtol=2e-6, atol=1e-9)
    xt = np.ascontiguousarray(x.transpose(0, 2, 1))  # rows <-> cols
    via_dim0 = orc.softmax_forward(cols, rows * bd, xt.reshape(bd * rows, cols)).reshape(bd, rows, cols)
    assert np.array_equal(fx, via_dim0.transpose(0, 2, 1))
    for dim, axis in ((0, 2), (1, 1)):
        m, z = orc.logsumexp_dim_forward(rows, cols, bd, x, dim)
        np.testing.assert_allclose(z, logsumexp(x.astype(np.float64), axis=axis), rtol=2e-6)
        assert np.array_equal(m, x.max(axis=axis))
    m0, z0 = orc.logsumexp_dim_forward(rows, cols, bd, x, 0)
    m_c, z_c = orc.logsumexp_cols(rows, cols * bd, x.reshape(bd * cols, rows))
    assert np.array_equal(z0.ravel(), z_c) and np.array_equal(m0.ravel(), m_c)
    # gradients: loss = sum w * f(x), central differences in fp64
    w = rng.standard_normal((bd, cols, rows))
    g = orc.softmax_rows_backward(rows, cols, bd, fx, w.astype(np.float32), np.zeros((bd, cols, rows), np.float32))
    x64, h = x.astype(np.float64), 1e-6
    num = np.zeros_like(x64)
    for idx in np.ndindex(x64.shape):
        xp, xm = x64.copy(), x64.copy()
        xp[idx] += h
        xm[idx] -= h
        num[idx] = ((softmax(xp, axis=1) - softmax(xm, axis=1)) * w.astype(np.float32)).sum() / (2 * h)
    np.testing.assert_allclose(g, num, rtol=2e-4, atol=2e-5)
    for dim, axis in ((0, 2), (1, 1)):
        m, z = orc.logsumexp_dim_forward(rows, cols, bd, x, dim)
        wz = rng.standard_normal(z.shape).astype(np.float32)
        g = orc.logsumexp_dim_backward(rows, cols, bd, x, z, wz, dim, np.zeros((bd, cols, rows), np.float32))
        num = np.zeros_like(x64)
        for idx in np.ndindex(x64.shape):
            xp, xm = x64.copy(), x64.copy()
            xp[idx] += h
            xm[idx] -= h
            num[idx] = ((logsumexp(xp, axis=axis) - logsumexp(xm, axis=axis)) * wz).sum() / (2 * h)
        np.testing.assert_allclose(g, num, rtol=2e-4, atol=2e-5)
