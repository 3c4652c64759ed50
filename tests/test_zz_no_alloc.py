"""dyhip_layer_norm_backward_static: the LayerNorm backward entry point that allocates nothing (its scratch is a
static device array of the library) against dyhip_layer_norm_backward with a caller-provided workspace, through
the C-ABI: two calls in a row, the second on a smaller input, on the fast path and on the generic path."""
import numpy as np
import pytest

from dynet_amd import DyhipError, lib
from oracle import cpu_oracle as orc
from util import GRAD_RTOL, assert_close, f32, rms

pytestmark = pytest.mark.gpu


def _case(dev, n, bd, seed, cols=True):
    rng = np.random.default_rng(seed)
    x, dy = f32(rng.standard_normal((bd, n))), f32(rng.standard_normal((bd, n)))
    g = f32(rng.uniform(0.5, 1.5, n))
    dx0, dg0, db0 = f32(rng.standard_normal((bd, n))), f32(rng.standard_normal(n)), f32(rng.standard_normal(n))
    xt, gt, dyt = dev.tensor(x), dev.tensor(g), dev.tensor(dy)
    outs = []
    for static in (False, True):
        dxt, dgt, dbt = dev.tensor(dx0), dev.tensor(dg0), dev.tensor(db0)
        if not cols:   # dx only: the call needs no scratch at all
            (dev.layer_norm_backward_static if static else dev.layer_norm_backward)(n, bd, xt, gt, dyt, dxt, None, None)
        elif static:
            dev.layer_norm_backward_static(n, bd, xt, gt, dyt, dxt, dgt, dbt)
        else:
            dev.layer_norm_backward(n, bd, xt, gt, dyt, dxt, dgt, dbt)
        outs.append((dxt.numpy(), dgt.numpy(), dbt.numpy()))
    for a, b, what in zip(outs[0], outs[1], ("dx", "dg", "db")):
        assert a.tobytes() == b.tobytes(), (what, n, bd)   # same kernels, same order: the same bits
    # and against the CPU oracle, to the gradient bar
    want = orc.layer_norm_backward(n, bd, x, g, dy, dx0.copy(), dg0.copy(), db0.copy())
    if not cols:
        want = (want[0], dg0, db0)
    floors = (1.0, np.sqrt(bd) * rms(dy), np.sqrt(bd) * rms(dy))
    for got, ref, fl, what in zip(outs[1], want, floors, ("dx", "dg", "db")):
        assert_close(got, ref.reshape(got.shape), GRAD_RTOL, "static layer_norm bwd " + what, floor=fl)


def test_static_scratch_entry_point_two_calls_in_a_row(dev):
    _case(dev, 1024, 4096, 1)     # the baseline's shape: 256 blocks of partial rows
    _case(dev, 256, 40, 2)        # smaller: the scratch still holds the previous call's partials
    _case(dev, 2048, 3000, 3)     # the largest fast-path row
    _case(dev, 1027, 33, 4)       # generic path: per-row statistics in the scratch
    _case(dev, 8, 1, 5)


def test_static_scratch_is_sized_for_the_path_the_call_takes(dev):
    """The size query covers both paths (it does not know the pointers); the static entry point knows them and
    must accept what its own path fits: fast-path rows with so many batch elements that the generic path's
    8 bytes per row would not fit, and any shape when neither dg nor db is asked for."""
    assert dev.layer_norm_backward_workspace(64, 600000) > lib.LN_STATIC_SCRATCH_BYTES
    _case(dev, 64, 600000, 6)
    assert dev.layer_norm_backward_workspace(3, 600000) > lib.LN_STATIC_SCRATCH_BYTES
    _case(dev, 3, 600000, 7, cols=False)
    _case(dev, 16, 7, 8)          # and a small call afterwards


def test_static_scratch_entry_point_rejects_what_does_not_fit(dev):
    t = dev.zeros(8)
    need = dev.layer_norm_backward_workspace(4100, 1 << 20)   # generic path: 8 bytes per row
    assert need > lib.LN_STATIC_SCRATCH_BYTES
    with pytest.raises(DyhipError) as e:
        dev.layer_norm_backward_static(4100, 1 << 20, t, t, t, t, t, t)
    assert e.value.status == lib.ERR_INVALID_ARG and "scratch" in str(e.value)
