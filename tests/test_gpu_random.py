"""Random tensors on the GPU (randomize_uniform / bernoulli / normal, dropout, reset_rng) against the
oracle's Philox4x32-10 restatement: words, uniforms, Bernoulli masks and dropout bit for bit; normals
(device log/sin/cos vs libm) to the forward tolerance.  What pins the oracle itself is in test_oracle.py."""
import numpy as np
import pytest

from oracle import cpu_oracle as orc
from dynet_amd import DyhipError, lib
from util import assert_close, FWD_RTOL, f32

pytestmark = pytest.mark.gpu
F32 = np.float32


@pytest.mark.parametrize("n", [1, 3, 4, 5, 1023, 4096, 100003])
def test_uniform_and_bernoulli_bit_exact(dev, n):
    dev.reset_rng(41)
    key, pos, q = dev.rng_state()
    assert (key, pos, q) == (42, 0, 0)  # key = seed + 1 as in Device_GPU::reset_rng
    out = dev.empty(n + 2)
    dev.constant(out, -7.0)
    view = out.offset(1, (n,))  # misaligned start: the scalar store path
    dev.randomize_uniform(view)
    got = out.numpy()
    assert got[0] == -7.0 and got[-1] == -7.0  # nothing written outside the tensor
    assert np.array_equal(got[1:-1], orc.randomize_uniform(key, 0, 0, n))
    # the position advanced by ceil(n / 4) blocks; the next call continues the stream
    blocks = (n + 3) // 4
    assert dev.rng_state()[1] == blocks
    dev.randomize_uniform(view, -2.5, 4.0)
    assert np.array_equal(out.numpy()[1:-1], orc.randomize_uniform(key, blocks, 0, n, -2.5, 4.0))
    dev.randomize_bernoulli(view, 0.3, 1.0 / 0.3)
    want = orc.randomize_bernoulli(key, 2 * blocks, 0, n, 0.3, 1.0 / 0.3)
    assert np.array_equal(out.numpy()[1:-1], want)
    assert set(np.unique(want)) <= {F32(0.0), F32(F32(1.0) / F32(0.3))}


def test_uniform_aligned_vector_path(dev):
    dev.reset_rng(0)
    n = 1 << 20
    out = dev.empty(n)
    dev.randomize_uniform(out)
    got = out.numpy()
    assert np.array_equal(got, orc.randomize_uniform(1, 0, 0, n))
    assert got.min() > 0.0 and got.max() <= 1.0
    assert abs(got.mean() - 0.5) < 2e-3 and abs(got.var() * 12 - 1) < 1e-2


@pytest.mark.parametrize("n", [2, 7, 4096, 100001])
def test_normal_matches_oracle(dev, n):
    dev.reset_rng(7)
    out = dev.empty(n)
    dev.randomize_normal(out, 1.5, 0.25)
    want = orc.randomize_normal(8, 0, 0, n, 1.5, 0.25)
    # device log/sin/cos differ from libm by a few ulp of values of size <= ~6 before scaling
    assert_close(out.numpy(), want, FWD_RTOL, "normal", floor=1.5)
    if n > 10000:
        z = (out.numpy().astype(np.float64) - 1.5) / 0.25
        assert abs(z.mean()) < 2e-2 and abs(z.std() - 1) < 2e-2


def test_reset_rng_restarts_the_stream_and_positions_can_be_restored(dev):
    out = dev.empty(1000)
    dev.reset_rng(5)
    dev.randomize_uniform(out)
    a = out.numpy()
    dev.randomize_uniform(out)
    b = out.numpy()
    assert not np.array_equal(a, b)
    dev.reset_rng(5)
    dev.randomize_uniform(out)
    assert np.array_equal(out.numpy(), a)
    dev.rng_set_position(250)  # where the second call started
    dev.randomize_uniform(out)
    assert np.array_equal(out.numpy(), b)
    dev.reset_rng(6)
    dev.randomize_uniform(out)
    assert not np.array_equal(out.numpy(), a)


def test_forked_queue_draws_its_own_stream(dev):
    dev.reset_rng(3)
    q = dev.fork()
    a, b = dev.empty(4096), dev.empty(4096)
    dev.randomize_uniform(a)
    q.randomize_uniform(b)
    q.sync()
    key, _, qid = q.rng_state()
    assert key == 4 and qid >= 1
    assert np.array_equal(a.numpy(), orc.randomize_uniform(4, 0, 0, 4096))
    assert np.array_equal(b.numpy(), orc.randomize_uniform(4, 0, qid, 4096))
    assert not np.array_equal(a.numpy(), b.numpy())
    dev.reset_rng(9)  # reseeds the forked queues too
    q.randomize_uniform(b)
    q.sync()
    assert np.array_equal(b.numpy(), orc.randomize_uniform(10, 0, qid, 4096))
    q.close()


def test_graph_replays_draw_fresh_numbers(dev):
    dev.reset_rng(11)
    out = dev.empty(1024)
    dev.graph_begin()
    dev.randomize_bernoulli(out, 0.5, 2.0)
    g = dev.graph_end()
    seen = []
    for r in range(3):
        g.launch()
        dev.sync()
        seen.append(out.numpy())
        assert np.array_equal(seen[-1], orc.randomize_bernoulli(12, r * 256, 0, 1024, 0.5, 2.0)), r
    assert not np.array_equal(seen[0], seen[1])
    g.destroy()


@pytest.mark.parametrize("n,p", [(5, 0.5), (4099, 0.1), (1 << 16, 0.75), (64, 0.0)])
def test_dropout_forward_backward(dev, n, p):
    rng = np.random.default_rng(n)
    x, dy, dx0 = f32(rng.standard_normal(n)), f32(rng.standard_normal(n)), f32(rng.standard_normal(n))
    dev.reset_rng(1)
    xt, mask, fx = dev.tensor(x), dev.empty(n), dev.empty(n)
    dev.dropout_forward(p, xt, mask, fx)
    ref_mask, ref_fx = orc.dropout_forward(2, 0, 0, p, x)
    assert np.array_equal(mask.numpy(), ref_mask)
    assert np.array_equal(fx.numpy(), ref_fx)
    keep = 1.0 - p
    assert set(np.unique(ref_mask)) <= {F32(0.0), F32(F32(1.0) / F32(keep))}
    if n >= 4096:
        assert abs((ref_mask != 0).mean() - keep) < 0.02
    dxt = dev.tensor(dx0)
    dev.dropout_backward(mask, dev.tensor(dy), dxt)
    assert np.array_equal(dxt.numpy(), orc.dropout_backward(ref_mask, dy, dx0.copy()))


def test_lstm_dropout_masks_from_the_generator(dev):
    """CompactVanillaLSTMBuilder::set_dropout_masks (dynet/lstm.cc:964-982): masks are random_bernoulli
    tensors of Dim({dim}, batch) with p = retention and scale = 1 / retention, fed to VanillaLSTMGates."""
    I, H, B, rate = 12, 16, 5, 0.25
    rng = np.random.default_rng(2)
    keep, scale = 1.0 - rate, 1.0 / (1.0 - rate)
    dev.reset_rng(17)
    mx, mh = dev.empty((B, I)), dev.empty((B, H))
    dev.randomize_bernoulli(mx, keep, scale)
    dev.randomize_bernoulli(mh, keep, scale)
    ref_mx = orc.randomize_bernoulli(18, 0, 0, B * I, keep, scale).reshape(B, I)
    ref_mh = orc.randomize_bernoulli(18, (B * I + 3) // 4, 0, B * H, keep, scale).reshape(B, H)
    assert np.array_equal(mx.numpy(), ref_mx) and np.array_equal(mh.numpy(), ref_mh)
    x, h = f32(rng.standard_normal((B, I))), f32(rng.standard_normal((B, H)))
    Wx, Wh = f32(rng.uniform(-0.3, 0.3, (I, 4 * H))), f32(rng.uniform(-0.3, 0.3, (H, 4 * H)))
    b = f32(rng.normal(0, 0.1, 4 * H))
    want = orc.lstm_gates_forward([x], [I], H, B, h, Wx, Wh, b, mask_x=ref_mx, mask_x_bd=B, mask_h=ref_mh, mask_h_bd=B)
    fx = dev.empty((B, 4 * H))
    dev.lstm_gates_forward([dev.tensor(x)], [I], H, B, dev.tensor(h), dev.tensor(Wx), dev.tensor(Wh), dev.tensor(b),
                           fx, mask_x=mx, mask_x_bd=B, mask_h=mh, mask_h_bd=B)
    assert_close(fx.numpy(), want, FWD_RTOL, "gates under generated dropout masks", floor=1.0)


def test_random_rejects_bad_arguments(dev):
    t = dev.empty(8)
    with pytest.raises(DyhipError) as e:
        dev.randomize_bernoulli(t, 1.5)
    assert e.value.status == lib.ERR_INVALID_ARG
    with pytest.raises(DyhipError):
        dev.dropout_forward(1.0, t, t, t)
    dev.randomize_uniform(dev.empty(0))  # empty tensors are no-ops and leave the position alone
