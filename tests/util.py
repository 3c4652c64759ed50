"""Shared helpers of the parity tests: seeded inputs, tolerance checks, a GPU fixture."""
import numpy as np

F32 = np.float32

# parity bar of the hot path: fp32 forward within 1e-5 relative, gradients within
# 1e-4 relative, gathers / picks / argmax bit exact
FWD_RTOL = 1e-5
GRAD_RTOL = 1e-4


def f32(a):
    return np.ascontiguousarray(a, dtype=F32)


def assert_close(got, ref, rtol, what, floor=0.0):
    """|got - ref| <= rtol * max(|ref|, floor), elementwise.

    floor = 0 is a pure relative check.  Operators whose result is a difference
    or a long sum of terms (LayerNorm, GEMM, batch sums, scatter-add) pass the
    magnitude of those terms as `floor`, because a relative bound on a value
    that cancels to ~0 is not meaningful in fp32.
    """
    got = np.asarray(got, np.float64)
    ref = np.asarray(ref, np.float64)
    assert got.shape == ref.shape, (what, got.shape, ref.shape)
    assert np.all(np.isfinite(got)), what + ": non-finite output"
    bound = rtol * np.maximum(np.abs(ref), floor)
    err = np.abs(got - ref)
    bad = err > bound
    if np.any(bad):
        k = np.argmax(err - bound)
        raise AssertionError("%s: %d/%d outside tolerance; worst at %d: got %r ref %r (err %g, bound %g)" % (
            what, int(bad.sum()), bad.size, k, got.flat[k], ref.flat[k], err.flat[k], bound.flat[k]))


def rms(a):
    a = np.asarray(a, np.float64)
    return float(np.sqrt(np.mean(a * a))) if a.size else 0.0


from dynet_amd.synth import glorot, zipf_ids  # noqa: E402,F401
