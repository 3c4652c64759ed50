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


def assert_shadow(got, ref, exact, what, k=4.0, abs_slack=2e-7, rel_slack=1e-6, rel_min=0.0):
    """The device result is as close to the fp64 value `exact` (computed from the same fp32 inputs) as the
    CPU path `ref` is, up to a factor k: in absolute terms over all elements, and in relative terms over
    the elements with |exact| > rel_min.  Unlike a floor on a relative bound this holds small outputs (a
    gate near 0.01) to the accuracy the CPU path itself has there.  The slacks cover the case where the CPU
    path happens to hit the fp64 value almost exactly."""
    got, ref, exact = (np.asarray(a, np.float64) for a in (got, ref, exact))
    assert got.shape == ref.shape == exact.shape, (what, got.shape, ref.shape, exact.shape)
    assert np.all(np.isfinite(got)), what + ": non-finite output"
    eg, er = np.abs(got - exact), np.abs(ref - exact)
    assert eg.max() <= max(k * er.max(), abs_slack), "%s: abs error vs fp64 %g, CPU path %g" % (what, eg.max(), er.max())
    sel = np.abs(exact) > rel_min
    if np.any(sel):
        rg, rr = eg[sel] / np.abs(exact[sel]), er[sel] / np.abs(exact[sel])
        assert rg.max() <= max(k * rr.max(), rel_slack), "%s: rel error vs fp64 %g, CPU path %g" % (
            what, rg.max(), rr.max())


def rms(a):
    a = np.asarray(a, np.float64)
    return float(np.sqrt(np.mean(a * a))) if a.size else 0.0


from dynet_amd.synth import glorot, zipf_ids  # noqa: E402,F401
