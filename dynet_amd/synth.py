"""Synthetic inputs of the baseline configurations (seeded host generators; DyNet's own RNG is
not used because its seed 0 means "nondeterministic", dynet/init.cc:238-241)."""
import numpy as np


def zipf_ids(rng, n, vocab, s=1.1):
    """n ids from Zipf(s) truncated to [0, vocab): p(k) ~ (k+1)^-s, inverse-CDF sampling."""
    p = (np.arange(1, vocab + 1, dtype=np.float64)) ** (-s)
    cdf = np.cumsum(p)
    cdf /= cdf[-1]
    return np.minimum(np.searchsorted(cdf, rng.random(n)), vocab - 1).astype(np.uint32)


def glorot(rng, rows, cols):
    """ParameterInitGlorot (dynet/param-init.cc:26-40): U(+-sqrt(6)/sqrt(rows+cols)).
    Returned in DyNet's column-major layout of a rows x cols matrix, i.e. numpy shape (cols, rows)."""
    s = np.sqrt(6.0) / np.sqrt(rows + cols)
    return np.ascontiguousarray(rng.uniform(-s, s, (cols, rows)), dtype=np.float32)
