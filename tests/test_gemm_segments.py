"""The hand-off between blocks of the 256 x 256-tile GEMM (dynet_amd/csrc/gemm_wide.hip), checked on the segment plan
the kernels use, without a GPU: a block that finishes a cut tile waits for flags that other blocks raise, so every flag
it waits for must be raised by exactly one block, no raised flag may be left unconsumed (it would satisfy the next
launch's wait too early), and a block may only wait for blocks dispatched before it (lower block index)."""
import numpy as np
import pytest

from dynet_amd.device import Device

SHAPES = [(10000, 4480, 1024), (1024, 4480, 10000), (10000, 1024, 4480), (4096, 1024, 4480), (1024, 4480, 4096),
          (4096, 4096, 1024), (4096, 4480, 256), (1000, 1000, 8200), (4352, 4096, 512), (7936, 4096, 256),
          (5000, 4400, 520), (300, 300, 65536), (257, 4480, 2048), (129, 129, 262144), (8192, 8192, 2048)]


def _random_shapes():
    rng = np.random.default_rng(7)
    return [(int(rng.integers(192, 12000)), int(rng.integers(192, 9000)), 32 * int(rng.integers(8, 400)))
            for _ in range(40)]


@pytest.mark.parametrize("segments", [256, 304, 64, 1, 2, 255, 257])
@pytest.mark.parametrize("M,N,K", SHAPES + _random_shapes())
def test_every_flag_is_raised_once_and_waited_for_once(M, N, K, segments):
    starts, nt, in_kernel = Device.gemm_wide_segments(M, N, K, segments)
    tiles = -(-M // 256) * -(-N // 256)
    assert nt == K // 32 and len(starts) == segments + 1
    assert starts[0] == 0 and starts[-1] == tiles * nt
    assert all(a <= b for a, b in zip(starts, starts[1:]))
    lengths = [b - a for a, b in zip(starts, starts[1:])]
    assert max(lengths) - min(lengths) <= 1                       # equal segments
    assert in_kernel == (tiles * nt // segments >= nt)
    # the kernel's walk: segment s is block segments - 1 - s
    raised = {}
    for s in range(segments):
        if starts[s] < starts[s + 1] and starts[s] % nt != 0:
            raised[s] = 0                                         # its first item starts inside a tile: a partial tile
    for s in range(segments):
        pos, end = starts[s], starts[s + 1]
        while pos < end:
            tile = pos // nt
            k0, k1 = pos - tile * nt, min(nt, end - tile * nt)
            pos += k1 - k0
            if k0 == 0 and k1 < nt:                               # holds the tile's first k-tiles: finishes it
                s2 = s + 1
                while s2 < segments and starts[s2] < (tile + 1) * nt:
                    assert s2 in raised, "segment %d waits for segment %d, which raises no flag" % (s, s2)
                    assert segments - 1 - s2 < segments - 1 - s   # a block dispatched earlier
                    raised[s2] += 1
                    s2 += 1
                if in_kernel:
                    assert s2 - s - 1 <= 1                        # a tile is cut at most once
    assert all(v == 1 for v in raised.values())
