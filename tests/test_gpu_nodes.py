"""GPU parity: GEMM shim, fused LSTM nodes, LookupNode, PickNegLogSoftmax /
logsumexp / argmax, the dynet::gpu helpers and the trainer kernels against the
CPU oracle on identical seeded inputs, through the C-ABI.
"""
import numpy as np
import pytest

from dynet_amd import DyhipError, lib
from oracle import cpu_oracle as orc
from util import F32, FWD_RTOL, GRAD_RTOL, assert_close, assert_shadow, f32, glorot, rms, zipf_ids

pytestmark = pytest.mark.gpu


# ---------------------------------------------------------------------------
# GEMM shim
# ---------------------------------------------------------------------------
def lib_pools():
    from dynet_amd import lib

    return (lib.POOL_FXS, lib.POOL_DEDFS, lib.POOL_SCS)


GEMM_SHAPES = [(1024, 32, 128), (1024, 32, 256), (4096, 128, 1280), (256, 128, 4096), (130, 33, 17), (5, 4, 6),
               (64, 1, 64), (1000, 128, 1024), (129, 65, 100),
               # small outputs with deep sums: the transposed form takes the fragment-order product (ragged edges,
               # one and several depth ranges)
               (100, 37, 1152), (64, 1, 2048), (33, 256, 1024), (2048, 200, 2560),
               # more tiles than two per CU with a thin last round: the trailing tile columns run as a GEMM of their own
               (4096, 2304, 40), (4100, 2310, 33),
               # operands of a few hundred KB: the one-launch product on 32 x 32 wavefront tiles (a tile a wavefront for
               # a shallow depth, the depth over four or eight wavefronts otherwise; 128-bit, 64-bit and scalar loads
               # along the depth by the leading dimensions' divisibility; ragged rows, columns and depth)
               (128, 128, 128), (200, 100, 50), (64, 64, 16), (33, 65, 9), (650, 1, 650), (1, 1, 1000), (35, 1, 1024),
               (1, 35, 1024), (300, 300, 300), (100, 7, 600), (31, 33, 520), (333, 333, 333), (512, 512, 512),
               (650, 3, 1300), (2000, 70, 100), (4096, 4, 256), (129, 1000, 64), (40, 40, 3), (6, 2, 70),
               # a row vector times a matrix and a depth of one (v^T * X of an attention's scores and its gradients): the same
               # bytes as a transposed product / a matrix times a vector / a rank-one update, and taken as those
               (1, 4480, 512), (1, 256, 1000), (1, 1024, 36), (1024, 36, 1), (512, 300, 1), (1, 300, 1024),
               # a tagger's output layer: a handful of rows over thousands of columns
               (20, 4480, 512), (3, 5000, 128), (20, 512, 4480), (1, 256, 300), (32, 300, 1000), (7, 1000, 257), (20, 128, 1024), (3, 64, 512), (31, 250, 1000),
               (2, 9, 1000)]


@pytest.mark.parametrize("M,N,K", GEMM_SHAPES)
def test_gemm_three_forms(dev, M, N, K):
    rng = np.random.default_rng(M * 7 + N * 3 + K)
    y0 = f32(rng.standard_normal((N, M)))
    floor = np.sqrt(K)  # size of the sum of K products of N(0,1) terms
    # NN: y = beta*y + l*r
    l, r = f32(rng.standard_normal((K, M))), f32(rng.standard_normal((N, K)))
    lt, rt = dev.tensor(l), dev.tensor(r)
    for beta in (1.0, 0.0):
        yt = dev.tensor(y0)
        dev.gemm_nn(M, N, K, lt, rt, beta, yt)
        assert_close(yt.numpy(), orc.gemm_nn(M, N, K, l, r, beta, y0.copy()), FWD_RTOL, "gemm_nn beta=%g" % beta,
                     floor=floor)
    # TN: y += l^T r with l stored K x M
    l2 = f32(rng.standard_normal((M, K)))
    yt = dev.tensor(y0)
    dev.gemm_tn_acc(M, N, K, dev.tensor(l2), rt, yt)
    assert_close(yt.numpy(), orc.gemm_tn_acc(M, N, K, l2, r, y0.copy()), FWD_RTOL, "gemm_tn", floor=floor)
    yt = dev.tensor(y0)
    dev.gemm_tn(M, N, K, dev.tensor(l2), rt, 0.0, yt)  # overwrites
    assert_close(yt.numpy(), orc.gemm_tn_acc(M, N, K, l2, r, np.zeros_like(y0)), FWD_RTOL, "gemm_tn beta=0", floor=floor)
    # NT: y += l r^T with r stored N x K
    r2 = f32(rng.standard_normal((K, N)))
    yt = dev.tensor(y0)
    dev.gemm_nt_acc(M, N, K, lt, dev.tensor(r2), yt)
    assert_close(yt.numpy(), orc.gemm_nt_acc(M, N, K, l, r2, y0.copy()), FWD_RTOL, "gemm_nt", floor=floor)


# Shallow products l * r^T (the weight gradient of one timestep, depth = batch <= 128) fetch both operand tiles whole:
# full depth (two halves), half depth, a depth with an odd number of groups of 8, ragged edges.
@pytest.mark.parametrize("M,N,K", [(4096, 1024, 128), (2052, 1028, 96), (4096, 512, 40), (1024, 4096, 64), (2048, 2048, 32)])
def test_gemm_nt_shallow(dev, M, N, K):
    rng = np.random.default_rng(M + N + K)
    y0 = f32(rng.standard_normal((N, M)))
    l, r2 = f32(rng.standard_normal((K, M))), f32(rng.standard_normal((K, N)))
    lt, rt = dev.tensor(l), dev.tensor(r2)
    yt = dev.tensor(y0)
    dev.gemm_nt_acc(M, N, K, lt, rt, yt)
    assert_close(yt.numpy(), orc.gemm_nt_acc(M, N, K, l, r2, y0.copy()), FWD_RTOL, "shallow gemm_nt_acc", floor=np.sqrt(K))
    yt = dev.tensor(y0)
    dev.gemm_nt(M, N, K, lt, rt, 0.0, yt)
    assert_close(yt.numpy(), orc.gemm_nt_acc(M, N, K, l, r2, np.zeros_like(y0)), FWD_RTOL, "shallow gemm_nt beta=0",
                 floor=np.sqrt(K))
    yt = dev.tensor(y0)
    dev.gemm_nt(M, N, K, lt, rt, 0.5, yt)
    assert_close(yt.numpy(), orc.gemm_nt_acc(M, N, K, l, r2, f32(0.5 * y0)), FWD_RTOL, "shallow gemm_nt beta=0.5",
                 floor=np.sqrt(K))


# l * r^T with a depth of at most 32 (the weight gradient of one timestep at a small batch) is a rank-K update of a matrix
# read and written once: depths on both sides of every multiple of four, column counts that do not fill the last group
# of eight, the baseline's smallest cell (1024 x 128 x 32), accumulate and overwrite.  Outputs above 4 MB at depths 24
# and 32 take the burst-fetch matrix-core kernel (ragged tile edges included).
@pytest.mark.parametrize("M,N,K", [(1024, 128, 32), (4096, 1024, 20), (2052, 1030, 7), (256, 5, 1), (6000, 1500, 13),
                                   (1024, 256, 4), (1024, 255, 29), (512, 9, 16), (4096, 1024, 24), (4096, 1024, 32),
                                   (2052, 1028, 24), (1500, 1000, 32)])
def test_gemm_nt_thin(dev, M, N, K):
    rng = np.random.default_rng(M + N + K)
    y0 = f32(rng.standard_normal((N, M)))
    l, r2 = f32(rng.standard_normal((K, M))), f32(rng.standard_normal((K, N)))
    lt, rt = dev.tensor(l), dev.tensor(r2)
    ref64 = r2.astype(np.float64).T @ l.astype(np.float64)
    yt = dev.tensor(y0)
    dev.gemm_nt_acc(M, N, K, lt, rt, yt)
    assert_close(yt.numpy(), (y0 + ref64).astype(np.float32), FWD_RTOL, "thin gemm_nt_acc", floor=np.sqrt(K))
    first = yt.numpy().copy()
    yt = dev.tensor(y0)
    dev.gemm_nt_acc(M, N, K, lt, rt, yt)
    assert yt.numpy().tobytes() == first.tobytes()  # a fixed order of additions
    yt = dev.tensor(y0)
    dev.gemm_nt(M, N, K, lt, rt, 0.0, yt)
    assert_close(yt.numpy(), ref64.astype(np.float32), FWD_RTOL, "thin gemm_nt beta=0", floor=np.sqrt(K))


# l^T * r with at most 32 columns of r (dx and dh of the gates node at a small batch): up to four columns the left
# operand streamed once, four of its columns a block; 5..32 columns on the matrix cores through LDS tiles (or the
# fragment-order product where the depth is a multiple of 128).  Column counts on both sides of every multiple of
# four, row counts that do not fill the last block or tile, depths that end inside a 64-index round, any beta.
@pytest.mark.parametrize("M,N,K", [(1024, 20, 4096), (128, 32, 1024), (650, 20, 2600), (1000, 1, 4000), (37, 7, 256),
                                   (1024, 13, 6000), (258, 4, 1024), (255, 29, 2048), (1024, 20, 10000), (33, 5, 260),
                                   (100, 32, 1004), (2048, 9, 516), (4100, 31, 772), (32, 16, 100000), (1024, 6, 300),
                                   (256, 128, 4096), (500, 47, 1028), (1024, 40, 2000), (100, 256, 512), (333, 65, 1300)])
def test_gemm_tn_thin(dev, M, N, K):
    rng = np.random.default_rng(M + N + K)
    y0 = f32(rng.standard_normal((N, M)))
    l, r2 = f32(rng.standard_normal((M, K))), f32(rng.standard_normal((N, K)))
    lt, rt = dev.tensor(l), dev.tensor(r2)
    ref64 = r2.astype(np.float64) @ l.astype(np.float64).T
    for beta in (1.0, 0.0, 0.5):
        yt = dev.tensor(y0)
        dev.gemm_tn(M, N, K, lt, rt, beta, yt)
        assert_close(yt.numpy(), (beta * y0 + ref64).astype(np.float32), FWD_RTOL, "thin gemm_tn beta=%g" % beta,
                     floor=np.sqrt(K))
    again = dev.tensor(y0)
    dev.gemm_tn(M, N, K, lt, rt, 0.5, again)
    assert again.numpy().tobytes() == yt.numpy().tobytes()  # a fixed order of additions


# l * r with at most 8 columns of r (matrix times vector: the un-batched graph's affine layers and projections): the
# depth split into slabs over blocks, their partial sums added by a second kernel with the epilogue (beta or bias).
# From 1024 rows on (and a depth of at most 4096 whose share of r fits LDS) one launch: a block owns 32 rows and the
# whole depth; rows that do not fill the last block, a depth that is not a multiple of eight, r at the LDS limit.
@pytest.mark.parametrize("M,N,K", [(4096, 1, 1024), (10000, 1, 1024), (1024, 3, 1000), (256, 8, 37), (6000, 5, 1500),
                                   (260, 2, 8), (4096, 4, 2048), (512, 1, 20000), (1028, 2, 77), (2052, 7, 1535), (2052, 7, 2047),
                                   (1024, 8, 1536), (1024, 8, 2048), (1024, 4, 4096), (1024, 1, 4100), (3000, 1, 5)])
def test_gemm_nn_thin(dev, M, N, K):
    rng = np.random.default_rng(M + N + K)
    y0 = f32(rng.standard_normal((N, M)))
    l, r2, bias = f32(rng.standard_normal((K, M))), f32(rng.standard_normal((N, K))), f32(rng.standard_normal(M))
    lt, rt, bt = dev.tensor(l), dev.tensor(r2), dev.tensor(bias)
    ref64 = r2.astype(np.float64) @ l.astype(np.float64)
    for beta in (1.0, 0.0, 0.5):
        yt = dev.tensor(y0)
        dev.gemm_nn(M, N, K, lt, rt, beta, yt)
        assert_close(yt.numpy(), (beta * y0 + ref64).astype(np.float32), FWD_RTOL, "thin gemm_nn beta=%g" % beta,
                     floor=np.sqrt(K))
    again = dev.tensor(y0)
    dev.gemm_nn(M, N, K, lt, rt, 0.5, again)
    assert again.numpy().tobytes() == yt.numpy().tobytes()  # a fixed order of additions
    yt = dev.tensor(y0)
    dev.affine_forward(M, N, K, bt, lt, rt, yt)
    assert_close(yt.numpy(), (bias[None, :] + ref64).astype(np.float32), FWD_RTOL, "thin affine", floor=np.sqrt(K))


# l * r with 9..32 columns of r (a small batch's affine layers): rows in 128-row wavefront tiles on the matrix cores,
# the depth split over a block's wavefronts and over blocks; depths that are not multiples of 4 or 16, rows that do not
# fill the last tile, a column count of 32, and a depth long enough for hundreds of slabs.
# Depths that are multiples of 128 take the one-launch fragment-order product instead (32- or 64-row blocks, rows past
# the end dropped, up to 256 columns).
@pytest.mark.parametrize("M,N,K", [(4096, 20, 1024), (4096, 32, 2048), (132, 9, 16), (128, 9, 17), (2600, 20, 650),
                                   (1000, 31, 1001), (10000, 16, 1024), (512, 20, 512), (256, 12, 50000), (1024, 20, 256),
                                   (4096, 20, 1000), (1030, 17, 384), (33, 9, 128), (4100, 200, 256), (100, 256, 1280),
                                   (8192, 64, 128), (1200, 20, 300), (400, 16, 100), (2000, 12, 500), (64, 9, 4),
                                   (640, 33, 132), (1000, 20, 2044), (1300, 20, 650), (300, 9, 2), (515, 40, 1030),
                                   (999, 12, 390)])
def test_gemm_nn_mid(dev, M, N, K):
    rng = np.random.default_rng(M + N + K)
    y0 = f32(rng.standard_normal((N, M)))
    l, r2, bias = f32(rng.standard_normal((K, M))), f32(rng.standard_normal((N, K))), f32(rng.standard_normal(M))
    lt, rt, bt = dev.tensor(l), dev.tensor(r2), dev.tensor(bias)
    ref64 = r2.astype(np.float64) @ l.astype(np.float64)
    for beta in (1.0, 0.0, 0.5):
        yt = dev.tensor(y0)
        dev.gemm_nn(M, N, K, lt, rt, beta, yt)
        assert_close(yt.numpy(), (beta * y0 + ref64).astype(np.float32), FWD_RTOL, "mid gemm_nn beta=%g" % beta,
                     floor=np.sqrt(K))
    again = dev.tensor(y0)
    dev.gemm_nn(M, N, K, lt, rt, 0.5, again)
    assert again.numpy().tobytes() == yt.numpy().tobytes()  # a fixed order of additions
    yt = dev.tensor(y0)
    dev.affine_forward(M, N, K, bt, lt, rt, yt)
    assert_close(yt.numpy(), (bias[None, :] + ref64).astype(np.float32), FWD_RTOL, "mid affine", floor=np.sqrt(K))
    # every entry of r matters once: a product with one-hot columns returns columns of l
    hot = np.zeros((N, K), np.float32)
    picks = rng.integers(0, K, N)
    hot[np.arange(N), picks] = 1.0
    yt = dev.empty((N, M))
    dev.gemm_nn(M, N, K, lt, dev.tensor(hot), 0.0, yt)
    assert yt.numpy().tobytes() == l[picks].tobytes()


# Large outputs go to the 256 x 256-tile kernel, which deals the k-tiles of all tiles to the CUs in equal segments:
# (a) fewer tiles than CUs: every tile spans several segments, whose partial tiles a second kernel adds; ragged edges
# and a depth that is not a multiple of 32 (the rest of the depth is added by the 128-wide kernel); (b), (c) a little
# more than one tile, and about two shallow tiles, per CU: a cut tile is finished inside the kernel; (d) a transposed
# left operand whose row count is not a multiple of 4.
# Checked against the fp64 product of the same fp32 inputs (the oracle's triple loop is the same sum, too slow here).
# (e) a shallow product whose leading 4096 columns are one full round of tiles: those go to the 256-wide kernel, the
# other 384 columns run as a product of their own.
# (f) more tiles than CUs with ragged edges and a depth remainder: every block finishes one cut tile from another
# block's partial tile inside the kernel; (g) the cfg-5 output projection.
WIDE_GEMM_SHAPES = [(1000, 1000, 8200), (4352, 4096, 512), (7936, 4096, 256), (1001, 1000, 8192), (2048, 2304, 2080),
                    (4096, 4480, 264), (5000, 4400, 520), (10000, 4480, 1024)]


@pytest.mark.parametrize("M,N,K", WIDE_GEMM_SHAPES)
def test_gemm_wide_tiles_three_forms(dev, M, N, K):
    want = 2 if (M, N) == (4096, 4480) else 1
    assert dev.gemm_uses_wide_tiles(1, 0, M, N, K) == want and (M % 4 != 0 or dev.gemm_uses_wide_tiles(0, 0, M, N, K) == want)
    rng = np.random.default_rng(M + 3 * N + 7 * K)
    y0 = f32(rng.standard_normal((N, M)))
    floor = np.sqrt(K)
    l, r = f32(rng.standard_normal((K, M))), f32(rng.standard_normal((N, K)))  # l: M x K, r: K x N, column-major
    exact = r.astype(np.float64) @ l.astype(np.float64)                        # (N, M) = column-major M x N
    lt, rt = dev.tensor(l), dev.tensor(r)
    if M % 4 == 0:
        for beta in (1.0, 0.0):
            yt = dev.tensor(y0)
            dev.gemm_nn(M, N, K, lt, rt, beta, yt)
            assert_close(yt.numpy(), beta * y0 + exact, FWD_RTOL, "wide gemm_nn beta=%g" % beta, floor=floor)
        again = dev.tensor(y0)  # partial tiles are added in a fixed order: the same bits every time
        dev.gemm_nn(M, N, K, lt, rt, 0.0, again)
        assert again.numpy().tobytes() == yt.numpy().tobytes()
        r2 = f32(r.T)  # N x K column-major = (K, N) row-major
        yt = dev.tensor(y0)
        dev.gemm_nt_acc(M, N, K, lt, dev.tensor(r2), yt)
        assert_close(yt.numpy(), y0 + exact, FWD_RTOL, "wide gemm_nt", floor=floor)
        bias = f32(rng.standard_normal(M))
        yt = dev.empty((N, M))
        dev.affine_forward(M, N, K, dev.tensor(bias), lt, rt, yt)
        assert_close(yt.numpy(), bias[None, :] + exact, FWD_RTOL, "wide affine", floor=floor)
    l2 = f32(l.T)  # K x M column-major
    for beta in (1.0, 0.0):
        yt = dev.tensor(y0)
        dev.gemm_tn(M, N, K, dev.tensor(l2), rt, beta, yt)
        assert_close(yt.numpy(), beta * y0 + exact, FWD_RTOL, "wide gemm_tn beta=%g" % beta, floor=floor)


def test_gemm_wide_tiles_random_shapes(dev):
    """Seeded random shapes -- fewer tiles than CUs (every tile spans several segments of k-tiles; a second kernel
    adds the parts), a little more than one tile per CU (a cut tile is finished inside the kernel), whole rounds plus
    a few tile columns that run as a product of their own, many shallow tiles -- with ragged edges and depths with
    and without a remainder of 32; all three forms against the fp64 product."""
    rng = np.random.default_rng(2024)
    r4 = lambda lo, hi: 4 * int(rng.integers(lo, hi))
    shapes = []
    for _ in range(4):  # few tiles, deep
        a, b = int(rng.integers(2, 5)), int(rng.integers(2, 5))
        nt = -(-4096 // (a * b)) + int(rng.integers(0, 8))
        shapes.append((256 * a - r4(0, 10), 256 * b - r4(0, 10), 32 * nt + r4(0, 8)))
    for _ in range(2):  # one round and a few tile columns more
        shapes.append((256 * 17 - r4(0, 10), 256 * int(rng.integers(17, 19)) - r4(0, 10), 32 * int(rng.integers(16, 22)) + r4(0, 8)))
    for _ in range(2):  # one exact round of tile columns and some columns more
        shapes.append((4096, 4096 + r4(10, 100), 32 * int(rng.integers(8, 12)) + r4(0, 8)))
    shapes.append((256 * 19 - r4(0, 10), 256 * 24 - r4(0, 10), 256 + r4(0, 8)))  # 456 tiles of 8 k-tiles
    taken = set()
    for M, N, K in shapes:
        kind = dev.gemm_uses_wide_tiles(0, 0, M, N, K)
        taken.add(kind)
        l, r = f32(rng.standard_normal((K, M))), f32(rng.standard_normal((N, K)))
        y0 = f32(rng.standard_normal((N, M)))
        exact = r.astype(np.float64) @ l.astype(np.float64)
        lt, rt = dev.tensor(l), dev.tensor(r)
        what = "M=%d N=%d K=%d kernel choice %d" % (M, N, K, kind)
        assert kind != 0, what
        yt = dev.tensor(y0)
        dev.gemm_nn(M, N, K, lt, rt, 1.0, yt)
        assert_close(yt.numpy(), y0 + exact, FWD_RTOL, "gemm_nn " + what, floor=np.sqrt(K))
        yt = dev.tensor(y0)
        dev.gemm_nt(M, N, K, lt, dev.tensor(f32(r.T)), 0.0, yt)
        assert_close(yt.numpy(), exact, FWD_RTOL, "gemm_nt " + what, floor=np.sqrt(K))
        yt = dev.tensor(y0)
        dev.gemm_tn(M, N, K, dev.tensor(f32(l.T)), rt, 1.0, yt)
        assert_close(yt.numpy(), y0 + exact, FWD_RTOL, "gemm_tn " + what, floor=np.sqrt(K))
        for w in lib_pools():
            dev.sync()
            dev.free_pool(w)
    assert taken == {1, 2}


def test_gemm_small_batch_random_shapes(dev):
    """Seeded random products with 1..40 columns on one side: the matrix-times-vector kernels (slab and one-launch
    forms), the 9..32-column matrix-core kernel, the rank-K update and the streamed transposed product, and the
    general kernels where a size is off their grid (row counts that are not a multiple of four, depths down to 1,
    operands that start off a 16-byte boundary).  All three forms against the fp64 product of the same inputs."""
    rng = np.random.default_rng(77)
    for it in range(40):
        M = int(rng.choice([int(rng.integers(1, 300)), 4 * int(rng.integers(32, 1200)), int(rng.integers(300, 5000))]))
        N = int(rng.integers(1, 41))
        K = int(rng.choice([int(rng.integers(1, 64)), int(rng.integers(64, 3000)), 4 * int(rng.integers(16, 600))]))
        off = int(rng.choice([0, 0, 1, 4]))  # floats before each operand's first element
        l, r = f32(rng.standard_normal(K * M + off)), f32(rng.standard_normal(N * K + off))
        y0 = f32(rng.standard_normal((N, M)))
        lm, rm = l[off:].reshape(K, M), r[off:].reshape(N, K)
        exact = rm.astype(np.float64) @ lm.astype(np.float64)
        what = "M=%d N=%d K=%d offset %d" % (M, N, K, off)
        lt, rt = dev.tensor(l).offset(off, (K, M)), dev.tensor(r).offset(off, (N, K))
        for beta in (0.0, 1.0):
            yt = dev.tensor(y0)
            dev.gemm_nn(M, N, K, lt, rt, beta, yt)
            assert_close(yt.numpy(), beta * y0 + exact, FWD_RTOL, "gemm_nn " + what, floor=np.sqrt(K))
        lT = np.concatenate([l[:off], f32(lm.T).ravel()])
        rT = np.concatenate([r[:off], f32(rm.T).ravel()])
        yt = dev.tensor(y0)
        dev.gemm_nt(M, N, K, lt, dev.tensor(rT).offset(off, (K, N)), 1.0, yt)
        assert_close(yt.numpy(), y0 + exact, FWD_RTOL, "gemm_nt " + what, floor=np.sqrt(K))
        yt = dev.tensor(y0)
        dev.gemm_tn(M, N, K, dev.tensor(lT).offset(off, (M, K)), rt, 1.0, yt)
        assert_close(yt.numpy(), y0 + exact, FWD_RTOL, "gemm_tn " + what, floor=np.sqrt(K))
        # the roles swapped: a wide right operand against a thin left one
        yt = dev.zeros((M, N))
        dev.gemm_nn(N, M, K, dev.tensor(f32(rm.T)), dev.tensor(f32(lm.T)), 0.0, yt)
        assert_close(yt.numpy(), exact.T, FWD_RTOL, "gemm_nn swapped " + what, floor=np.sqrt(K))
        for w in lib_pools():
            dev.sync()
            dev.free_pool(w)


def test_gemm_wide_give_up_is_reported_by_every_synchronising_call_and_leaves_clean_flags():
    """The error path of the hand-off between blocks, forced from the host: producers store their partial tiles but
    leave their flags down and the consumers' bounded wait is set to zero polls, so every cut tile's consumer gives
    up at once and every kernel still runs to its end.  dyhip_device_sync and dyhip_memcpy_d2h must both report it,
    and the next product (defaults restored) must be right: no stale flag."""
    from dynet_amd import Device
    from dynet_amd.device import DyhipError

    d = Device(0, mem_mb=(512, 64, 64, 64))
    try:
        M, N, K = 4352, 4096, 512  # 272 tiles of 16 k-tiles on 256 segments: cut tiles are finished inside the kernel
        assert d.gemm_uses_wide_tiles(0, 0, M, N, K) == 1
        assert Device.gemm_wide_segments(M, N, K, 256)[2]
        rng = np.random.default_rng(11)
        l, r = f32(rng.standard_normal((K, M))), f32(rng.standard_normal((N, K)))
        exact = r.astype(np.float64) @ l.astype(np.float64)
        lt, rt, yt = d.tensor(l), d.tensor(r), d.empty((N, M))
        d.set_gemm_handoff(0, False)
        d.gemm_nn(M, N, K, lt, rt, 0.0, yt)
        with pytest.raises(DyhipError, match="gave up"):
            d.sync()
        d.sync()  # reported once; the queue is usable again
        d.gemm_nn(M, N, K, lt, rt, 0.0, yt)
        with pytest.raises(DyhipError, match="gave up"):
            yt.numpy()
        d.set_gemm_handoff()
        d.gemm_nn(M, N, K, lt, rt, 0.0, yt)
        d.sync()
        assert_close(yt.numpy(), exact, FWD_RTOL, "wide gemm after a reported give-up", floor=np.sqrt(K))
    finally:
        d.close()


def test_gemm_wide_tiles_first_used_inside_a_graph_and_scaled_accumulate():
    """A device whose first large product is recorded into a graph (the kernel's dynamic-LDS opt-in then happens
    during the capture), replayed with eager work between the replays; and beta other than 0 or 1."""
    from dynet_amd import Device

    d = Device(0, mem_mb=(256, 64, 64, 64))
    try:
        M, N, K = 1024, 1024, 8192
        assert d.gemm_uses_wide_tiles(0, 0, M, N, K) == 1
        rng = np.random.default_rng(5)
        l, r = f32(rng.standard_normal((K, M))), f32(rng.standard_normal((N, K)))
        y0 = f32(rng.standard_normal((N, M)))
        exact = r.astype(np.float64) @ l.astype(np.float64)
        lt, rt, yt, y0t = d.tensor(l), d.tensor(r), d.empty((N, M)), d.tensor(y0)
        d.graph_begin()
        d.scale_copy(M * N, y0t, 1.0, yt)
        d.gemm_nn(M, N, K, lt, rt, 0.5, yt)
        g = d.graph_end()
        for replay in range(3):
            g.launch()
            d.sync()
            assert_close(yt.numpy(), 0.5 * y0 + exact, FWD_RTOL, "wide gemm in a graph, replay %d" % replay,
                         floor=np.sqrt(K))
            d.constant(yt, 7.0)  # eager work between the replays
            d.sync()
        g.destroy()
    finally:
        d.close()


@pytest.mark.parametrize("M,N,K,B", [(64, 48, 32, 5), (130, 70, 33, 3), (7, 5, 3, 17), (256, 128, 256, 4), (31, 1, 9, 2),
                                     (7, 5, 9, 1000), (1, 35, 1024, 128), (35, 1, 1024, 128), (64, 64, 64, 128),
                                     (35, 35, 64, 512), (512, 1, 512, 32), (33, 2, 130, 3), (300, 300, 2048, 2),
                                     # an attention over a batch: context H*a, its gradients dctx*a^T (a rank-one update an item)
                                     # and H^T*dctx: the streaming kernels with the item in the grid
                                     (1024, 1, 35, 16), (256, 2, 40, 5), (512, 4, 300, 3), (1024, 35, 1, 16), (256, 7, 32, 4),
                                     (35, 1, 1024, 16), (9, 3, 512, 7), (35, 1, 260, 3), (1000, 8, 24, 6)])
def test_gemm_strided_batched(dev, M, N, K, B):
    """The batched-left-operand branches of the three GEMM shims: per batch item the plain product, as the
    reference's CPU path loops it (dynet/matrix-multiply.h:90-93, 148-150, 213-215)."""
    rng = np.random.default_rng(M + 3 * N + 5 * K + B)
    floor = np.sqrt(K)
    y0 = f32(rng.standard_normal((B, N, M)))
    l, r = f32(rng.standard_normal((B, K, M))), f32(rng.standard_normal((B, N, K)))
    lT, rT = f32(rng.standard_normal((B, M, K))), f32(rng.standard_normal((B, K, N)))
    # l * r, both batched, beta 0 and 1; then with r shared by the items (stride 0)
    for beta in (0.0, 1.0):
        yt = dev.tensor(y0)
        dev.gemm_strided_batched(0, 0, M, N, K, dev.tensor(l), M * K, dev.tensor(r), K * N, beta, yt, M * N, B)
        want = np.stack([orc.gemm_nn(M, N, K, l[b], r[b], beta, y0[b].copy()) for b in range(B)])
        assert_close(yt.numpy(), want, FWD_RTOL, "batched l*r beta=%g" % beta, floor=floor)
    yt = dev.tensor(y0)
    dev.gemm_strided_batched(0, 0, M, N, K, dev.tensor(l), M * K, dev.tensor(r[0]), 0, 1.0, yt, M * N, B)
    want = np.stack([orc.gemm_nn(M, N, K, l[b], r[0], 1.0, y0[b].copy()) for b in range(B)])
    assert_close(yt.numpy(), want, FWD_RTOL, "batched l*r, shared r", floor=floor)
    # l^T * r
    yt = dev.tensor(y0)
    dev.gemm_strided_batched(1, 0, M, N, K, dev.tensor(lT), M * K, dev.tensor(r), K * N, 1.0, yt, M * N, B)
    want = np.stack([orc.gemm_tn_acc(M, N, K, lT[b], r[b], y0[b].copy()) for b in range(B)])
    assert_close(yt.numpy(), want, FWD_RTOL, "batched l^T*r", floor=floor)
    # l * r^T with l shared
    yt = dev.tensor(y0)
    dev.gemm_strided_batched(0, 1, M, N, K, dev.tensor(l[1]), 0, dev.tensor(rT), K * N, 1.0, yt, M * N, B)
    want = np.stack([orc.gemm_nt_acc(M, N, K, l[1], rT[b], y0[b].copy()) for b in range(B)])
    assert_close(yt.numpy(), want, FWD_RTOL, "batched l*r^T, shared l", floor=floor)
    # overlapping outputs and the doubly transposed form are refused
    with pytest.raises(DyhipError):
        dev.gemm_strided_batched(0, 0, M, N, K, dev.tensor(l), M * K, dev.tensor(r), K * N, 0.0, yt, M * N - 1, B)
    with pytest.raises(DyhipError):
        dev.gemm_strided_batched(1, 1, M, N, K, dev.tensor(l), M * K, dev.tensor(r), K * N, 0.0, yt, M * N, B)


@pytest.mark.parametrize("off_l,off_r", [(0, 0), (1, 0), (2, 2), (0, 3), (2, 0), (4, 2)])
@pytest.mark.parametrize("M,N,K", [(96, 40, 200), (70, 33, 64), (650, 2, 652)])
def test_gemm_small_products_on_operands_off_the_16_byte_grid(dev, M, N, K, off_l, off_r):
    """Operands that start 4, 8 or 12 bytes into a 16-byte line: the loads along the depth fall back from 128 to 64 or
    32 bits; same products as dynet/matrix-multiply.h:70-215."""
    from dynet_amd.device import DevTensor

    rng = np.random.default_rng(M + N + K + 10 * off_l + off_r)
    floor = np.sqrt(K)
    y0 = f32(rng.standard_normal((N, M)))
    lbuf, rbuf = f32(rng.standard_normal(M * K + off_l)), f32(rng.standard_normal(N * K + off_r))
    lt, rt = dev.tensor(lbuf), dev.tensor(rbuf)
    lv = DevTensor(dev, lt.ptr + 4 * off_l, (M * K,))
    rv = DevTensor(dev, rt.ptr + 4 * off_r, (N * K,))
    l, r = lbuf[off_l:], rbuf[off_r:]
    for beta in (0.0, 1.0):
        yt = dev.tensor(y0)
        dev.gemm_nn(M, N, K, lv, rv, beta, yt)
        assert_close(yt.numpy(), orc.gemm_nn(M, N, K, l.reshape(K, M), r.reshape(N, K), beta, y0.copy()), FWD_RTOL,
                     "l*r", floor=floor)
    yt = dev.tensor(y0)
    dev.gemm_tn_acc(M, N, K, lv, rv, yt)
    assert_close(yt.numpy(), orc.gemm_tn_acc(M, N, K, l.reshape(M, K), r.reshape(N, K), y0.copy()), FWD_RTOL, "l^T*r",
                 floor=floor)
    yt = dev.tensor(y0)
    dev.gemm_nt_acc(M, N, K, lv, rv, yt)
    assert_close(yt.numpy(), orc.gemm_nt_acc(M, N, K, l.reshape(K, M), r.reshape(K, N), y0.copy()), FWD_RTOL, "l*r^T",
                 floor=floor)


def test_gemm_is_fp32_accurate_against_fp64(dev):
    """No reduced-precision shortcut on the matrix cores: error vs fp64 stays at fp32 rounding level."""
    rng = np.random.default_rng(5)
    M, N, K = 512, 64, 2048
    l, r = f32(rng.standard_normal((K, M))), f32(rng.standard_normal((N, K)))
    yt = dev.zeros((N, M))
    dev.gemm_nn(M, N, K, dev.tensor(l), dev.tensor(r), 0.0, yt)
    want = r.astype(np.float64) @ l.astype(np.float64)
    assert np.max(np.abs(yt.numpy() - want)) < 2e-6 * np.sqrt(K) * 10


@pytest.mark.parametrize("M,N,K", [(1000, 128, 64), (10000, 96, 256), (37, 5, 20), (300, 192, 128), (4096, 4, 1024),
                                   (4100, 2310, 24), (650, 1, 650), (100, 7, 100), (3, 3, 3), (33, 100, 5000), (200, 100, 50),
                                   (650, 2, 1300)])
def test_affine_forward(dev, M, N, K):
    """AffineTransform: bias broadcast + W x (direct and split-K routes of the GEMM)."""
    rng = np.random.default_rng(M + N + K)
    W, x, b = f32(rng.standard_normal((K, M))), f32(rng.standard_normal((N, K))), f32(rng.standard_normal(M))
    want = np.ascontiguousarray(np.broadcast_to(b, (N, M))).copy()
    orc.gemm_nn(M, N, K, W, x, 1.0, want)
    fx = dev.empty((N, M))
    dev.constant(fx, 7.0)  # forward overwrites
    dev.affine_forward(M, N, K, dev.tensor(b), dev.tensor(W), dev.tensor(x), fx)
    assert_close(fx.numpy(), want, FWD_RTOL, "affine", floor=np.sqrt(K))


# ---------------------------------------------------------------------------
# fused LSTM nodes
# ---------------------------------------------------------------------------
def test_lstm_golden_vectors(dev, golden):
    gd = golden["lstm_nodes"]
    rel = gd["rel_tol"]
    t = gd["lstm_node_h_fwd"]
    H, B = t["hidden_dim"], t["batch_size"]
    out = dev.empty((B, H))
    dev.lstm_h_forward(H, B, dev.tensor(f32(t["c_t"])), dev.tensor(f32(t["gates_t"])), out)
    h = out.numpy().reshape(-1)
    assert abs(h[0]) < t["small_abs"]
    assert_close(h[1:], np.array(t["h_t"][1:]), rel, "lstm_node_h_fwd")
    t = gd["lstm_node_c_fwd"]
    dev.lstm_c_forward(H, B, dev.tensor(f32(t["c_tm1"])), dev.tensor(f32(t["gates_t"])), out)
    c = out.numpy().reshape(-1)
    assert np.all(np.abs(c[:3]) < t["small_abs"])
    assert_close(c[3:], np.array(t["c_t"][3:]), rel, "lstm_node_c_fwd")
    for name, mode in (("lstm_node_gates_fwd", lib.LOGISTIC_PACKET), ("lstm_node_gates_fwd", lib.LOGISTIC_SCALAR),
                       ("lstm_node_gates_dropout_fwd", lib.LOGISTIC_PACKET)):
        t = gd[name]
        I, H, B = t["input_dim"], t["hidden_dim"], t["batch_size"]
        fx = dev.empty((B, 4 * H))
        kw = {}
        if "mask_x" in t:
            kw = dict(mask_x=dev.tensor(f32(t["mask_x"])), mask_x_bd=B, mask_h=dev.tensor(f32(t["mask_h"])), mask_h_bd=B)
        dev.lstm_gates_forward([dev.tensor(f32(t["x_t"]))], [I], H, B, dev.tensor(f32(t["h_tm1"])),
                               dev.tensor(f32(t["Wx"])), dev.tensor(f32(t["Wh"])), dev.tensor(f32(t["b"])), fx,
                               logistic_mode=mode, **kw)
        assert_close(fx.numpy().reshape(-1), np.array(t["gates"]), rel, name)


def _sig64(v):
    return 1.0 / (1.0 + np.exp(-v))


def _lstm_exact_step(x, h_prev, c_prev, Wx, Wh, b, mask_x=None, mask_h=None):
    """One VanillaLSTMGates -> C -> H step in fp64 from fp32 inputs (true sigmoid / tanh): the yardstick
    for assert_shadow.  Weights are stored [k][row], so the pre-activation is x Wx + h Wh + b (+1 on f)."""
    f64 = lambda a: np.asarray(a, np.float64)
    H = h_prev.shape[1]
    xm = f64(x) * (f64(mask_x) if mask_x is not None else 1.0)
    hm = f64(h_prev) * (f64(mask_h) if mask_h is not None else 1.0)
    pre = xm @ f64(Wx) + hm @ f64(Wh) + f64(b)
    pre[:, H:2 * H] += 1.0
    g = np.concatenate([_sig64(pre[:, :3 * H]), np.tanh(pre[:, 3 * H:])], axis=1)
    c = g[:, :H] * g[:, 3 * H:] + g[:, H:2 * H] * f64(c_prev)
    h = g[:, 2 * H:3 * H] * np.tanh(c)
    return g, c, h


def _assert_gates_shadow(got, ref, exact, H, what):
    """Sigmoid gates: relative everywhere (a small gate has a large negative pre-activation, so its relative
    error is the absolute error of that sum).  The tanh gate, c and h pass through zero, where a relative
    error measures nothing (tanh(s) ~ s for a sum s of O(1) terms that cancels): absolute everywhere,
    relative above 0.1."""
    assert_shadow(got[:, :3 * H], ref[:, :3 * H], exact[:, :3 * H], what + " (i,f,o)")
    assert_shadow(got[:, 3 * H:], ref[:, 3 * H:], exact[:, 3 * H:], what + " (g)", rel_min=0.1)


def _lstm_case(rng, I, H, B):
    x = f32(rng.standard_normal((B, I)))
    h = f32(rng.standard_normal((B, H)))
    c = f32(rng.standard_normal((B, H)))
    Wx, Wh = glorot(rng, 4 * H, I), glorot(rng, 4 * H, H)
    b = np.zeros(4 * H, F32)
    return x, h, c, Wx, Wh, b


@pytest.mark.parametrize("I,H,B,dims,dropout,mask_full", [
    (128, 256, 32, None, False, True),      # the single-cell configuration of the baseline
    (256, 1024, 128, None, False, True),    # layer 1 of the LM configuration
    (5, 3, 2, None, False, True),           # tests/test-rnn.cc:341-357
    (3, 5, 2, None, True, True),            # :402-431
    (3, 5, 2, None, True, False),           # :601-630 (batch-broadcast masks)
    (4, 5, 2, [1, 3], False, True),         # :433-460 (multi-input)
    (4, 5, 2, [1, 3], True, True),          # :499-529
    (37, 19, 7, [5, 32], True, False),
    # up to 8 columns with at least 256 gate rows: the matrix-times-vector kernels (forward over both depth segments
    # with the gates' epilogue in its second kernel; streaming kernels for dx / dh and the weight gradients)
    (128, 128, 1, None, False, True),
    (200, 64, 3, None, False, True),
    (256, 512, 8, None, True, True),
    (96, 72, 2, [32, 64], False, True),
    # 9..32 columns: the forward takes the small-batch product over both depth segments (weights above 4 MB, or
    # sizes the fragment-order kernel does not take), 128-bit and one-by-one reads of x and h
    (512, 768, 20, None, False, True),
    (200, 64, 12, None, False, True),
    (330, 200, 20, [130, 200], True, True),
    (256, 256, 9, None, False, True),
    # depths that are multiples of four only: the one-launch forward's leftover groups (100 = 12 groups and a half,
    # 300 + 200: a leading 256 and 128 split over the waves, the rest dealt out one group a wave)
    (100, 200, 16, None, False, True),
    (300, 200, 20, None, True, True),
    (132, 64, 10, [100, 32], False, True),
    # even depths that are not multiples of four: x and h columns start on 8-byte boundaries only
    (650, 650, 20, None, False, True),
    (50, 30, 12, None, True, True),
    (6, 10, 9, None, False, True),
])
def test_lstm_cell_forward_backward(dev, I, H, B, dims, dropout, mask_full):
    rng = np.random.default_rng(I * 100 + H * 10 + B)
    x, h, c_prev, Wx, Wh, b = _lstm_case(rng, I, H, B)
    if H < 64:
        b = f32(rng.standard_normal(4 * H) * 0.1)
    dims = dims or [I]
    offs = np.cumsum([0] + dims)
    xs = [np.ascontiguousarray(x[:, offs[k]:offs[k + 1]]) for k in range(len(dims))]
    mx = mh = None
    mbd = 0
    if dropout:
        mbd = B if mask_full else 1
        mx, mh = f32(rng.integers(0, 2, (mbd, I)) * 0.9), f32(rng.integers(0, 2, (mbd, H)) * 0.8)
    xs_t = [dev.tensor(a) for a in xs]
    ht, ct, Wxt, Wht, bt = (dev.tensor(a) for a in (h, c_prev, Wx, Wh, b))
    mxt = dev.tensor(mx) if dropout else None
    mht = dev.tensor(mh) if dropout else None
    mask_kw = dict(mask_x=mxt, mask_x_bd=mbd, mask_h=mht, mask_h_bd=mbd)
    o_mask = dict(mask_x=mx, mask_x_bd=mbd, mask_h=mh, mask_h_bd=mbd)
    scale = float(np.sqrt(I + H) * max(rms(Wx), rms(Wh)))  # size of the pre-activation terms

    # ---- forward: gates -> c -> h -------------------------------------------
    fx_t = dev.empty((B, 4 * H))
    dev.lstm_gates_forward(xs_t, dims, H, B, ht, Wxt, Wht, bt, fx_t, **mask_kw)
    fx_ref = orc.lstm_gates_forward(xs, dims, H, B, h, Wx, Wh, b, **o_mask)
    # an fp32 GEMM in another summation order moves the pre-activation by ~1e-7*scale;
    # the gate moves by at most that (|sigma'|, |tanh'| <= 1)
    assert_close(fx_t.numpy(), fx_ref, FWD_RTOL, "gates fwd", floor=max(1.0, scale))
    # ... and every gate, however small, is as close to the fp64 value as the CPU path is
    g64, _, _ = _lstm_exact_step(x, h, c_prev, Wx, Wh, b, mx, mh)
    _assert_gates_shadow(fx_t.numpy(), fx_ref, g64, H, "gates fwd")
    c_t, h_t = dev.empty((B, H)), dev.empty((B, H))
    fxo_t = dev.tensor(fx_ref)  # downstream nodes are compared from identical inputs
    dev.lstm_c_forward(H, B, ct, fxo_t, c_t)
    c_ref = orc.lstm_c_forward(H, B, c_prev, fx_ref)
    assert_close(c_t.numpy(), c_ref, FWD_RTOL, "c fwd", floor=1e-3)
    f64 = lambda a: a.astype(np.float64)
    c64 = f64(fx_ref[:, :H]) * f64(fx_ref[:, 3 * H:]) + f64(fx_ref[:, H:2 * H]) * f64(c_prev)
    assert_shadow(c_t.numpy(), c_ref, c64, "c fwd", rel_min=0.1)
    dev.lstm_h_forward(H, B, dev.tensor(c_ref), fxo_t, h_t)
    h_ref = orc.lstm_h_forward(H, B, c_ref, fx_ref)
    assert_close(h_t.numpy(), h_ref, FWD_RTOL, "h fwd", floor=1e-6)
    assert_shadow(h_t.numpy(), h_ref, f64(fx_ref[:, 2 * H:3 * H]) * np.tanh(f64(c_ref)), "h fwd", rel_min=1e-6)

    # ---- backward: h -> c -> gates, every argument, into non-zero buffers ----
    dh, dc_up = f32(rng.standard_normal((B, H))), f32(rng.standard_normal((B, H)))
    dht = dev.tensor(dh)
    cr_t = dev.tensor(c_ref)
    for i, shape in ((0, (B, H)), (1, (B, 4 * H))):
        g0 = f32(rng.standard_normal(shape))
        gt = dev.tensor(g0)
        dev.lstm_h_backward(H, B, cr_t, fxo_t, dht, i, gt)
        assert_close(gt.numpy(), orc.lstm_h_backward(H, B, c_ref, fx_ref, dh, i, g0.copy()), GRAD_RTOL, "h bwd %d" % i,
                     floor=np.maximum(np.abs(g0), 1e-4))
        gt = dev.tensor(g0)
        dev.lstm_c_backward(H, B, ct, fxo_t, dev.tensor(dc_up), i, gt)
        assert_close(gt.numpy(), orc.lstm_c_backward(H, B, c_prev, fx_ref, dc_up, i, g0.copy()), GRAD_RTOL,
                     "c bwd %d" % i, floor=np.maximum(np.abs(g0), 1e-4))
    dgates = f32(rng.standard_normal((B, 4 * H)))
    dgt = dev.tensor(dgates)
    dpre_t = dev.empty((B, 4 * H))
    dev.lstm_gates_dpre(H, B, fxo_t, dgt, dpre_t)
    k_in = len(dims)
    shapes = [(B, d) for d in dims] + [(B, H), (I, 4 * H), (H, 4 * H), (4 * H,)]
    floors = [np.sqrt(4 * H) * rms(Wx)] * k_in + [np.sqrt(4 * H) * rms(Wh), np.sqrt(B), np.sqrt(B), np.sqrt(B)]
    for i, shape in enumerate(shapes):
        g0 = f32(rng.standard_normal(shape))
        want = orc.lstm_gates_backward(xs, dims, H, B, h, Wx, Wh, fx_ref, dgates, i, g0.copy(), **o_mask)
        for cached in (False, True):
            gt = dev.tensor(g0)
            dev.lstm_gates_backward(xs_t, dims, H, B, ht, Wxt, Wht, fxo_t, dgt, i, gt,
                                    dpre=dpre_t if cached else None, **mask_kw)
            assert_close(gt.numpy(), want, GRAD_RTOL, "gates bwd arg %d cached=%s" % (i, cached),
                         floor=max(1.0, float(floors[i])))


def test_fused_nodes_equal_unfused_path_over_three_steps(dev):
    """tests/test-rnn.cc:155-184,214-243: gates/C/H equal affine -> logistic/tanh -> cmult."""
    rng = np.random.default_rng(9)
    I, H, B = 3, 5, 2
    x, h, c, Wx, Wh, b = _lstm_case(rng, I, H, B)
    b = f32(rng.standard_normal(4 * H) * 0.1)
    xt, Wxt, Wht, bt = dev.tensor(x), dev.tensor(Wx), dev.tensor(Wh), dev.tensor(b)
    ht, ct = dev.tensor(h), dev.tensor(c)
    h64, c64 = h.astype(np.float64), c.astype(np.float64)
    W64x, W64h = Wx.T.astype(np.float64), Wh.T.astype(np.float64)
    sig = lambda v: 1 / (1 + np.exp(-v))
    for _ in range(3):
        fx, c2, h2 = dev.empty((B, 4 * H)), dev.empty((B, H)), dev.empty((B, H))
        dev.lstm_gates_forward([xt], [I], H, B, ht, Wxt, Wht, bt, fx, logistic_mode=lib.LOGISTIC_SCALAR)
        dev.lstm_c_forward(H, B, ct, fx, c2)
        dev.lstm_h_forward(H, B, c2, fx, h2)
        tmp = x.astype(np.float64) @ W64x.T + h64 @ W64h.T + b
        i_t, f_t, o_t = sig(tmp[:, :H]), sig(tmp[:, H:2 * H] + 1), sig(tmp[:, 2 * H:3 * H])
        c64 = f_t * c64 + i_t * np.tanh(tmp[:, 3 * H:])
        h64 = o_t * np.tanh(c64)
        assert_close(h2.numpy(), h64, 1e-5, "fused vs unfused", floor=1e-3)
        ht, ct = h2, c2


@pytest.mark.parametrize("I,H,B", [(128, 256, 32), (24, 50, 7), (256, 1024, 128), (5, 3, 1)])
def test_fused_cell_path_equals_node_composition(dev, I, H, B):
    """dyhip_lstm_recurrent_* + dyhip_lstm_cell_* over two timesteps (the first from the zero state)
    against the oracle's VanillaLSTMGates -> C -> H nodes and their backward."""
    rng = np.random.default_rng(I + H + B)
    Wx, Wh, b = glorot(rng, 4 * H, I), glorot(rng, 4 * H, H), f32(rng.normal(0, 0.1, 4 * H))
    xs = [f32(rng.standard_normal((B, I))) for _ in range(2)]
    zeros = np.zeros((B, H), F32)
    # oracle: node by node
    ref = []
    h_prev, c_prev = zeros, zeros
    for x in xs:
        g = orc.lstm_gates_forward([x], [I], H, B, h_prev, Wx, Wh, b)
        c = orc.lstm_c_forward(H, B, c_prev, g)
        h = orc.lstm_h_forward(H, B, c, g)
        ref.append((g, c, h, h_prev, c_prev))
        h_prev, c_prev = h, c
    # device: xproj for both steps at once, then cell steps
    Wxt, Wht, bt = dev.tensor(Wx), dev.tensor(Wh), dev.tensor(b)
    X = dev.tensor(np.stack(xs))
    gates, cs, hs = dev.empty((2, B, 4 * H)), dev.empty((2, B, H)), dev.empty((2, B, H))
    fb, bb = dev.lstm_cell_workspace(H, B)
    wf, wfb = dev.workspace(fb)
    wb, wbb = dev.workspace(bb)
    dev.gemm_nn(4 * H, 2 * B, I, Wxt, X, 0.0, gates)
    sl = lambda t, k, w: t.offset(k * B * w, (B, w))
    dev.lstm_cell_forward(H, B, sl(gates, 0, 4 * H), bt, None, 0, None, sl(gates, 0, 4 * H), sl(cs, 0, H), sl(hs, 0, H))
    n = dev.lstm_recurrent_forward(H, B, Wht, sl(hs, 0, H), wf, wfb)
    assert n >= 1
    dev.lstm_cell_forward(H, B, sl(gates, 1, 4 * H), bt, wf, n, sl(cs, 0, H), sl(gates, 1, 4 * H), sl(cs, 1, H),
                          sl(hs, 1, H))
    # another summation order moves a pre-activation by ~1e-7 * (size of its terms); the gate, c and h
    # move by at most that (|sigma'|, |tanh'| <= 1)
    floor = max(1.0, float(np.sqrt(I + H) * max(rms(Wx), rms(Wh))))
    h64, c64 = zeros, zeros
    for k in range(2):
        assert_close(sl(gates, k, 4 * H).numpy(), ref[k][0], FWD_RTOL, f"gates[{k}]", floor=floor)
        assert_close(sl(cs, k, H).numpy(), ref[k][1], FWD_RTOL, f"c[{k}]", floor=floor)
        assert_close(sl(hs, k, H).numpy(), ref[k][2], FWD_RTOL, f"h[{k}]", floor=floor)
        g64, c64, h64 = _lstm_exact_step(xs[k], h64, c64, Wx, Wh, b)
        _assert_gates_shadow(sl(gates, k, 4 * H).numpy(), ref[k][0], g64, H, f"gates[{k}]")
        assert_shadow(sl(cs, k, H).numpy(), ref[k][1], c64, f"c[{k}]", rel_min=0.1)
        assert_shadow(sl(hs, k, H).numpy(), ref[k][2], h64, f"h[{k}]", rel_min=0.1)
    # backward: gradients arrive at h of both steps
    dh = [f32(rng.standard_normal((B, H))) for _ in range(2)]
    r_dh = [d.copy() for d in dh]
    r_dc = [np.zeros((B, H), F32) for _ in range(2)]
    r_dpre = [None, None]
    for k in (1, 0):
        g, c, h, hp, cp = ref[k]
        dg = np.zeros((B, 4 * H), F32)
        orc.lstm_h_backward(H, B, c, g, r_dh[k], 0, r_dc[k])
        orc.lstm_h_backward(H, B, c, g, r_dh[k], 1, dg)
        if k > 0:
            orc.lstm_c_backward(H, B, cp, g, r_dc[k], 0, r_dc[k - 1])
        orc.lstm_c_backward(H, B, cp, g, r_dc[k], 1, dg)
        r_dpre[k] = np.where(np.arange(4 * H) < 3 * H, dg * g * (F32(1) - g), dg * (F32(1) - g * g)).astype(F32)
        if k > 0:
            orc.lstm_gates_backward([xs[k]], [I], H, B, hp, Wx, Wh, g, dg, 1, r_dh[k - 1])
    dht = dev.tensor(np.stack(dh))
    dct, dpre = dev.empty((2, B, H)), dev.empty((2, B, 4 * H))
    dev.lstm_cell_backward(H, B, sl(gates, 1, 4 * H), sl(cs, 1, H), sl(cs, 0, H), sl(dht, 1, H), None, 0, None,
                           sl(dpre, 1, 4 * H), sl(dct, 0, H))
    n = dev.lstm_recurrent_backward(H, B, Wht, sl(dpre, 1, 4 * H), wb, wbb)
    dev.lstm_cell_backward(H, B, sl(gates, 0, 4 * H), sl(cs, 0, H), None, sl(dht, 0, H), wb, n, sl(dct, 0, H),
                           sl(dpre, 0, 4 * H), None)
    for k in range(2):
        assert_close(sl(dpre, k, 4 * H).numpy(), r_dpre[k], GRAD_RTOL, f"dpre[{k}]",
                     floor=max(float(np.abs(r_dpre[k]).max()) * 1e-2, 1e-6))


def lib_slices(dev, ws, n, size):
    """The n split slices of `size` floats a recurrent product left in the workspace `ws`."""
    from dynet_amd.device import DevTensor
    return DevTensor(dev, ws, (n, size), np.float32).numpy()


@pytest.mark.parametrize("I,H,B", [(24, 128, 1), (40, 128, 33), (16, 256, 32), (64, 384, 70), (32, 1024, 128)])
def test_single_launch_step_equals_node_composition(dev, I, H, B):
    """dyhip_lstm_step_forward (recurrent product + cell update in one kernel, packed Wh) over three
    timesteps against the oracle's VanillaLSTMGates -> C -> H nodes and against the two-call form."""
    rng = np.random.default_rng(7 * I + H + B)
    Wx, Wh, b = glorot(rng, 4 * H, I), glorot(rng, 4 * H, H), f32(rng.normal(0, 0.1, 4 * H))
    T = 3
    xs = [f32(rng.standard_normal((B, I))) for _ in range(T)]
    zeros = np.zeros((B, H), F32)
    ref = []
    h_prev, c_prev = zeros, zeros
    for x in xs:
        g = orc.lstm_gates_forward([x], [I], H, B, h_prev, Wx, Wh, b)
        c = orc.lstm_c_forward(H, B, c_prev, g)
        h = orc.lstm_h_forward(H, B, c, g)
        ref.append((g, c, h))
        h_prev, c_prev = h, c
    assert dev.lstm_step_supported(H, B)
    Wxt, Wht, bt = dev.tensor(Wx), dev.tensor(Wh), dev.tensor(b)
    packed = dev.empty(4 * H * H)
    dev.lstm_pack_recurrent(H, Wht, packed)
    # the packed copy is a permutation of Wh (stored [k][row]): tile rt, group kg, lane 32*lhi + g*8 + u, slot s
    # <- row g*H + rt*8 + u, k = 8*kg + 4*lhi + s
    want = Wh.reshape(H // 8, 2, 4, 4, H // 8, 8).transpose(4, 0, 1, 3, 5, 2).reshape(-1)
    assert np.array_equal(packed.numpy(), want)
    # and the packed state of h (stored [col][k]): tile ct, group kg, lane 32*lhi + l32, slot s, zero past B
    Bp = (B + 31) // 32 * 32
    assert dev.lstm_packed_state_floats(H, B) == H * Bp
    hv = f32(rng.standard_normal((B, H)))
    hp_t = dev.empty(H * Bp)
    dev.lstm_pack_state(H, B, dev.tensor(hv), hp_t)
    hpad = np.zeros((Bp, H), F32)
    hpad[:B] = hv
    pack_cols = lambda a, K: a.reshape(Bp // 32, 32, K // 8, 2, 4).transpose(0, 2, 3, 1, 4).reshape(-1)
    assert np.array_equal(hp_t.numpy(), pack_cols(hpad, H))
    X = dev.tensor(np.stack(xs))
    xproj = dev.empty((T, B, 4 * H))
    dev.gemm_nn(4 * H, T * B, I, Wxt, X, 0.0, xproj)
    sl = lambda t, k, w: t.offset(k * B * w, (B, w))
    fb, _ = dev.lstm_cell_workspace(H, B)
    wf, wfb = dev.workspace(fb)
    out = {}
    for name in ("step", "chain", "two_call"):
        gates, cs, hs = dev.empty((T, B, 4 * H)), dev.empty((T, B, H)), dev.empty((T, B, H))
        if name == "chain":  # every timestep one launch, the packed h handed from step to step
            hp = [dev.empty(H * Bp), dev.empty(H * Bp)]
            dev.lstm_step_forward_packed(H, B, None, None, sl(xproj, 0, 4 * H), bt, None, sl(gates, 0, 4 * H),
                                         sl(cs, 0, H), sl(hs, 0, H), hp[0])
            for t in range(1, T):
                dev.lstm_step_forward_packed(H, B, packed, hp[(t - 1) % 2], sl(xproj, t, 4 * H), bt, sl(cs, t - 1, H),
                                             sl(gates, t, 4 * H), sl(cs, t, H), sl(hs, t, H),
                                             hp[t % 2] if t + 1 < T else None)
            out[name] = (gates.numpy(), cs.numpy(), hs.numpy())
            continue
        dev.lstm_cell_forward(H, B, sl(xproj, 0, 4 * H), bt, None, 0, None, sl(gates, 0, 4 * H), sl(cs, 0, H),
                              sl(hs, 0, H))
        for t in range(1, T):
            if name == "step":
                dev.lstm_step_forward(H, B, packed, sl(hs, t - 1, H), sl(xproj, t, 4 * H), bt, sl(cs, t - 1, H),
                                      sl(gates, t, 4 * H), sl(cs, t, H), sl(hs, t, H))
            else:
                n = dev.lstm_recurrent_forward(H, B, Wht, sl(hs, t - 1, H), wf, wfb)
                dev.lstm_cell_forward(H, B, sl(xproj, t, 4 * H), bt, wf, n, sl(cs, t - 1, H), sl(gates, t, 4 * H),
                                      sl(cs, t, H), sl(hs, t, H))
        out[name] = (gates.numpy(), cs.numpy(), hs.numpy())
    floor = max(1.0, float(np.sqrt(I + H) * max(rms(Wx), rms(Wh))))
    h64, c64 = zeros, zeros
    for k in range(T):
        for q, what in enumerate(("gates", "c", "h")):
            assert_close(out["step"][q][k], ref[k][q], FWD_RTOL, f"{what}[{k}] vs oracle", floor=floor)
            assert_close(out["step"][q][k], out["two_call"][q][k], FWD_RTOL, f"{what}[{k}] vs two-call", floor=floor)
        exact = _lstm_exact_step(xs[k], h64, c64, Wx, Wh, b)
        _, c64, h64 = exact
        assert out["chain"][0][k].tobytes() == out["step"][0][k].tobytes()  # same kernel, same operands
        for name in ("step", "chain", "two_call"):
            _assert_gates_shadow(out[name][0][k], ref[k][0], exact[0], H, f"gates[{k}] {name}")
            assert_shadow(out[name][1][k], ref[k][1], exact[1], f"c[{k}] {name}", rel_min=0.1)
            assert_shadow(out[name][2][k], ref[k][2], exact[2], f"h[{k}] {name}", rel_min=0.1)


@pytest.mark.parametrize("H,B", [(128, 1), (128, 33), (256, 32), (384, 70), (1024, 128)])
def test_packed_backward_timestep_equals_the_two_call_form(dev, H, B):
    """dyhip_lstm_cell_backward_packed + dyhip_lstm_recurrent_backward_packed (packed Wh^T and dpre) against
    dyhip_lstm_cell_backward + dyhip_lstm_recurrent_backward and against fp64."""
    rng = np.random.default_rng(3 * H + B)
    Wh = glorot(rng, 4 * H, H)
    gates = f32(rng.uniform(0.05, 0.95, (B, 4 * H)))
    gates[:, 3 * H:] = f32(rng.uniform(-0.9, 0.9, (B, H)))
    c, c_tm1 = f32(rng.standard_normal((B, H))), f32(rng.standard_normal((B, H)))
    dh, dc = f32(rng.standard_normal((B, H))), f32(rng.standard_normal((B, H)))
    Wht = dev.tensor(Wh)
    packedT = dev.empty(4 * H * H)
    dev.lstm_pack_recurrent_transposed(H, Wht, packedT)
    # Wh is stored [j][r] (column j of the 4H x H matrix): tile rt of Wh^T, group kg, lane 32*lhi + l32, slot s
    # <- Wh[r = 8*kg + 4*lhi + s, j = rt*32 + l32]
    want = Wh.reshape(H // 32, 32, 4 * H // 8, 2, 4).transpose(0, 2, 3, 1, 4).reshape(-1)
    assert np.array_equal(packedT.numpy(), want)
    _, bb = dev.lstm_cell_workspace(H, B)
    ws, wsb = dev.workspace(bb)
    Bp = (B + 31) // 32 * 32
    gt, ct, cpt, dht, dct = (dev.tensor(a) for a in (gates, c, c_tm1, dh, dc))
    # plain form
    dpre0, dcp0 = dev.empty((B, 4 * H)), dev.empty((B, H))
    dev.lstm_cell_backward(H, B, gt, ct, cpt, dht, None, 0, dct, dpre0, dcp0)
    n0 = dev.lstm_recurrent_backward(H, B, Wht, dpre0, ws, wsb)
    rec0 = lib_slices(dev, ws, n0, H * B).sum(axis=0, dtype=np.float64)
    # packed form
    dpre1, dcp1 = dev.empty((B, 4 * H)), dev.empty((B, H))
    dpp = dev.empty(4 * H * Bp)
    dev.zero(dpp)
    dev.lstm_cell_backward_packed(H, B, gt, ct, cpt, dht, None, 0, dct, dpre1, dcp1, dpp)
    assert dpre1.numpy().tobytes() == dpre0.numpy().tobytes() and dcp1.numpy().tobytes() == dcp0.numpy().tobytes()
    pad = np.zeros((Bp, 4 * H), F32)
    pad[:B] = dpre1.numpy()
    assert np.array_equal(dpp.numpy(), pad.reshape(Bp // 32, 32, 4 * H // 8, 2, 4).transpose(0, 2, 3, 1, 4).reshape(-1))
    n1 = dev.lstm_recurrent_backward_packed(H, B, packedT, dpp, ws, wsb)
    rec1 = lib_slices(dev, ws, n1, H * B).sum(axis=0, dtype=np.float64)
    exact = dpre1.numpy().astype(np.float64) @ Wh.astype(np.float64).T  # (B, 4H) x (4H, H)
    floor = np.sqrt(4 * H) * rms(Wh) * rms(dpre1.numpy())
    assert_close(rec1.reshape(B, H), exact, FWD_RTOL, "packed Wh^T dpre vs fp64", floor=floor)
    assert_close(rec1.reshape(B, H), rec0.reshape(B, H), FWD_RTOL, "packed vs plain recurrent product", floor=floor)
    # the next timestep down consumes the slices exactly like the plain ones
    dpre2, dcp2 = dev.empty((B, 4 * H)), dev.empty((B, H))
    dev.lstm_cell_backward_packed(H, B, gt, ct, cpt, dht, ws, n1, dct, dpre2, dcp2, None)
    want_dh = dh.astype(np.float64) + rec1.reshape(B, H)
    t = np.tanh(c.astype(np.float64))
    dcv = dc + want_dh * gates[:, 2 * H:3 * H] * (1 - t * t)
    assert_close(dcp2.numpy(), dcv * gates[:, H:2 * H], GRAD_RTOL, "dc_tm1 after the packed product", floor=1.0)


@pytest.mark.parametrize("H,B", [(128, 1), (128, 33), (256, 32), (384, 70), (1024, 128)])
def test_single_launch_backward_timestep(dev, H, B):
    """dyhip_lstm_step_backward_packed over three timesteps (T-1: no recurrent term; T-2 and T-3: Wh^T * dpre of the
    step above from the fragment-order copy the launch above wrote) against the cell-backward + recurrent-product
    entry points on plain operands, the packed layouts against their definition, and the product against fp64."""
    rng = np.random.default_rng(5 * H + B)
    Wh = glorot(rng, 4 * H, H)
    Wht = dev.tensor(Wh)
    pT = dev.empty(4 * H * H)
    dev.lstm_pack_recurrent_transposed16(H, Wht, pT)
    # Wh is stored [unit j][depth k]: tile rt of Wh^T, group kg, lane 16*lq + l16, slot s <- Wh[k = 16kg + 4lq + s, j = 16rt + l16]
    want = Wh.reshape(H // 16, 16, 4 * H // 16, 4, 4).transpose(0, 2, 3, 1, 4).reshape(-1)
    assert np.array_equal(pT.numpy(), want)
    n16 = dev.lstm_packed_state16_floats(4 * H, B)
    Bp = (B + 31) // 32 * 32
    assert n16 == 4 * H * Bp
    _, bb = dev.lstm_cell_workspace(H, B)
    ws, wsb = dev.workspace(bb)
    steps = []
    for t in range(3):
        gates = f32(rng.uniform(0.05, 0.95, (B, 4 * H)))
        gates[:, 3 * H:] = f32(rng.uniform(-0.9, 0.9, (B, H)))
        steps.append(tuple(dev.tensor(a) for a in (gates, f32(rng.standard_normal((B, H))), f32(rng.standard_normal((B, H))),
                                                   f32(rng.standard_normal((B, H))))))
    dpp = [dev.empty(n16), dev.empty(n16)]
    for q in dpp:
        dev.zero(q)
    dc_new, dc_ref = None, None
    prev_packed, n_slices, dpre_ref_prev = None, 0, None
    for t, (gt, ct, cpt, dht) in enumerate(steps):
        dpre1, dcp1 = dev.empty((B, 4 * H)), dev.empty((B, H))
        dev.lstm_step_backward_packed(H, B, pT, prev_packed, gt, ct, cpt, dht, dc_new, dpre1, dcp1, dpp[t % 2])
        # reference: slices of Wh^T * dpre of the step above (plain operands), then the cell backward
        dpre0, dcp0 = dev.empty((B, 4 * H)), dev.empty((B, H))
        if dpre_ref_prev is not None:
            n_slices = dev.lstm_recurrent_backward(H, B, Wht, dpre_ref_prev, ws, wsb)
        dev.lstm_cell_backward(H, B, gt, ct, cpt, dht, ws if n_slices else None, n_slices, dc_ref, dpre0, dcp0)
        what = "H=%d B=%d step %d" % (H, B, t)
        if t == 0:  # no product: the same arithmetic on the same values
            assert dpre1.numpy().tobytes() == dpre0.numpy().tobytes() and dcp1.numpy().tobytes() == dcp0.numpy().tobytes(), what
        else:
            floor = max(1.0, float(np.sqrt(4 * H) * rms(Wh) * rms(dpre_ref_prev.numpy())))
            assert_close(dpre1.numpy(), dpre0.numpy(), GRAD_RTOL, "dpre " + what, floor=floor)
            assert_close(dcp1.numpy(), dcp0.numpy(), GRAD_RTOL, "dc_tm1 " + what, floor=floor)
            # the product inside the launch against fp64: recover it from dc_tm1 = (dc + (dh + rec) o (1 - tanh^2 c)) f
            g = gt.numpy().astype(np.float64)
            tc = np.tanh(ct.numpy().astype(np.float64))
            rec = dpre_ref_prev.numpy().astype(np.float64) @ Wh.astype(np.float64).T
            dcv = dc_ref.numpy() + (dht.numpy() + rec) * g[:, 2 * H:3 * H] * (1 - tc * tc)
            assert_close(dcp1.numpy(), dcv * g[:, H:2 * H], GRAD_RTOL, "dc_tm1 vs fp64 " + what, floor=floor)
        pad = np.zeros((Bp, 4 * H), F32)
        pad[:B] = dpre1.numpy()
        assert np.array_equal(dpp[t % 2].numpy(),
                              pad.reshape(Bp // 16, 16, 4 * H // 16, 4, 4).transpose(0, 2, 3, 1, 4).reshape(-1)), what
        prev_packed, dpre_ref_prev, dc_new, dc_ref = dpp[t % 2], dpre0, dcp1, dcp0
    # a dpre that did not come from a launch of the kernel
    other = dev.empty(n16)
    dev.lstm_pack_state16(4 * H, B, dpre_ref_prev, other)
    pad = np.zeros((Bp, 4 * H), F32)
    pad[:B] = dpre_ref_prev.numpy()
    assert np.array_equal(other.numpy(), pad.reshape(Bp // 16, 16, 4 * H // 16, 4, 4).transpose(0, 2, 3, 1, 4).reshape(-1))


@pytest.mark.parametrize("I,H,B", [(128, 256, 32), (256, 128, 1), (128, 128, 45), (384, 256, 70)])
def test_single_launch_step_with_input_product(dev, I, H, B):
    """dyhip_lstm_step_forward_x: Wx*x, Wh*h_tm1, bias, activations, c and h in one launch, from the zero state
    (no recurrent operand) and from a given state, against the oracle's gates -> C -> H nodes."""
    rng = np.random.default_rng(I + 3 * H + B)
    Wx, Wh, b = glorot(rng, 4 * H, I), glorot(rng, 4 * H, H), f32(rng.normal(0, 0.1, 4 * H))
    Wxt, Wht, bt = dev.tensor(Wx), dev.tensor(Wh), dev.tensor(b)
    pWx, pWh = dev.empty(4 * H * I), dev.empty(4 * H * H)
    dev.lstm_pack_input(I, H, Wxt, pWx)
    dev.lstm_pack_recurrent(H, Wht, pWh)
    assert np.array_equal(pWx.numpy(), Wx.reshape(I // 8, 2, 4, 4, H // 8, 8).transpose(4, 0, 1, 3, 5, 2).reshape(-1))
    zeros = np.zeros((B, H), F32)
    h_prev, c_prev = zeros, zeros
    ht = ct = None
    floor = max(1.0, float(np.sqrt(I + H) * max(rms(Wx), rms(Wh))))
    for t in range(3):
        x = f32(rng.standard_normal((B, I)))
        g_ref = orc.lstm_gates_forward([x], [I], H, B, h_prev, Wx, Wh, b)
        c_ref = orc.lstm_c_forward(H, B, c_prev, g_ref)
        h_ref = orc.lstm_h_forward(H, B, c_ref, g_ref)
        g64, c64, h64 = _lstm_exact_step(x, h_prev, c_prev, Wx, Wh, b)  # both sides start the step from h_ref, c_ref
        g2, c2, h2 = dev.empty((B, 4 * H)), dev.empty((B, H)), dev.empty((B, H))
        if t == 0:
            dev.lstm_step_forward_x(I, H, B, pWx, dev.tensor(x), None, None, bt, None, g2, c2, h2)
        else:
            dev.lstm_step_forward_x(I, H, B, pWx, dev.tensor(x), pWh, ht, bt, ct, g2, c2, h2)
        assert_close(g2.numpy(), g_ref, FWD_RTOL, f"gates[{t}]", floor=floor)
        assert_close(c2.numpy(), c_ref, FWD_RTOL, f"c[{t}]", floor=floor)
        assert_close(h2.numpy(), h_ref, FWD_RTOL, f"h[{t}]", floor=floor)
        if t > 0:
            ht.set(h_prev)   # the device step starts from the CPU path's state, as the fp64 yardstick does
            ct.set(c_prev)
            dev.lstm_step_forward_x(I, H, B, pWx, dev.tensor(x), pWh, ht, bt, ct, g2, c2, h2)
        _assert_gates_shadow(g2.numpy(), g_ref, g64, H, f"gates[{t}]")
        assert_shadow(c2.numpy(), c_ref, c64, f"c[{t}]", rel_min=0.1)
        assert_shadow(h2.numpy(), h_ref, h64, f"h[{t}]", rel_min=0.1)
        ht, ct, h_prev, c_prev = h2, c2, h_ref, c_ref
    with pytest.raises(DyhipError):
        dev.lstm_step_forward_x(96, H, B, pWx, ht, pWh, ht, bt, ct, g2, c2, h2)
    with pytest.raises(DyhipError):
        dev.lstm_step_forward_x(I, H, B, pWx, ht, pWh, None, bt, ct, g2, c2, h2)


def test_single_launch_step_rejects_unsupported_sizes(dev):
    assert not dev.lstm_step_supported(96, 4)
    assert not dev.lstm_step_supported(130, 4)
    t = dev.zeros(4 * 96 * 96)
    with pytest.raises(DyhipError) as e:
        dev.lstm_pack_recurrent(96, t, t)
    assert e.value.status == lib.ERR_INVALID_ARG
    with pytest.raises(DyhipError):
        dev.lstm_step_forward(96, 4, t, t, t, t, t, t, t, t)


def test_more_than_65535_batch_elements(dev):
    """The grid's second dimension holds 65535 blocks; kernels that put a batch element (or a block / sequence of
    the gpu-ops helpers) there stride over the rest, as the reference's launches do (dynet/cuda.h:82-103)."""
    rng = np.random.default_rng(70)
    B, H = 70000, 4
    c_prev, gates = f32(rng.standard_normal((B, H))), f32(rng.uniform(0.1, 0.9, (B, 4 * H)))
    ct, gt = dev.tensor(c_prev), dev.tensor(gates)
    c2, h2 = dev.empty((B, H)), dev.empty((B, H))
    dev.lstm_c_forward(H, B, ct, gt, c2)
    c_ref = orc.lstm_c_forward(H, B, c_prev, gates)
    assert_close(c2.numpy(), c_ref, FWD_RTOL, "c fwd", floor=1e-3)
    dev.lstm_h_forward(H, B, dev.tensor(c_ref), gt, h2)
    assert_close(h2.numpy(), orc.lstm_h_forward(H, B, c_ref, gates), FWD_RTOL, "h fwd", floor=1e-6)
    dg = f32(rng.standard_normal((B, 4 * H)))
    dpre = dev.empty((B, 4 * H))
    dev.lstm_gates_dpre(H, B, gt, dev.tensor(dg), dpre)
    want = np.where(np.arange(4 * H) < 3 * H, dg * gates * (F32(1) - gates), dg * (F32(1) - gates * gates)).astype(F32)
    assert_close(dpre.numpy(), want, GRAD_RTOL, "dpre", floor=1e-6)
    # mean_elems backward over 70000 batch elements
    d, dx0 = f32(rng.standard_normal(B)), f32(rng.standard_normal((B, 3)))
    dxt = dev.tensor(dx0)
    dev.mean_elems_backward(3, B, dev.tensor(d), dxt)
    assert_close(dxt.numpy(), orc.mean_elems_backward(3, B, d, dx0.copy()), GRAD_RTOL, "mean_elems bwd", floor=1e-3)
    # block gather / scatter helpers with 70000 blocks
    table = f32(rng.standard_normal((100, 5)))
    bidx = rng.integers(0, 100, B).astype(np.uint32)
    out = dev.empty((B, 5))
    dev.sparse_to_dense_block_assign_and_multiply(B, dev.tensor(bidx, np.uint32), 5, 2.0, dev.tensor(table), out)
    want = orc.sparse_to_dense_block_assign_and_multiply(bidx, 5, 2.0, table)
    assert out.numpy().tobytes() == want.tobytes()
    acc = dev.zeros((100, 5))
    dev.dense_to_sparse_block_add(B, dev.tensor(bidx, np.uint32), 5, dev.tensor(want), acc)
    assert_close(acc.numpy(), orc.dense_to_sparse_block_add(bidx, 5, want, np.zeros((100, 5), F32)), GRAD_RTOL,
                 "dense_to_sparse_block_add", floor=np.sqrt(B / 100) * 2)
    # ragged movers with 70000 sequences of 2 floats
    src = dev.tensor(f32(rng.standard_normal((B, 2))))
    dst = dev.zeros((B, 2))
    ptrs = dev.tensor(np.concatenate([src.ptr + 8 * np.arange(B, dtype=np.uint64), dst.ptr + 8 * np.arange(B, dtype=np.uint64)]),
                      np.uint64)
    lens = dev.tensor(np.full(B, 2, np.uint64), np.uint64)
    dev.parallel_memcpy(B, 2, ptrs.ptr, ptrs.ptr + 8 * B, lens)
    assert dst.numpy().tobytes() == src.numpy().tobytes()


def test_lstm_rejects_bad_arguments(dev):
    t = dev.zeros(64)
    with pytest.raises(DyhipError) as e:
        dev.lstm_gates_forward([t], [2], 2, 2, t, t, t, t, t, mask_x=t, mask_x_bd=3, mask_h=t, mask_h_bd=2)
    assert e.value.status == lib.ERR_INVALID_ARG and "dropout_mask_x" in str(e.value)
    with pytest.raises(DyhipError):
        dev.lstm_c_backward(2, 2, t, t, t, 2, t)


# ---------------------------------------------------------------------------
# LookupNode
# ---------------------------------------------------------------------------
@pytest.mark.parametrize("vocab,dim,n", [(50000, 512, 256 * 64), (10000, 256, 128), (7, 3, 40), (33, 130, 1000),
                                         (5, 4, 1),
                                         # id counts around powers of two, key widths from 9 to 18 bits, a vocabulary that is
                                         # a power of two
                                         (4096, 8, 2048), (4096, 8, 2049), (300, 4, 4097), (70000, 4, 8193),
                                         (1 << 16, 4, 16383), (200000, 4, 16385), (1000, 16, 40000),
                                         # long runs (split by columns) at every thread-group shape: rows of 1..3
                                         # vector elements, non-vector rows, rows wider than a thread group
                                         (50, 4, 3000), (50, 12, 3000), (50, 3, 3000), (40, 130, 5000), (40, 2052, 900),
                                         (30, 1028, 2000), (3, 64, 700), (5000, 256, 4480)])
def test_lookup_gather_bit_exact_and_scatter_add(dev, vocab, dim, n):
    rng = np.random.default_rng(vocab + dim + n)
    table = f32(rng.uniform(-0.1, 0.1, (vocab, dim)))
    ids = zipf_ids(rng, n, vocab)
    tt = dev.tensor(table, pool=lib.POOL_FXS)
    ids_t = dev.empty(n, np.uint32)
    fx = dev.empty((n, dim))
    dev.lookup_forward(ids, ids_t, dim, vocab, tt, fx)
    assert fx.numpy().tobytes() == table[ids].tobytes()  # bit-exact gather
    assert ids_t.numpy().tobytes() == ids.tobytes()
    dev.lookup_forward(None, ids_t, dim, vocab, tt, fx, mult=0.5)  # ids already on the device
    assert fx.numpy().tobytes() == orc.lookup_forward(ids, dim, vocab, table, 0.5).tobytes()
    # scatter-add into a non-zero gradient table
    g = f32(rng.standard_normal((n, dim)))
    grads0 = f32(rng.standard_normal((vocab, dim)))
    gt = dev.tensor(grads0)
    dev.lookup_accumulate_grads(ids_t, dim, vocab, dev.tensor(g), gt)
    got = gt.numpy()
    want = orc.lookup_accumulate_grads(ids, dim, vocab, g, grads0.copy())  # sequential fp32, the CPU path
    counts = np.bincount(ids, minlength=vocab).astype(np.float64)
    floor = np.sqrt(np.maximum(counts, 1.0))[:, None] * np.ones((1, dim))
    assert_close(got, want, GRAD_RTOL, "lookup scatter-add", floor=floor)
    untouched = counts == 0
    assert got[untouched].tobytes() == grads0[untouched].tobytes()
    # as close to the fp64 sum as the sequential fp32 path is (both are chains of fp32 adds whose worst element
    # over the table is a random-walk maximum: a factor of 8 between two such maxima is noise, 100 is a bug)
    exact = grads0.astype(np.float64)
    np.add.at(exact, ids, g.astype(np.float64))
    assert np.max(np.abs(got - exact)) <= max(8 * np.max(np.abs(want - exact)), 1e-5)
    # deterministic: the same call gives the same bits
    gt2 = dev.tensor(grads0)
    dev.lookup_accumulate_grads(ids_t, dim, vocab, dev.tensor(g), gt2)
    assert gt2.numpy().tobytes() == got.tobytes()
    # two-phase form: plan built once (e.g. at forward time), reduction kernel at backward time
    plan = dev.lookup_build_plan(ids_t, vocab)
    _check_plan(dev, plan, ids, vocab)
    gt3 = dev.tensor(grads0)
    dev.lookup_accumulate_grads_planned(n, plan, dim, vocab, dev.tensor(g), gt3)
    assert gt3.numpy().tobytes() == got.tobytes()
    # rows that fewer than 15 ids name are summed in the CPU path's order: the same bits
    short = (counts > 0) & (counts < 15)
    assert got[short].tobytes() == want[short].tobytes()


def _check_plan(dev, plan, ids, vocab):
    """A plan is a grouping of the ids: a permutation of the positions, equal ids consecutive, positions
    ascending inside a run, and run offsets that say where each run starts and ends."""
    n = ids.size
    gid, gpos, roff, rrem = dev.lookup_plan_parts(plan.numpy(), n)
    assert np.array_equal(np.sort(gpos), np.arange(n))
    clamped = np.minimum(ids, vocab)
    assert np.array_equal(gid, clamped[gpos])
    heads = np.flatnonzero(np.concatenate([[True], gid[1:] != gid[:-1]]))
    assert heads.size == np.unique(clamped).size           # every id is one run
    ends = np.concatenate([heads[1:], [n]])
    k = np.arange(n)
    run = np.searchsorted(heads, k, side="right") - 1
    assert np.array_equal(roff, k - heads[run]) and np.array_equal(rrem, ends[run] - k)
    inside = roff > 0
    assert np.all(gpos[inside] > gpos[np.flatnonzero(inside) - 1])  # stable: the CPU path's order inside a run
    assert dev.lookup_plan_invalid_ids(n, plan) == int((ids >= vocab).sum())


@pytest.mark.parametrize("vocab,n,kind", [
    (50000, 65535, "zipf"),        # the largest id vector of the one-kernel plan
    (50000, 4480, "zipf"),         # 16-bit keys, 5 steps of 64 ids per wavefront: the 8-step form of the direct kernel
    (50000, 32768, "zipf"),        # ... 32 steps: the longest the direct kernel takes
    (50000, 32769, "zipf"),        # ... 33: the compact-and-sort kernel although the keys fit 16 bits
    (50000, 65536, "zipf"),        # the first size of the radix-sort plan (two passes)
    (300000, 70001, "zipf"),       # ... three passes
    (200, 70000, "uniform"),       # ... one pass
    (1 << 30, 66000, "uniform"),   # ... four
    (50000, 600000, "zipf"),       # ... pieces of more than 2048 ids a block
    (1000, 70000, "same"),         # ... every id beyond the vocabulary: one run that the reduction skips
    (70000, 100000, "same"),       # ... one id only
    (1 << 20, 30000, "uniform"),   # 21-bit ids: two sort passes beyond the bucket digit
    (1 << 30, 5000, "uniform"),    # 31-bit ids: three
    (256, 20000, "uniform"),       # vocab fits the bucket digit plus the sentinel's extra bit
    (200, 3000, "uniform"),        # ... and without it: no sort pass at all
    (1000, 40000, "one_bucket"),   # every id = 7 mod 256: a bucket too large for LDS takes the global-memory route
    (50000, 60000, "same"),        # one id only
    (97, 1, "uniform"), (97, 17, "uniform"),
])
def test_lookup_plan_is_a_stable_grouping(dev, vocab, n, kind):
    rng = np.random.default_rng(vocab % 1000 + n)
    if kind == "zipf":
        ids = zipf_ids(rng, n, vocab)
    elif kind == "uniform":
        ids = rng.integers(0, vocab, n).astype(np.uint32)
    elif kind == "one_bucket":
        ids = (7 + 256 * rng.integers(0, (vocab - 7) // 256, n)).astype(np.uint32)
    else:
        ids = np.full(n, 12345, np.uint32)
    for misalign in (0, 1):  # 128-bit id loads need alignment; a view one element in takes the scalar route
        base = dev.empty(n + 1, np.uint32)
        ids_t = base.offset(misalign, (n,))
        ids_t.set(ids)
        plan = dev.lookup_build_plan(ids_t, vocab)
        _check_plan(dev, plan, ids, vocab)


def test_lookup_ids_beyond_the_vocabulary_are_skipped_and_counted(dev):
    """Device-resident ids are not validated by the reference's GPU path; here an id >= vocab never aliases onto a
    valid row: it is left out of the sum and counted."""
    rng = np.random.default_rng(77)
    vocab, dim, n = 1000, 24, 5000
    ids = zipf_ids(rng, n, vocab)
    bad = rng.choice(n, 40, replace=False)
    ids[bad] = rng.choice([vocab, vocab + 1, 1 << 16, (1 << 16) + 5, 0xFFFFFFFF, 0x80000000 + 3], 40).astype(np.uint32)
    g = f32(rng.standard_normal((n, dim)))
    ids_t = dev.tensor(ids, np.uint32)
    plan = dev.lookup_build_plan(ids_t, vocab)
    _check_plan(dev, plan, ids, vocab)
    gt = dev.zeros((vocab, dim))
    dev.lookup_accumulate_grads_planned(n, plan, dim, vocab, dev.tensor(g), gt)
    ok = ids < vocab
    want = orc.lookup_accumulate_grads(ids[ok], dim, vocab, np.ascontiguousarray(g[ok]), np.zeros((vocab, dim), F32))
    counts = np.bincount(ids[ok], minlength=vocab)
    assert_close(gt.numpy(), want, GRAD_RTOL, "scatter-add with invalid ids", floor=np.sqrt(np.maximum(counts, 1))[:, None]
                 * np.ones((1, dim)))


def test_lookup_all_ids_equal_and_all_distinct(dev):
    rng = np.random.default_rng(3)
    vocab, dim = 64, 32
    for ids in (np.full(1000, 5, np.uint32), rng.permutation(vocab).astype(np.uint32)):
        g = f32(rng.standard_normal((ids.size, dim)))
        gt = dev.zeros((vocab, dim))
        dev.lookup_accumulate_grads(dev.tensor(ids, np.uint32), dim, vocab, dev.tensor(g), gt)
        want = orc.lookup_accumulate_grads(ids, dim, vocab, g, np.zeros((vocab, dim), F32))
        assert_close(gt.numpy(), want, GRAD_RTOL, "lookup edge", floor=np.sqrt(ids.size))


def test_lookup_out_of_range_index_is_an_error(dev):
    t = dev.zeros((4, 4))
    with pytest.raises(DyhipError) as e:
        dev.lookup_forward(np.array([0, 4], np.uint32), dev.empty(2, np.uint32), 4, 4, t, dev.empty((2, 4)))
    assert e.value.status == lib.ERR_INVALID_ARG and "Out-of-bounds" in str(e.value)


# ---------------------------------------------------------------------------
# logsumexp / PickNegLogSoftmax / LogSumExp / argmax
# ---------------------------------------------------------------------------
@pytest.mark.parametrize("rows,bd", [(50000, 512), (10000, 128), (37, 5), (1027, 3), (1, 4), (4, 1),
                                     # short columns: a thread per column up to 64 rows, a wavefront per column up to
                                     # 512 (1, 2, 4 or 8 loads a lane), then a block per column whose ends are peeled
                                     # off around 128-bit groups whatever the column's offset
                                     (33, 1000), (64, 300), (65, 7), (128, 9), (200, 70), (256, 5), (511, 6),
                                     (512, 3), (513, 3), (2050, 2), (50001, 16)])
def test_pnls_forward_backward(dev, rows, bd):
    rng = np.random.default_rng(rows + bd)
    x = f32(rng.standard_normal((bd, rows)) * 2.0)
    labels = rng.integers(0, rows, bd).astype(np.uint32)
    xt = dev.tensor(x)
    aux = dev.empty(3 * bd)
    fx = dev.empty(bd)
    dev.pnls_forward(rows, bd, xt, labels, aux, fx)
    ref_fx, ref_aux = orc.pnls_forward(rows, bd, x, labels)
    a = aux.numpy()
    assert a.view(np.uint32)[2 * bd:].tobytes() == ref_aux.view(np.uint32)[2 * bd:].tobytes()  # picks: bit exact
    assert a[bd:2 * bd].tobytes() == ref_aux[bd:2 * bd].tobytes()  # row maxima: bit exact
    assert_close(a[:bd], ref_aux[:bd], FWD_RTOL, "logsumexp z")
    assert_close(fx.numpy(), ref_fx, FWD_RTOL, "pnls fwd", floor=1.0)
    m_t, z_t = dev.empty(bd), dev.empty(bd)
    dev.logsumexp_cols(rows, bd, xt, m_t, z_t)
    assert z_t.numpy().tobytes() == a[:bd].tobytes()
    # backward from the oracle's aux so that both sides see identical z
    dy = f32(rng.standard_normal(bd))
    dx0 = f32(rng.standard_normal((bd, rows)) * 0.01)
    dxt = dev.tensor(dx0)
    dev.pnls_backward(rows, bd, xt, dev.tensor(ref_aux), dev.tensor(dy), dxt)
    want = orc.pnls_backward(rows, bd, x, ref_aux, dy, dx0.copy())
    assert_close(dxt.numpy(), want, GRAD_RTOL, "pnls bwd", floor=np.maximum(np.abs(dx0), 1e-7))
    # sum_v (softmax - onehot) == 0 per row
    delta = (dxt.numpy().astype(np.float64) - dx0).sum(1)
    assert np.max(np.abs(delta)) < 1e-4 * max(1.0, np.max(np.abs(dy)))
    # the gradient itself, without a buffer that hides its small terms: accumulate into zeros and the
    # overwriting form, each against the oracle element by element.  Every softmax term exp(x - z) * dy is
    # held to 1e-4 relative down to p = 1e-7 (the floor |dy| * 1e-7); the picked element is p*dy - dy.
    want0 = orc.pnls_backward(rows, bd, x, ref_aux, dy, np.zeros((bd, rows), F32))
    floor0 = np.abs(dy)[:, None] * 1e-7 * np.ones((1, rows))
    floor0[np.arange(bd), labels] = np.abs(dy)
    dxz = dev.zeros((bd, rows))
    dev.pnls_backward(rows, bd, xt, dev.tensor(ref_aux), dev.tensor(dy), dxz)
    assert_close(dxz.numpy(), want0, GRAD_RTOL, "pnls bwd into zeros", floor=floor0)
    # the overwriting form: the same, whatever the buffer held before
    dxa = dev.empty((bd, rows))
    dev.pnls_backward(rows, bd, xt, dev.tensor(ref_aux), dev.tensor(dy), dxa, assign=True)
    assert_close(dxa.numpy(), want0, GRAD_RTOL, "pnls bwd assign", floor=floor0)
    assert dxa.numpy().tobytes() == dxz.numpy().tobytes()


@pytest.mark.parametrize("rows", [64, 4099, 13])
def test_logsumexp_with_minus_infinity_entries(dev, rows):
    """Masked logits: -inf entries contribute exp(-inf - m) = 0, as in the reference's max-first form
    (dynet/tensor.cc:468-507), wherever they sit: the first 128-bit group of a thread, the scalar tail of a
    row count that is not a multiple of four, whole wavefronts.  A column of nothing but -inf gives NaN there
    (exp(-inf + inf)) and here."""
    rng = np.random.default_rng(rows)
    bd = 7
    x = f32(rng.standard_normal((bd, rows)) * 2.0)
    x[0, :4] = -np.inf                      # a thread's first float4
    x[1, :min(rows, 4096)] = -np.inf        # every thread's first group (all of the column when rows <= 4096)
    x[1, -1] = 0.5
    x[2, ::2] = -np.inf
    x[3, 1:] = -np.inf                      # a single finite entry
    x[4, :] = -np.inf                       # nothing finite at all
    x[5, -3:] = -np.inf                     # the scalar tail
    labels = rng.integers(0, rows, bd).astype(np.uint32)
    labels[3] = 0
    xt = dev.tensor(x)
    m_t, z_t = dev.empty(bd), dev.empty(bd)
    dev.logsumexp_cols(rows, bd, xt, m_t, z_t)
    aux, fx = dev.empty(3 * bd), dev.empty(bd)
    dev.pnls_forward(rows, bd, xt, labels, aux, fx)
    ref_fx, ref_aux = orc.pnls_forward(rows, bd, x, labels)
    ref_z, ref_m = ref_aux[:bd], ref_aux[bd:2 * bd]
    assert np.isnan(ref_z[4]) and np.isnan(z_t.numpy()[4]) and np.isnan(fx.numpy()[4])
    ok = np.arange(bd) != 4
    assert m_t.numpy().tobytes() == ref_m.tobytes()
    assert_close(z_t.numpy()[ok], ref_z[ok], FWD_RTOL, "logsumexp with -inf", floor=1e-3)
    fin = ok & np.isfinite(ref_fx)
    assert np.array_equal(np.isfinite(fx.numpy()[ok]), np.isfinite(ref_fx[ok]))
    assert_close(fx.numpy()[fin], ref_fx[fin], FWD_RTOL, "pnls fwd with -inf", floor=1.0)
    keep = np.array([0, 1, 2, 3, 5, 6])
    xs = np.ascontiguousarray(x[keep])
    sm = dev.empty((keep.size, rows))
    dev.softmax_forward(rows, keep.size, dev.tensor(xs), sm)
    assert_close(sm.numpy(), orc.softmax_forward(rows, keep.size, xs), FWD_RTOL, "softmax with -inf", floor=1e-30)


def test_logsumexp_shift_invariance_and_no_overflow(dev):
    rng = np.random.default_rng(8)
    rows, bd = 4096, 16
    x = f32(rng.standard_normal((bd, rows)))
    m, z, z2 = dev.empty(bd), dev.empty(bd), dev.empty(bd)
    dev.logsumexp_cols(rows, bd, dev.tensor(x), m, z)
    dev.logsumexp_cols(rows, bd, dev.tensor(x + F32(64.0)), m, z2)
    assert np.max(np.abs(z2.numpy() - z.numpy() - 64.0)) < 1e-4
    big = np.full((1, 8), -1000.0, F32)
    big[0, :2] = 1000.0
    dev.logsumexp_cols(8, 1, dev.tensor(big), m, z)
    assert abs(float(z.numpy()[0]) - (1000.0 + np.log(2.0))) < 1e-3


def test_pnls_label_out_of_range_is_an_error(dev):
    with pytest.raises(DyhipError) as e:
        dev.pnls_forward(4, 2, dev.zeros((2, 4)), np.array([0, 4], np.uint32), dev.empty(6), dev.empty(2))
    assert e.value.status == lib.ERR_INVALID_ARG and "Index error in PickNegLogSoftmax" in str(e.value)


@pytest.mark.parametrize("rows,cols", [(10000, 128), (37, 5), (1027, 3), (1, 4), (4, 1), (50000, 64), (33, 700), (130, 9),
                                       (300, 40), (513, 3), (100, 6), (3000, 5), (5000, 3), (16384, 2), (16385, 2), (40001, 3), (20001, 20)])
def test_softmax_and_log_softmax(dev, rows, cols):
    rng = np.random.default_rng(rows + cols)
    x = f32(rng.standard_normal((cols, rows)) * 2)
    dy = f32(rng.standard_normal((cols, rows)))
    g0 = f32(rng.standard_normal((cols, rows)))
    xt, dyt = dev.tensor(x), dev.tensor(dy)
    # softmax
    ref = orc.softmax_forward(rows, cols, x)
    fx = dev.empty((cols, rows))
    dev.softmax_forward(rows, cols, xt, fx)
    assert_close(fx.numpy(), ref, FWD_RTOL, "softmax fwd", floor=1e-30)
    dx = dev.tensor(g0)
    dev.softmax_backward(rows, cols, dev.tensor(ref), dyt, dx)
    want = orc.softmax_backward(rows, cols, ref, dy, g0.copy())
    assert_close(dx.numpy(), want, GRAD_RTOL, "softmax bwd", floor=np.maximum(np.abs(g0), 1e-4))
    # log-softmax
    ref, aux_ref = orc.log_softmax_forward(rows, cols, x)
    aux = dev.empty(2 * cols)
    dev.log_softmax_forward(rows, cols, xt, aux, fx)
    # x - z: an error of 1e-5 relative in z moves every element by 1e-5 * |z|
    assert_close(fx.numpy(), ref, FWD_RTOL, "log_softmax fwd", floor=float(np.abs(aux_ref[:cols]).max()) + 1.0)
    assert_close(aux.numpy(), aux_ref, FWD_RTOL, "log_softmax aux")
    dx = dev.tensor(g0)
    dev.log_softmax_backward(rows, cols, dev.tensor(ref), dyt, aux, dx)
    want = orc.log_softmax_backward(rows, cols, ref, dy, g0.copy())
    scale = np.abs(dy).sum(axis=1, keepdims=True) * np.exp(ref) + np.abs(dy) + np.abs(g0)
    assert_close(dx.numpy(), want, GRAD_RTOL, "log_softmax bwd", floor=np.maximum(scale, 1e-4))


def test_logsumexp_node(dev):
    rng = np.random.default_rng(15)
    n, bd = 600, 4
    a, b, c1 = f32(rng.standard_normal((bd, n))), f32(rng.standard_normal((bd, n))), f32(rng.standard_normal((1, n)))
    ts = [dev.tensor(v) for v in (a, b, c1)]
    bds = [bd, bd, 1]
    fx = dev.empty((bd, n))
    dev.logsumexp_node_forward(n, bd, ts, bds, fx)
    ref = orc.logsumexp_node_forward(n, bd, [a, b, c1], bds)
    assert_close(fx.numpy(), ref, FWD_RTOL, "LogSumExp fwd", floor=1e-2)
    dy = f32(rng.standard_normal((bd, n)))
    for i, shape in ((0, (bd, n)), (2, (1, n))):
        g0 = f32(rng.standard_normal(shape))
        gt = dev.tensor(g0)
        dev.logsumexp_node_backward(n, bd, ts, bds, dev.tensor(ref), dev.tensor(dy), i, gt)
        want = orc.logsumexp_node_backward(n, bd, [a, b, c1], bds, ref, dy, i, g0.copy())
        assert_close(gt.numpy(), want, GRAD_RTOL, "LogSumExp bwd %d" % i, floor=1e-2)


@pytest.mark.parametrize("k,n,bd", [(9, 300, 4), (32, 50, 3), (33, 50, 3), (35, 1, 128), (100, 7, 2), (64, 1, 1)])
def test_logsumexp_node_many_arguments(dev, k, n, bd):
    """More arguments than one launch takes (32): chained through the output.  Mixed batch sizes, a few -inf entries,
    every argument's gradient."""
    rng = np.random.default_rng(k + n + bd)
    bds = [bd if (i % 3 != 1 or bd == 1) else 1 for i in range(k)]
    xs = [f32(rng.standard_normal((b, n)) * 3) for b in bds]
    xs[0][0, 0] = -np.inf
    ts = [dev.tensor(v) for v in xs]
    fx = dev.empty((bd, n))
    dev.logsumexp_node_forward(n, bd, ts, bds, fx)
    ref = orc.logsumexp_node_forward(n, bd, xs, bds)
    assert_close(fx.numpy(), ref, FWD_RTOL, "LogSumExp fwd", floor=1.0)
    exact = np.log(sum(np.exp(np.broadcast_to(v, (bd, n)).astype(np.float64)) for v in xs))
    assert_close(fx.numpy(), exact, FWD_RTOL, "LogSumExp fwd vs fp64", floor=1.0)
    dy = f32(rng.standard_normal((bd, n)))
    for i in (0, 1, k - 1):
        g0 = f32(rng.standard_normal((bds[i], n)))
        gt = dev.tensor(g0)
        dev.logsumexp_node_backward(n, bd, ts, bds, dev.tensor(ref), dev.tensor(dy), i, gt)
        want = orc.logsumexp_node_backward(n, bd, xs, bds, ref, dy, i, g0.copy())
        assert_close(gt.numpy(), want, GRAD_RTOL, "LogSumExp bwd %d" % i, floor=1e-2 * np.sqrt(bd))
    # every argument -inf in one entry: NaN there, as the reference's exp(-inf + inf)
    for v in xs:
        v[-1, -1] = -np.inf
    dev.logsumexp_node_forward(n, bd, [dev.tensor(v) for v in xs], bds, fx)
    got = fx.numpy()
    assert np.isnan(got[-1, -1]) and np.isfinite(got.ravel()[:-1]).all()


def test_argmax(dev, golden):
    t = golden["node_values"]["argmax"]
    idx = dev.empty(t["bd"], np.int64)
    dev.argmax_cols(t["rows"], t["bd"], dev.tensor(f32(t["x"])), idx)
    assert list(idx.numpy()) == t["expected"]
    rng = np.random.default_rng(4)
    x = f32(rng.integers(0, 50, (9, 5000)))  # many ties: first maximum wins
    idx = dev.empty(9, np.int64)
    dev.argmax_cols(5000, 9, dev.tensor(x), idx)
    assert idx.numpy().tobytes() == orc.argmax_cols(5000, 9, x).tobytes()


@pytest.mark.parametrize("rows,bd", [(1, 7), (4, 100001), (32, 1000), (33, 999), (64, 5), (2048, 33), (2049, 3), (8192, 4),
                                     (8193, 2), (50000, 9), (100003, 1)])
def test_argmax_shapes_with_ties(dev, rows, bd):
    """A thread, a wavefront or a block (256 / 1024 threads) per column, on both sides of each limit; small integer
    values, so that every column holds its maximum many times: the first one wins, as in the oracle."""
    rng = np.random.default_rng(rows + bd)
    x = f32(rng.integers(0, 7, (bd, rows)))
    idx = dev.empty(bd, np.int64)
    dev.argmax_cols(rows, bd, dev.tensor(x), idx)
    assert idx.numpy().tobytes() == orc.argmax_cols(rows, bd, x).tobytes()
    x = f32(rng.standard_normal((bd, rows)))
    dev.argmax_cols(rows, bd, dev.tensor(x), idx)
    assert np.array_equal(idx.numpy(), x.argmax(axis=1))


@pytest.mark.parametrize("rows,bd", [(65536, 2), (70001, 1), (131072, 3), (300001, 2)])
def test_vocabulary_length_columns_of_a_small_batch(dev, rows, bd):
    """Columns of 65 536 rows and more in a batch of a few are cut into chunks over many blocks (log-sum-exp, the dot
    of the softmax backward, argmax).  The oracle's sequential fp32 sums drift at this length, so the references are
    the same formulas in fp64 (dynet/tensor.cc:468-507, nodes-pickneglogsoftmax.cc:72-145, nodes-softmaxes.cc:40-213,
    nodes-argmax.cc:44-55); maxima, picks and argmax are exact."""
    rng = np.random.default_rng(rows + bd)
    x = f32(rng.standard_normal((bd, rows)) * 3)
    x[0, : rows // 3] = -np.inf  # masked logits
    x64 = x.astype(np.float64)
    mx = x.max(axis=1)
    lse = np.log(np.exp(x64 - mx[:, None].astype(np.float64)).sum(axis=1)) + mx
    xt = dev.tensor(x)
    m, z = dev.empty(bd), dev.empty(bd)
    dev.logsumexp_cols(rows, bd, xt, m, z)
    assert m.numpy().tobytes() == mx.tobytes()
    assert_close(z.numpy(), lse, FWD_RTOL, "logsumexp", floor=1.0)
    labels = rng.integers(rows // 3, rows, bd).astype(np.uint32)
    aux, fx = dev.empty(3 * bd), dev.empty(bd)
    dev.pnls_forward(rows, bd, xt, labels, aux, fx)
    assert_close(fx.numpy(), lse - x64[np.arange(bd), labels], FWD_RTOL, "pnls", floor=1.0)
    sm = np.exp(x64 - lse[:, None])
    y = dev.empty((bd, rows))
    dev.softmax_forward(rows, bd, xt, y)
    assert_close(y.numpy(), sm, FWD_RTOL, "softmax", floor=1.0 / rows)
    dy, g0 = f32(rng.standard_normal((bd, rows))), f32(rng.standard_normal((bd, rows)))
    gt = dev.tensor(g0)
    dev.softmax_backward(rows, bd, dev.tensor(f32(sm)), dev.tensor(dy), gt)
    smf = f32(sm).astype(np.float64)
    want = g0 + (dy - (smf * dy).sum(axis=1, keepdims=True)) * smf
    assert_close(gt.numpy(), want, GRAD_RTOL, "softmax bwd", floor=1.0)
    aux2 = dev.empty(2 * bd)
    dev.log_softmax_forward(rows, bd, xt, aux2, y)
    got = y.numpy()
    fin = np.isfinite(x)
    assert np.array_equal(np.isneginf(got), ~fin)
    assert_close(np.where(fin, got, 0.0), np.where(fin, x64 - lse[:, None], 0.0), FWD_RTOL, "log_softmax", floor=1.0)
    lsm = f32(np.where(fin, x64 - lse[:, None], -50.0))
    gt = dev.tensor(g0)
    dev.log_softmax_backward(rows, bd, dev.tensor(lsm), dev.tensor(dy), aux2, gt)
    want = g0 + dy - np.exp(lsm.astype(np.float64)) * dy.astype(np.float64).sum(axis=1, keepdims=True)
    assert_close(gt.numpy(), want, GRAD_RTOL, "log_softmax bwd", floor=np.sqrt(rows))
    idx = dev.empty(bd, np.int64)
    xi = f32(rng.integers(0, 9, (bd, rows)))  # every column holds its maximum thousands of times: the first wins
    dev.argmax_cols(rows, bd, dev.tensor(xi), idx)
    assert np.array_equal(idx.numpy(), xi.argmax(axis=1))
    dev.argmax_cols(rows, bd, xt, idx)
    assert np.array_equal(idx.numpy(), x.argmax(axis=1))


def test_argmax_node(dev, golden):
    """The Argmax node (dynet/nodes-argmax.cc:44-68): one-hot forward with the reference test's vector, bit-exact against
    the oracle on a larger case with ties, straight-through backward = accumulate."""
    t = golden["node_values"]["argmax_node"]
    idx, fx = dev.empty(t["bd"], np.int64), dev.empty((t["bd"], t["rows"]))
    dev.argmax_onehot_forward(t["rows"], t["bd"], dev.tensor(f32(t["x"])), idx, fx)
    assert list(fx.numpy().ravel()) == t["expected"]
    dx = dev.zeros((t["bd"], t["rows"]), pool=lib.POOL_DEDFS)
    dev.accumulate(dev.tensor(f32(t["x"])), dx)        # straight-through: dEdxi += dEdf, with dEdf = x_ = batch_vals
    assert list(dx.numpy().ravel()) == list(f32(t["straight_through_dx"]))
    rng = np.random.default_rng(13)
    x = f32(np.round(rng.standard_normal((300, 1001)) * 2))  # many ties: the first maximum wins
    idx, fx = dev.empty(300, np.int64), dev.empty((300, 1001))
    dev.argmax_onehot_forward(1001, 300, dev.tensor(x), idx, fx)
    want_idx, want_fx = orc.argmax_onehot_forward(1001, 300, x)
    assert idx.numpy().tobytes() == want_idx.tobytes() and fx.numpy().tobytes() == want_fx.tobytes()


# ---------------------------------------------------------------------------
# dynet::gpu helpers, parameter copy, trainer
# ---------------------------------------------------------------------------
def test_gpu_ops_helpers(dev):
    rng = np.random.default_rng(16)
    n, size = 1000, 5000
    src = f32(rng.standard_normal(size))
    idx = rng.permutation(size)[:n].astype(np.uint32)  # distinct targets
    it = dev.tensor(idx, np.uint32)
    out = dev.empty(n)
    dev.sparse_to_dense_assign(n, it, dev.tensor(src), out)
    assert out.numpy().tobytes() == orc.sparse_to_dense_assign(idx, src).tobytes()
    trg = dev.zeros(size)
    dev.dense_to_sparse_assign(n, it, dev.tensor(src[:n]), trg)
    assert trg.numpy().tobytes() == orc.dense_to_sparse_assign(idx, src[:n], np.zeros(size, F32)).tobytes()
    trg = dev.tensor(src)
    dev.dense_to_sparse_subtract(n, it, dev.tensor(src[:n]), trg)
    assert trg.numpy().tobytes() == orc.dense_to_sparse_subtract(idx, src[:n], src.copy()).tobytes()
    table = f32(rng.standard_normal((50, 37)))
    bidx = rng.integers(0, 50, 64).astype(np.uint32)
    out = dev.empty((64, 37))
    dev.sparse_to_dense_block_assign_and_multiply(64, dev.tensor(bidx, np.uint32), 37, 2.0, dev.tensor(table), out)
    want = orc.sparse_to_dense_block_assign_and_multiply(bidx, 37, 2.0, table)
    assert out.numpy().tobytes() == want.tobytes()
    acc = dev.zeros((50, 37))
    dev.dense_to_sparse_block_add(64, dev.tensor(bidx, np.uint32), 37, dev.tensor(want), acc)
    assert_close(acc.numpy(), orc.dense_to_sparse_block_add(bidx, 37, want, np.zeros((50, 37), F32)), GRAD_RTOL,
                 "dense_to_sparse_block_add", floor=1.0)


def test_parallel_memcpy_and_accumulate(dev):
    rng = np.random.default_rng(17)
    lens = np.array([5, 1024, 0, 333, 4096, 7], np.uint64)
    srcs = [f32(rng.standard_normal(int(n))) for n in lens]
    src_t = [dev.tensor(s) if s.size else dev.empty(1) for s in srcs]
    # ragged targets inside one buffer, deliberately not 16-byte aligned for some
    total = int(lens.sum()) + len(lens)
    big = dev.zeros(total)
    offs = np.concatenate([[0], np.cumsum(lens + 1)[:-1]]).astype(np.int64)
    ptr_arr = np.array([t.ptr for t in src_t] + [big.ptr + 4 * int(o) for o in offs], np.uint64)
    ptrs = dev.tensor(ptr_arr, np.uint64)
    lens_t = dev.tensor(lens, np.uint64)
    k = len(lens)
    dev.parallel_memcpy(k, int(lens.max()), ptrs.ptr, ptrs.ptr + 8 * k, lens_t)
    got = big.numpy()
    for s, o in zip(srcs, offs):
        assert got[o:o + s.size].tobytes() == s.tobytes()
    dev.parallel_accumulate(k, int(lens.max()), ptrs.ptr, ptrs.ptr + 8 * k, lens_t)
    got = big.numpy()
    for s, o in zip(srcs, offs):
        assert got[o:o + s.size].tobytes() == (s + s).tobytes()


def test_scale_copy_constant_accumulate_sgd_norm(dev):
    rng = np.random.default_rng(18)
    n = 100003
    p, g = f32(rng.standard_normal(n)), f32(rng.standard_normal(n))
    pt, gt, out = dev.tensor(p), dev.tensor(g), dev.empty(n)
    dev.scale_copy(n, pt, 1.0, out)
    assert out.numpy().tobytes() == p.tobytes()
    dev.scale_copy(n, pt, 0.25, out)
    assert out.numpy().tobytes() == orc.scale_copy(p, 0.25).tobytes()
    dev.constant(out, 3.5)
    assert np.all(out.numpy() == F32(3.5))
    dev.accumulate(gt, out)
    assert out.numpy().tobytes() == (g + F32(3.5)).tobytes()
    dev.sgd_update(n, pt, gt, 0.1, 0.5, 1.0)
    assert pt.numpy().tobytes() == orc.sgd_update(p.copy(), g, 0.1, 0.5, 1.0).tobytes()
    nrm = dev.empty(1)
    dev.squared_l2norm(n, gt, nrm)
    assert abs(float(nrm.numpy()[0]) - float((g.astype(np.float64) ** 2).sum())) < 1e-5 * n


@pytest.mark.parametrize("n,shift", [(1, 0), (3, 1), (1000003, 0), (1000003, 1), (1000003, 3), (4096, 2), (24 * 1024 * 1024 + 5, 0)])
def test_squared_l2norm_any_length_and_alignment(dev, n, shift):
    """The vector body of the squared norm starts at the first 16-byte boundary: lengths that are not multiples of 4
    and inputs that start 4, 8 or 12 bytes past one; the largest case takes the full grid."""
    rng = np.random.default_rng(n + shift)
    g = f32(rng.standard_normal(n + shift))
    gt = dev.tensor(g).offset(shift, (n,))
    nrm = dev.empty(1)
    dev.squared_l2norm(n, gt, nrm)
    want = float((g[shift:].astype(np.float64) ** 2).sum())
    assert abs(float(nrm.numpy()[0]) - want) <= 2e-6 * want + 1e-6


def test_device_side_clipping_and_sparse_rows(dev):
    rng = np.random.default_rng(19)
    vocab, dim, n = 500, 48, 700
    ids = zipf_ids(rng, n, vocab)
    table, grads = f32(rng.standard_normal((vocab, dim))), np.zeros((vocab, dim), F32)
    used = np.unique(ids)
    grads[used] = f32(rng.standard_normal((used.size, dim)))
    g2 = f32(rng.standard_normal(1000))
    plan = dev.lookup_build_plan(dev.tensor(ids, np.uint32), vocab)
    sq = dev.zeros(2)
    gt, tt, g2t = dev.tensor(grads), dev.tensor(table), dev.tensor(g2)
    dev.squared_l2norm_rows(n, plan, dim, vocab, gt, sq)
    dev.squared_l2norm(g2.size, g2t, sq.offset(1, (1,)))
    want_sq = (grads.astype(np.float64) ** 2).sum()
    assert abs(float(sq.numpy()[0]) - want_sq) < 1e-5 * want_sq
    total = np.sqrt(want_sq + (g2.astype(np.float64) ** 2).sum())
    scale = dev.empty(1)
    for thr, want in ((5.0, 5.0 / total), (1e9, 1.0), (0.0, 1.0)):
        dev.clip_scale(2, sq, thr, scale)
        assert abs(float(scale.numpy()[0]) - want) < 1e-5 * want
    dev.clip_scale(2, sq, 5.0, scale)
    s = scale.numpy()[0]
    dev.sgd_update_rows(n, plan, dim, vocab, tt, gt, 0.1, scale, 1.0)
    want_t = table.copy()
    for r in used:
        orc.sgd_update(want_t[r], grads[r], 0.1, float(s), 1.0)
    assert tt.numpy().tobytes() == want_t.tobytes()
    assert not gt.numpy().any()
    p = f32(rng.standard_normal(1000))
    pt = dev.tensor(p)
    dev.sgd_update_scaled(1000, pt, g2t, 0.1, scale, 1.0, clear_grad=False)
    assert pt.numpy().tobytes() == orc.sgd_update(p.copy(), g2, 0.1, float(s), 1.0).tobytes()
    assert g2t.numpy().tobytes() == g2.tobytes()
    dev.sgd_update_scaled(1000, pt, g2t, 0.1, scale, 1.0, clear_grad=True)
    assert not g2t.numpy().any()
    # a NaN or infinite gradient norm: scale 0, the norm is reported, and the updates leave the parameters alone
    norm = dev.empty(1)
    dev.clip_scale(2, sq, 5.0, scale, norm)
    assert abs(float(norm.numpy()[0]) - total) < 1e-5 * total and scale.numpy()[0] == s
    for bad in (np.nan, np.inf):
        dev.clip_scale(2, dev.tensor(np.array([1.0, bad], F32)), 5.0, scale, norm)
        assert scale.numpy()[0] == 0.0
        assert np.isnan(norm.numpy()[0]) if np.isnan(bad) else np.isinf(norm.numpy()[0])
        before, before_t = pt.numpy().copy(), tt.numpy().copy()
        g_bad = dev.tensor(np.full(1000, bad, F32))
        dev.sgd_update_scaled(1000, pt, g_bad, 0.1, scale, 1.0, clear_grad=True)
        assert pt.numpy().tobytes() == before.tobytes() and not g_bad.numpy().any()
        gt.set(np.full((vocab, dim), bad, F32))
        dev.sgd_update_rows(n, plan, dim, vocab, tt, gt, 0.1, scale, 1.0)
        assert tt.numpy().tobytes() == before_t.tobytes()
        # clipping disabled: the reference does not look at the norm (dynet/training.cc:174), the scale is 1
        for off in (0.0, -1.0):
            dev.clip_scale(2, dev.tensor(np.array([1.0, bad], F32)), off, scale, norm)
            assert scale.numpy()[0] == 1.0
            assert np.isnan(norm.numpy()[0]) if np.isnan(bad) else np.isinf(norm.numpy()[0])


@pytest.mark.parametrize("n", [4 * 1024 * 3 + 5, 5_000_003])
def test_sgd_update_of_a_large_slab(dev, n):
    """The slab update's unrolled and streaming forms (whole chunks of 1024 groups of four, the remaining groups, the
    last odd floats; 20 MB takes the streaming accesses), with and without clearing the gradient, and from an address
    that is not 16-byte aligned: the oracle's p -= g * (lr * scale / wd), bit for bit."""
    rng = np.random.default_rng(n)
    for shift in (0, 1):
        p, g = f32(rng.standard_normal(n + shift)), f32(rng.standard_normal(n + shift))
        pt, gt = dev.tensor(p), dev.tensor(g)
        scale = dev.tensor(np.array([0.37], F32))
        pv, gv = pt.offset(shift, (n,)), gt.offset(shift, (n,))
        want = orc.sgd_update(p[shift:].copy(), g[shift:], 0.1, 0.37, 1.0)
        dev.sgd_update_scaled(n, pv, gv, 0.1, scale, 1.0, clear_grad=False)
        assert pt.numpy()[shift:].tobytes() == want.tobytes() and gt.numpy().tobytes() == g.tobytes()
        dev.sgd_update_scaled(n, pv, gv, 0.1, scale, 1.0, clear_grad=True)
        assert pt.numpy()[shift:].tobytes() == orc.sgd_update(want.copy(), g[shift:], 0.1, 0.37, 1.0).tobytes()
        assert not gt.numpy()[shift:].any() and gt.numpy()[:shift].tobytes() == g[:shift].tobytes()
        assert pt.numpy()[:shift].tobytes() == p[:shift].tobytes()
        for w in lib_pools():
            dev.sync()
            dev.free_pool(w)


def test_zero_sized_calls_are_no_ops(dev):
    """Empty tensors (a batch of zero columns, zero ids, K = 0) must not launch anything or fail."""
    sentinel = f32(np.arange(8))
    t = dev.tensor(sentinel)
    e = dev.empty((0,))
    dev.unary_forward(lib.OP_TANH, e, e, n=0)
    dev.unary_backward(lib.OP_TANH, e, e, e, n=0)
    dev.cmult_forward(0, 1, 1, e, e, e)
    dev.scale_copy(0, e, 2.0, e)
    dev.sgd_update(0, e, e, 0.1)
    dev.lookup_forward(None, dev.empty((0,), np.uint32), 4, 10, t, e)
    dev.pnls_forward_staged(5, 0, e, e, e)
    dev.pnls_backward(5, 0, e, e, e, e)
    dev.logsumexp_cols(5, 0, e, e, e)
    dev.gemm_nn(0, 3, 4, e, t, 0.0, e)
    dev.gemm_nn(3, 0, 4, t, e, 0.0, e)
    # K = 0: y = beta * y
    y = dev.tensor(f32([1, 2, 3, 4, 5, 6]))
    dev.gemm_nn(3, 2, 0, t, t, 1.0, y)
    assert y.numpy().tobytes() == f32([1, 2, 3, 4, 5, 6]).tobytes()
    dev.gemm_nn(3, 2, 0, t, t, 0.0, y)
    assert not y.numpy().any()
    dev.layer_norm_forward(4, 0, e, t, t, e)
    dev.sum_forward(0, 3, [e], [3], e)
    dev.sync()
    assert t.numpy().tobytes() == sentinel.tobytes()


def test_forked_queue_ordering_and_errors(dev):
    """dyhip_device_fork / dyhip_device_wait: a chain that hops between two queues sees every earlier write."""
    rng = np.random.default_rng(20)
    n = 1 << 20
    x = f32(rng.standard_normal(n))
    q = dev.fork()
    a, b, c = dev.tensor(x), dev.empty(n), dev.empty(n)
    want = x.copy()
    for _ in range(6):
        dev.scale_copy(n, a, 0.5, b)      # device queue: b = a / 2
        q.wait(dev)
        q.scale_copy(n, b, 3.0, c)        # forked queue: c = 3 b
        dev.wait(q)
        dev.scale_copy(n, c, 1.0, a)      # device queue again: a = c
        want = orc.scale_copy(orc.scale_copy(want, 0.5), 3.0)
    assert a.numpy().tobytes() == want.tobytes()
    # a GEMM on each queue at the same time: separate split-K workspaces
    M, N, K = 256, 64, 2048
    l, r = f32(rng.standard_normal((K, M))), f32(rng.standard_normal((N, K)))
    lt, rt = dev.tensor(l), dev.tensor(r)
    y0, y1 = dev.zeros((N, M)), dev.zeros((N, M))
    q.wait(dev)
    for _ in range(4):
        dev.gemm_nn(M, N, K, lt, rt, 0.0, y0)
        q.gemm_nn(M, N, K, lt, rt, 0.0, y1)
    dev.wait(q)
    ref = orc.gemm_nn(M, N, K, l, r, 0.0, np.zeros((N, M), F32))
    assert_close(y0.numpy(), ref, FWD_RTOL, "gemm on the device queue", floor=np.sqrt(K))
    assert y0.numpy().tobytes() == y1.numpy().tobytes()
    with pytest.raises(DyhipError):
        q.fork()  # only the device itself can be forked
    q.close()


def test_device_scalars_and_pools(dev):
    vals = [np.frombuffer(dev_scalar(dev, k), F32)[0] for k in range(3)]
    assert vals == [-1.0, 1.0, 0.0]
    pool = dev.pool(lib.POOL_SCS)
    pool.free()
    a = pool.allocate(1)
    b = pool.allocate(1)
    assert b - a == 256 and a % 256 == 0  # GPUAllocator alignment
    assert pool.used() == 512
    z = dev.zeros(1000, pool=lib.POOL_DEDFS)
    dev.constant(z, 2.0)
    dev.pool(lib.POOL_DEDFS).zero_allocated()  # what the executor does before backward
    assert not z.numpy().any()


def dev_scalar(dev, which):
    from dynet_amd.device import DevTensor

    return DevTensor(dev, dev.scalar_ptr(which), (1,)).numpy().tobytes()


# ---- PickRange and the unfused builder step ---------------------------------------------------
@pytest.mark.parametrize("inner,length,outer,start,end", [(1, 8, 5, 2, 6), (1, 4096, 128, 1024, 2048), (7, 5, 3, 0, 5),
                                                          (3, 9, 70000, 4, 5), (33, 4, 1, 1, 3), (7, 9, 10001, 2, 5),
                                                          (1, 1500, 9, 100, 1123), (1, 1500, 9, 100, 1124), (5, 3, 1, 1, 2),
                                                          (1, 2, 1025, 1, 2)])
def test_pick_range(dev, inner, length, outer, start, end):
    rng = np.random.default_rng(inner + length)
    x = f32(rng.standard_normal(inner * length * outer))
    want = orc.pick_range_forward(inner, length, outer, start, end, x)
    fx = dev.empty(want.size)
    dev.pick_range_forward(inner, length, outer, start, end, dev.tensor(x), fx)
    assert np.array_equal(fx.numpy(), want)
    dy, dx0 = f32(rng.standard_normal(want.size)), f32(rng.standard_normal(x.size))
    dxt = dev.tensor(dx0)
    dev.pick_range_backward(inner, length, outer, start, end, dev.tensor(dy), dxt)
    assert np.array_equal(dxt.numpy(), orc.pick_range_backward(inner, length, outer, start, end, dy, dx0.copy()))
    with pytest.raises(DyhipError):
        dev.pick_range_forward(inner, length, outer, end, end, dxt, fx)


def _builder_step(dev, H, B, x_in, d_in, h_prev, c_prev, P, ln):
    """One layer of VanillaLSTMBuilder::add_input_impl (dynet/lstm.cc:477-546) issued op by op:
    affine_transform (or bias + layer_norm(Wx x) + layer_norm(Wh h)), pick_range x4, logistic / tanh
    (forget gate through ConstantPlusX 1.0), cmult / sum, tanh (of layer_norm(c) under ln_lstm), cmult."""
    G = 4 * H
    tmp = dev.empty((B, G))
    if ln:
        a, an = dev.empty((B, G)), dev.empty((B, G))
        b_, bn = dev.empty((B, G)), dev.empty((B, G))
        dev.gemm_nn(G, B, d_in, P["Wx"], x_in, 0.0, a)
        dev.layer_norm_forward(G, B, a, P["gx"], P["bx"], an)
        dev.gemm_nn(G, B, H, P["Wh"], h_prev, 0.0, b_)
        dev.layer_norm_forward(G, B, b_, P["gh"], P["bh"], bn)
        dev.sum_forward(G, B, [P["b"], an, bn], [1, B, B], tmp)
    else:
        dev.affine_forward(G, B, d_in, P["b"], P["Wx"], x_in, tmp)
        dev.gemm_nn(G, B, H, P["Wh"], h_prev, 1.0, tmp)
    parts = []
    for q in range(4):
        t = dev.empty((B, H))
        dev.pick_range_forward(1, G, B, q * H, (q + 1) * H, tmp, t)
        parts.append(t)
    a_i, a_f, a_o, a_g = parts
    one = dev.empty((H,))
    dev.constant(one, 1.0)
    a_f1 = dev.empty((B, H))
    dev.csum_forward(H, B, 1, a_f, one, a_f1)  # i_aft + forget_bias
    i_t, f_t, o_t, g_t = (dev.empty((B, H)) for _ in range(4))
    for src, dst in ((a_i, i_t), (a_f1, f_t), (a_o, o_t)):
        dev.unary_forward(lib.OP_LOGISTIC, src, dst)
    dev.unary_forward(lib.OP_TANH, a_g, g_t)
    fc, ig, c = dev.empty((B, H)), dev.empty((B, H)), dev.empty((B, H))
    dev.cmult_forward(H, B, B, f_t, c_prev, fc)
    dev.cmult_forward(H, B, B, i_t, g_t, ig)
    dev.sum_forward(H, B, [fc, ig], [B, B], c)
    tc, h = dev.empty((B, H)), dev.empty((B, H))
    if ln:
        cn = dev.empty((B, H))
        dev.layer_norm_forward(H, B, c, P["gc"], P["bc"], cn)
        dev.unary_forward(lib.OP_TANH, cn, tc)
    else:
        dev.unary_forward(lib.OP_TANH, c, tc)
    dev.cmult_forward(H, B, B, o_t, tc, h)
    return h, c


def test_unfused_builder_step_equals_fused_nodes(dev):
    """tests/test-rnn.cc:155-184: VanillaLSTMBuilder (unfused ops) and the fused gates/C/H nodes agree over
    three timesteps to 1e-5, here with both sides running on the device."""
    rng = np.random.default_rng(21)
    I, H, B = 6, 8, 4
    Wx, Wh, b = glorot(rng, 4 * H, I), glorot(rng, 4 * H, H), f32(rng.normal(0, 0.1, 4 * H))
    P = {"Wx": dev.tensor(Wx), "Wh": dev.tensor(Wh), "b": dev.tensor(b)}
    h_u = h_f = dev.tensor(f32(rng.standard_normal((B, H)) * 0.5))
    c_u = c_f = dev.tensor(f32(rng.standard_normal((B, H)) * 0.5))
    for t in range(3):
        x = dev.tensor(f32(rng.standard_normal((B, I))))
        h_u, c_u = _builder_step(dev, H, B, x, I, h_u, c_u, P, ln=False)
        g, c2, h2 = dev.empty((B, 4 * H)), dev.empty((B, H)), dev.empty((B, H))
        dev.lstm_gates_forward([x], [I], H, B, h_f, P["Wx"], P["Wh"], P["b"], g)
        dev.lstm_c_forward(H, B, c_f, g, c2)
        dev.lstm_h_forward(H, B, c2, g, h2)
        h_f, c_f = h2, c2
        assert_close(h_u.numpy(), h_f.numpy(), 1e-5, f"h step {t}", floor=1e-2)
        assert_close(c_u.numpy(), c_f.numpy(), 1e-5, f"c step {t}", floor=1e-2)


def test_ln_lstm_builder_step(dev):
    """The ln_lstm variant (dynet/lstm.cc:513-518,540-542), the in-tree consumer of layer_norm, against
    the same step composed from the oracle's nodes."""
    rng = np.random.default_rng(22)
    I, H, B = 10, 12, 5
    G = 4 * H
    Wx, Wh, b = glorot(rng, G, I), glorot(rng, G, H), f32(rng.normal(0, 0.1, G))
    ln = {k: f32(rng.uniform(0.5, 1.5, n)) if k[0] == "g" else f32(rng.normal(0, 0.1, n))
          for k, n in (("gx", G), ("bx", G), ("gh", G), ("bh", G), ("gc", H), ("bc", H))}
    P = {"Wx": dev.tensor(Wx), "Wh": dev.tensor(Wh), "b": dev.tensor(b)}
    P.update({k: dev.tensor(v) for k, v in ln.items()})
    h, c = f32(rng.standard_normal((B, H)) * 0.5), f32(rng.standard_normal((B, H)) * 0.5)
    ht, ct = dev.tensor(h), dev.tensor(c)
    for t in range(2):
        x = f32(rng.standard_normal((B, I)))
        ht, ct = _builder_step(dev, H, B, dev.tensor(x), I, ht, ct, P, ln=True)
        # oracle composition of the same nodes
        a = orc.gemm_nn(G, B, I, Wx, x, 0.0, np.zeros((B, G), F32))
        bb = orc.gemm_nn(G, B, H, Wh, h, 0.0, np.zeros((B, G), F32))
        tmp = orc.sum_forward(G, B, [b, orc.layer_norm_forward(G, B, a, ln["gx"], ln["bx"]),
                                     orc.layer_norm_forward(G, B, bb, ln["gh"], ln["bh"])], [1, B, B]).reshape(B, G)
        pick = lambda q: np.ascontiguousarray(tmp[:, q * H:(q + 1) * H])
        i_t = orc.unary_forward(orc.OP_LOGISTIC, pick(0))
        f_t = orc.unary_forward(orc.OP_LOGISTIC, pick(1) + F32(1.0))
        o_t = orc.unary_forward(orc.OP_LOGISTIC, pick(2))
        g_t = orc.unary_forward(orc.OP_TANH, pick(3))
        c = (f_t * c + i_t * g_t).astype(F32)
        h = (o_t * orc.unary_forward(orc.OP_TANH, orc.layer_norm_forward(H, B, c, ln["gc"], ln["bc"]).reshape(B, H))
             ).astype(F32)
        # layer_norm divides by sigma of a GEMM output: differences of 1e-7 in it come back scaled by g / sigma
        assert_close(ct.numpy(), c, FWD_RTOL, f"c step {t}", floor=1.0)
        assert_close(ht.numpy(), h, FWD_RTOL, f"h step {t}", floor=1.0)


def test_zero_any_alignment_and_inside_a_graph(dev):
    """dyhip_zero is a kernel for every address and size (no memset node), so it can be captured."""
    n = 4096
    buf = dev.empty(n, np.uint32)
    ones = np.full(n, 0xFFFFFFFF, np.uint32)
    for off, nbytes in [(0, 16), (1, 1), (3, 13), (5, 64), (15, 17), (16, 4000), (7, 4001), (9, 2), (2, 0)]:
        buf.set(ones)
        dev.zero_bytes(buf.ptr + off, nbytes)
        got = buf.numpy().view(np.uint8)
        want = ones.view(np.uint8).copy()
        want[off:off + nbytes] = 0
        assert np.array_equal(got, want), (off, nbytes)
    buf.set(ones)
    dev.graph_begin()
    dev.zero_bytes(buf.ptr + 6, 999)
    g = dev.graph_end()
    for _ in range(2):
        buf.set(ones)
        g.launch()
        dev.sync()
        want = ones.view(np.uint8).copy()
        want[6:6 + 999] = 0
        assert np.array_equal(buf.numpy().view(np.uint8), want)
    g.destroy()


@pytest.mark.parametrize("rows,cols,bd", [(7, 5, 3), (64, 100, 2), (130, 9, 1), (1, 300, 4), (1000, 33, 2), (3, 1, 5),
                                          # few rows and many columns (a wavefront folds its lanes over the columns), column
                                          # counts around the eight loads a thread has in flight
                                          (3, 8000, 2), (2, 1000, 3), (5, 4097, 1), (512, 512, 2), (33, 70, 2), (16, 129, 3),
                                          # few row groups: the columns are cut into slabs over the blocks as well
                                          (100, 3000, 2), (2048, 300, 1), (64, 256, 3), (40, 257, 5), (1, 6000, 1), (700, 511, 1)])
def test_softmax_and_logsumexp_along_dim_1(dev, rows, cols, bd):
    rng = np.random.default_rng(rows + cols + bd)
    x = f32(rng.standard_normal((bd, cols, rows)) * 3)
    xt = dev.tensor(x)
    fx = dev.empty((bd, cols, rows))
    dev.softmax_rows_forward(rows, cols, bd, xt, fx)
    ref = orc.softmax_rows_forward(rows, cols, bd, x)
    assert_close(fx.numpy(), ref, FWD_RTOL, "softmax dim 1", floor=1.0 / cols)
    np.testing.assert_allclose(fx.numpy().sum(axis=1), 1.0, rtol=1e-5)
    dy = f32(rng.standard_normal((bd, cols, rows)))
    dx0 = f32(rng.standard_normal((bd, cols, rows)))
    dxt = dev.tensor(dx0)
    dev.softmax_rows_backward(rows, cols, bd, dev.tensor(ref), dev.tensor(dy), dxt)
    assert_close(dxt.numpy(), orc.softmax_rows_backward(rows, cols, bd, ref, dy, dx0.copy()), GRAD_RTOL, "softmax dim 1 bwd",
                 floor=1.0)
    for dim in (0, 1):
        others = cols if dim == 0 else rows
        m, z = dev.empty((bd, others)), dev.empty((bd, others))
        dev.logsumexp_dim_forward(rows, cols, bd, xt, dim, m, z)
        rm, rz = orc.logsumexp_dim_forward(rows, cols, bd, x, dim)
        assert m.numpy().tobytes() == rm.tobytes()
        assert_close(z.numpy(), rz, FWD_RTOL, "logsumexp dim %d" % dim, floor=1.0)
        dz = f32(rng.standard_normal((bd, others)))
        dxt = dev.tensor(dx0)
        dev.logsumexp_dim_backward(rows, cols, bd, xt, dev.tensor(rz), dev.tensor(dz), dim, dxt)
        assert_close(dxt.numpy(), orc.logsumexp_dim_backward(rows, cols, bd, x, rz, dz, dim, dx0.copy()), GRAD_RTOL,
                     "logsumexp dim %d bwd" % dim, floor=1.0)
    with pytest.raises(DyhipError):
        dev.logsumexp_dim_forward(rows, cols, bd, xt, 2, m, z)


@pytest.mark.parametrize("rows,cols,bd", [(6, 40, 2), (6, 1500, 2), (70, 300, 1)])
def test_softmax_and_logsumexp_along_dim_1_with_infinite_entries(dev, rows, cols, bd):
    """-inf entries drop out of a row; a row that is all -inf is NaN (exp(-inf - -inf)), as in
    dynet/tensor.cc TensorTools::logsumexp and nodes-softmaxes.cc Softmax with dimension 1."""
    rng = np.random.default_rng(5)
    x = f32(rng.standard_normal((bd, cols, rows)) * 3)
    x[:, ::3, 1] = -np.inf
    x[:, : cols // 2, 2] = -np.inf
    x[:, :, 4] = -np.inf
    xt = dev.tensor(x)
    fx = dev.empty((bd, cols, rows))
    dev.softmax_rows_forward(rows, cols, bd, xt, fx)
    ref = orc.softmax_rows_forward(rows, cols, bd, x)
    got = fx.numpy()
    assert np.array_equal(np.isnan(got), np.isnan(ref)) and np.isnan(got[:, :, 4]).all() and not np.isnan(got[:, :, :4]).any()
    assert_close(np.nan_to_num(got), np.nan_to_num(ref), FWD_RTOL, "softmax dim 1", floor=1.0 / cols)
    m, z = dev.empty((bd, rows)), dev.empty((bd, rows))
    dev.logsumexp_dim_forward(rows, cols, bd, xt, 1, m, z)
    rm, rz = orc.logsumexp_dim_forward(rows, cols, bd, x, 1)
    assert m.numpy().tobytes() == rm.tobytes()
    assert np.array_equal(np.isnan(z.numpy()), np.isnan(rz)) and np.isnan(rz[:, 4]).all()
    assert_close(np.nan_to_num(z.numpy()), np.nan_to_num(rz), FWD_RTOL, "logsumexp dim 1", floor=1.0)


def test_pool_growth_is_ordered_with_forked_queues_and_refused_inside_a_capture(gpu):
    """A pool that grows zero-fills its new block before any queue can use it; growth while a graph is being
    recorded is refused with a clear error and leaves the capture usable."""
    from dynet_amd import Device

    gpu.sync()
    d = Device(0, mem_mb=(1, 1, 1, 1))
    try:
        small = d.empty(100)
        d.graph_begin()
        with pytest.raises(DyhipError, match="capture"):
            d.empty(1 << 20)  # 4 MB from a 1 MB pool: would have to grow
        d.constant(small, 2.0)
        g = d.graph_end()
        g.launch()
        d.sync()
        assert np.all(small.numpy() == F32(2.0))
        g.destroy()
        q = d.fork()
        big = q.empty(1 << 21)  # the shared pool grows through the forked queue ...
        q.constant(big, 1.0)    # ... whose next kernel must find the block already cleared
        q.sync()
        d.sync()
        assert np.all(big.numpy() == F32(1.0))
        fresh = d.empty(1 << 22)
        assert not fresh.numpy().any()
        d.sync()
        d.free_pool(lib.POOL_FXS)  # consolidates the blocks into one
        again = d.empty(1 << 22)
        assert not again.numpy().any()
    finally:
        d.close()
