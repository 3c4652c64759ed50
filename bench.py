#!/usr/bin/env python3
"""Benchmark of the fused-layer hot path on one MI355X.

    python bench.py --gpus 1 --steps K --warmup W

Workload (config.workload = "cfg2_elementwise_reduction_sweep"): the
elementwise / reduction sweep of the baseline on a 4096 x 1024 fp32 tensor with
values ~ N(0,1): tanh, logistic, rectify, cmult, sum_batches (batch 64 of
64 x 1024) and layer_norm over the 1024 dim (g ~ U(0.5,1.5), b ~ N(0,0.1)),
forward and backward.  One "step" is one pass of that sweep (13 kernel
launches) over one of several rotating buffer sets, so that successive steps
do not find their inputs in the 256 MB Infinity Cache.  Inputs are resident in
HBM before the timed region.

Reported: value = algorithmic bytes of one step / step time (GB/s), the
per-kernel achieved bandwidth of every kernel of the sweep and of the lookup /
PickNegLogSoftmax kernels (cfg 3 / 4), the latency of one fused LSTM cell step
(cfg 1), a roofline object for the dominant kernel, and the CPU oracle timed on
the host cores next to it (a reported baseline, not the target).

Per-kernel durations are measured with HIP events on the library's stream
around a replayed HIP graph that holds one launch per rotating buffer set, so
the figure is the back-to-back device time per launch, not Python's launch
latency.
"""
import argparse
import gc
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBPS = 8000.0
S_ELEMS = 4096 * 1024
S_BYTES = S_ELEMS * 4
LN_N, LN_BD = 1024, 4096
SB_N, SB_BD = 64 * 1024, 64


def parse_args():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--sets", type=int, default=24,
                    help="rotating buffer sets; 24 x 33.5 MB (the smallest kernel footprint) = 3x the Infinity Cache")
    ap.add_argument("--stream-threshold", type=int, default=None,
                    help="override the library's non-temporal access threshold in bytes (tuning experiments)")
    ap.add_argument("--kernel-reps", type=int, default=20, help="graph replays per per-kernel measurement")
    ap.add_argument("--no-graph", action="store_true",
                    help="plain back-to-back launches instead of HIP-graph replays everywhere (for profiler runs)")
    ap.add_argument("--one-pass", action="store_true",
                    help="counter-collection mode: launch every kernel of the sweep (and a 16.8 MB calibration copy) "
                         "a few times with plain launches, print nothing but a short note, and exit")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--pmc-summary", nargs=2, metavar=("FETCH_DB", "WRITE_DB"),
                    help="print the hardware-counter summary of two --one-pass runs under rocprofv3 --pmc and exit")
    ap.add_argument("--unique-ids", type=int, default=None,
                    help="with --pmc-summary: distinct ids of the cfg-3 id vector (the bench prints it as unique_ids)")
    ap.add_argument("--no-extras", action="store_true", help="skip the cfg 1 / 3 / 4 kernel measurements")
    ap.add_argument("--cpu-seconds", type=float, default=12.0, help="bound on the CPU-baseline leg")
    ap.add_argument("--cpu-config-seconds", type=float, default=3.0,
                    help="bound on each leg of the per-configuration CPU baseline (cfg 1, 3, 4 and the reduced cfg 5)")
    ap.add_argument("--no-lm", action="store_true", help="skip the cfg 5 LSTM-LM training-step measurement")
    ap.add_argument("--no-large", action="store_true", help="skip the 16x larger repeat of the cfg 2 sweep")
    ap.add_argument("--lm-steps", type=int, default=30)
    return ap.parse_args()


class Sweep:
    """The cfg-2 sweep: buffers for R rotating sets and the list of kernels."""

    def __init__(self, dev, lib, sets, seed=0, scale=1):
        """scale multiplies the number of rows / batch elements (1 = the baseline's 4096 x 1024 tensor)."""
        self.dev, self.lib, self.R = dev, lib, sets
        S_ELEMS, LN_BD, SB_BD = globals()["S_ELEMS"] * scale, globals()["LN_BD"] * scale, globals()["SB_BD"] * scale
        S_BYTES = S_ELEMS * 4
        self.elems = S_ELEMS
        rng = np.random.default_rng(seed)
        self.g = dev.tensor(rng.uniform(0.5, 1.5, LN_N).astype(np.float32), pool=lib.POOL_PS)
        self.b = dev.tensor((rng.standard_normal(LN_N) * 0.1).astype(np.float32), pool=lib.POOL_PS)
        self.dg = dev.zeros(LN_N, pool=lib.POOL_PS)
        self.db = dev.zeros(LN_N, pool=lib.POOL_PS)
        self.sets = []
        host = [rng.standard_normal(S_ELEMS).astype(np.float32) for _ in range(3)] if scale > 1 else None
        for _ in range(sets):
            draw = (lambda k: host[k]) if host else (lambda k: rng.standard_normal(S_ELEMS).astype(np.float32))
            s = {
                "x": dev.tensor(draw(0)),
                "x2": dev.tensor(draw(1)),
                "y": dev.empty(S_ELEMS),
                "dy": dev.tensor(draw(2)),
                "dx": dev.zeros(S_ELEMS, pool=lib.POOL_DEDFS),
                "s": dev.empty(SB_N),
            }
            self.sets.append(s)
        self.ws_ln, self.ws_ln_bytes = dev.workspace(dev.layer_norm_backward_workspace(LN_N, LN_BD))
        self.ws_br, self.ws_br_bytes = dev.workspace(max(dev.batch_reduce_workspace(SB_N, SB_BD), 256))
        L = lib
        S = S_BYTES
        d = dev
        # (name, algorithmic bytes per launch, launcher taking a buffer set)
        self.kernels = [
            ("tanh_fwd", 2 * S, lambda b: d.unary_forward(L.OP_TANH, b["x"], b["y"])),
            ("tanh_bwd", 4 * S, lambda b: d.unary_backward(L.OP_TANH, b["y"], b["dy"], b["dx"])),
            ("logistic_fwd", 2 * S, lambda b: d.unary_forward(L.OP_LOGISTIC, b["x"], b["y"])),
            ("logistic_bwd", 4 * S, lambda b: d.unary_backward(L.OP_LOGISTIC, b["y"], b["dy"], b["dx"])),
            ("rectify_fwd", 2 * S, lambda b: d.unary_forward(L.OP_RECTIFY, b["x"], b["y"])),
            ("rectify_bwd", 4 * S, lambda b: d.unary_backward(L.OP_RECTIFY, b["y"], b["dy"], b["dx"])),
            ("cmult_fwd", 3 * S, lambda b: d.cmult_forward(S_ELEMS, 1, 1, b["x"], b["x2"], b["y"])),
            ("cmult_bwd_arg0", 4 * S, lambda b: self._cmult_bwd(b, 0)),
            ("cmult_bwd_arg1", 4 * S, lambda b: self._cmult_bwd(b, 1)),
            ("sum_batches_fwd", S + S // 64,
             lambda b: d.sum_batches_forward(SB_N, SB_BD, b["x"], b["s"], self.ws_br, self.ws_br_bytes)),
            ("sum_batches_bwd", 2 * S + S // 64, lambda b: d.sum_batches_backward(SB_N, SB_BD, b["s"], b["dx"])),
            ("layer_norm_fwd", 2 * S + 2 * LN_N * 4,
             lambda b: d.layer_norm_forward(LN_N, LN_BD, b["x"], self.g, self.b, b["y"])),
            ("layer_norm_bwd", 4 * S + 4 * LN_N * 4,
             lambda b: d.layer_norm_backward(LN_N, LN_BD, b["x"], self.g, b["dy"], b["dx"], self.dg, self.db,
                                             self.ws_ln, self.ws_ln_bytes)),
        ]
        self.step_bytes = sum(k[1] for k in self.kernels)

    def _cmult_bwd(self, b, i):
        from dynet_amd.device import _check, _p, _sz, _u, _vp, cdll

        _check(cdll.dyhip_cmult_backward(self.dev.handle, _sz(self.elems), _u(1), _u(1), _p(b["x"]), _p(b["x2"]),
                                         _p(b["dy"]), _u(i), _p(b["dx"]), _vp(None), _sz(0)))

    def run_step(self, r):
        b = self.sets[r % self.R]
        for _, _, fn in self.kernels:
            fn(b)


def time_graph(dev, graph, reps, launches_per_replay):
    """Average device time per launch (us) of a captured graph replayed `reps` times."""
    for _ in range(3):
        graph.launch()
    dev.sync()
    dev.timer_start()
    for _ in range(reps):
        graph.launch()
    ms = dev.timer_stop()
    return ms * 1e3 / (reps * launches_per_replay)


def capture(dev, fn_list):
    dev.graph_begin()
    try:
        for fn in fn_list:
            fn()
    finally:
        g = dev.graph_end()
    return g


def time_loop(dev, fns, reps):
    """Average device time per call (us) of plain back-to-back launches (no graph)."""
    for fn in fns:
        fn()
    dev.sync()
    dev.timer_start()
    for _ in range(reps):
        for fn in fns:
            fn()
    ms = dev.timer_stop()
    return ms * 1e3 / (reps * len(fns))


def per_kernel_table(dev, named, sets, reps, use_graph=True):
    """named: list of (name, bytes, fn(set)); returns a list of dicts with us / GB/s / fraction of peak."""
    out = []
    # One replay holds at least 192 launches (the set list repeated): the boundary between two replays of a graph
    # costs about 5 us on this GPU (measured from inside the kernels: 6.5 us from the last block of one replay to the
    # first block of the next, against 1.5 us between two launches of one replay), which a graph of 8 launches would
    # add to every launch as 0.6 us and one of 24 as 0.2 us.  The figure is then what a launch costs inside a long
    # graph, such as the 2500-node LSTM-LM step.
    rounds = max(1, -(-192 // max(len(sets), 1)))
    for name, nbytes, fn in named:
        fns = [(lambda s=s: fn(s)) for s in sets] * rounds
        if use_graph:
            g = capture(dev, fns)
            us = time_graph(dev, g, reps, len(fns))
            g.destroy()
        else:
            us = time_loop(dev, fns, reps)
        gbps = nbytes / us / 1e3
        out.append({"kernel": name, "bytes": int(nbytes), "us": round(us, 3), "GBps": round(gbps, 1),
                    "frac_of_8TBps": round(gbps / HBM_PEAK_GBPS, 4)})
    return out


def extras_kernels(dev, lib, n_sets=None):
    """cfg 3 (lookup) and cfg 4 (PickNegLogSoftmax): yields (name, info, [(kernel, bytes, launcher)], buffer sets),
    one configuration at a time (the caller frees the pools in between).  Enough rotating buffer sets that a
    kernel's working set over one rotation exceeds the 256 MB Infinity Cache."""
    from dynet_amd.synth import zipf_ids

    rng = np.random.default_rng(0)
    # ---- cfg 3: lookup 50000 x 512, 16384 Zipf(1.1) ids -----------------------
    V, D, n = CFG3["V"], CFG3["D"], CFG3["n"]
    G = n * D * 4
    sets = []
    for _ in range(n_sets or 8):  # 8 x (33.5 MB of gradient rows + ~8 MB of touched table rows) = 335 MB
        ids = zipf_ids(rng, n, V)
        sets.append({
            "table": dev.tensor(rng.uniform(-0.1, 0.1, (V, D)).astype(np.float32)),
            "grads": dev.zeros((V, D), pool=lib.POOL_DEDFS),
            "ids": dev.tensor(ids, np.uint32), "fx": dev.empty((n, D)),
            "g": dev.tensor(rng.standard_normal((n, D)).astype(np.float32)),
            "uniq": int(np.unique(ids).size),
        })
    ws, wsb = dev.workspace(dev.lookup_accumulate_grads_workspace(n, D, V))
    uniq = sets[0]["uniq"]
    for s in sets:
        s["plan"], s["plan_ws"], s["plan_wsb"] = dev.lookup_plan_buffers(n, V)
        dev.lookup_build_plan_into(s["ids"], V, s["plan"], s["plan_ws"], s["plan_wsb"])
    ws2, wsb2 = dev.workspace(dev.lookup_accumulate_grads_planned_workspace(n, D))
    scatter_bytes = G + 2 * uniq * D * 4
    named = [
        ("lookup_gather", 2 * G + n * 4, lambda s: dev.lookup_forward(None, s["ids"], D, V, s["table"], s["fx"])),
        ("lookup_scatter_add(plan built at forward)", scatter_bytes,
         lambda s: dev.lookup_accumulate_grads_planned(n, s["plan"], D, V, s["g"], s["grads"], ws2, wsb2)),
        ("lookup_scatter_add(plan + segmented sum)", scatter_bytes,
         lambda s: dev.lookup_accumulate_grads(s["ids"], D, V, s["g"], s["grads"], ws, wsb)),
        ("lookup_plan (one kernel; no float data moved, bytes as for the scatter-add)", scatter_bytes,
         lambda s: dev.lookup_build_plan_into(s["ids"], V, s["plan"], s["plan_ws"], s["plan_wsb"])),
    ]
    yield "cfg3_lookup", {"vocab": V, "dim": D, "n_ids": n, "unique_ids": uniq, "rotating_buffer_sets": len(sets)}, named, sets
    # ---- the plan beyond 65535 ids (device-wide radix sort + run offsets) and for keys wider than 16 bits ---------
    big_n, wide_v = 262144, 200000
    sets = []
    for _ in range(n_sets or 4):
        sets.append({"ids_big": dev.tensor(zipf_ids(rng, big_n, V), np.uint32), "ids_wide": dev.tensor(zipf_ids(rng, n, wide_v), np.uint32)})
    pb, pbw, pbb = dev.lookup_plan_buffers(big_n, V)
    pw, pww, pwb = dev.lookup_plan_buffers(n, wide_v)
    named = [
        ("lookup_plan, 262144 ids (radix sort + run offsets; bytes = ids read + plan written)", big_n * 20,
         lambda s: dev.lookup_build_plan_into(s["ids_big"], V, pb, pbw, pbb)),
        ("lookup_plan, 16384 ids over a vocabulary of 200000 (one kernel, keys of 18 bits)", n * 20,
         lambda s: dev.lookup_build_plan_into(s["ids_wide"], wide_v, pw, pww, pwb)),
    ]
    yield "lookup_plan_other_routes", {"rotating_buffer_sets": len(sets)}, named, sets
    # ---- cwise with a dimension broadcast at the layer_norm composite's shape (x - mean, x / sigma) ----------------
    cn, cbd = LN_N, LN_BD
    da, db_ = (cn, 1, 1, 1, cbd), (1, 1, 1, 1, cbd)
    S = cn * cbd * 4
    sets = [{"a": dev.tensor(rng.standard_normal((cbd, cn)).astype(np.float32)),
             "b": dev.tensor(rng.uniform(0.5, 1.5, cbd).astype(np.float32)), "y": dev.empty((cbd, cn)),
             "dy": dev.tensor(rng.standard_normal((cbd, cn)).astype(np.float32)),
             "da": dev.zeros((cbd, cn), pool=lib.POOL_DEDFS), "db": dev.zeros(cbd, pool=lib.POOL_DEDFS)}
            for _ in range(n_sets or 12)]
    wsc, wscb = dev.workspace(max(dev.cwise_backward_workspace(da, db_, 1), 256))
    named = [
        ("cwise_quotient_fwd(1024 x 4096 by 1 x 4096)", 2 * S + cbd * 4,
         lambda s: dev.cwise_forward(lib.CWISE_QUOTIENT, da, db_, s["a"], s["b"], s["y"])),
        ("cwise_quotient_bwd_arg0", 3 * S + cbd * 4,
         lambda s: dev.cwise_backward(lib.CWISE_QUOTIENT, da, db_, s["a"], s["b"], s["dy"], 0, s["da"], wsc, wscb)),
        ("cwise_quotient_bwd_arg1(sum over the 1024 dim)", 2 * S + 3 * cbd * 4,
         lambda s: dev.cwise_backward(lib.CWISE_QUOTIENT, da, db_, s["a"], s["b"], s["dy"], 1, s["db"], wsc, wscb)),
    ]
    yield "cwise_dimension_broadcast", {"dims_a": list(da), "dims_b": list(db_), "rotating_buffer_sets": len(sets)}, named, sets
    # ---- cfg 4: PickNegLogSoftmax 50000 x 512 ----------------------------------
    rows, bd = CFG4["rows"], CFG4["bd"]
    X = rows * bd * 4
    sets = []
    for _ in range(n_sets or 3):
        labels = rng.integers(0, rows, bd).astype(np.uint32)
        aux = dev.empty(3 * bd)
        aux.offset(2 * bd, (bd,)).set((np.arange(bd, dtype=np.uint32) * rows + labels).view(np.float32))
        sets.append({"x": dev.tensor((rng.standard_normal((bd, rows)) * 2).astype(np.float32)), "aux": aux,
                     "fx": dev.empty(bd), "dy": dev.tensor(rng.standard_normal(bd).astype(np.float32)),
                     "dx": dev.zeros((bd, rows), pool=lib.POOL_DEDFS)})
    for s in sets:
        dev.pnls_forward_staged(rows, bd, s["x"], s["aux"], s["fx"])
    named = [
        ("pnls_fwd", X, lambda s: dev.pnls_forward_staged(rows, bd, s["x"], s["aux"], s["fx"])),
        ("pnls_bwd", 3 * X, lambda s: dev.pnls_backward(rows, bd, s["x"], s["aux"], s["dy"], s["dx"])),
    ]
    yield "cfg4_pnls", {"rows": rows, "bd": bd, "rotating_buffer_sets": len(sets)}, named, sets
    # ---- layer_norm over rows wider than the one-wave-per-row kernels take (> 2048 floats) ---------------------
    n, bd = 4096, 1024
    S = n * bd * 4
    sets = [{"x": dev.tensor(rng.standard_normal((bd, n)).astype(np.float32)), "y": dev.empty((bd, n)),
             "dy": dev.tensor(rng.standard_normal((bd, n)).astype(np.float32)),
             "dx": dev.zeros((bd, n), pool=lib.POOL_DEDFS)} for _ in range(n_sets or 6)]
    g, b = dev.tensor(rng.uniform(0.5, 1.5, n).astype(np.float32)), dev.tensor(np.zeros(n, np.float32))
    dg, db = dev.zeros(n, pool=lib.POOL_DEDFS), dev.zeros(n, pool=lib.POOL_DEDFS)
    ws_ln, ws_lnb = dev.workspace(dev.layer_norm_backward_workspace(n, bd))
    named = [
        ("layer_norm_fwd(n=4096)", 2 * S + 2 * n * 4, lambda s: dev.layer_norm_forward(n, bd, s["x"], g, b, s["y"])),
        ("layer_norm_bwd(n=4096)", 4 * S + 4 * n * 4,
         lambda s: dev.layer_norm_backward(n, bd, s["x"], g, s["dy"], s["dx"], dg, db, ws_ln, ws_lnb)),
    ]
    yield "layer_norm_wide_rows", {"n": n, "bd": bd, "rotating_buffer_sets": len(sets)}, named, sets
    # ---- shapes off the baseline's grid: small and transposed products, long elements of a small batch, reductions
    # along dim 1, vocabulary-length columns of a batch of one or two, short and long reduced axes of the broadcast
    # gradients, sums of scalars over a batch.  One buffer set each (a few MB at most: these live in the caches in
    # use too); the figure is the time of one call inside a long graph. -----------------------------------------
    R = lambda *shape: dev.tensor(rng.standard_normal(shape).astype(np.float32))
    Z = lambda *shape: dev.zeros(shape, pool=lib.POOL_DEDFS)
    s0 = {}
    named = []

    def add(name, nbytes, fn):
        named.append((name, nbytes, lambda s, fn=fn: fn()))

    a, b, y = R(128, 128), R(128, 128), Z(128, 128)
    add("gemm l^T*r 128x128x128", 3 * 128 * 128 * 4, lambda a=a, b=b, y=y: dev.gemm_tn_acc(128, 128, 128, a, b, y))
    a, b, y = R(512, 512), R(512, 512), Z(512, 512)
    add("gemm l^T*r 512x512x512", 3 * 512 * 512 * 4, lambda a=a, b=b, y=y: dev.gemm_tn_acc(512, 512, 512, a, b, y))
    a, b, y = R(650, 650), R(1, 650), Z(1, 650)
    add("gemm l*r 650x1x650 (leading dimension not a multiple of 4)", (650 * 650 + 1300) * 4,
        lambda a=a, b=b, y=y: dev.gemm_nn(650, 1, 650, a, b, 0.0, y))
    a, b, y = R(128, 1024, 1), R(128, 1024, 35), Z(128, 35, 1)
    add("gemm strided-batched l*r^T 1x35x1024 x 128 items", 128 * (1024 + 35 * 1024 + 35) * 4,
        lambda a=a, b=b, y=y: dev.gemm_strided_batched(0, 1, 1, 35, 1024, a, 1024, b, 35 * 1024, 0.0, y, 35, 128))
    a, b, y = R(128, 35, 1024), R(128, 1, 35), Z(128, 1, 1024)
    add("gemm strided-batched l*r 1024x1x35 x 128 items (attention context)", 128 * (1024 * 35 + 35 + 1024) * 4,
        lambda a=a, b=b, y=y: dev.gemm_strided_batched(0, 0, 1024, 1, 35, a, 1024 * 35, b, 35, 0.0, y, 1024, 128))
    dctx, dH = R(128, 1, 1024), Z(128, 35, 1024)
    add("gemm strided-batched l*r^T 1024x35x1 x 128 items (rank-one update an item)", 128 * (2 * 1024 * 35 + 35 + 1024) * 4,
        lambda dctx=dctx, b=b, dH=dH: dev.gemm_strided_batched(0, 1, 1024, 35, 1, dctx, 1024, b, 35, 1.0, dH, 1024 * 35, 128))
    a, b, y = R(1000, 9, 7), R(1000, 5, 9), Z(1000, 5, 7)
    add("gemm strided-batched l*r 7x5x9 x 1000 items", 1000 * (63 + 45 + 35) * 4,
        lambda a=a, b=b, y=y: dev.gemm_strided_batched(0, 0, 7, 5, 9, a, 63, b, 45, 0.0, y, 35, 1000))
    n, bd = 1 << 20, 4
    x, m, dy, dx = R(bd, n), dev.empty(bd), R(bd), Z(bd, n)
    add("mean_elems 1048576 x 4", n * bd * 4, lambda x=x, m=m: dev.mean_elems_forward(1 << 20, 4, x, m))
    add("std_elems 1048576 x 4", n * bd * 4, lambda x=x, m=m: dev.std_elems_forward(1 << 20, 4, x, m))
    add("std_elems_bwd 1048576 x 4", 3 * n * bd * 4, lambda x=x, m=m, dy=dy, dx=dx: dev.std_elems_backward(1 << 20, 4, x, m, dy, dx))
    x, y = R(1, 2048, 2048), dev.empty((1, 2048, 2048))
    add("softmax along dim 1, 2048 x 2048", 2 * 2048 * 2048 * 4, lambda x=x, y=y: dev.softmax_rows_forward(2048, 2048, 1, x, y))
    rows, bd = 300000, 2
    x, m, z, dy, dx = R(bd, rows), dev.empty(bd), dev.empty(bd), R(bd, rows), Z(bd, rows)
    add("logsumexp_cols 300000 x 2", rows * bd * 4, lambda x=x, m=m, z=z: dev.logsumexp_cols(300000, 2, x, m, z))
    add("softmax_bwd 300000 x 2", 4 * rows * bd * 4, lambda x=x, dy=dy, dx=dx: dev.softmax_backward(300000, 2, x, dy, dx))
    x, idx = R(1, 1000000), dev.empty(1, np.int64)
    add("argmax_cols 1000000 x 1", 4000000, lambda x=x, idx=idx: dev.argmax_cols(1000000, 1, x, idx))
    da, db_ = (1024, 35, 1, 1, 16), (1024, 1, 1, 1, 16)
    a, b, dy, g = R(16, 35, 1024), R(16, 1024), R(16, 35, 1024), Z(16, 1024)
    add("cwise_mult_bwd_arg1 1024x35x16 by 1024x1x16 (sum over the 35)", 2 * 16 * 35 * 1024 * 4,
        lambda a=a, b=b, dy=dy, g=g, da=da, db_=db_: dev.cwise_backward(lib.CWISE_MULT, da, db_, a, b, dy, 1, g))
    da2, db2 = (100000, 3, 1, 1, 1), (1, 3, 1, 1, 1)
    a, b, dy, g = R(3, 100000), R(3), R(3, 100000), Z(3)
    add("cwise_quotient_bwd_arg1 100000x3 by 1x3 (three sums of 100000 terms)", 3 * 300000 * 4,
        lambda a=a, b=b, dy=dy, g=g, da2=da2, db2=db2: dev.cwise_backward(lib.CWISE_QUOTIENT, da2, db2, a, b, dy, 1, g))
    x, y = R(1000000, 1), dev.empty(1)
    wsb_, wsbb = dev.workspace(dev.batch_reduce_workspace(1, 1000000))
    add("sum_batches of 1000000 scalars", 4000000, lambda x=x, y=y: dev.sum_batches_forward(1, 1000000, x, y, wsb_, wsbb))
    x, y = R(100000, 9, 7), dev.empty((100000, 3, 7))
    add("pick_range 7x9x100000 [2,5)", 2 * 100000 * 21 * 4, lambda x=x, y=y: dev.pick_range_forward(7, 9, 100000, 2, 5, x, y))
    xs, y = [R(128, 1) for _ in range(35)], dev.empty((128, 1))
    add("logsumexp node, 35 arguments of 1 x 128", 36 * 128 * 4, lambda xs=xs, y=y: dev.logsumexp_node_forward(1, 128, xs, [128] * 35, y))
    yield "off_grid_shapes", {"rotating_buffer_sets": 1}, named, [s0]


def extras(dev, lib, reps, use_graph=True):
    """cfg 3 (lookup), cfg 4 (PickNegLogSoftmax) kernels and the cfg 1 LSTM cell latency."""
    from dynet_amd.synth import glorot

    rng = np.random.default_rng(1)
    res = {}
    for name, info, named, sets in extras_kernels(dev, lib):
        info["kernels"] = per_kernel_table(dev, named, sets, reps, use_graph=use_graph)
        res[name] = info
        for w in (lib.POOL_FXS, lib.POOL_DEDFS, lib.POOL_SCS):
            dev.sync()
            dev.free_pool(w)
    # ---- cfg 1: one fused LSTM cell step, fwd + bwd ------------------------------
    I, H, B = 128, 256, 32
    t = {k: dev.tensor(v) for k, v in {
        "x": rng.standard_normal((B, I)), "h": rng.standard_normal((B, H)), "c": rng.standard_normal((B, H)),
        "Wx": glorot(rng, 4 * H, I), "Wh": glorot(rng, 4 * H, H), "b": np.zeros(4 * H),
        "dh": rng.standard_normal((B, H)), "dc": rng.standard_normal((B, H))}.items()}
    fx, c2, h2 = dev.empty((B, 4 * H)), dev.empty((B, H)), dev.empty((B, H))
    dgates, dcp, dx, dhp = (dev.zeros(s, pool=lib.POOL_DEDFS) for s in ((B, 4 * H), (B, H), (B, I), (B, H)))
    dWx, dWh, db = (dev.zeros(s, pool=lib.POOL_DEDFS) for s in ((I, 4 * H), (H, 4 * H), (4 * H,)))
    dct = dev.zeros((B, H), pool=lib.POOL_DEDFS)
    dpre = dev.empty((B, 4 * H))

    def cell():
        dev.lstm_gates_forward([t["x"]], [I], H, B, t["h"], t["Wx"], t["Wh"], t["b"], fx)
        dev.lstm_c_forward(H, B, t["c"], fx, c2)
        dev.lstm_h_forward(H, B, c2, fx, h2)
        dev.lstm_h_backward(H, B, c2, fx, t["dh"], 0, dct)
        dev.lstm_h_backward(H, B, c2, fx, t["dh"], 1, dgates)
        dev.lstm_c_backward(H, B, t["c"], fx, dct, 0, dcp)
        dev.lstm_c_backward(H, B, t["c"], fx, dct, 1, dgates)
        dev.lstm_gates_dpre(H, B, fx, dgates, dpre)
        for i, out in enumerate((dx, dhp, dWx, dWh, db)):
            dev.lstm_gates_backward([t["x"]], [I], H, B, t["h"], t["Wx"], t["Wh"], fx, dgates, i, out, dpre=dpre)

    cell()
    dev.sync()
    dev.free_pool(lib.POOL_SCS)
    if use_graph:
        g = capture(dev, [cell])
        us = time_graph(dev, g, max(reps, 50), 1)
        g.destroy()
    else:
        us = time_loop(dev, [cell], max(reps, 50))
    res["cfg1_lstm_cell"] = {"I": I, "H": H, "B": B, "fwd_bwd_us": round(us, 2), "launches": 13 + 5,
                             "gemm_flops": 3 * 2 * 4 * H * (I + H) * B,
                             "path": "VanillaLSTMGates / C / H nodes, every backward argument"}
    # the same step through the fused cell entry points
    fb, bb = dev.lstm_cell_workspace(H, B)
    wf, _ = dev.workspace(fb)
    wb, _ = dev.workspace(bb)
    xproj, dcp2 = dev.empty((B, 4 * H)), dev.empty((B, H))

    def cell_fused():
        dev.gemm_nn(4 * H, B, I, t["Wx"], t["x"], 0.0, xproj)
        n = dev.lstm_recurrent_forward(H, B, t["Wh"], t["h"], wf, fb)
        dev.lstm_cell_forward(H, B, xproj, t["b"], wf, n, t["c"], fx, c2, h2)
        dev.lstm_cell_backward(H, B, fx, c2, t["c"], t["dh"], None, 0, t["dc"], dpre, dcp2)
        dev.lstm_recurrent_backward(H, B, t["Wh"], dpre, wb, bb)       # d h_prev as split-K slices
        dev.gemm_tn(I, B, 4 * H, t["Wx"], dpre, 1.0, dx)
        dev.gemm_nt_acc(4 * H, I, B, dpre, t["x"], dWx)
        dev.gemm_nt_acc(4 * H, H, B, dpre, t["h"], dWh)
        dev.csum_backward(4 * H, 1, B, dpre, 0, db)

    cell_fused()
    dev.sync()
    if use_graph:
        g = capture(dev, [cell_fused])
        us2 = time_graph(dev, g, max(reps, 50), 1)
        g.destroy()
    else:
        us2 = time_loop(dev, [cell_fused], max(reps, 50))
    res["cfg1_lstm_cell"]["fused_cell_path_fwd_bwd_us"] = round(us2, 2)
    # forward in one launch (input product, recurrent product and cell update from packed weights); the two
    # packed copies are made once outside the timed region, as a caller does per weight update, not per timestep
    pWx, pWh = dev.empty(4 * H * I), dev.empty(4 * H * H)
    dev.lstm_pack_input(I, H, t["Wx"], pWx)
    dev.lstm_pack_recurrent(H, t["Wh"], pWh)

    def fwd_single():
        dev.lstm_step_forward_x(I, H, B, pWx, t["x"], pWh, t["h"], t["b"], t["c"], fx, c2, h2)

    def fwd_nodes():
        dev.lstm_gates_forward([t["x"]], [I], H, B, t["h"], t["Wx"], t["Wh"], t["b"], fx)
        dev.lstm_c_forward(H, B, t["c"], fx, c2)
        dev.lstm_h_forward(H, B, c2, fx, h2)

    def cell_single():
        fwd_single()
        dev.lstm_cell_backward(H, B, fx, c2, t["c"], t["dh"], None, 0, t["dc"], dpre, dcp2)
        dev.lstm_recurrent_backward(H, B, t["Wh"], dpre, wb, bb)
        dev.gemm_tn(I, B, 4 * H, t["Wx"], dpre, 1.0, dx)
        dev.gemm_nt_acc(4 * H, I, B, dpre, t["x"], dWx)
        dev.gemm_nt_acc(4 * H, H, B, dpre, t["h"], dWh)
        dev.csum_backward(4 * H, 1, B, dpre, 0, db)

    for key, fn in (("forward_only_nodes_us", fwd_nodes), ("forward_only_single_launch_us", fwd_single),
                    ("single_launch_forward_fwd_bwd_us", cell_single)):
        fn()
        dev.sync()
        if use_graph:
            g = capture(dev, [fn] * 4)
            us3 = time_graph(dev, g, max(reps, 50), 4)
            g.destroy()
        else:
            us3 = time_loop(dev, [fn], max(reps, 50))
        res["cfg1_lstm_cell"][key] = round(us3, 2)
    res["combine_tensors"] = movers(dev, lib, reps, use_graph)
    return res


def movers(dev, lib, reps, use_graph=True):
    """The batched executor's combine_tensors / accumulate_tensors on 128 nodes of 1024 floats each: the mover
    kernels alone (pointer table resident), and the whole host path per call (table written into page-locked
    memory, queued copy, kernel; no synchronisation between calls)."""
    from dynet_amd.device import PinnedArray

    rng = np.random.default_rng(2)
    k, sz = 128, 1024
    parts = [dev.tensor(rng.standard_normal(sz).astype(np.float32)) for _ in range(k)]
    grads = [dev.zeros(sz, pool=lib.POOL_DEDFS) for _ in range(k)]
    out = dev.empty(k * sz)
    table = dev.empty(3 * k, np.uint64)
    lens = np.full(k, sz, np.uint64)
    fwd = np.concatenate([np.array([t.ptr for t in parts], np.uint64), out.ptr + 4 * sz * np.arange(k, dtype=np.uint64), lens])
    bwd = np.concatenate([out.ptr + 4 * sz * np.arange(k, dtype=np.uint64), np.array([t.ptr for t in grads], np.uint64), lens])
    ring = [PinnedArray((3 * k,), np.uint64) for _ in range(64)]
    res = {"nodes": k, "floats_per_node": sz}
    for name, tab, call, nbytes in (("combine_tensors", fwd, dev.parallel_memcpy, 2 * k * sz * 4),
                                    ("accumulate_tensors", bwd, dev.parallel_accumulate, 3 * k * sz * 4)):
        table.set(tab)
        fn = lambda: call(k, sz, table.ptr, table.ptr + 8 * k, table.ptr + 16 * k)
        fn()
        dev.sync()
        if use_graph:
            g = capture(dev, [fn] * 8)
            us = time_graph(dev, g, max(reps, 50), 8)
            g.destroy()
        else:
            us = time_loop(dev, [fn], max(reps, 50))
        # host path: 64 calls back to back, each with its own slice of page-locked staging memory
        for p in ring:
            p.array[:] = tab
        dev.sync()
        t0 = time.perf_counter()
        for p in ring:
            dev.copy_h2d_async(table, p)
            fn()
        t_issue = time.perf_counter() - t0
        dev.sync()
        t_all = time.perf_counter() - t0
        res[name] = {"bytes": nbytes, "kernel_us": round(us, 2), "kernel_GBps": round(nbytes / us / 1e3, 1),
                     "host_path_us_per_call": round(t_all / len(ring) * 1e6, 2),
                     "host_issue_us_per_call": round(t_issue / len(ring) * 1e6, 2)}
    for p in ring:
        p.close()
    return res


FP32_MFMA_PEAK_TFLOPS = 157.3

PMC_PROFILE = os.path.join(ROOT, "profiles", "hbm_traffic_pmc_all_kernels.txt")


def measured_traffic():
    """HBM bytes per launch from the committed hardware-counter summary (rocprofv3 --pmc FETCH_SIZE, then
    WRITE_SIZE, on `bench.py --one-pass`, scaled as the summary says; written by `bench.py --pmc-summary`).
    The counters are not read in this run: the figures belong to the commit that wrote the file.  {} if absent."""
    out = {}
    try:
        with open(PMC_PROFILE) as f:
            for line in f:
                parts = line.split()
                if len(parts) == 3 and parts[0] == "TRAFFIC":
                    out[parts[1]] = float(parts[2])
    except OSError:
        pass
    return out


# device kernel (substring of its name) -> entry of the counter summary
PMC_KERNELS = [
    ("TanhFwd", "tanh_fwd"), ("TanhBwd", "tanh_bwd"), ("LogisticPacketFwd", "logistic_fwd"),
    ("LogisticBwd", "logistic_bwd"), ("RectifyFwd", "rectify_fwd"), ("RectifyBwd", "rectify_bwd"),
    ("AccMul2", "cmult_bwd"), ("Mul2", "cmult_fwd"), ("AccIn0", "sum_batches_bwd"),
    ("batch_reduce_kernel", "sum_batches_fwd"), ("ln_fwd_wave_kernel", "layer_norm_fwd"),
    ("ln_bwd_wave_kernel", "layer_norm_bwd_main"), ("combine_partials", "layer_norm_bwd_combine"),
    ("ln_fwd_team_kernel", "layer_norm_wide_fwd"), ("ln_bwd_team_kernel", "layer_norm_wide_bwd_main"),
    ("lookup_gather_kernel", "lookup_gather"), ("plan_direct_kernel", "lookup_plan"),
    ("cwise_bcast2_kernel<2,", "cwise_quotient_fwd"), ("cwise_bcast2_kernel<5,", "cwise_quotient_bwd_arg0"),
    ("cwise_reduce_row_kernel<6,", "cwise_quotient_bwd_arg1"),
    ("scatter_runs_kernel", "lookup_scatter_runs"), ("lse_cols_kernel", "pnls_fwd"), ("pnls_bwd_kernel", "pnls_bwd"),
    ("lstm_step_fwd_kernel", "lstm_step_fwd"), ("lstm_step_bwd_kernel", "lstm_step_bwd"),
    ("skinny_tn_kernel<false, false>", "lstm_rec_bwd_packed"),
    ("lstm_cell_bwd_kernel", "lstm_cell_bwd_packed"), ("gemm_wide_kernel<false, false>", "gemm_wide_nt_dW"),
    ("gemm_wide_fixup_kernel", "gemm_wide_nt_dW_fixup"),
]
CFG3 = {"V": 50000, "D": 512, "n": 256 * 64}
CFG4 = {"rows": 50000, "bd": 512}


def print_pmc_summary(fetch_db, write_db, unique_ids):
    """Text summary of two rocprofv3 --pmc runs of `bench.py --one-pass` (rocpd databases): KiB per dispatch of
    FETCH_SIZE and WRITE_SIZE per kernel, the scale factors from the calibration copies, and TRAFFIC lines
    (bench entry, HBM bytes per launch) that measured_traffic() reads back."""
    import re
    import sqlite3

    def table(path):
        # per kernel name; the combine kernel of the LayerNorm backward runs at two shapes (the sweep's 4096 rows of
        # 1024 and the wide-row extra's 1024 rows of 4096): its launches are told apart by grid size, the smaller
        # grid being the sweep's
        cur = sqlite3.connect(path).cursor()
        cols = [r[1] for r in cur.execute("pragma table_info(counters_collection)")]
        grid = next((c for c in ("grid_size", "grid_size_x", "grid_x") if c in cols), None)
        if grid is None:
            rows = cur.execute("select kernel_name, count(*), avg(value) from counters_collection group by kernel_name")
            return {k: (c, a) for k, c, a in rows}
        rows = cur.execute("select kernel_name, %s, count(*), avg(value) from counters_collection group by kernel_name, %s"
                           % (grid, grid)).fetchall()
        small = min((g for k, g, _, _ in rows if "combine_partials" in k), default=None)
        out = {}
        for k, g, c, a in rows:
            key = k + " [wide rows]" if "combine_partials" in k and g != small else k
            c0, a0 = out.get(key, (0, 0.0))
            out[key] = (c0 + c, (a0 * c0 + a * c) / (c0 + c))
        return out

    def entry(kname):
        if "IdentityFwd" in kname:  # the calibration copy: 4th template argument = streaming accesses or not
            m = re.search(r"ew_vec4_kernel<\s*\d+,\s*\w+,\s*\d+,\s*(true|false)", kname)
            return "copy_streaming" if (m and m.group(1) == "true") else "copy_plain"
        if "combine_partials" in kname and kname.endswith("[wide rows]"):
            return "layer_norm_wide_bwd_combine"
        for sub, name in PMC_KERNELS:
            if sub in kname:
                return name
        return None

    f, w = table(fetch_db), table(write_db)
    rows = {}
    for k in f:
        e = entry(k)
        if e is None:
            continue
        calls, fk = f[k]
        wk = w.get(k, (0, 0.0))[1]
        r = rows.setdefault(e, [0, 0.0, 0.0])
        r[1] = (r[1] * r[0] + fk * calls) / (r[0] + calls)
        r[2] = (r[2] * r[0] + wk * calls) / (r[0] + calls)
        r[0] += calls
    S = S_BYTES
    G = CFG3["n"] * CFG3["D"] * 4
    X = CFG4["rows"] * CFG4["bd"] * 4
    algo = {"tanh_fwd": 2 * S, "logistic_fwd": 2 * S, "rectify_fwd": 2 * S, "tanh_bwd": 4 * S, "logistic_bwd": 4 * S,
            "rectify_bwd": 4 * S, "cmult_fwd": 3 * S, "cmult_bwd": 4 * S, "sum_batches_fwd": S + S // 64,
            "sum_batches_bwd": 2 * S + S // 64, "layer_norm_fwd": 2 * S + 2 * LN_N * 4,
            "layer_norm_bwd_main": 4 * S + 4 * LN_N * 4, "layer_norm_wide_fwd": 2 * S + 2 * 4096 * 4,
            "layer_norm_wide_bwd_main": 4 * S + 4 * 4096 * 4, "lookup_gather": 2 * G + CFG3["n"] * 4,
            "lookup_scatter_runs": G + 2 * unique_ids * CFG3["D"] * 4, "pnls_fwd": X, "pnls_bwd": 3 * X,
            # 1024 x 4096 by 1 x 4096: S in and out + the divisor row; dy, the row and dx in and out; dy, both operands
            "cwise_quotient_fwd": 2 * S + 4096 * 4, "cwise_quotient_bwd_arg0": 3 * S + 4096 * 4,
            "cwise_quotient_bwd_arg1": 2 * S + 3 * 4096 * 4,
            # cfg-5 timestep at H = 1024, B = 128 (HB = H*B floats): packed Wh once + 13 HB; packed Wh^T once + 4 HB
            # in + 4 slices of HB out; 4+4+4+4+1 HB in and out of the packed cell backward
            "lstm_step_fwd": (4 * 1024 * 1024 + 13 * 1024 * 128) * 4, "lstm_rec_bwd_packed": (4 * 1024 * 1024 + 8 * 1024 * 128) * 4,
            "lstm_cell_bwd_packed": 21 * 1024 * 128 * 4,
            # packed Wh^T once + dpre of the step above (4 HB) + gates 4, c, c_tm1, dh, dc in + dpre twice and dc_tm1 out
            "lstm_step_bwd": (4 * 1024 * 1024 + 21 * 1024 * 128) * 4,
            # operands once + the output read and written (the partial tiles of its runs are traffic on top)
            "gemm_wide_nt_dW": (4096 * 4480 + 1024 * 4480 + 2 * 4096 * 1024) * 4}
    kib = S / 1024.0
    cs, cp = rows.get("copy_streaming"), rows.get("copy_plain")
    ff = kib / cs[1]
    fw = kib / cs[2]
    print("HBM traffic per launch from hardware counters, one MI355X")
    print()
    print("commands (each from /tmp with TMPDIR=/tmp, one counter per run):")
    print("  timeout -s KILL 120 rocprofv3 --pmc FETCH_SIZE -d <out> -o pmc -- python3 bench.py --one-pass --sets 4")
    print("  timeout -s KILL 120 rocprofv3 --pmc WRITE_SIZE -d <out> -o pmc -- python3 bench.py --one-pass --sets 4")
    print("  python3 bench.py --pmc-summary <FETCH run>/pmc_results.db <WRITE run>/pmc_results.db --unique-ids %d" % unique_ids)
    print("(--one-pass: plain launches of the cfg-2 sweep over 4 buffer sets, each preceded by the library's copy kernel on a")
    print(" 16 MiB tensor, once with streaming (non-temporal) and once with plain accesses; then the cfg-3 lookup kernels and")
    print(" the cfg-4 PickNegLogSoftmax kernels on 4 buffer sets each; then the kernels of one cfg-5 timestep (H = 1024, B = 128,")
    print(" packed operands) and the weight-gradient GEMM 4096x1024x4480.  KiB per dispatch, averaged, from the rocpd database.)")
    print()
    print("calibration: the copy kernel moves %.0f KiB each way." % kib)
    print("  streaming accesses: FETCH_SIZE reads %.1f, WRITE_SIZE reads %.1f" % (cs[1], cs[2]))
    if cp:
        print("  plain accesses:     FETCH_SIZE reads %.1f, WRITE_SIZE reads %.1f" % (cp[1], cp[2]))
        print("  -> the FETCH_SIZE ratio to the bytes moved is %.4f with streaming loads and %.4f with plain loads: the counter's"
              % (cs[1] / kib, cp[1] / kib))
        print("     scale does not depend on the kind of load, so one factor applies to every kernel below.")
    print("  -> scale factors: FETCH x %.4f, WRITE x %.4f" % (ff, fw))
    print()
    print("%-28s %6s %12s %12s %12s %15s %8s" % ("kernel", "calls", "FETCH KiB", "WRITE KiB", "scaled MB", "algorithmic MB", "ratio"))
    traffic = {}
    for name in sorted(rows):
        calls, fk, wk = rows[name]
        scaled = (fk * ff + wk * fw) * 1024.0
        traffic[name] = scaled
        al = algo.get(name)
        print("%-28s %6d %12.1f %12.1f %12.2f %15s %8s" % (name, calls, fk, wk, scaled / 1e6,
                                                         "%.2f" % (al / 1e6) if al else "-",
                                                         "%.3f" % (scaled / al) if al else "-"))
    print()
    print("bench entries (layer_norm_bwd = main kernel + its combine launch; both cmult_bwd calls launch one kernel):")
    t = dict(traffic)
    if "layer_norm_bwd_main" in t:
        t["layer_norm_bwd"] = t.pop("layer_norm_bwd_main") + t.pop("layer_norm_bwd_combine", 0.0)
    if "layer_norm_wide_bwd_main" in t:
        t["layer_norm_wide_bwd"] = t.pop("layer_norm_wide_bwd_main") + t.pop("layer_norm_wide_bwd_combine", 0.0)
    if "cmult_bwd" in t:
        t["cmult_bwd_arg0"] = t["cmult_bwd_arg1"] = t.pop("cmult_bwd")
    for name in sorted(t):
        if not name.startswith("copy_"):
            print("TRAFFIC %s %.0f" % (name, t[name]))


def lstm_one_pass(dev, launches=4):
    """For the counter runs: the kernels of one cfg-5 timestep (H = 1024, B = 128) on packed operands and the
    weight-gradient GEMM over all timesteps (4096 x 1024 x 4480, accumulating), `launches` plain launches each."""
    H, B, T = 1024, 128, 35
    Wh = dev.empty((H, 4 * H))
    h, c, c2, hh, dh, dc, dc2 = (dev.empty((B, H)) for _ in range(7))
    xp, g, dpre = (dev.empty((B, 4 * H)) for _ in range(3))
    bias = dev.empty((4 * H,))
    for t in (Wh, h, c, dh, dc, xp, bias):
        dev.randomize_normal(t, 0.0, 0.1)
    pk, pkT = dev.empty((4 * H * H,)), dev.empty((4 * H * H,))
    dev.lstm_pack_recurrent(H, Wh, pk)
    dev.lstm_pack_recurrent_transposed(H, Wh, pkT)
    nh, nd = dev.lstm_packed_state_floats(H, B), dev.lstm_packed_state_floats(4 * H, B)
    hp_in, hp_out, dpp = dev.empty((nh,)), dev.empty((nh,)), dev.empty((nd,))
    dev.lstm_pack_state(H, B, h, hp_in)
    _, bb = dev.lstm_cell_workspace(H, B)
    wb, _ = dev.workspace(bb)
    dev.lstm_step_forward_packed(H, B, pk, hp_in, xp, bias, c, g, c2, hh, hp_out)
    nb = 0
    for _ in range(launches):
        dev.lstm_step_forward_packed(H, B, pk, hp_in, xp, bias, c, g, c2, hh, hp_out)
        dev.lstm_cell_backward_packed(H, B, g, c2, c, dh, wb if nb else None, nb, dc, dpre, dc2, dpp)
        nb = dev.lstm_recurrent_backward_packed(H, B, pkT, dpp, wb, bb)
    pkT16 = dev.empty((4 * H * H,))
    dev.lstm_pack_recurrent_transposed16(H, Wh, pkT16)
    nd16 = dev.lstm_packed_state16_floats(4 * H, B)
    dp_in, dp_out = dev.empty((nd16,)), dev.empty((nd16,))
    dev.lstm_pack_state16(4 * H, B, dpre, dp_in)
    for _ in range(launches):
        dev.lstm_step_backward_packed(H, B, pkT16, dp_in, g, c2, c, dh, dc, dpre, dc2, dp_out)
    N = T * B
    a, b, y = dev.empty((N, 4 * H)), dev.empty((N, H)), dev.empty((H, 4 * H))
    for t in (a, b, y):
        dev.randomize_normal(t, 0.0, 0.1)
    for _ in range(launches):
        dev.gemm_nt_acc(4 * H, H, N, a, b, y)
    dev.sync()


def lstm_lm(steps, warmup=12, use_graph=True):
    """cfg 5: whole training step of the 2-layer LSTM LM (forward, backward, clip, SGD update), tokens/s."""
    from dynet_amd import Device
    from dynet_amd.lm import LstmLM
    from dynet_amd.synth import zipf_ids

    V, E, H, L, B, T = 10000, 256, 1024, 2, 128, 35
    rng = np.random.default_rng(0)
    batches = [zipf_ids(rng, (T + 1) * B, V).reshape(T + 1, B) for _ in range(8)]
    flops = 3 * T * (2 * 4 * H * (E + H) * B + 2 * 4 * H * (H + H) * B + 2 * V * H * B)
    res = {"config": {"V": V, "E": E, "H": H, "layers": L, "B": B, "T": T, "trainer": "SimpleSGD lr 0.1",
                      "clip_threshold": 5.0, "init": "Glorot (lookup: embedding dim only), LSTM biases 0",
                      "ids": "Zipf(1.1)"},
           "tokens_per_step": T * B, "gemm_flop_per_step": flops,
           "fused_path_schedule": "one device queue, layer by layer; a forward timestep is one kernel (recurrent "
                                  "product + cell update) and so is a backward one (Wh^T dpre of the step above + "
                                  "cell backward), operands handed from timestep to timestep in matrix-core "
                                  "fragment order",
           "node_path_schedule": "the three fused LSTM nodes per layer and timestep, every backward argument its own "
                                 "call; the gates nodes' backward calls for Wx, Wh and b record their operands and the "
                                 "T recorded products of a parameter are formed as one product over the gathered "
                                 "operands where the executor hands the gradient to the parameter "
                                 "(node_at_a_time_path); node_at_a_time_path_weight_gradients_per_node forms them "
                                 "node by node, T products of depth B each",
           "timed_region": "per step: host->device copy of ids and labels, id sort, forward, backward, "
                           "device-side clipping, update; one HIP-graph replay per step; loss read back after "
                           "the last step"}
    # Each path is measured on two instances (device, model and graph built afresh); both times are reported and
    # ms_per_step is the faster one.  The collector is off inside the timed loop: in this process, which holds the
    # tables of every earlier leg, one full collection is a 5-10 ms pause of the host thread that launches the steps
    # (7.1 instead of 6.6 ms per step over 30 steps; a kernel trace shows equal kernel durations either way).
    for path, tb in (("fused", True), ("fused_dropout", True), ("nodes", False), ("nodes_eager", False)):
        runs = []
        for _ in range(1 if path == "fused_dropout" else 2):
            dev = Device(0, mem_mb=(1024, 1024, 512, 1024))
            drop = 0.5 if path == "fused_dropout" else 0.0  # CompactVanillaLSTMBuilder::set_dropout(d, d_h)
            lm = LstmLM(dev, V, E, H, L, B, T, lr=0.1, clip=5.0, time_batched=tb, path=path.split("_")[0],
                        defer_weight_grads=path == "nodes", dropout=drop, dropout_h=drop)
            lm.stage(batches[0])
            if use_graph:
                lm.capture()
            first = None
            for i in range(warmup):
                loss = lm.step(batches[i % len(batches)])
                first = loss if first is None else first
            dev.sync()
            gc.collect()
            gc.disable()
            t0 = time.perf_counter()
            for i in range(steps):
                lm.step(batches[(warmup + i) % len(batches)], read_loss=False)
            dev.sync()
            dt = (time.perf_counter() - t0) / steps
            gc.enable()
            last = float(lm.loss.numpy()[0])
            runs.append((dt, first, last))
            if lm.graph is not None:
                lm.graph.destroy()
            dev.close()
        dt, first, last = min(runs)
        key = {"fused": "fused_cell_path", "fused_dropout": "fused_cell_path_with_dropout_0.5_0.5", "nodes": "node_at_a_time_path",
               "nodes_eager": "node_at_a_time_path_weight_gradients_per_node"}[path]
        res[key] = {"ms_per_step": round(dt * 1e3, 3), "tokens_per_s": round(T * B / dt, 1),
                    "ms_per_step_of_each_instance": [round(r[0] * 1e3, 3) for r in runs],
                    "gemm_tflops": round(flops / dt / 1e12, 2),
                    "frac_of_fp32_mfma_peak": round(flops / dt / 1e12 / FP32_MFMA_PEAK_TFLOPS, 4),
                    "steps": steps, "loss_per_token_first": round(first / (T * B), 4),
                    "loss_per_token_last": round(last / (T * B), 4)}
    return res


def lm_kernels(reps, use_graph=True):
    """The GEMMs and the non-GEMM kernels of the cfg-5 step at their in-situ shapes: TFLOP/s against the fp32
    MFMA peak, GB/s against the HBM peak."""
    from dynet_amd import Device, lib

    V, E, H, B, T = 10000, 256, 1024, 128, 35
    N = T * B
    dev = Device(0, mem_mb=(2048, 1024, 64, 1024))
    out = {"gemm": [], "kernels": []}
    shapes = [("input projection, layer 1 (NN)", "nn", 4 * H, N, H), ("input projection, layer 0 (NN)", "nn", 4 * H, N, E),
              ("output projection (NN, bias epilogue)", "affine", V, N, H), ("d h_top = R^T dlogits (TN)", "tn", H, N, V),
              ("dR = dlogits h^T (NT)", "nt", V, H, N), ("dWx1 / dWh = dpre x^T (NT)", "nt", 4 * H, H, N),
              ("dx = Wx^T dpre (TN)", "tn", H, N, 4 * H), ("dWx0 (NT)", "nt", 4 * H, E, N),
              ("dWh of one timestep = dpre h^T (NT, depth = batch; node-at-a-time path)", "nt", 4 * H, H, B),
              ("recurrent Wh h, one timestep (NN, split-K slices)", "rec_f", 4 * H, B, H),
              ("recurrent Wh^T dpre, one timestep (TN, depth-range slices, plain operands)", "rec_b", H, B, 4 * H)]
    for name, form, M, Nn, K in shapes:
        a, b, y = dev.empty((M * K,)), dev.empty((Nn * K,)), dev.empty((M * Nn,))
        bias = dev.empty((M,))
        # random operands: constant fills switch few bits in the matrix cores, and the clock under them is ~10 % higher
        for t in (a, b, bias):
            dev.randomize_normal(t, 0.0, 0.1)
        fb, bb = dev.lstm_cell_workspace(H, B)
        ws, _ = dev.workspace(max(fb, bb))
        fn = {"nn": lambda: dev.gemm_nn(M, Nn, K, a, b, 0.0, y), "tn": lambda: dev.gemm_tn(M, Nn, K, a, b, 0.0, y),
              "nt": lambda: dev.gemm_nt(M, Nn, K, a, b, 0.0, y), "affine": lambda: dev.affine_forward(M, Nn, K, bias, a, b, y),
              "rec_f": lambda: dev.lstm_recurrent_forward(H, B, a, b, ws, fb),
              "rec_b": lambda: dev.lstm_recurrent_backward(H, B, a, b, ws, bb)}[form]
        if use_graph:
            g = capture(dev, [fn] * 4)
            us = time_graph(dev, g, reps, 4)
            g.destroy()
        else:
            us = time_loop(dev, [fn], reps)
        tf = 2.0 * M * Nn * K / us / 1e6
        out["gemm"].append({"gemm": name, "M": M, "N": Nn, "K": K, "us": round(us, 2), "TFLOPs": round(tf, 1),
                            "frac_of_fp32_mfma_peak": round(tf / FP32_MFMA_PEAK_TFLOPS, 4)})
        for w in (lib.POOL_FXS, lib.POOL_SCS):
            dev.sync()
            dev.free_pool(w)
    # fused cell kernels at H = 1024, B = 128 with the split counts the recurrent GEMMs produce
    Wh, h, dpre = dev.empty((H, 4 * H)), dev.empty((B, H)), dev.empty((B, 4 * H))
    xp, bb_, c, c2, hh, g = (dev.empty(s) for s in ((B, 4 * H), (4 * H,), (B, H), (B, H), (B, H), (B, 4 * H)))
    dh, dc, dc2 = dev.empty((B, H)), dev.empty((B, H)), dev.empty((B, H))
    for t in (Wh, h, dpre, xp, bb_, c, dh, dc):
        dev.constant(t, 0.01)
    fb, bb = dev.lstm_cell_workspace(H, B)
    wf, _ = dev.workspace(fb)
    wb, _ = dev.workspace(bb)
    nf = dev.lstm_recurrent_forward(H, B, Wh, h, wf, fb)
    nb = dev.lstm_recurrent_backward(H, B, Wh, dpre, wb, bb)
    dev.lstm_cell_forward(H, B, xp, bb_, wf, nf, c, g, c2, hh)
    named = [("lstm_cell_fwd (%d slices)" % nf, (4 * (1 + nf) * H * B + 4 * H + 7 * H * B) * 4,
              lambda s: dev.lstm_cell_forward(H, B, xp, bb_, wf, nf, c, g, c2, hh)),
             ("lstm_cell_bwd (%d slices)" % nb, ((4 + 4 + nb + 4 + 1) * H * B) * 4,
              lambda s: dev.lstm_cell_backward(H, B, g, c2, c, dh, wb, nb, dc, dpre, dc2))]
    out["kernels"] = per_kernel_table(dev, named, [None] * 4, reps, use_graph=use_graph)
    # single-launch forward timestep: product and cell update in one kernel, Wh read from its packed copy
    pk = dev.empty((4 * H * H,))
    dev.lstm_pack_recurrent(H, Wh, pk)
    nh, nd = dev.lstm_packed_state_floats(H, B), dev.lstm_packed_state_floats(4 * H, B)
    hp_in, hp_out, dpp = dev.empty((nh,)), dev.empty((nh,)), dev.empty((nd,))
    dev.lstm_pack_state(H, B, h, hp_in)
    step = lambda: dev.lstm_step_forward_packed(H, B, pk, hp_in, xp, bb_, c, g, c2, hh, hp_out)
    pack = lambda: dev.lstm_pack_recurrent(H, Wh, pk)
    # backward timestep over packed operands: cell kernel (dpre plain and packed), then the slices of Wh^T dpre
    pkT = dev.empty((4 * H * H,))
    dev.lstm_pack_recurrent_transposed(H, Wh, pkT)
    dev.lstm_cell_backward_packed(H, B, g, c2, c, dh, None, 0, dc, dpre, dc2, dpp)
    nbp = dev.lstm_recurrent_backward_packed(H, B, pkT, dpp, wb, bb)
    rec_bwd = lambda: dev.lstm_recurrent_backward_packed(H, B, pkT, dpp, wb, bb)
    # the same backward timestep as one launch (what the fused path issues): 16x16x4 fragment order
    pkT16 = dev.empty((4 * H * H,))
    dev.lstm_pack_recurrent_transposed16(H, Wh, pkT16)
    nd16 = dev.lstm_packed_state16_floats(4 * H, B)
    dp16_in, dp16_out = dev.empty((nd16,)), dev.empty((nd16,))
    dev.lstm_pack_state16(4 * H, B, dpre, dp16_in)
    step_bwd = lambda: dev.lstm_step_backward_packed(H, B, pkT16, dp16_in, g, c2, c, dh, dc, dpre, dc2, dp16_out)
    cell_bwd = lambda: dev.lstm_cell_backward_packed(H, B, g, c2, c, dh, wb, nbp, dc, dpre, dc2, dpp)
    for name, fn, flops, nbytes in (("lstm_step_fwd (recurrent product + cell update)", step, 2.0 * 4 * H * H * B,
                                     (4 * H * H + H * B + 4 * H * B + 4 * H + H * B + 7 * H * B) * 4),
                                    ("lstm_step_bwd (Wh^T dpre over the whole depth + cell backward, one launch)", step_bwd,
                                     2.0 * 4 * H * H * B, (4 * H * H + 4 * H * B + 17 * H * B) * 4),
                                    ("lstm_rec_bwd (Wh^T dpre from packed operands, %d slices)" % nbp, rec_bwd,
                                     2.0 * 4 * H * H * B, (4 * H * H + 4 * H * B + nbp * H * B) * 4),
                                    ("lstm_cell_bwd_packed (%d slices, dpre plain + packed)" % nbp, cell_bwd, 0.0,
                                     ((4 + 4 + nbp + 4 + 4 + 1) * H * B) * 4),
                                    ("lstm_pack_recurrent (once per layer per step)", pack, 0.0, 2 * 4 * H * H * 4)):
        if use_graph:
            gr = capture(dev, [fn] * 4)
            us = time_graph(dev, gr, reps, 4)
            gr.destroy()
        else:
            us = time_loop(dev, [fn], reps)
        row = {"kernel": name, "bytes": nbytes, "us": round(us, 3), "GBps": round(nbytes / us / 1e3, 1),
               "frac_of_8TBps": round(nbytes / us / 1e3 / HBM_PEAK_GBPS, 4)}
        if flops:
            row["TFLOPs"] = round(flops / us / 1e6, 1)
            row["frac_of_fp32_mfma_peak"] = round(flops / us / 1e6 / FP32_MFMA_PEAK_TFLOPS, 4)
        out["kernels"].append(row)
    dev.close()
    return out


class _OneCore:
    """Pins the process to one host core for the duration (the CPU legs are single-threaded C)."""

    def __enter__(self):
        self.allowed, self.cpu = None, None
        try:
            self.allowed = sorted(os.sched_getaffinity(0))
            self.cpu = self.allowed[len(self.allowed) // 2]
            os.sched_setaffinity(0, {self.cpu})
        except (AttributeError, OSError):
            self.allowed = None
        return self

    def __exit__(self, *exc):
        if self.allowed is not None:
            os.sched_setaffinity(0, set(self.allowed))
        return False


def _time_cpu(fn, seconds, max_reps):
    fn()
    reps, t0 = 0, time.perf_counter()
    while True:
        fn()
        reps += 1
        el = time.perf_counter() - t0
        if el >= seconds or reps >= max_reps:
            return el / reps, reps


def cpu_baseline_per_config(seconds):
    """The CPU oracle on configurations 1, 3, 4 at their full sizes and on a reduced configuration 5, each on one
    pinned host core, the C functions called into preallocated outputs; `seconds` bounds each leg."""
    import ctypes as C

    from dynet_amd.synth import glorot, zipf_ids
    from oracle import cpu_oracle as orc
    from oracle import lm_oracle

    L = orc._lib
    rng = np.random.default_rng(0)
    f = lambda a: np.ascontiguousarray(a, dtype=np.float32)  # noqa: E731
    fp = lambda a: a.ctypes.data_as(C.POINTER(C.c_float))  # noqa: E731
    up = lambda a: a.ctypes.data_as(C.POINTER(C.c_uint))  # noqa: E731
    out = {"cores": 1, "kind": "port", "library": "oracle/libdynet_cpu_oracle.so"}
    with _OneCore() as core:
        out["pinned_to_cpu"] = core.cpu
        # ---- cfg 1: VanillaLSTMGates + C + H, forward and every backward argument ------------------------------
        I, H, B = 128, 256, 32
        x, h, c, dh = (f(rng.standard_normal((B, d))) for d in (I, H, H, H))
        Wx, Wh, b = f(glorot(rng, 4 * H, I)), f(glorot(rng, 4 * H, H)), np.zeros(4 * H, np.float32)
        fx, c2, h2 = np.empty((B, 4 * H), np.float32), np.empty((B, H), np.float32), np.empty((B, H), np.float32)
        dgates, dct, dcp = np.zeros((B, 4 * H), np.float32), np.zeros((B, H), np.float32), np.zeros((B, H), np.float32)
        outs = [np.zeros(sh, np.float32) for sh in ((B, I), (B, H), (I, 4 * H), (H, 4 * H), (4 * H,))]
        xs = (C.POINTER(C.c_float) * 1)(fp(x))
        dims = (C.c_uint * 1)(I)
        none = C.POINTER(C.c_float)()

        def cell():
            L.orc_lstm_gates_forward(1, xs, dims, H, B, fp(h), fp(Wx), fp(Wh), fp(b), none, 0, none, 0,
                                     orc.LOGISTIC_PACKET, fp(fx))
            L.orc_lstm_c_forward(H, B, fp(c), fp(fx), fp(c2))
            L.orc_lstm_h_forward(H, B, fp(c2), fp(fx), fp(h2))
            L.orc_lstm_h_backward(H, B, fp(c2), fp(fx), fp(dh), 0, fp(dct))
            L.orc_lstm_h_backward(H, B, fp(c2), fp(fx), fp(dh), 1, fp(dgates))
            L.orc_lstm_c_backward(H, B, fp(c), fp(fx), fp(dct), 0, fp(dcp))
            L.orc_lstm_c_backward(H, B, fp(c), fp(fx), fp(dct), 1, fp(dgates))
            for i, o in enumerate(outs):
                L.orc_lstm_gates_backward(1, xs, dims, H, B, fp(h), fp(Wx), fp(Wh), none, 0, none, 0, fp(fx), fp(dgates),
                                          i, fp(o))

        dt, reps = _time_cpu(cell, seconds, 2000)
        out["cfg1_lstm_cell"] = {"I": I, "H": H, "B": B, "fwd_bwd_us": round(dt * 1e6, 1), "reps": reps,
                                 "what": "gates, C, H forward; H and C backward (both arguments); gates backward for all "
                                         "five arguments, each recomputing the activation derivative as the reference does"}
        # ---- cfg 3: gather + scatter-add -----------------------------------------------------------------------
        V, D, n = CFG3["V"], CFG3["D"], CFG3["n"]
        ids = np.ascontiguousarray(zipf_ids(rng, n, V), dtype=np.uint32)
        table, g = f(rng.uniform(-0.1, 0.1, (V, D))), f(rng.standard_normal((n, D)))
        fxl, grads = np.empty((n, D), np.float32), np.zeros((V, D), np.float32)
        G, uniq = n * D * 4, int(np.unique(ids).size)
        dt_g, r1 = _time_cpu(lambda: L.orc_lookup_forward(n, up(ids), C.c_size_t(D), V, fp(table), C.c_float(1.0), fp(fxl)),
                             seconds / 2, 200)
        dt_s, r2 = _time_cpu(lambda: L.orc_lookup_accumulate_grads(n, up(ids), C.c_size_t(D), V, fp(g), fp(grads)),
                             seconds / 2, 200)
        out["cfg3_lookup"] = {"vocab": V, "dim": D, "n_ids": n, "unique_ids": uniq,
                              "gather_ms": round(dt_g * 1e3, 3), "gather_GBps": round((2 * G + 4 * n) / dt_g / 1e9, 2),
                              "scatter_add_ms": round(dt_s * 1e3, 3),
                              "scatter_add_GBps": round((G + 2 * uniq * D * 4) / dt_s / 1e9, 2), "reps": [r1, r2]}
        del table, g, fxl, grads
        # ---- cfg 4: PickNegLogSoftmax forward + backward -------------------------------------------------------
        rows, bd = CFG4["rows"], CFG4["bd"]
        xl = f(rng.standard_normal((bd, rows)) * 2)
        labels = rng.integers(0, rows, bd).astype(np.uint32)
        aux, err, dy = np.empty(3 * bd, np.float32), np.empty(bd, np.float32), f(rng.standard_normal(bd))
        dxl = np.zeros((bd, rows), np.float32)
        X = rows * bd * 4
        vp = lambda a: a.ctypes.data_as(C.c_void_p)  # noqa: E731
        dt_f, r1 = _time_cpu(lambda: L.orc_pnls_forward(C.c_size_t(rows), bd, fp(xl), up(labels), vp(aux), fp(err)),
                             seconds / 2, 50)
        dt_b, r2 = _time_cpu(lambda: L.orc_pnls_backward(C.c_size_t(rows), bd, fp(xl), vp(aux), fp(dy), fp(dxl)),
                             seconds / 2, 50)
        out["cfg4_pnls"] = {"rows": rows, "bd": bd, "fwd_ms": round(dt_f * 1e3, 2), "fwd_GBps": round(X / dt_f / 1e9, 2),
                            "bwd_ms": round(dt_b * 1e3, 2), "bwd_GBps": round(3 * X / dt_b / 1e9, 2), "reps": [r1, r2]}
        del xl, dxl
        # ---- cfg 5 at a reduced size (the oracle's matrix products are plain triple loops) ----------------------
        V5, E5, H5, L5, B5, T5 = 1000, 64, 128, 2, 16, 8
        from dynet_amd.lm import LstmLM

        params = LstmLM.init_params(V5, E5, H5, L5, seed=3)
        tokens = zipf_ids(rng, (T5 + 1) * B5, V5).reshape(T5 + 1, B5).astype(np.uint32)
        dt5, r5 = _time_cpu(lambda: lm_oracle.step(params, tokens, L5), seconds, 20)
        flops = 3 * T5 * (2 * 4 * H5 * (E5 + H5) * B5 + 2 * 4 * H5 * (H5 + H5) * B5 + 2 * V5 * H5 * B5)
        out["cfg5_lstm_lm_reduced"] = {
            "V": V5, "E": E5, "H": H5, "layers": L5, "B": B5, "T": T5, "ms_per_step": round(dt5 * 1e3, 2),
            "tokens_per_s": round(T5 * B5 / dt5, 1), "gemm_gflops": round(flops / dt5 / 1e9, 2), "reps": r5,
            "note": "timed at this reduced size; the full configuration (V 10000, E 256, H 1024, B 128, T 35) has %.0f "
                    "times the matrix-product work" % (3 * 35 * (2 * 4 * 1024 * 1280 * 128 + 2 * 4 * 1024 * 2048 * 128
                                                                   + 2 * 10000 * 1024 * 128) / flops)}
    return out


def cpu_baseline(step_bytes, seconds):
    """The CPU oracle (plain-C restatement of DyNet's CPU path) on the same sweep: one host core (the process is
    pinned to it for the duration), the C functions called directly into preallocated outputs."""
    import ctypes as C

    from oracle import cpu_oracle as orc

    L = orc._lib
    rng = np.random.default_rng(0)
    x = rng.standard_normal(S_ELEMS).astype(np.float32)
    x2 = rng.standard_normal(S_ELEMS).astype(np.float32)
    dy = rng.standard_normal(S_ELEMS).astype(np.float32)
    dx, y = np.zeros(S_ELEMS, np.float32), np.empty(S_ELEMS, np.float32)
    s_out = np.empty(SB_N, np.float32)
    g = rng.uniform(0.5, 1.5, LN_N).astype(np.float32)
    b = (rng.standard_normal(LN_N) * 0.1).astype(np.float32)
    dg, db = np.zeros(LN_N, np.float32), np.zeros(LN_N, np.float32)
    fp = lambda a: a.ctypes.data_as(C.POINTER(C.c_float))  # noqa: E731
    X, X2, DY, DX, Y, SO, G, B, DG, DB = (fp(a) for a in (x, x2, dy, dx, y, s_out, g, b, dg, db))
    n, one = C.c_size_t(S_ELEMS), C.c_uint(1)

    def sweep():
        for op in (orc.OP_TANH, orc.OP_LOGISTIC, orc.OP_RECTIFY):
            L.orc_unary_forward(op, orc.LOGISTIC_PACKET, n, X, Y)
            L.orc_unary_backward(op, n, Y, DY, DX)
        L.orc_cmult_forward(n, one, one, X, X2, Y)
        L.orc_cmult_backward(n, one, one, X, X2, DY, C.c_uint(0), DX)
        L.orc_cmult_backward(n, one, one, X, X2, DY, C.c_uint(1), DX)
        L.orc_sum_batches_forward(C.c_size_t(SB_N), C.c_uint(SB_BD), X, SO)
        L.orc_sum_batches_backward(C.c_size_t(SB_N), C.c_uint(SB_BD), SO, DX)
        L.orc_layer_norm_forward(C.c_size_t(LN_N), C.c_uint(LN_BD), X, G, B, Y)
        L.orc_layer_norm_backward(C.c_size_t(LN_N), C.c_uint(LN_BD), X, G, DY, DX, DG, DB)

    with _OneCore() as core:
        pinned = core.cpu
        dt, reps = _time_cpu(sweep, seconds, 50)
        el = dt * reps
    return {"value": round(step_bytes * reps / el / 1e9, 3), "unit": "GB/s", "cores": 1, "kind": "port",
            "sample": "%d full passes of the same cfg-2 sweep (4096x1024 fp32) through oracle/libdynet_cpu_oracle.so "
                      "in %.1f s on one host core (pinned to cpu %s) of %d" % (reps, el, pinned, os.cpu_count() or 0)}


def main():
    args = parse_args()
    if args.pmc_summary:
        uniq = args.unique_ids
        if uniq is None:
            from dynet_amd.synth import zipf_ids

            uniq = int(np.unique(zipf_ids(np.random.default_rng(0), CFG3["n"], CFG3["V"])).size)
        print_pmc_summary(args.pmc_summary[0], args.pmc_summary[1], uniq)
        return
    if args.gpus != 1:
        print("bench.py measures one GPU: the hot path has no multi-GPU leg (it would shard along the batch "
              "dimension with one gradient all-reduce per step). Run with --gpus 1.", file=sys.stderr)
        sys.exit(2)
    from dynet_amd import Device, lib

    traced = "rocprofiler" in os.environ.get("LD_PRELOAD", "") or bool(os.environ.get("ROCP_TOOL_LIBRARIES"))
    if traced and not args.no_graph and not args.one_pass:
        # the kernel tracer of this ROCm release crashes on the host once ~32k graph-launched kernels have
        # been replayed in one process; the per-dispatch durations it records do not need graphs anyway
        print("bench.py: running under rocprofiler, switching to plain launches (--no-graph)", file=sys.stderr)
        args.no_graph = True
    dev = Device(0, mem_mb=(2560, 2048, 64, 256))  # pools grow on demand (cfg 3 takes ~1.4 GB + 0.8 GB)
    if args.stream_threshold is not None:
        dev.set_stream_threshold(args.stream_threshold)
    sweep = Sweep(dev, lib, args.sets)
    if args.one_pass:
        # hardware-counter runs (rocprofv3 --pmc ...): plain launches so that every dispatch is attributed
        default_threshold = 8 << 20
        for r in range(min(4, sweep.R)):
            b = sweep.sets[r]
            # calibration: reads 16 MiB, writes 16 MiB; with streaming accesses, then with plain ones
            dev.scale_copy(S_ELEMS, b["x"], 1.0, b["y"])
            dev.set_stream_threshold(1 << 62)
            dev.scale_copy(S_ELEMS, b["x"], 1.0, b["y"])
            dev.set_stream_threshold(args.stream_threshold if args.stream_threshold is not None else default_threshold)
            sweep.run_step(r)
        dev.sync()
        for w in (lib.POOL_FXS, lib.POOL_DEDFS, lib.POOL_SCS):
            dev.free_pool(w)
        for _, _, fns, sets in extras_kernels(dev, lib, n_sets=4):
            for st in sets:
                for kname, _, fn in fns:
                    if "plan + segmented" not in kname:  # the combined call repeats the two kernels timed apart
                        fn(st)
            dev.sync()
            for w in (lib.POOL_FXS, lib.POOL_DEDFS, lib.POOL_SCS):
                dev.free_pool(w)
        lstm_one_pass(dev)
        dev.close()
        print(json.dumps({"one_pass": True, "calibration": "ew_vec4_kernel<..IdentityFwd> moves 16384 KiB each way"}))
        return
    # ---- whole-step timing: one captured graph per buffer set ---------------------
    sweep.run_step(0)
    dev.sync()
    if args.no_graph:
        class _Eager:
            def __init__(self, r):
                self.r = r

            def launch(self):
                sweep.run_step(self.r)

            def destroy(self):
                pass

        graphs = [_Eager(r) for r in range(sweep.R)]
    else:
        graphs = [capture(dev, [lambda r=r: sweep.run_step(r)]) for r in range(sweep.R)]
    # Eight consecutive steps per graph where the step count allows: the boundary between two graph replays costs
    # about 5 us here (see per_kernel_table), 4 % of a 127 us step if every step is a replay of its own.  The rest of
    # the K steps, and the warmup, are single-step replays.
    G = 8
    multi = [] if args.no_graph or sweep.R % G else [
        capture(dev, [lambda r=r: sweep.run_step(r) for r in range(k, k + G)]) for k in range(0, sweep.R, G)]
    for s in range(args.warmup):
        graphs[s % sweep.R].launch()
    for g in multi:
        g.launch()
    dev.sync()
    t0 = time.perf_counter()
    dev.timer_start()
    s = 0
    while multi and args.steps - s >= G:
        multi[(s // G) % len(multi)].launch()
        s += G
    for s in range(s, args.steps):
        graphs[s % sweep.R].launch()
    ms = dev.timer_stop()
    dev.sync()
    wall_ms = (time.perf_counter() - t0) * 1e3
    ms_per_step = ms / args.steps
    value = sweep.step_bytes / (ms_per_step * 1e-3) / 1e9
    for g in graphs + multi:
        g.destroy()
    # ---- per-kernel achieved bandwidth ---------------------------------------------
    table = per_kernel_table(dev, sweep.kernels, sweep.sets, args.kernel_reps, use_graph=not args.no_graph)
    # The ceiling a kernel of this size can reach here: the library's plain copy (streaming 128-bit loads and stores,
    # nothing else) on the same 16.8 MB tensors, measured in the same way.  Every entry is also given as a fraction
    # of it: what is left above that fraction is the memory system and the fixed cost of a launch, not the kernel.
    copy = per_kernel_table(dev, [("copy", 2 * S_BYTES, lambda b: dev.scale_copy(S_ELEMS, b["x"], 1.0, b["y"]))],
                            sweep.sets, args.kernel_reps, use_graph=not args.no_graph)[0]
    for k in table:
        k["frac_of_copy_ceiling"] = round(k["GBps"] / copy["GBps"], 4)
    # the runtime's own device-to-device copy (hipMemcpyAsync through dyhip_memcpy_d2d: not one of this library's
    # kernels) on the same tensors, as a ceiling that does not share code with what it is a ceiling for
    copy_rt = per_kernel_table(dev, [("hipMemcpyAsync", 2 * S_BYTES, lambda b: dev.copy_d2d(b["y"], b["x"], S_BYTES))],
                               sweep.sets, args.kernel_reps, use_graph=not args.no_graph)[0]
    traffic_table = measured_traffic()
    # Dominant kernel = the device kernel with the largest share of the sweep's device time, as the first row
    # of a kernel-trace summary of the sweep would name it.  cmult_bwd_arg0 and cmult_bwd_arg1 launch the same
    # device kernel (ew_vec4_kernel<.., AccMul2>); every other row is a device kernel of its own, except
    # layer_norm_bwd, which is two dispatches (ln_bwd_wave_kernel + combine_partials_kernel) timed together.
    same_kernel = {"cmult_bwd_arg0": "cmult_bwd", "cmult_bwd_arg1": "cmult_bwd"}
    groups = {}
    for k in table:
        groups.setdefault(same_kernel.get(k["kernel"], k["kernel"]), []).append(k)

    def roofline_of(name, rows):
        us = sum(r["us"] for r in rows) / len(rows)
        nbytes = sum(r["bytes"] for r in rows) / len(rows)
        gbps = nbytes / us / 1e3
        traffic = [traffic_table.get(r["kernel"]) for r in rows]
        return {"bound": "hbm", "kernel": name, "achieved": round(gbps, 1), "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                "frac": round(gbps / HBM_PEAK_GBPS, 4),
                "traffic": None if None in traffic else sum(traffic) / len(traffic),
                "traffic_source": "profiles/" + os.path.basename(PMC_PROFILE) + " (offline counter runs, not this run)",
                "algorithmic_bytes_per_launch": int(nbytes), "avg_launch_us": round(us, 3),
                "launches_per_step": len(rows),
                "share_of_step_device_time": round(sum(r["us"] for r in rows) / sum(k["us"] for k in table), 4)}

    top = max(groups, key=lambda n: sum(r["us"] for r in groups[n]))
    roofline = roofline_of(top, groups[top])
    slowest = max(table, key=lambda k: k["us"])  # the longest single entry of the sweep (layer_norm_bwd)
    roofline_slowest = roofline_of(slowest["kernel"], [slowest])
    out = {
        "metric": "fused-kernel HBM GB/s (cfg-2 elementwise/reduction sweep, algorithmic bytes / device time)",
        "value": round(value, 1), "unit": "GB/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 5), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f32", "data": "synthetic",
        "config": {"workload": "cfg2_elementwise_reduction_sweep", "tensor": "4096x1024 fp32",
                   "kernels_per_step": len(sweep.kernels), "rotating_buffer_sets": sweep.R,
                   "steps_per_graph_replay": G if multi else 1,
                   "bytes_per_step": int(sweep.step_bytes)},
        "frac_of_hbm_peak": round(value / HBM_PEAK_GBPS, 4),
        "wall_ms_per_step": round(wall_ms / args.steps, 5),
        "roofline": roofline, "roofline_longest_entry": roofline_slowest,
        "hbm_copy_ceiling": {"kernel": "copy of one 4096x1024 fp32 tensor (streaming loads and stores)", "bytes": 2 * S_BYTES,
                             "us": copy["us"], "GBps": copy["GBps"], "frac_of_8TBps": copy["frac_of_8TBps"],
                             "runtime_memcpy_d2d": {"what": "hipMemcpyAsync device-to-device on the same rotating tensors",
                                                    "us": copy_rt["us"], "GBps": copy_rt["GBps"],
                                                    "frac_of_8TBps": copy_rt["frac_of_8TBps"]}},
        "kernels": table,
        # cfg 5, both paths named: the drop-in one (DyNet's nodes called one at a time, as its executor does) and the
        # time-batched / fused one, which needs a builder-level call sequence (the timesteps of a layer issued together)
        "lstm_lm_tokens_per_s_node_api": None, "lstm_lm_tokens_per_s_fused_path": None,
    }
    for w in (lib.POOL_FXS, lib.POOL_DEDFS, lib.POOL_SCS):
        dev.sync()
        dev.free_pool(w)
    if not args.no_extras:
        out.update(extras(dev, lib, args.kernel_reps, use_graph=not args.no_graph))
    dev.close()
    if not args.no_large:
        # the same kernels on tensors 16 times larger (65536 x 1024 fp32, 268 MB each): how much of the gap to the
        # HBM peak at the baseline's shape is the fixed cost of a launch
        dev = Device(0, mem_mb=(3584, 1280, 64, 256))
        if args.stream_threshold is not None:
            dev.set_stream_threshold(args.stream_threshold)
        big = Sweep(dev, lib, 2, scale=16)
        out["cfg2_sweep_16x_larger_tensors"] = {
            "tensor": "65536x1024 fp32", "rotating_buffer_sets": big.R,
            "kernels": per_kernel_table(dev, big.kernels, big.sets, max(4, args.kernel_reps // 4),
                                        use_graph=not args.no_graph)}
        dev.close()
    if not args.no_lm:
        out["cfg5_lstm_lm"] = lstm_lm(args.lm_steps, use_graph=not args.no_graph)
        out["cfg5_lstm_lm"]["in_situ"] = lm_kernels(args.kernel_reps, use_graph=not args.no_graph)
        out["lstm_lm_tokens_per_s_node_api"] = out["cfg5_lstm_lm"]["node_at_a_time_path"]["tokens_per_s"]
        out["lstm_lm_tokens_per_s_fused_path"] = out["cfg5_lstm_lm"]["fused_cell_path"]["tokens_per_s"]
    if not args.no_cpu_baseline:
        out["cpu_baseline_per_config"] = cpu_baseline_per_config(args.cpu_config_seconds)
        out["cpu_baseline"] = cpu_baseline(sweep.step_bytes, args.cpu_seconds)
    # the long tables first, the headline fields last: a reader who keeps only the end of the line keeps those
    head = ("metric", "value", "unit", "n_gpus", "steps", "warmup", "ms_per_step", "higher_is_better", "scaling",
            "vs_baseline", "dtype", "data", "config", "frac_of_hbm_peak", "wall_ms_per_step", "hbm_copy_ceiling",
            "lstm_lm_tokens_per_s_node_api", "lstm_lm_tokens_per_s_fused_path", "roofline_longest_entry", "roofline",
            "cpu_baseline")
    ordered = {k: v for k, v in out.items() if k not in head}
    ordered.update({k: out[k] for k in head if k in out})
    print(json.dumps(ordered))


if __name__ == "__main__":
    main()
