"""CPU oracle (test infrastructure, never the product path) for one training step of the batched LSTM
language model, composed node by node from the oracle's own functions in the order DyNet executes them:

  forward   examples/batching/rnnlm-batch.h:110-151  (per timestep: lookup, CompactVanillaLSTMBuilder::add_input_impl
            dynet/lstm.cc:1044-1080, i_bias + i_R * i_y_t, pickneglogsoftmax; then sum_batches(sum(errs)))
  backward  reverse topological order, every node's backward accumulating into its arguments' gradients
            (dynet/exec.cc:178-225)
  update    Trainer::update (dynet/training.cc:195-226): clip_gradients (:173-187) over
            ParameterCollection::gradient_l2_norm (dynet/model.cc:806-848), SimpleSGD rule (:619-637) with sparse
            lookup rows, then clear().

Parity of the composition is pinned by its parts (each node function has its own known-answer checks) and by
tests/test_oracle.py::test_lm_step_gradient_check, a central-difference check of the loss gradient in fp64-free
form (directional derivative against <grad, direction>).
"""
import numpy as np

from . import cpu_oracle as orc


def _mask_args(masks, l, B):
    """Keyword arguments of the gates node for layer l: the sequence's dropout masks (dynet/lstm.cc:964-982), or none."""
    if masks is None:
        return {}
    mx, mh = masks[l]
    return {"mask_x": mx, "mask_x_bd": B, "mask_h": mh, "mask_h_bd": B}


def forward(p, tokens, L, masks=None):
    """tokens[T+1, B]; masks = per layer (mask_x[B, d_in], mask_h[B, H]) for vanilla_lstm_gates_dropout
    (dynet/lstm.cc:1068-1073), or None.  Returns (loss, cache)."""
    T, B = tokens.shape[0] - 1, tokens.shape[1]
    V, E = p["C"].shape
    H = p["Wh0"].shape[0]
    zeros = np.zeros((B, H), np.float32)
    cache = {"emb": [], "gates": [[None] * L for _ in range(T)], "c": [[None] * L for _ in range(T)],
             "h": [[None] * L for _ in range(T)], "logits": [], "aux": [], "errs": []}
    for t in range(T):
        x = orc.lookup_forward(tokens[t], E, V, p["C"])
        cache["emb"].append(x)
        d_in = E
        for l in range(L):
            h_tm1 = cache["h"][t - 1][l] if t > 0 else zeros
            c_tm1 = cache["c"][t - 1][l] if t > 0 else zeros
            g = orc.lstm_gates_forward([x], [d_in], H, B, h_tm1, p[f"Wx{l}"], p[f"Wh{l}"], p[f"b{l}"],
                                       **_mask_args(masks, l, B))
            c = orc.lstm_c_forward(H, B, c_tm1, g)
            h = orc.lstm_h_forward(H, B, c, g)
            cache["gates"][t][l], cache["c"][t][l], cache["h"][t][l] = g, c, h
            x, d_in = h, H
        # i_bias + i_R * i_y_t: AffineTransform order (dynet/nodes-affinetransform.cc:77-113): bias first, GEMM added
        r = np.ascontiguousarray(np.broadcast_to(p["bias"], (B, V)), dtype=np.float32).copy()
        orc.gemm_nn(V, B, H, p["R"], x, 1.0, r)
        err, aux = orc.pnls_forward(V, B, r, tokens[t + 1])
        cache["logits"].append(r)
        cache["aux"].append(aux)
        cache["errs"].append(err)
    total = np.zeros(B, np.float32)
    for e in cache["errs"]:  # Sum node over the T error expressions
        total = (total + e).astype(np.float32)
    loss = orc.sum_batches_forward(1, B, total)[0]
    return loss, cache


def backward(p, tokens, L, cache, masks=None):
    T, B = tokens.shape[0] - 1, tokens.shape[1]
    V, E = p["C"].shape
    H = p["Wh0"].shape[0]
    g = {n: np.zeros_like(a) for n, a in p.items()}
    zeros = np.zeros((B, H), np.float32)
    d_h = [[np.zeros((B, H), np.float32) for _ in range(L)] for _ in range(T)]
    d_c = [[np.zeros((B, H), np.float32) for _ in range(L)] for _ in range(T)]
    ones = np.ones(B, np.float32)
    for t in reversed(range(T)):
        top = cache["h"][t][L - 1]
        d_r = np.zeros((B, V), np.float32)
        orc.pnls_backward(V, B, cache["logits"][t], cache["aux"][t], ones, d_r)
        orc.csum_backward(V, 1, B, d_r, 0, g["bias"])
        orc.gemm_nt_acc(V, H, B, d_r, top, g["R"])
        orc.gemm_tn_acc(H, B, V, p["R"], d_r, d_h[t][L - 1])
        d_x_below = None
        for l in reversed(range(L)):
            gates, c = cache["gates"][t][l], cache["c"][t][l]
            c_tm1 = cache["c"][t - 1][l] if t > 0 else zeros
            h_tm1 = cache["h"][t - 1][l] if t > 0 else zeros
            x, d_in = (cache["h"][t][l - 1], H) if l > 0 else (cache["emb"][t], E)
            d_g = np.zeros((B, 4 * H), np.float32)
            orc.lstm_h_backward(H, B, c, gates, d_h[t][l], 0, d_c[t][l])
            orc.lstm_h_backward(H, B, c, gates, d_h[t][l], 1, d_g)
            d_c_tm1 = d_c[t - 1][l] if t > 0 else np.zeros((B, H), np.float32)
            orc.lstm_c_backward(H, B, c_tm1, gates, d_c[t][l], 0, d_c_tm1)
            orc.lstm_c_backward(H, B, c_tm1, gates, d_c[t][l], 1, d_g)
            d_x = d_h[t][l - 1] if l > 0 else np.zeros((B, E), np.float32)
            d_h_tm1 = d_h[t - 1][l] if t > 0 else np.zeros((B, H), np.float32)
            args = ([x], [d_in], H, B, h_tm1, p[f"Wx{l}"], p[f"Wh{l}"], gates, d_g)
            mk = _mask_args(masks, l, B)
            orc.lstm_gates_backward(*args, 0, d_x, **mk)
            orc.lstm_gates_backward(*args, 1, d_h_tm1, **mk)
            orc.lstm_gates_backward(*args, 2, g[f"Wx{l}"], **mk)
            orc.lstm_gates_backward(*args, 3, g[f"Wh{l}"], **mk)
            orc.lstm_gates_backward(*args, 4, g[f"b{l}"], **mk)
            if l == 0:
                d_x_below = d_x
        orc.lookup_accumulate_grads(tokens[t], E, V, d_x_below, g["C"])
    return g


def update(p, g, tokens, lr, clip):
    """In place on p; returns the clip scale.  The lookup's norm and update run over the rows its gradient
    touched (non_zero_grads), everything else is dense."""
    names = [n for n in p if n != "C"]
    rows = np.unique(tokens[:-1])
    sq = np.float32(0)
    for n in names:
        sq = np.float32(sq + orc.squared_l2norm(g[n]))
    sq_c = np.float32(0)
    for r in rows:
        sq_c = np.float32(sq_c + orc.squared_l2norm(g["C"][r]))
    gg = np.sqrt(np.float32(sq + sq_c))
    gscale = np.float32(clip / gg) if (clip > 0 and gg > clip) else np.float32(1.0)
    for n in names:
        orc.sgd_update(p[n].reshape(-1), g[n].reshape(-1), lr, float(gscale), 1.0)
    for r in rows:
        orc.sgd_update(p["C"][r], g["C"][r], lr, float(gscale), 1.0)
    return gscale


def step(p, tokens, L, lr=0.1, clip=5.0, masks=None):
    """One training step; p is updated in place.  Returns (loss, grads before the update, clip scale)."""
    tokens = np.ascontiguousarray(tokens, dtype=np.uint32)
    loss, cache = forward(p, tokens, L, masks)
    g = backward(p, tokens, L, cache, masks)
    gscale = update(p, g, tokens, lr, clip)
    return loss, g, gscale
