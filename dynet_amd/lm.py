"""Batched LSTM language-model training step on the HIP device: the graph of
examples/batching/rnnlm-batch.h:86-151 (lookup -> CompactVanillaLSTMBuilder, dynet/lstm.cc:905-926,1044-1080
-> bias + R*h -> pickneglogsoftmax -> sum_batches(sum(errs))) followed by cg.backward and
SimpleSGDTrainer::update (dynet/training.cc:173-256,619-637), issued as one launch sequence and replayed as a
HIP graph.

What differs from DyNet's node-at-a-time execution (results agree to fp32 rounding):
  * the T lookups, the T projections and the T PickNegLogSoftmax nodes of a step run as one call each over
    T*B columns (what DyNet's autobatching does to them);
  * gradient clipping never leaves the device: squared norms -> clip scale -> update all read device memory;
  * ``path="nodes"`` issues the three fused LSTM nodes per layer and timestep exactly as
    CompactVanillaLSTMBuilder::add_input_impl does; with ``time_batched=True`` the weight/bias gradients of the
    gate GEMMs are formed once per layer over the K = T*B columns of all timesteps instead of T times over B;
    with ``defer_weight_grads=True`` every gates node's backward call for Wx, Wh and b only records its operands
    (they stay alive until the graph is freed), and the recorded products of a parameter are formed as one
    product over the gathered operands at the point where the executor hands the gradient to the parameter: what
    an adapter behind the unchanged node API can do (it sees one node at a time and does not know that its
    operands sit in one array here, so it gathers them);
  * ``path="fused"`` (default) runs layer by layer: one GEMM forms Wx*x for all timesteps, a timestep is then
    the recurrent GEMM Wh*h plus one cell kernel (gates + c + h); backward mirrors it, and dx, dWx, dWh, db are
    GEMMs/reductions over all timesteps;
  * a timestep of the fused path is one kernel forward (recurrent product + cell update) and one backward (Wh^T *
    dpre of the step above + cell backward), both reading their operands from packed copies in matrix-core
    fragment order that the previous timestep's kernel wrote (``single_launch``, where the sizes allow);
  * with ``overlap=True`` the fused path cuts the time axis into chunks and runs the layers as a pipeline on one
    queue per layer: layer l works on chunk k while layer l-1 is already on chunk k+1 (backward: l on chunk k, l+1
    on chunk k-1).  It paid off while a timestep's kernels left most of the GPU idle; the packed kernels keep the
    matrix cores of every CU busy on their own, two of them side by side only slow each other, and the default is
    one queue.

Dropout (``dropout`` / ``dropout_h`` > 0) is CompactVanillaLSTMBuilder's (dynet/lstm.cc:964-982,1068-1073): per layer
one input mask (d_in x B) and one recurrent mask (H x B), Bernoulli(retention) / retention, drawn once per sequence,
i.e. once per step here, on the device; the gates see x (.) mask_x and h_tm1 (.) mask_h at every timestep.  The node
path hands the masks to the gates node.  The fused path multiplies the layer's input by mask_x once for all
timesteps before the input product (and dx by it after the transposed product), the one-launch timesteps take mask_h
as an argument (the packed copy of h for the next timestep is written masked; the recurrent gradient passes through
the mask), and the weight gradients over all timesteps read the masked copies.
"""
import numpy as np

from . import lib
from .synth import glorot


class LstmLM:
    """V-word LM: embedding E, L layers of hidden H, batch B, T timesteps per step."""

    def __init__(self, dev, V, E, H, L, B, T, seed=0, lr=0.1, clip=5.0, time_batched=True, params=None, path="fused",
                 overlap=None, chunk=7, single_launch=None, dropout=0.0, dropout_h=None, defer_weight_grads=False):
        assert path in ("fused", "nodes")
        # node path: the weight and bias gradients of the gates nodes are not formed node by node (T products of
        # depth B into the same parameter gradient) but recorded and formed once, where the executor hands the
        # gradient to the parameter (ParameterNode::accumulate_grad, dynet/exec.cc:274-280)
        self.defer = bool(defer_weight_grads) and path == "nodes" and not time_batched
        self.dropout = float(dropout)
        self.dropout_h = self.dropout if dropout_h is None else float(dropout_h)
        assert 0.0 <= self.dropout < 1.0 and 0.0 <= self.dropout_h < 1.0
        self.use_dropout = self.dropout > 0.0 or self.dropout_h > 0.0
        self.overlap = False if overlap is None else bool(overlap)
        self.overlap = self.overlap and path == "fused" and L > 1 and not self.use_dropout
        self.chunk = max(1, int(chunk))
        self.dev, self.V, self.E, self.H, self.L, self.B, self.T = dev, V, E, H, L, B, T
        self.lr, self.clip, self.time_batched, self.path = float(lr), float(clip), bool(time_batched), path
        N = self.N = T * B
        PS, FXS, DE = lib.POOL_PS, lib.POOL_FXS, lib.POOL_DEDFS
        if params is None:
            params = self.init_params(V, E, H, L, seed)
        # parameters and their gradients (PS pool), names as in the reference model
        self.p, self.g = {}, {}
        # The dense parameters sit in one slab and their gradients in another (each tensor starts on a
        # 256-byte boundary, the gaps stay zero), so that the trainer's norm and update are one launch each
        # over the slab instead of one per parameter.  The lookup table is updated by rows and stays apart.
        self.dense = [n for n in params if n != "C"]
        pad = lambda k: (k + 63) // 64 * 64
        self.dense_elems = sum(pad(params[n].size) for n in self.dense)
        self.p_dense = dev.zeros((self.dense_elems,), pool=PS)
        self.g_dense = dev.zeros((self.dense_elems,), pool=PS)
        off = 0
        for name in self.dense:
            a = params[name]
            self.p[name] = self.p_dense.offset(off, a.shape).set(np.ascontiguousarray(a, dtype=np.float32))
            self.g[name] = self.g_dense.offset(off, a.shape)
            off += pad(a.size)
        self.p["C"] = dev.tensor(params["C"], pool=PS)
        self.g["C"] = dev.zeros(params["C"].shape, pool=PS)
        self.sqnorms = dev.zeros((2,), pool=PS)  # [dense slab, touched lookup rows]
        self.gscale = dev.zeros((1,), pool=PS)
        self.gnorm = dev.zeros((1,), pool=PS)  # gradient norm of the last step, for the host to check
        # forward values (FXS pool); [t] slices are contiguous so [T, B, *] is one matrix with T*B columns
        self.ids = dev.empty((N,), np.uint32, pool=FXS)
        self.emb = dev.empty((T, B, E), pool=FXS)
        self.h0 = dev.zeros((B, H), pool=FXS)  # zeros(): the initial h and c of every layer
        self.h = [dev.empty((T, B, H), pool=FXS) for _ in range(L)]
        self.c = [dev.empty((T, B, H), pool=FXS) for _ in range(L)]
        self.gates = [dev.empty((T, B, 4 * H), pool=FXS) for _ in range(L)]
        self.logits = dev.empty((N, V), pool=FXS)
        self.aux = dev.empty((3 * N,), pool=FXS)  # [z | m | ids] of PickNegLogSoftmax
        self.errs = dev.empty((N,), pool=FXS)
        self.loss = dev.empty((1,), pool=FXS)
        # dropout masks of the sequence, and the masked copies of every layer's input and state that the weight
        # gradients over all timesteps (and the fused path's input product) read
        self.mask_x, self.mask_h, self.xm, self.hm = [], [], [], []
        if self.use_dropout:
            for l in range(L):
                d_in = E if l == 0 else H
                self.mask_x.append(dev.empty((B, d_in), pool=FXS))
                self.mask_h.append(dev.empty((B, H), pool=FXS))
                self.xm.append(dev.empty((T, B, d_in), pool=FXS))
                self.hm.append(dev.empty((T, B, H), pool=FXS))
            self.dh_rec = dev.empty((B, H), pool=FXS)  # (Wh^T dpre) of one timestep where no one-launch step exists
        # gradients of the forward values (DEDFS pool), zeroed at the start of every backward pass
        self.de_begin = dev.pool(DE).used()
        self.d_errs = dev.empty((N,), pool=DE)
        self.d_logits = dev.empty((N, V), pool=DE)
        self.d_emb = dev.empty((T, B, E), pool=DE)
        self.d_h = [dev.empty((T, B, H), pool=DE) for _ in range(L)]
        self.d_c = [dev.empty((T, B, H), pool=DE) for _ in range(L)]
        self.d_gates = [dev.empty((T, B, 4 * H), pool=DE) for _ in range(L)]
        self.de_bytes = dev.pool(DE).used() - self.de_begin
        if self.defer:  # the gathered operands of a layer's recorded products
            self.gath_dpre = dev.empty((T, B, 4 * H), pool=DE)
            self.gath_x = dev.empty((T, B, max(E, H)), pool=DE)
            self.gath_h = dev.empty((T, B, H), pool=DE)
        self.d_pre = [dev.empty((T, B, 4 * H), pool=DE) for _ in range(L)]  # overwritten, never accumulated into
        fb, bb = dev.lstm_cell_workspace(H, B)
        self.rec_f_bytes, self.rec_b_bytes = fb, bb
        self.rec_f = [dev.workspace(fb)[0] for _ in range(L)]  # one per layer: layers run side by side
        self.rec_b = [dev.workspace(bb)[0] for _ in range(L)]
        # forward timesteps as one kernel each (recurrent product + cell update) where the size allows
        ok = path == "fused" and dev.lstm_step_supported(H, B)
        self.single_launch = ok if single_launch is None else (bool(single_launch) and ok)
        self.Wh_packed = [dev.empty((4 * H * H,), pool=PS) for _ in range(L)] if self.single_launch else []
        self.WhT_packed = [dev.empty((4 * H * H,), pool=PS) for _ in range(L)] if self.single_launch else []
        # packed copies of h and of dpre for the next timestep's recurrent product, two per layer used in turn
        nh = dev.lstm_packed_state_floats(H, B) if self.single_launch else 0
        nd = dev.lstm_packed_state16_floats(4 * H, B) if self.single_launch else 0
        self.h_packed = [[dev.empty((nh,), pool=FXS) for _ in range(2)] for _ in range(L)] if self.single_launch else []
        self.dpre_packed = [[dev.empty((nd,), pool=DE) for _ in range(2)] for _ in range(L)] if self.single_launch else []
        # queue l runs layer l; queue 0 is the device itself
        self.queues = [dev] + ([dev.fork() for _ in range(L - 1)] if self.overlap else [])
        self.plan, self.plan_ws, self.plan_ws_bytes = dev.lookup_plan_buffers(N, V)
        self.graph = None
        # page-locked staging for the ids and the flattened label offsets, two sets used in turn: a set is
        # rewritten only after a device sync that follows the copy that read it
        from .device import PinnedArray
        self._stage = [(PinnedArray((N,), np.uint32), PinnedArray((N,), np.uint32)) for _ in range(2)]
        self._stage_at = 0

    @staticmethod
    def init_params(V, E, H, L, seed=0):
        """ParameterInitGlorot as the reference model's constructors apply it (dynet/param-init.cc:26-40):
        lookup table scaled by its embedding dimension only, LSTM biases zero (dynet/lstm.cc:916)."""
        rng = np.random.default_rng(seed)
        s = np.sqrt(3.0) / np.sqrt(E)
        p = {"C": rng.uniform(-s, s, (V, E)).astype(np.float32)}
        d_in = E
        for l in range(L):
            p[f"Wx{l}"] = glorot(rng, 4 * H, d_in)
            p[f"Wh{l}"] = glorot(rng, 4 * H, H)
            p[f"b{l}"] = np.zeros(4 * H, np.float32)
            d_in = H
        p["R"] = glorot(rng, V, H)
        s = np.sqrt(3.0) / np.sqrt(V)
        p["bias"] = rng.uniform(-s, s, V).astype(np.float32)
        return p

    # ---- one step ---------------------------------------------------------------
    def stage(self, tokens):
        """Host -> device: tokens[T+1, B]; rows 0..T-1 are the inputs, rows 1..T the words to predict.
        Asynchronous copies from page-locked staging buffers; the host blocks only every second call."""
        tokens = np.ascontiguousarray(tokens, dtype=np.uint32)
        assert tokens.shape == (self.T + 1, self.B), tokens.shape
        if tokens.max() >= self.V:
            raise ValueError("token id out of the vocabulary")
        if self.N * self.V > 2 ** 32:
            raise ValueError("PickNegLogSoftmax indexes its input with 32-bit offsets")
        if self._stage_at == 0:
            self.dev.sync()  # both staging sets are free again
        ids, flat = self._stage[self._stage_at]
        self._stage_at ^= 1
        ids.array[:] = tokens[:-1].reshape(-1)
        flat.array[:] = (np.arange(self.N, dtype=np.uint64) * self.V + tokens[1:].reshape(-1)).astype(np.uint32)
        self.dev.copy_h2d_async(self.ids, ids)
        self.dev.copy_h2d_async(self.aux.offset(2 * self.N, (self.N,)), flat)

    def _t(self, buf, t, width):
        return buf.offset(t * self.B * width, (self.B, width))

    def draw_masks(self):
        """set_dropout_masks (dynet/lstm.cc:964-982): per layer the input mask, then the recurrent mask, each
        random_bernoulli(retention, 1 / retention) with one column per batch element."""
        for l in range(self.L):
            self.dev.randomize_bernoulli(self.mask_x[l], 1.0 - self.dropout, 1.0 / (1.0 - self.dropout))
            self.dev.randomize_bernoulli(self.mask_h[l], 1.0 - self.dropout_h, 1.0 / (1.0 - self.dropout_h))

    def _x_of(self, l):
        """(input of layer l over all timesteps as the gates see it, its width)."""
        if self.use_dropout:
            return self.xm[l], (self.H if l > 0 else self.E)
        return (self.h[l - 1], self.H) if l > 0 else (self.emb, self.E)

    def _mask_inputs(self, q, l):
        """xm[l] = input of layer l (.) mask_x[l], the mask broadcast over the timesteps."""
        x, d_in = (self.h[l - 1], self.H) if l > 0 else (self.emb, self.E)
        q.cmult_forward(self.B * d_in, self.T, 1, x, self.mask_x[l], self.xm[l])

    def forward(self):
        d, V, E, H, L, B, T, N = self.dev, self.V, self.E, self.H, self.L, self.B, self.T, self.N
        d.lookup_forward(None, self.ids, E, V, self.p["C"], self.emb)
        if self.path == "fused":
            self._forward_layers_fused()
        else:
            self._forward_layers_nodes()
        d.affine_forward(V, N, H, self.p["bias"], self.p["R"], self.h[L - 1], self.logits)
        d.pnls_forward_staged(V, N, self.logits, self.aux, self.errs)
        d.sum_batches_forward(1, N, self.errs, self.loss)

    def _chunks(self):
        return [(k, min(k + self.chunk, self.T)) for k in range(0, self.T, self.chunk)]

    def _cell_steps_forward(self, q, l, t0, t1):
        H, B = self.H, self.B
        for t in range(t0, t1):
            g = self._t(self.gates[l], t, 4 * H)
            if self.single_launch:
                hp = self.h_packed[l]
                q.lstm_step_forward_packed(H, B, self.Wh_packed[l] if t > 0 else None, hp[(t - 1) % 2] if t > 0 else None,
                                           g, self.p[f"b{l}"], self._t(self.c[l], t - 1, H) if t > 0 else None, g,
                                           self._t(self.c[l], t, H), self._t(self.h[l], t, H),
                                           hp[t % 2] if t + 1 < self.T else None,
                                           mask_h=self.mask_h[l] if self.use_dropout else None)
            elif t > 0:
                h_tm1 = self._t(self.h[l], t - 1, H)
                if self.use_dropout:  # the recurrent product reads h_tm1 (.) mask_h
                    q.cmult_forward(B * H, 1, 1, h_tm1, self.mask_h[l], self._t(self.hm[l], t - 1, H))
                    h_tm1 = self._t(self.hm[l], t - 1, H)
                n = q.lstm_recurrent_forward(H, B, self.p[f"Wh{l}"], h_tm1, self.rec_f[l],
                                             self.rec_f_bytes)
                q.lstm_cell_forward(H, B, g, self.p[f"b{l}"], self.rec_f[l], n, self._t(self.c[l], t - 1, H), g,
                                    self._t(self.c[l], t, H), self._t(self.h[l], t, H))
            else:
                q.lstm_cell_forward(H, B, g, self.p[f"b{l}"], None, 0, None, g, self._t(self.c[l], t, H),
                                    self._t(self.h[l], t, H))

    def _forward_layers_fused(self):
        d, E, H, L, B, T, N = self.dev, self.E, self.H, self.L, self.B, self.T, self.N
        if self.single_launch:  # the weights moved in the last update
            for l in range(L):
                d.lstm_pack_recurrent(H, self.p[f"Wh{l}"], self.Wh_packed[l])
                d.lstm_pack_recurrent_transposed16(H, self.p[f"Wh{l}"], self.WhT_packed[l])
        if not self.overlap:
            for l in range(L):
                if self.use_dropout:
                    self._mask_inputs(d, l)
                x, d_in = self._x_of(l)
                d.gemm_nn(4 * H, N, d_in, self.p[f"Wx{l}"], x, 0.0, self.gates[l])  # Wx*x of every timestep
                self._cell_steps_forward(d, l, 0, T)
                if self.use_dropout and self.single_launch and T > 1:  # for dWh: h (.) mask_h of every timestep
                    d.cmult_forward(B * H, T, 1, self.h[l], self.mask_h[l], self.hm[l])
            return
        # pipeline over time chunks: queue l runs layer l, one chunk behind queue l-1
        qs = self.queues
        d.gemm_nn(4 * H, N, E, self.p["Wx0"], self.emb, 0.0, self.gates[0])
        for l in range(1, L):
            qs[l].wait(d)  # joins the capture; nothing of layer l may start before the step does
        for (t0, t1) in self._chunks():
            for l in range(L):
                q = qs[l]
                if l > 0:
                    q.wait(qs[l - 1])  # h of the layer below for this chunk
                    nb = (t1 - t0) * B
                    q.gemm_nn(4 * H, nb, H, self.p[f"Wx{l}"], self._t(self.h[l - 1], t0, H),
                              0.0, self._t(self.gates[l], t0, 4 * H))
                self._cell_steps_forward(q, l, t0, t1)
        for l in range(1, L):
            d.wait(qs[l])

    def _forward_layers_nodes(self):
        d, E, H, L, B, T = self.dev, self.E, self.H, self.L, self.B, self.T
        for t in range(T):
            x, d_in = self._t(self.emb, t, E), E
            for l in range(L):
                h_tm1 = self._t(self.h[l], t - 1, H) if t > 0 else self.h0
                c_tm1 = self._t(self.c[l], t - 1, H) if t > 0 else self.h0
                g, c, h = self._t(self.gates[l], t, 4 * H), self._t(self.c[l], t, H), self._t(self.h[l], t, H)
                d.lstm_gates_forward([x], [d_in], H, B, h_tm1, self.p[f"Wx{l}"], self.p[f"Wh{l}"], self.p[f"b{l}"], g,
                                     **self._node_masks(l))
                d.lstm_c_forward(H, B, c_tm1, g, c)
                d.lstm_h_forward(H, B, c, g, h)
                x, d_in = h, H
        if self.use_dropout and self.time_batched:  # the masked copies for the weight gradients over all timesteps
            for l in range(L):
                self._mask_inputs(d, l)
                if T > 1:
                    d.cmult_forward(B * H, T, 1, self.h[l], self.mask_h[l], self.hm[l])

    def _node_masks(self, l):
        if not self.use_dropout:
            return {}
        return {"mask_x": self.mask_x[l], "mask_x_bd": self.B, "mask_h": self.mask_h[l], "mask_h_bd": self.B}

    def backward(self):
        d, V, E, H, L, B, T, N = self.dev, self.V, self.E, self.H, self.L, self.B, self.T, self.N
        fused = self.path == "fused"
        # the node path accumulates into every gradient buffer (zeroed first, as the executor does); the fused
        # path overwrites them all
        if not fused:
            d.zero(lib_tensor(d, self.d_errs.ptr, self.de_bytes))
        d.constant(self.d_errs, 1.0)  # d loss / d errs[b] through sum_batches(sum(errs))
        d.pnls_backward(V, N, self.logits, self.aux, self.d_errs, self.d_logits, assign=fused)
        top = self.h[L - 1]
        d.csum_backward(V, 1, N, self.d_logits, 0, self.g["bias"])
        d.gemm_nt_acc(V, H, N, self.d_logits, top, self.g["R"])
        d.gemm_tn(H, N, V, self.p["R"], self.d_logits, 0.0 if fused else 1.0, self.d_h[L - 1])
        if fused:
            self._backward_layers_fused()
        else:
            self._backward_layers_nodes()
        d.lookup_accumulate_grads_planned(N, self.plan, E, V, self.d_emb, self.g["C"])

    def _cell_steps_backward(self, q, l, t0, t1):
        """Timesteps t1-1 .. t0 of layer l; the recurrent slices of step t1 (if any) are in rec_b[l]."""
        H, B, T = self.H, self.B, self.T
        Wh = self.p[f"Wh{l}"]
        for t in reversed(range(t0, t1)):
            last, first = t == T - 1, t == 0
            dpre = self._t(self.d_pre[l], t, 4 * H)
            if self.single_launch:
                # one launch: Wh^T * dpre of the step above (from the fragment-order copy that step's launch wrote)
                # and this step's cell backward, which writes dpre plain and in fragment order for the step below
                q.lstm_step_backward_packed(H, B, self.WhT_packed[l], None if last else self.dpre_packed[l][(t + 1) % 2],
                                            self._t(self.gates[l], t, 4 * H), self._t(self.c[l], t, H),
                                            None if first else self._t(self.c[l], t - 1, H), self._t(self.d_h[l], t, H),
                                            None if last else self._t(self.d_c[l], t, H), dpre,
                                            None if first else self._t(self.d_c[l], t - 1, H),
                                            None if first else self.dpre_packed[l][t % 2],
                                            mask_h=self.mask_h[l] if self.use_dropout else None)
                continue
            if self.use_dropout:
                # no one-launch step at this size: (Wh^T dpre) as a plain product, through the mask, into d_h[t-1]
                q.lstm_cell_backward(H, B, self._t(self.gates[l], t, 4 * H), self._t(self.c[l], t, H),
                                     None if first else self._t(self.c[l], t - 1, H), self._t(self.d_h[l], t, H), None, 0,
                                     None if last else self._t(self.d_c[l], t, H), dpre,
                                     None if first else self._t(self.d_c[l], t - 1, H))
                if not first:
                    q.gemm_tn(H, B, 4 * H, Wh, dpre, 0.0, self.dh_rec)
                    q.cmult_forward(B * H, 1, 1, self.dh_rec, self.mask_h[l], self.dh_rec)
                    q.accumulate(self.dh_rec, self._t(self.d_h[l], t - 1, H))
                continue
            args = (H, B, self._t(self.gates[l], t, 4 * H), self._t(self.c[l], t, H),
                    None if first else self._t(self.c[l], t - 1, H), self._t(self.d_h[l], t, H),
                    None if last else self.rec_b[l], 0 if last else self._rec_b_n[l],
                    None if last else self._t(self.d_c[l], t, H), dpre, None if first else self._t(self.d_c[l], t - 1, H))
            q.lstm_cell_backward(*args)
            if not first:
                self._rec_b_n[l] = q.lstm_recurrent_backward(H, B, Wh, dpre, self.rec_b[l], self.rec_b_bytes)

    def _weight_grads(self, q, l):
        E, H, B, T, N = self.E, self.H, self.B, self.T, self.N
        x, d_in = self._x_of(l)
        q.gemm_nt_acc(4 * H, d_in, N, self.d_pre[l], x, self.g[f"Wx{l}"])
        if T > 1:
            q.gemm_nt_acc(4 * H, H, N - B, self._t(self.d_pre[l], 1, 4 * H), self.hm[l] if self.use_dropout else self.h[l],
                          self.g[f"Wh{l}"])
        q.csum_backward(4 * H, 1, N, self.d_pre[l], 0, self.g[f"b{l}"])

    def _backward_layers_fused(self):
        d, E, H, L, B, T, N = self.dev, self.E, self.H, self.L, self.B, self.T, self.N
        self._rec_b_n = [0] * L
        if not self.overlap:
            for l in reversed(range(L)):
                self._cell_steps_backward(d, l, 0, T)
                d_in, dx = (H, self.d_h[l - 1]) if l > 0 else (E, self.d_emb)
                d.gemm_tn(d_in, N, 4 * H, self.p[f"Wx{l}"], self.d_pre[l], 0.0, dx)
                if self.use_dropout:  # the gradient reaches the layer's input through mask_x
                    d.cmult_forward(B * d_in, T, 1, dx, self.mask_x[l], dx)
                self._weight_grads(d, l)
            return
        # pipeline, newest chunk first: the top layer runs on the device queue (it owns d_h[L-1]),
        # layer l on queue L-1-l, one chunk behind the layer above
        qs = self.queues
        qof = lambda l: qs[L - 1 - l]
        for l in range(L - 1):
            qof(l).wait(d)
        for (t0, t1) in reversed(self._chunks()):
            for l in reversed(range(L)):
                q = qof(l)
                if l < L - 1:
                    q.wait(qof(l + 1))  # d_h[l] of this chunk
                self._cell_steps_backward(q, l, t0, t1)
                nb = (t1 - t0) * B
                d_in, dx = (H, self.d_h[l - 1]) if l > 0 else (E, self.d_emb)
                q.gemm_tn(d_in, nb, 4 * H, self.p[f"Wx{l}"], self._t(self.d_pre[l], t0, 4 * H), 0.0,
                          self._t(dx, t0, d_in))
        for l in reversed(range(L)):
            self._weight_grads(qof(l), l)  # each on its own queue, side by side with the layers still running
        for l in range(L - 1):
            d.wait(qof(l))

    def _flush_recorded(self):
        """The recorded products of every parameter as one product each: the operands of the T backward calls are
        gathered in ascending timestep order (the addresses go to the kernel as arguments), then
        dWx += dpre x^T, dWh += dpre[1:] h[:-1]^T, db += sum over the columns of dpre, each over all timesteps."""
        d, E, H, B, T = self.dev, self.E, self.H, self.B, self.T
        for l in range(self.L):
            rec = sorted(self._recorded[l], key=lambda r: r[0])
            d_in = H if l > 0 else E
            n = len(rec) * B
            gx = self.gath_x.offset(0, (len(rec), B, d_in))
            d.gather_segments([r[1] for r in rec], 4 * H * B, self.gath_dpre)
            d.gather_segments([r[2] for r in rec], d_in * B, gx)
            if self.use_dropout:  # the gates saw x (.) mask_x and h_tm1 (.) mask_h
                d.cmult_forward(B * d_in, len(rec), 1, gx, self.mask_x[l], gx)
            d.gemm_nt_acc(4 * H, d_in, n, self.gath_dpre, gx, self.g[f"Wx{l}"])
            later = [r for r in rec if r[0] > 0]  # h_tm1 of the first step is the zero state: its product adds nothing
            if later:
                assert rec[0][0] == 0 and len(later) == len(rec) - 1
                gh = self.gath_h.offset(0, (len(later), B, H))
                d.gather_segments([r[3] for r in later], H * B, gh)
                if self.use_dropout:
                    d.cmult_forward(B * H, len(later), 1, gh, self.mask_h[l], gh)
                d.gemm_nt_acc(4 * H, H, len(later) * B, self._t(self.gath_dpre, 1, 4 * H), gh, self.g[f"Wh{l}"])
            d.csum_backward(4 * H, 1, n, self.gath_dpre, 0, self.g[f"b{l}"])
            if l == 0:
                # the T recorded products Wx^T dpre_t into the lookup nodes' gradients as one product over the gathered
                # dpre (here the T gradients are one array; an executor's are T tensors, which the product's columns
                # are added to with one dyhip_parallel_accumulate)
                assert len(rec) == T
                d.gemm_tn_acc(E, n, 4 * H, self.p["Wx0"], self.gath_dpre, self.d_emb)
                if self.use_dropout:
                    d.cmult_forward(B * E, T, 1, self.d_emb, self.mask_x[0], self.d_emb)

    def _backward_layers_nodes(self):
        d, E, H, L, B, T, N = self.dev, self.E, self.H, self.L, self.B, self.T, self.N
        self._recorded = [[] for _ in range(L)]
        for t in reversed(range(T)):
            for l in reversed(range(L)):
                g, c = self._t(self.gates[l], t, 4 * H), self._t(self.c[l], t, H)
                c_tm1 = self._t(self.c[l], t - 1, H) if t > 0 else self.h0
                h_tm1 = self._t(self.h[l], t - 1, H) if t > 0 else self.h0
                dh, dc, dg = self._t(self.d_h[l], t, H), self._t(self.d_c[l], t, H), self._t(self.d_gates[l], t, 4 * H)
                dpre = self._t(self.d_pre[l], t, 4 * H)
                d.lstm_h_backward(H, B, c, g, dh, 0, dc)
                d.lstm_h_backward(H, B, c, g, dh, 1, dg)
                if t > 0:
                    d.lstm_c_backward(H, B, c_tm1, g, dc, 0, self._t(self.d_c[l], t - 1, H))
                d.lstm_c_backward(H, B, c_tm1, g, dc, 1, dg)
                d.lstm_gates_dpre(H, B, g, dg, dpre)
                if l > 0:
                    x, d_in, dx = self._t(self.h[l - 1], t, H), H, self._t(self.d_h[l - 1], t, H)
                else:
                    x, d_in, dx = self._t(self.emb, t, E), E, self._t(self.d_emb, t, E)
                # The gradient of layer 0's input belongs to a lookup node, an arity-0 node whose gradient nobody reads
                # before the executor hands it over at the end of backward: its product is recorded as well.
                lazy_dx = self.defer and l == 0
                if self.use_dropout:
                    # the gates node's own backward: it applies the masks to dx / dh and to the operands of dWx / dWh
                    mk = self._node_masks(l)
                    args = ([x], [d_in], H, B, h_tm1, self.p[f"Wx{l}"], self.p[f"Wh{l}"], g, dg)
                    if not lazy_dx:
                        d.lstm_gates_backward(*args, 0, dx, dpre=dpre, **mk)
                    if t > 0:
                        d.lstm_gates_backward(*args, 1, self._t(self.d_h[l], t - 1, H), dpre=dpre, **mk)
                    if self.defer:
                        self._recorded[l].append((t, dpre, x, h_tm1))
                    elif not self.time_batched:
                        d.lstm_gates_backward(*args, 2, self.g[f"Wx{l}"], dpre=dpre, **mk)
                        if t > 0:
                            d.lstm_gates_backward(*args, 3, self.g[f"Wh{l}"], dpre=dpre, **mk)
                        d.lstm_gates_backward(*args, 4, self.g[f"b{l}"], dpre=dpre, **mk)
                    continue
                if not lazy_dx:
                    d.gemm_tn_acc(d_in, B, 4 * H, self.p[f"Wx{l}"], dpre, dx)
                if t > 0:
                    d.gemm_tn_acc(H, B, 4 * H, self.p[f"Wh{l}"], dpre, self._t(self.d_h[l], t - 1, H))
                if self.defer:
                    self._recorded[l].append((t, dpre, x, h_tm1))
                elif not self.time_batched:
                    d.gemm_nt_acc(4 * H, d_in, B, dpre, x, self.g[f"Wx{l}"])
                    if t > 0:  # h_tm1 of the first step is the zero state: its product adds nothing
                        d.gemm_nt_acc(4 * H, H, B, dpre, h_tm1, self.g[f"Wh{l}"])
                    d.csum_backward(4 * H, 1, B, dpre, 0, self.g[f"b{l}"])
        if self.defer:
            self._flush_recorded()
        if self.time_batched:
            for l in range(L):
                x, d_in = self._x_of(l)
                d.gemm_nt_acc(4 * H, d_in, N, self.d_pre[l], x, self.g[f"Wx{l}"])
                if T > 1:
                    d.gemm_nt_acc(4 * H, H, N - B, self._t(self.d_pre[l], 1, 4 * H),
                                  self.hm[l] if self.use_dropout else self.h[l], self.g[f"Wh{l}"])
                d.csum_backward(4 * H, 1, N, self.d_pre[l], 0, self.g[f"b{l}"])

    def update(self):
        d = self.dev
        d.squared_l2norm(self.dense_elems, self.g_dense, self.sqnorms.offset(0, (1,)))
        d.squared_l2norm_rows(self.N, self.plan, self.E, self.V, self.g["C"], self.sqnorms.offset(1, (1,)))
        d.clip_scale(2, self.sqnorms, self.clip, self.gscale, self.gnorm)
        d.sgd_update_scaled(self.dense_elems, self.p_dense, self.g_dense, self.lr, self.gscale, 1.0, True)
        d.sgd_update_rows(self.N, self.plan, self.E, self.V, self.p["C"], self.g["C"], self.lr, self.gscale, 1.0)

    def issue(self):
        """The whole step on the device stream (ids and labels already staged)."""
        self.dev.lookup_build_plan_into(self.ids, self.V, self.plan, self.plan_ws, self.plan_ws_bytes)
        if self.use_dropout:
            self.draw_masks()
        self.forward()
        self.backward()
        self.update()

    def capture(self):
        """Record the step; ``step`` then replays it.

        The step is recorded and instantiated twice and the first graph thrown away: in a process that has built and
        destroyed many small graphs before, the first large graph replays ~3 % slower than one instantiated after
        it (6.77 against 6.55 ms per step here; kernel durations are the same, the time goes between the nodes).
        """
        for attempt in range(2):
            self.dev.sync()
            self.dev.graph_begin()
            try:
                self.issue()
            finally:
                graph = self.dev.graph_end()
            if attempt == 0:
                graph.destroy()
        self.graph = graph
        return self.graph

    def step(self, tokens, read_loss=True):
        self.stage(tokens)
        if self.graph is not None:
            self.graph.launch()
        else:
            self.issue()
        if read_loss:
            self.check_gradient_norm()
            return float(self.loss.numpy()[0])
        return None

    def check_gradient_norm(self):
        """Trainer::clip_gradients's check (dynet/training.cc:176-180), made when the host looks: a step whose
        gradient norm was NaN or infinite has already been dropped on the device."""
        nrm = float(self.gnorm.numpy()[0])
        if not np.isfinite(nrm):
            raise RuntimeError("Magnitude of gradient is bad: %r" % nrm)
        return nrm

    def get_masks(self):
        """The dropout masks of the last step, per layer (mask_x[B, d_in], mask_h[B, H]); None without dropout."""
        if not self.use_dropout:
            return None
        return [(self.mask_x[l].numpy(), self.mask_h[l].numpy()) for l in range(self.L)]

    def get_params(self):
        return {n: t.numpy() for n, t in self.p.items()}

    def get_grads(self):
        return {n: t.numpy() for n, t in self.g.items()}


def lib_tensor(dev, ptr, nbytes):
    from .device import DevTensor
    return DevTensor(dev, ptr, (nbytes,), np.uint8)
