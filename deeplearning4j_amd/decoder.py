"""GPT-2-shaped decoder driven op by op through the NativeOps C ABI.

Stands in for what a SameDiff inference session does with such a graph in the reference
(nd4j-api .../autodiff/samediff/internal/InferenceSession.java: one native call per graph node): every step below is
one reference op executed through `execCustomOp2` or a legacy `exec*` entry point -- `gather` (token and position
embeddings), broadcastable `add`, `layer_norm`, `xw_plus_b` (the linear layers), transform-strict GELU (opNum 53),
transform-any Assign (the write into the key/value cache), `dot_product_attention_v2`, pairwise Add (residuals),
`matmul` (tied output embedding), `argmax`.  Nothing is fused on the Python side and no array leaves the device
between ops.  The linear layers' weights are uploaded k-contiguous ([out, in]) and `xw_plus_b` is called with its
weight-transpose flag (IArg 1, generic/nn/xw_plus_b.cpp:38,99-104): a single token's projection then reads whole
weight rows, which streams several times faster than column strips of an [in, out] matrix.

Memory layout (all activations token-major, so the head split needs no copy):
  x, attention output ... [B, T, d_model]
  qkv ................... [B, T, 3 * d_model]; q / k / v are column slices, heads are views [B, H, T, 64]
                          with strides [T * 3d, 64, 3d, 1]
  key / value cache ..... per layer [B, max_len, d_model]; the keys seen by attention at length L are the view
                          [B, H, L, 64] with strides [max_len * d, 64, d, 1]
Op contexts are built once per (phase, sequence length) and replayed, as SameDiff caches its OpContext per node.
"""
import math

import numpy as np

from . import nativeops as N
from .executioner import Executioner, Pairwise, TransformStrict
from .ndarray import BFLOAT16, FLOAT32, HALF, INT64, NDArray


class DecoderConfig:
    def __init__(self, n_layer=12, d_model=768, n_head=12, d_ff=3072, vocab=50257, max_len=1024):
        assert d_model % n_head == 0
        self.n_layer, self.d_model, self.n_head, self.d_ff, self.vocab, self.max_len = n_layer, d_model, n_head, d_ff, vocab, max_len
        self.d_head = d_model // n_head

    @staticmethod
    def gpt2_small():
        return DecoderConfig()


def init_weights(cfg, seed):
    """Random-init parameters of the GPT-2 architecture as fp32 numpy arrays: N(0, 0.02) everywhere, layer-norm
    gains N(1, 0.02).  Linear weights are stored [in, out] (x @ W), as GPT-2's Conv1D does."""
    rng = np.random.default_rng(seed)
    nrm = lambda *s: rng.normal(0.0, 0.02, s).astype(np.float32)
    d, ff = cfg.d_model, cfg.d_ff
    w = {"wte": nrm(cfg.vocab, d), "wpe": nrm(cfg.max_len, d), "lnf_g": 1 + nrm(d), "lnf_b": nrm(d), "layers": []}
    for _ in range(cfg.n_layer):
        w["layers"].append({
            "ln1_g": 1 + nrm(d), "ln1_b": nrm(d), "w_qkv": nrm(d, 3 * d), "b_qkv": nrm(3 * d), "w_o": nrm(d, d), "b_o": nrm(d),
            "ln2_g": 1 + nrm(d), "ln2_b": nrm(d), "w_fc": nrm(d, ff), "b_fc": nrm(ff), "w_proj": nrm(ff, d), "b_proj": nrm(d)})
    return w


class Decoder:
    """Greedy decoding with a key/value cache.  `dtype` is the storage type of weights and activations."""

    def __init__(self, cfg, weights, dtype=BFLOAT16, batch=1, executioner=None):
        self.cfg, self.dtype, self.B = cfg, dtype, batch
        self.ex = executioner or Executioner()
        self.L = self.ex.L
        up = lambda a: self._resident(NDArray.from_numpy(a, dtype))
        self.wte, self.wpe = up(weights["wte"]), up(weights["wpe"])
        self.lnf_g, self.lnf_b = up(weights["lnf_g"]), up(weights["lnf_b"])
        linear = ("w_qkv", "w_o", "w_fc", "w_proj")   # stored [in, out] in `weights`, kept [out, in] on the device
        self.layers = [{k: up(np.ascontiguousarray(v.T) if k in linear else v) for k, v in lw.items()} for lw in weights["layers"]]
        d = cfg.d_model
        self.kcache = [NDArray.empty((batch, cfg.max_len, d), dtype) for _ in range(cfg.n_layer)]
        self.vcache = [NDArray.empty((batch, cfg.max_len, d), dtype) for _ in range(cfg.n_layer)]
        self.length = 0            # tokens in the cache
        self._programs = {}        # (T_new, past) -> list of bound op calls
        self._buffers = {}         # T_new -> activation arrays
        self.use_graphs = False    # replay each single-token step as one captured HIP graph (one graph per cache length)
        self._graphs = {}          # (past, source of the fed-back ids) -> captured graph handle

    @staticmethod
    def _resident(arr):
        arr.sync_to_device()
        return arr

    # ---- op binding helpers: each returns a zero-argument callable that runs one native op -----------------------------
    def _custom(self, name, ins, outs, **kw):
        return self.ex.bind_custom(name, ins, outs, **kw)

    def _legacy(self, fn, name, arrays, *args):
        """`arrays` are the NDArray objects behind the handles in `args`; the call keeps them alive (a view's native
        handle is released when its Python object is collected)."""
        L, check = self.L, N.check

        def call():
            fn(*args)
            if L.lastErrorCode() != 0:
                check(name)
        call.keep = arrays
        return call

    def _pairwise_add(self, x, y, z):
        return self._legacy(self.L.execPairwiseTransform, "execPairwiseTransform", (x, y, z), None, Pairwise.Add, x.handle, y.handle, z.handle, None)

    def _gelu(self, x, z):
        return self._legacy(self.L.execTransformStrict, "execTransformStrict", (x, z), None, TransformStrict.GELU, x.handle, None, z.handle)

    def _assign(self, x, z):
        return self._legacy(self.L.execTransformAny, "execTransformAny", (x, z), None, 0, x.handle, None, z.handle)

    # ---- program construction --------------------------------------------------------------------------------------------------
    def _activations(self, T):
        if T in self._buffers:
            return self._buffers[T]
        c, B, dt = self.cfg, self.B, self.dtype
        d, ff = c.d_model, c.d_ff
        a = {
            "ids": NDArray.empty((B, T), INT64),
            "tok": NDArray.empty((B, T, d), dt), "x": NDArray.empty((B, T, d), dt), "ln": NDArray.empty((B, T, d), dt),
            "qkv": NDArray.empty((B, T, 3 * d), dt), "att": NDArray.empty((B, T, d), dt), "proj": NDArray.empty((B, T, d), dt),
            "h": NDArray.empty((B, T, ff), dt), "g": NDArray.empty((B, T, ff), dt),
            "last": NDArray.empty((B, d), dt), "logits": NDArray.empty((B, c.vocab), dt), "next": NDArray.empty((B,), INT64),
        }
        if T == 1:
            # single-token steps: argmax writes the next ids where the following step's gather reads them (one array seen
            # as [B] and as [B, 1]), so consecutive steps need no feedback copy
            a["next"] = a["ids"].view((B,), (1,), 0)
        self._buffers[T] = a
        return a

    def _program(self, T, past):
        key = (T, past)
        if key in self._programs:
            return self._programs[key]
        c, B = self.cfg, self.B
        d, H, Dh, ff, M = c.d_model, c.n_head, c.d_head, c.d_ff, c.max_len
        a = self._activations(T)
        total = past + T
        assert total <= M, "sequence exceeds max_len"
        ops = []
        two_d = lambda arr, cols: arr.view((B * T, cols), (cols, 1))
        # embeddings: x = wte[ids] + wpe[past : past + T]
        ops.append(self._custom("gather", [self.wte, a["ids"]], [a["tok"]], i_args=[0]))
        ops.append(self._custom("add", [a["tok"], self.wpe.slice(0, past, total)], [a["x"]]))
        x2, ln2, qkv2, att2, proj2 = two_d(a["x"], d), two_d(a["ln"], d), two_d(a["qkv"], 3 * d), two_d(a["att"], d), two_d(a["proj"], d)
        h2, g2 = two_d(a["h"], ff), two_d(a["g"], ff)
        q4 = a["qkv"].view((B, H, T, Dh), (T * 3 * d, Dh, 3 * d, 1), 0)
        knew = a["qkv"].view((B, T, d), (T * 3 * d, 3 * d, 1), d)
        vnew = a["qkv"].view((B, T, d), (T * 3 * d, 3 * d, 1), 2 * d)
        o4 = a["att"].view((B, H, T, Dh), (T * d, Dh, d, 1), 0)
        scale = 1.0 / math.sqrt(Dh)
        for li, w in enumerate(self.layers):
            kc, vc = self.kcache[li], self.vcache[li]
            ops.append(self._custom("layer_norm", [x2, w["ln1_g"], w["ln1_b"]], [ln2], i_args=[1], b_args=[False]))
            ops.append(self._custom("xw_plus_b", [ln2, w["w_qkv"], w["b_qkv"]], [qkv2], i_args=[0, 1]))
            # append this chunk's keys / values to the cache
            ops.append(self._assign(knew, kc.view((B, T, d), (M * d, d, 1), past * d)))
            ops.append(self._assign(vnew, vc.view((B, T, d), (M * d, d, 1), past * d)))
            k4 = kc.view((B, H, total, Dh), (M * d, Dh, d, 1), 0)
            v4 = vc.view((B, H, total, Dh), (M * d, Dh, d, 1), 0)
            # a chunk that starts at position 0 attends causally; a single new token sees the whole cache
            ops.append(self._custom("dot_product_attention_v2", [q4, v4, k4], [o4], t_args=[scale, 0.0], b_args=[past == 0 and T > 1, False]))
            ops.append(self._custom("xw_plus_b", [att2, w["w_o"], w["b_o"]], [proj2], i_args=[0, 1]))
            ops.append(self._pairwise_add(x2, proj2, x2))
            ops.append(self._custom("layer_norm", [x2, w["ln2_g"], w["ln2_b"]], [ln2], i_args=[1], b_args=[False]))
            ops.append(self._custom("xw_plus_b", [ln2, w["w_fc"], w["b_fc"]], [h2], i_args=[0, 1]))
            ops.append(self._gelu(h2, g2))
            ops.append(self._custom("xw_plus_b", [g2, w["w_proj"], w["b_proj"]], [proj2], i_args=[0, 1]))
            ops.append(self._pairwise_add(x2, proj2, x2))
        # final layer norm on the last position only, tied output projection, greedy pick
        xlast = a["x"].view((B, d), (T * d, 1), (T - 1) * d)
        ops.append(self._custom("layer_norm", [xlast, self.lnf_g, self.lnf_b], [a["last"]], i_args=[1], b_args=[False]))
        ops.append(self._custom("matmul", [a["last"], self.wte], [a["logits"]], i_args=[0, 1]))
        ops.append(self._custom("argmax", [a["logits"]], [a["next"]], i_args=[1]))
        assert past > 0 or T >= 1
        self._programs[key] = ops
        return ops

    # ---- running ----------------------------------------------------------------------------------------------------------------------
    def reset(self):
        self.length = 0

    def forward(self, ids=None):
        """Run one chunk: `ids` [B, T] int64 host array, or None to feed back the previous step's argmax (T = 1, no
        host round trip).  Returns the NDArray of greedy next-token ids [B] (device-resident)."""
        if ids is None:
            T = 1
            a = self._activations(1)
            prog = self._program(1, self.length)
            # previous `next` [B] -> ids [B, 1]
            src = self._last_next
            if not hasattr(self, "_feed") or self._feed[0] is not src:
                # (every feedback copy ever built stays alive: a recorded step may hold its views)
                if not hasattr(self, "_feeds"):
                    self._feeds = {}
                if id(src) not in self._feeds:
                    copy = (lambda: None) if src is a["next"] else self._assign(src.view((self.B, 1), (1, 1)), a["ids"])
                    self._feeds[id(src)] = (src, copy)
                self._feed = self._feeds[id(src)]
            if self.use_graphs:
                self._graph_step(prog)
                self.length += 1
                self._last_next = a["next"]
                return a["next"]
            self._feed[1]()
        else:
            ids = np.asarray(ids, dtype=np.int64)
            assert ids.ndim == 2 and ids.shape[0] == self.B
            T = ids.shape[1]
            assert self.length == 0 or T == 1, "a chunk longer than one token must start an empty cache"
            a = self._activations(T)
            prog = self._program(T, self.length)
            a["ids"].assign_numpy(ids)
        for op in prog:
            op()
        self.length += T
        self._last_next = a["next"]
        return a["next"]

    def _graph_step(self, prog):
        """One decode step through a captured graph: the ops of the step (feedback copy of the last id included) are recorded
        the first time this cache length is seen -- the kernels' arguments depend on it -- and replayed from then on.
        Arrays, views and op contexts are built before the capture starts, so recording only launches kernels."""
        L = self.L
        key = (self.length, id(self._last_next))   # the recorded feedback copy reads the array the last ids were written to
        g = self._graphs.get(key)
        if g is None:
            if L.nd4jhipGraphBeginCapture() != 0:
                N.check("nd4jhipGraphBeginCapture")
            try:
                self._feed[1]()
                for op in prog:
                    op()
            finally:
                g = L.nd4jhipGraphEndCapture()
            if not g:
                N.check("nd4jhipGraphEndCapture")
                raise N.NativeOpsError("nd4jhipGraphEndCapture returned no graph")
            self._graphs[key] = g
        if L.nd4jhipGraphLaunch(g) != 0:
            N.check("nd4jhipGraphLaunch")

    def close(self):
        for g in self._graphs.values():
            self.L.nd4jhipGraphDestroy(g)
        self._graphs = {}

    def logits(self, T=None):
        """Logits [B, vocab] of the last forward call (as float32 on the host)."""
        T = T or max(k for k in self._buffers if self._buffers[k]["next"] is self._last_next)
        return self._buffers[T]["logits"].to_float()

    def generate(self, prompt_ids, n_steps):
        """Prefill with `prompt_ids` [B, T0], then `n_steps - 1` further greedy steps; returns ids [B, n_steps]."""
        self.reset()
        hist = self._history(n_steps)
        nxt = self.forward(prompt_ids)
        self._snapshot(nxt, hist, 0)
        for i in range(1, n_steps):
            nxt = self.forward(None)
            self._snapshot(nxt, hist, i)
        self.ex.synchronize()
        return np.ascontiguousarray(hist[0].to_numpy().T)

    def _history(self, n_steps):
        """[n_steps, B] id buffer with one row view per step, kept between calls so that steady-state generation allocates nothing."""
        h = getattr(self, "_hist", None)
        if h is None or h[0].shape[0] < n_steps:
            buf = NDArray.empty((n_steps, self.B), INT64)
            h = (buf, [buf.view((self.B,), (1,), i * self.B) for i in range(n_steps)])
            self._hist = h
        if h[0].shape[0] != n_steps:
            buf = NDArray.empty((n_steps, self.B), INT64)
            h = (buf, [buf.view((self.B,), (1,), i * self.B) for i in range(n_steps)])
            self._hist = h
        return h

    def _snapshot(self, arr, hist, i):
        """Device-side copy of the step's ids into row i of the history, so that generate() reads back once at the end."""
        self.L.execTransformAny(None, 0, arr.handle, None, hist[1][i].handle)
        N.check("execTransformAny")
