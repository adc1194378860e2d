"""CPU composition of the GPT-2-shaped decode step out of the oracle's ops -- test infrastructure only.

Mirrors deeplearning4j_amd/decoder.py op for op (gather, add, layer_norm, xw_plus_b = mmul against the transposed
[out, in] weights followed by the bias row as in generic/nn/xw_plus_b.cpp:99-133, GELU opNum 53, dot_product_attention_v2, argmax), each executed by the CPU
restatement in nd4j_oracle.c, so that greedy token ids
and logits of the HIP path can be compared on the same seeded weights.  Arrays are numpy: float32, or uint16 bit
patterns for bf16.
"""
import math

import numpy as np

from . import oracle as O


class OracleDecoder:
    def __init__(self, cfg, weights, dtype=O.FLOAT32, batch=1):
        self.cfg, self.dt, self.B = cfg, dtype, batch
        conv = (lambda a: O.f32_to_bf16(a)) if dtype == O.BFLOAT16 else (lambda a: np.ascontiguousarray(a, dtype=np.float32))
        self.w = {k: conv(v) for k, v in weights.items() if k != "layers"}
        # the linear layers' weights are kept [out, in] and multiplied with the transpose flag, as the device harness does
        linear = ("w_qkv", "w_o", "w_fc", "w_proj")
        self.layers = [{k: conv(np.ascontiguousarray(v.T) if k in linear else v) for k, v in lw.items()} for lw in weights["layers"]]
        self.np_dt = np.uint16 if dtype == O.BFLOAT16 else np.float32
        d = cfg.d_model
        self.kc = [np.zeros((batch, cfg.max_len, d), self.np_dt) for _ in range(cfg.n_layer)]
        self.vc = [np.zeros((batch, cfg.max_len, d), self.np_dt) for _ in range(cfg.n_layer)]
        self.length = 0
        self.last_logits = None

    def _a(self, arr):
        return O.Arr(arr, self.dt)

    def _empty(self, *shape):
        return np.zeros(shape, self.np_dt)

    def _matmul(self, x, w, trans_y=False):
        n = w.shape[0] if trans_y else w.shape[1]
        z = self._empty(x.shape[0], n)
        O.matmul(self._a(x), self._a(w), self._a(z), trans_y=trans_y, accumulate=1)
        return z

    def _bias(self, x, b):
        O.add_row_vector(self._a(x), self._a(b), self._a(x))
        return x

    def _ln(self, x, g, b):
        z = self._empty(*x.shape)
        O.layer_norm(self._a(x), self._a(g), self._a(b), self._a(z), [1], channels_first=False)
        return z

    def _add(self, x, y):
        z = self._empty(*x.shape)
        O.pairwise(0, self._a(x), self._a(y), self._a(z))
        return z

    def forward(self, ids):
        c, B = self.cfg, self.B
        d, H, Dh = c.d_model, c.n_head, c.d_head
        ids = np.asarray(ids, dtype=np.int64)
        T = ids.shape[1]
        past, total = self.length, self.length + T
        assert past == 0 or T == 1
        tok = self.w["wte"][ids.reshape(-1)]                                     # gather, axis 0
        pos = np.ascontiguousarray(np.broadcast_to(self.w["wpe"][past:total], (B, T, d))).reshape(B * T, d)
        x = self._add(tok, pos)
        scale = 1.0 / math.sqrt(Dh)
        for li, w in enumerate(self.layers):
            ln = self._ln(x, w["ln1_g"], w["ln1_b"])
            qkv = self._bias(self._matmul(ln, w["w_qkv"], trans_y=True), w["b_qkv"]).reshape(B, T, 3, H, Dh)
            self.kc[li][:, past:total] = qkv[:, :, 1].reshape(B, T, d)
            self.vc[li][:, past:total] = qkv[:, :, 2].reshape(B, T, d)
            att = self._empty(B, T, H, Dh)
            for b in range(B):
                q3 = qkv[b, :, 0].transpose(1, 0, 2)                                        # [H, T, Dh] view
                k3 = self.kc[li][b, :total].reshape(total, H, Dh).transpose(1, 0, 2)        # [H, total, Dh] view
                v3 = self.vc[li][b, :total].reshape(total, H, Dh).transpose(1, 0, 2)
                o3 = att[b].transpose(1, 0, 2)
                O.attention_v2(self._a(q3), self._a(v3), self._a(k3), self._a(o3), scale=scale, causal=(past == 0 and T > 1))
            proj = self._bias(self._matmul(att.reshape(B * T, d), w["w_o"], trans_y=True), w["b_o"])
            x = self._add(x, proj)
            ln = self._ln(x, w["ln2_g"], w["ln2_b"])
            h = self._bias(self._matmul(ln, w["w_fc"], trans_y=True), w["b_fc"])
            g = self._empty(*h.shape)
            O.transform_strict(53, self._a(h), self._a(g))
            proj = self._bias(self._matmul(g, w["w_proj"], trans_y=True), w["b_proj"])
            x = self._add(x, proj)
        last = np.ascontiguousarray(x.reshape(B, T, d)[:, T - 1])
        last = self._ln(last, self.w["lnf_g"], self.w["lnf_b"])
        logits = self._matmul(last, self.w["wte"], trans_y=True)
        nxt = np.zeros((B,), np.int64)
        O.index_reduce(0, self._a(logits), nxt, [1])
        self.length = total
        self.last_logits = O.bf16_to_f32(logits) if self.dt == O.BFLOAT16 else logits
        return nxt

    def generate(self, prompt_ids, n_steps):
        self.length = 0
        out = [self.forward(prompt_ids)]
        for _ in range(n_steps - 1):
            out.append(self.forward(out[-1].reshape(self.B, 1)))
        return np.stack(out, axis=1)
