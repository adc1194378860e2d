"""Pins the mask arguments of the oracle's dot_product_attention_v2 restatement.  The reference holds no enabled test
with masks (its Java tests for v2 are @Disabled), so the restatement is pinned by what the mathematics fixes:
  * an fp64 numpy composition of matmul -> scale -> clip -> penalty where the merged mask is false -> softmax -> matmul;
  * the padded-batch identity: masking the trailing keys equals truncating keys and values;
  * the query mask multiplies the weights output and leaves `out` alone (the reference forms `out` first);
  * one penalty, not two, where the causal mask and the value mask both hide a key (boolean AND of the masks).
"""
import numpy as np

from oracle import oracle as O


def _np_attention(q, k, v, scale, causal, v_mask, q_mask, penalty=1e9):
    lg = np.einsum("bid,bjd->bij", q.astype(np.float64), k.astype(np.float64)) * scale
    lg = np.clip(lg, -1e4, 1e4)
    B, Tq, Tv = lg.shape
    keep = np.ones((B, Tq, Tv), bool)
    if causal:
        keep &= np.tril(np.ones((Tq, Tv), bool))[None]
    if v_mask is not None:
        keep &= (v_mask != 0)[:, None, :]
    lg = lg - penalty * (~keep)
    e = np.exp(lg - lg.max(-1, keepdims=True))
    w = e / e.sum(-1, keepdims=True)
    out = w @ v.astype(np.float64)
    if q_mask is not None:
        w = w * q_mask[:, :, None]
    return out, w, lg


def _run(q, k, v, scale=1.0, causal=False, q_mask=None, v_mask=None):
    B, Tq, _ = q.shape
    Tv, Dv = v.shape[1], v.shape[2]
    out, w, lg = np.zeros((B, Tq, Dv), np.float32), np.zeros((B, Tq, Tv), np.float32), np.zeros((B, Tq, Tv), np.float32)
    O.attention_v2(q, v, k, out, w, lg, scale=scale, causal=causal, q_mask=q_mask, v_mask=v_mask)
    return out, w, lg


def _data(seed, B=3, Tq=7, Tv=9, D=8):
    rng = np.random.default_rng(seed)
    return (rng.normal(0, 1, (B, Tq, D)).astype(np.float32), rng.normal(0, 1, (B, Tv, D)).astype(np.float32),
            rng.normal(0, 1, (B, Tv, D)).astype(np.float32), rng)


def test_value_mask_against_numpy_composition():
    q, k, v, rng = _data(1)
    for mask_dtype in (np.float32, np.int32, np.int64, np.bool_):
        vm = (rng.random((3, 9)) > 0.4)
        vm[:, 0] = True                                  # every query keeps at least one key
        vm = vm.astype(mask_dtype)
        for causal in (False, True):
            out, w, lg = _run(q, k, v, 0.35, causal, v_mask=vm)
            eo, ew, el = _np_attention(q, k, v, 0.35, causal, vm, None)
            np.testing.assert_allclose(out, eo, rtol=1e-5, atol=1e-6)
            np.testing.assert_allclose(w, ew, rtol=1e-5, atol=1e-7)
            np.testing.assert_allclose(lg, el, rtol=1e-6, atol=1e-3)   # 1e9 in fp32 carries 64 units of rounding; masked entries only


def test_padded_batch_identity():
    q, k, v, _ = _data(2, Tv=12)
    vm = np.ones((3, 12), np.float32)
    vm[:, 8:] = 0
    out, w, _ = _run(q, k, v, 0.5, False, v_mask=vm)
    out_t, w_t, _ = _run(q, k[:, :8].copy(), v[:, :8].copy(), 0.5, False)
    np.testing.assert_allclose(out, out_t, rtol=1e-6, atol=1e-7)
    np.testing.assert_allclose(w[:, :, :8], w_t, rtol=1e-6, atol=1e-8)
    assert np.abs(w[:, :, 8:]).max() < 1e-30


def test_query_mask_scales_weights_only():
    q, k, v, rng = _data(3)
    qm = rng.integers(0, 2, (3, 7)).astype(np.float32)
    qm[0, 0] = 2.0                                       # the mask is cast to the arrays' type, not to BOOL: a 2 doubles the row
    out_m, w_m, lg_m = _run(q, k, v, 1.0, True, q_mask=qm)
    out, w, lg = _run(q, k, v, 1.0, True)
    assert np.array_equal(out_m, out) and np.array_equal(lg_m, lg)
    np.testing.assert_array_equal(w_m, w * qm[:, :, None])


def test_causal_and_value_mask_merge_into_one_penalty():
    q, k, v, _ = _data(4, Tq=9)
    vm = np.ones((3, 9), np.float32)
    vm[:, 5] = 0
    _, _, lg = _run(q, k, v, 1.0, True, v_mask=vm)
    _, _, lg0 = _run(q, k, v, 1.0, False)
    hidden_twice = np.triu(np.ones((9, 9), bool), 1)[:, 5]      # rows where key 5 is also after the query
    d = (lg0 - lg)[:, hidden_twice, 5]
    np.testing.assert_allclose(d, 1e9, rtol=1e-6)               # not 2e9


def test_all_keys_hidden_spreads_the_weight():
    """fp32: every logit of the row sits near -1e9, where fp32 resolves 64 units, so the row comes out (nearly) uniform
    over all keys -- also the ones after the query."""
    q, k, v, _ = _data(5, Tq=4, Tv=6)
    vm = np.ones((3, 6), np.float32)
    vm[1, :] = 0
    out, w, _ = _run(q, k, v, 1.0, True, v_mask=vm)
    np.testing.assert_allclose(w[1], np.full((4, 6), 1 / 6), rtol=1e-6)
    np.testing.assert_allclose(out[1], np.broadcast_to(v[1].mean(0), (4, 8)), rtol=1e-5, atol=1e-6)
