"""BASELINE configs 3 and 4 at their full sizes: size-independent properties over the whole result, and the oracle
on a sample of rows / batch entries (the oracle would need minutes for the whole arrays).

Config 3: x [16, 1024, 768] -> layer_norm over the last axis -> gelu; softmax over the last axis of logits
[16, 12, 1024, 1024], dense and through the permuted [0, 2, 1, 3] view.  Config 4: causal attention on
[96, 1024, 64] (8 x 12 heads folded into the batch)."""
import numpy as np
import pytest

from conftest import assert_close
from deeplearning4j_amd.executioner import TransformStrict
from deeplearning4j_amd.ndarray import BFLOAT16, FLOAT32, HALF, NDArray, bf16_bits_to_f32, f32_to_bf16_bits

pytestmark = pytest.mark.gpu


def _store(a, dt):
    """fp32 draw -> (values as stored, device array)."""
    if dt == BFLOAT16:
        bits = f32_to_bf16_bits(a)
        return bf16_bits_to_f32(bits), NDArray.from_numpy(bits, BFLOAT16)
    if dt == HALF:
        h = a.astype(np.float16)
        return h.astype(np.float32), NDArray.from_numpy(h)
    return a, NDArray.from_numpy(a)


def _oracle_arr(oracle, vals, dt):
    if dt == BFLOAT16:
        return oracle.Arr(f32_to_bf16_bits(vals), oracle.BFLOAT16)
    if dt == HALF:
        return oracle.Arr(vals.astype(np.float16))
    return oracle.Arr(vals.astype(np.float32))


def _as_float(oa):
    return bf16_bits_to_f32(oa.a) if oa.dt == 17 else oa.a.astype(np.float32)


@pytest.mark.parametrize("dt,tol", [(FLOAT32, 1e-5), (BFLOAT16, 1e-2)])
def test_config3_layer_norm_then_gelu(ex, oracle, dt, tol):
    rng = np.random.default_rng(3003)
    x, X = _store(rng.normal(0, 1, (16, 1024, 768)).astype(np.float32), dt)
    g, G = _store(rng.normal(1, 0.02, 768).astype(np.float32), dt)
    b, B = _store(rng.normal(0, 0.02, 768).astype(np.float32), dt)
    y = ex.exec_custom("layer_norm", [X, G, B], i_args=[2], b_args=[False])[0]
    z = ex.exec_transform_strict(TransformStrict.GELU, y)
    yf, zf = y.to_float(), z.to_float()
    # whole result: undoing gain and bias leaves rows of mean 0 and variance var / (var + 1e-5)
    u = (yf.astype(np.float64) - b) / g
    atol = 3e-2 if dt == BFLOAT16 else 1e-4
    assert np.abs(u.mean(-1)).max() < atol
    var = x.astype(np.float64).var(-1)
    assert np.abs(u.var(-1) - var / (var + 1e-5)).max() < (5e-2 if dt == BFLOAT16 else 1e-3)
    # gelu(y) = y * sigmoid(1.702 y) has the sign of y and never exceeds |y|
    assert np.all(np.abs(zf) <= np.abs(yf) + 1e-6) and np.all((zf >= 0) | (yf < 0))
    # sampled rows against the oracle, both ops
    rows = [(0, 0), (3, 517), (15, 1023), (8, 64)]
    xs = np.stack([x[i, j] for i, j in rows])
    oy = _oracle_arr(oracle, np.zeros_like(xs), dt)
    oracle.layer_norm(_oracle_arr(oracle, xs, dt), _oracle_arr(oracle, g, dt), _oracle_arr(oracle, b, dt), oy, [1], channels_first=False)
    got_y = np.stack([yf[i, j] for i, j in rows])
    assert_close(got_y, _as_float(oy), tol, tol, "layer_norm rows")
    oz = _oracle_arr(oracle, np.zeros_like(xs), dt)
    oracle.transform_strict(TransformStrict.GELU, _oracle_arr(oracle, got_y, dt), oz)
    assert_close(np.stack([zf[i, j] for i, j in rows]), _as_float(oz), tol, tol, "gelu rows")


@pytest.mark.parametrize("dt,tol", [(FLOAT32, 1e-5), (BFLOAT16, 1e-2)])
def test_config3_softmax_dense_and_permuted_view(ex, oracle, dt, tol):
    rng = np.random.default_rng(3003)
    shape = (16, 12, 1024, 1024)
    logits, L = _store(rng.normal(0, 2, shape).astype(np.float32), dt)
    z = ex.exec_custom("softmax", [L])[0].to_float()
    # whole result: rows sum to one, entries lie in [0, 1], the largest logit keeps the largest weight
    sums = z.sum(-1, dtype=np.float64)
    assert np.abs(sums - 1).max() < (2e-2 if dt == BFLOAT16 else 1e-5)
    assert z.min() >= 0 and z.max() <= 1
    am = logits.argmax(-1)
    assert np.all(np.take_along_axis(z, am[..., None], -1)[..., 0] >= z.max(-1) - 1e-7)
    # sampled rows against the oracle
    idx = [(0, 0, 0), (7, 5, 333), (15, 11, 1023)]
    xs = np.stack([logits[i] for i in idx])
    oz = _oracle_arr(oracle, np.zeros_like(xs), dt)
    oracle.softmax(_oracle_arr(oracle, xs, dt), oz, 1)
    assert_close(np.stack([z[i] for i in idx]), _as_float(oz), tol, tol * 1e-2, "softmax rows")
    # the same numbers laid out [16, 1024, 12, 1024] and seen through permute(0, 2, 1, 3): bit-identical result
    # (both layouts go through fp32 arithmetic and one rounding to the storage type)
    _, P = _store(np.ascontiguousarray(logits.transpose(0, 2, 1, 3)), dt)
    zp = ex.exec_custom("softmax", [P.permute(0, 2, 1, 3)], [NDArray.empty(shape, dt)])[0].to_float()
    assert np.array_equal(zp, z)


@pytest.mark.parametrize("dt", [HALF, BFLOAT16, FLOAT32])
def test_config4_causal_attention(ex, oracle, dt):
    tol = 1e-4 if dt == FLOAT32 else 1e-2        # the fp32 tile kernel at the config's shape, to the fp32 gate
    rng = np.random.default_rng(4004)
    B, T, D = 96, 1024, 64
    q, Q = _store(rng.normal(0, 1, (B, T, D)).astype(np.float32), dt)
    k, K = _store(rng.normal(0, 1, (B, T, D)).astype(np.float32), dt)
    v, V = _store(rng.normal(0, 1, (B, T, D)).astype(np.float32), dt)
    out = ex.exec_custom("dot_product_attention_v2", [Q, V, K], [NDArray.empty((B, T, D), dt)], t_args=[0.125, 0.0], b_args=[True, False])[0].to_float()
    assert np.isfinite(out).all()
    # whole result: the first query sees one key, so its output is that value row; every output is a convex
    # combination of the value rows it may see
    assert_close(out[:, 0], v[:, 0], tol, tol, "query 0")
    vmax, vmin = np.maximum.accumulate(v, axis=1), np.minimum.accumulate(v, axis=1)
    assert np.all(out <= vmax + 2 * tol) and np.all(out >= vmin - 2 * tol)
    # sampled batch entries against the oracle (the reference's unfused sequence on [1, T, D])
    for bi in (0, 41, 95):
        oo = _oracle_arr(oracle, np.zeros((1, T, D), np.float32), dt)
        oracle.attention_v2(_oracle_arr(oracle, q[bi:bi + 1], dt), _oracle_arr(oracle, v[bi:bi + 1], dt), _oracle_arr(oracle, k[bi:bi + 1], dt), oo,
                            scale=0.125, causal=True)
        assert_close(out[bi:bi + 1], _as_float(oo), tol, tol, "batch entry %d" % bi)


@pytest.mark.parametrize("dt", [BFLOAT16, FLOAT32])
@pytest.mark.parametrize("B,T", [(40, 1024), (50, 768), (37, 1280), (72, 512), (264, 384)])
def test_causal_attention_in_every_block_order(ex, oracle, dt, B, T):
    """Launches whose blocks all fit on the chip at once take their query tiles in an order the host lays out (with a
    multiple of 8 batch entries, and without), larger ones heavy tiles first, small ones in mirrored pairs: the same
    results whichever applies.  Sampled batch entries against the oracle, and every row inside the hull of the value rows
    it may see."""
    tol = 1e-4 if dt == FLOAT32 else 1e-2
    rng = np.random.default_rng(B * 10000 + T)
    D = 64
    q, Q = _store(rng.normal(0, 1, (B, T, D)).astype(np.float32), dt)
    k, K = _store(rng.normal(0, 1, (B, T, D)).astype(np.float32), dt)
    v, V = _store(rng.normal(0, 1, (B, T, D)).astype(np.float32), dt)
    out = ex.exec_custom("dot_product_attention_v2", [Q, V, K], [NDArray.empty((B, T, D), dt)], t_args=[0.125, 0.0], b_args=[True, False])[0].to_float()
    assert np.isfinite(out).all()
    assert_close(out[:, 0], v[:, 0], tol, tol, "query 0")
    vmax, vmin = np.maximum.accumulate(v, axis=1), np.minimum.accumulate(v, axis=1)
    assert np.all(out <= vmax + 2 * tol) and np.all(out >= vmin - 2 * tol)
    for bi in (0, B // 2 + 1, B - 1):
        oo = _oracle_arr(oracle, np.zeros((1, T, D), np.float32), dt)
        oracle.attention_v2(_oracle_arr(oracle, q[bi:bi + 1], dt), _oracle_arr(oracle, v[bi:bi + 1], dt), _oracle_arr(oracle, k[bi:bi + 1], dt), oo,
                            scale=0.125, causal=True)
        assert_close(out[bi:bi + 1], _as_float(oo), tol, tol, "batch entry %d" % bi)


@pytest.mark.parametrize("dt", [BFLOAT16, FLOAT32])
def test_causal_prefill_over_token_major_heads_equals_the_dense_layout(ex, dt):
    """A decoder's prefill: [batch, heads, T, 64] views of a token-major qkv buffer (batch and head strides that do not
    nest), 5 x 12 heads x 8 query tiles -- a launch that is on the chip at once and takes the host-made block order with a
    number of batch entries that is no multiple of 8.  The same numbers laid out densely [60, T, 64] give the same bits."""
    rng = np.random.default_rng(77)
    B, H, T, D = 5, 12, 1024, 64
    d = H * D
    qkv = rng.normal(0, 1, (B, T, 3 * d)).astype(np.float32)
    _, Q = _store(qkv, dt)
    qkv_r = Q.to_float().reshape(B, T, 3, H, D)
    att = NDArray.empty((B, T, d), dt)
    views = [Q.view((B, H, T, D), (T * 3 * d, D, 3 * d, 1), which * d) for which in range(3)]
    o4 = att.view((B, H, T, D), (T * d, D, d, 1), 0)
    ex.exec_custom("dot_product_attention_v2", [views[0], views[2], views[1]], [o4], t_args=[0.125, 0.0], b_args=[True, False])
    got = att.to_float().reshape(B, T, H, D).transpose(0, 2, 1, 3).reshape(B * H, T, D)
    dense = [NDArray.from_numpy(np.ascontiguousarray(qkv_r[:, :, which].transpose(0, 2, 1, 3).reshape(B * H, T, D)), dt) for which in range(3)]
    want = ex.exec_custom("dot_product_attention_v2", [dense[0], dense[2], dense[1]], [NDArray.empty((B * H, T, D), dt)], t_args=[0.125, 0.0],
                          b_args=[True, False])[0].to_float()
    assert np.isfinite(got).all() and np.array_equal(got, want)
    v = qkv_r[:, :, 2].transpose(0, 2, 1, 3).reshape(B * H, T, D)
    tol = 1e-4 if dt == FLOAT32 else 1e-2
    assert_close(got[:, 0], v[:, 0], tol, tol, "query 0")


@pytest.mark.parametrize("dt", [HALF, BFLOAT16])
def test_config4_weights_and_logits_outputs(ex, oracle, dt):
    """The same op with its second and third outputs requested (attention weights and clipped, masked logits) at the
    config's sequence length: [12, 1024, 64] -> weights and logits [12, 1024, 1024].  Whole-result properties, then two
    batch entries against the oracle."""
    rng = np.random.default_rng(4004)
    B, T, D = 12, 1024, 64
    q, Q = _store(rng.normal(0, 1, (B, T, D)).astype(np.float32), dt)
    k, K = _store(rng.normal(0, 1, (B, T, D)).astype(np.float32), dt)
    v, V = _store(rng.normal(0, 1, (B, T, D)).astype(np.float32), dt)
    outs = ex.exec_custom("dot_product_attention_v2", [Q, V, K], [NDArray.empty((B, T, D), dt), NDArray.empty((B, T, T), dt), NDArray.empty((B, T, T), dt)],
                          t_args=[0.125, 0.0], b_args=[True, False])
    out, w, lg = (o.to_float() for o in outs)
    # weights: rows are distributions over the keys a query may see (the mask leaves exact zeros)
    upper = np.triu(np.ones((T, T), bool), 1)
    assert np.all(w[:, upper] == 0.0) and np.all(w >= 0.0)
    assert np.abs(w.astype(np.float64).sum(-1) - 1.0).max() < (2e-2 if dt == BFLOAT16 else 3e-3)
    # logits: the scaled products below the diagonal, the penalty above it
    assert np.all(lg[:, upper] < -6.0e4)
    i, j = 700, 123
    assert_close(lg[:, i, j], 0.125 * (q[:, i].astype(np.float64) * k[:, j]).sum(-1), 1e-2, 2e-2, "one logit per batch entry")
    # the output is the weights applied to the values
    assert_close(out[5], w[5].astype(np.float64) @ v[5], 1e-2, 2e-2, "out = weights v")
    for bi in (0, 11):
        oo, ow, ol = (_oracle_arr(oracle, np.zeros(s_, np.float32), dt) for s_ in ((1, T, D), (1, T, T), (1, T, T)))
        oracle.attention_v2(_oracle_arr(oracle, q[bi:bi + 1], dt), _oracle_arr(oracle, v[bi:bi + 1], dt), _oracle_arr(oracle, k[bi:bi + 1], dt), oo,
                            weights=ow, logits=ol, scale=0.125, causal=True)
        assert_close(out[bi:bi + 1], _as_float(oo), 1e-2, 1e-2, "out, batch entry %d" % bi)
        assert_close(w[bi:bi + 1], _as_float(ow), 1e-2, 1e-2, "weights, batch entry %d" % bi)
        lo, lgot = _as_float(ol), lg[bi:bi + 1]
        keep = ~upper[None]
        assert_close(lgot[keep], lo[keep], 1e-2, 2e-2, "logits below the diagonal, batch entry %d" % bi)
        assert np.array_equal(lgot[~keep], lo[~keep]) or np.allclose(lgot[~keep], lo[~keep], rtol=1e-2)


@pytest.mark.parametrize("dt,L,tol", [(BFLOAT16, 768, 1e-2), (HALF, 768, 2e-3), (FLOAT32, 384, 1e-5),
                                      (BFLOAT16, 384, 1e-2), (HALF, 1152, 2e-3), (BFLOAT16, 1152, 1e-2), (HALF, 640, 2e-3)])
@pytest.mark.parametrize("rows,has_bias,pitched", [(4097, True, False), (4608, False, False), (4099, True, True)])
def test_layer_norm_rows_of_one_and_a_half_passes(ex, oracle, dt, L, tol, rows, has_bias, pitched):
    """Many rows (two per wave) whose length is not a whole number of 16-byte wave passes: 16-bit rows of 384, 768 and
    1152 go in 12-byte vectors (one, two, three full passes), fp32 rows of 384 and 16-bit rows of 640 in 16-byte vectors
    with the last pass partly masked.  An odd row count (the last wave has a lone row), no bias, and rows at a pitch (the
    left columns of a wider matrix), every row against the oracle."""
    rng = np.random.default_rng(rows + L + int(has_bias))
    width = L + 64 if pitched else L
    full, Full = _store(rng.normal(0.3, 2.0, (rows, width)).astype(np.float32), dt)
    x = full[:, :L]
    X = Full.slice(1, 0, L) if pitched else Full
    g, G = _store(rng.normal(1, 0.1, L).astype(np.float32), dt)
    b, B = _store(rng.normal(0, 0.1, L).astype(np.float32), dt)
    ins = [X, G, B] if has_bias else [X, G]
    y = ex.exec_custom("layer_norm", ins, i_args=[1], b_args=[False])[0].to_float()
    oy = _oracle_arr(oracle, np.zeros_like(x), dt)
    oins = [_oracle_arr(oracle, np.ascontiguousarray(x), dt), _oracle_arr(oracle, g, dt)] + ([_oracle_arr(oracle, b, dt)] if has_bias else [None])
    oracle.layer_norm(oins[0], oins[1], oins[2], oy, [1], channels_first=False)
    assert_close(y, _as_float(oy), tol, tol, "layer_norm, %d rows of %d" % (rows, L))
