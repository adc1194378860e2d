"""Recorded sequences of a transformer block's linear layers on 5 to 32 rows (a batched decode step): the merging pass lets the
product that reads a layer_norm's output normalise the rows itself, and the product in front of the residual Add write
the sum.  Every array any of the separate ops would have written must come out with the same bits, in both replay modes."""
import numpy as np
import pytest

from deeplearning4j_amd import nativeops as N
from deeplearning4j_amd.executioner import Pairwise
from deeplearning4j_amd.ndarray import BFLOAT16, HALF, NDArray, bf16_bits_to_f32, f32_to_bf16_bits

pytestmark = pytest.mark.gpu


def _arr(a, dt):
    if dt == BFLOAT16:
        return NDArray.from_numpy(f32_to_bf16_bits(a.astype(np.float32)), BFLOAT16)
    return NDArray.from_numpy(a.astype(np.float16))


def _bits(A):
    a = A.to_numpy()
    return a if a.dtype == np.uint16 else a.view(np.uint16)


@pytest.mark.parametrize("dt", [BFLOAT16, HALF])
@pytest.mark.parametrize("rows,k,n1,n2", [(32, 768, 768, 2304), (8, 768, 768, 3072), (5, 512, 256, 512), (17, 320, 320, 64), (32, 576, 128, 1024),
                                          (32, 256, 256, 256), (32, 1024, 1024, 256)])
def test_add_layer_norm_product_chain_on_few_rows(ex, dt, rows, k, n1, n2):
    """p = a W1' + b1;  h += p;  ln = layer_norm(h);  z = ln W2' + b2;  act = gelu(z).  Row lengths the in-product
    normalisation takes (320 to 768) and ones it leaves to the separate kernel (256, 1024)."""
    L = ex.L
    rng = np.random.default_rng(rows * 1000 + k + n2)
    a, h = rng.normal(0, 1, (rows, n1)), rng.normal(0, 1, (rows, k))
    w1, b1 = rng.normal(0, n1 ** -0.5, (k, n1)), rng.normal(0, 0.1, k)
    w2, b2 = rng.normal(0, k ** -0.5, (n2, k)), rng.normal(0, 0.1, n2)
    gain, bias = rng.normal(1, 0.05, k), rng.normal(0, 0.05, k)
    A, W1, B1, W2, B2, G, Bi = (_arr(v, dt) for v in (a, w1, b1, w2, b2, gain, bias))

    def run(record):
        H = _arr(h, dt)
        P, Ln, Z, Act = NDArray.empty((rows, k), dt), NDArray.empty((rows, k), dt), NDArray.empty((rows, n2), dt), NDArray.empty((rows, n2), dt)
        for arr in (A, W1, B1, W2, B2, G, Bi, H):
            arr.sync_to_device()
        for arr in (P, Ln, Z, Act):
            L.dbAllocateSpecialBuffer(arr.buffer.ptr)
        calls = [ex.bind_custom("xw_plus_b", [A, W1, B1], [P], i_args=[0, 1]),
                 lambda: (L.execPairwiseTransform(None, Pairwise.Add, H.handle, P.handle, H.handle, None), N.check("execPairwiseTransform")),
                 ex.bind_custom("layer_norm", [H, G, Bi], [Ln], i_args=[1], b_args=[False]),
                 ex.bind_custom("xw_plus_b", [Ln, W2, B2], [Z], i_args=[0, 1]),
                 lambda: (L.execTransformStrict(None, 53, Z.handle, None, Act.handle), N.check("execTransformStrict"))]
        fused = 0
        if record:
            assert L.nd4jhipGraphBeginCapture() == 0, L.lastErrorMessage()
            for c in calls:
                c()
            g = L.nd4jhipGraphEndCapture()
            N.check("nd4jhipGraphEndCapture")
            assert g
            fused = L.nd4jhipGraphFusedOps(g)
            assert L.nd4jhipGraphFusedApplied(g) == fused      # no merged step fell back to separate launches
            assert L.nd4jhipGraphAudit(g) == 0, L.lastErrorMessage()
            outs = []
            try:
                for mode in (1, 0):
                    L.nd4jhipSetGraphReplayMode(mode)
                    H.assign_numpy(_arr(h, dt).to_numpy())
                    assert L.nd4jhipGraphLaunch(g) == 0, L.lastErrorMessage()
                    outs.append([_bits(x).copy() for x in (P, H, Ln, Z, Act)])
            finally:
                L.nd4jhipSetGraphReplayMode(0)
                L.nd4jhipGraphDestroy(g)
            return outs, fused
        for c in calls:
            c()
        return [[_bits(x).copy() for x in (P, H, Ln, Z, Act)]], 0

    (want,), _ = run(False)
    got, fused = run(True)
    # the Add rides in the first product when the layer_norm behind it rides in the second; the GELU always rides
    in_product = 320 <= k <= 768
    assert fused == (3 if in_product else 2), fused
    for outs in got:
        for name, g_, w_ in zip(("p", "h", "ln", "z", "act"), outs, want):
            assert np.array_equal(g_, w_), (name, int((g_ != w_).sum()))
    ln = want[2]
    lnf = bf16_bits_to_f32(ln) if dt == BFLOAT16 else ln.view(np.float16).astype(np.float32)
    assert np.isfinite(lnf).all() and 0.5 < lnf.std() < 2.0


@pytest.mark.parametrize("dt", [BFLOAT16, HALF])
@pytest.mark.parametrize("heads,dh,tv", [(12, 64, 640), (6, 128, 900)])
def test_one_token_attention_merges_inside_the_projection(ex, dt, heads, dh, tv):
    """att = attention(q [1, H, 1, D]; cache [1, H, Tv, D]);  p = att W' + b;  h += p.  The attention cuts its key range into
    four parts; recorded, the projection merges the parts on its way in (no merge launch) and still writes `att`."""
    L = ex.L
    rng = np.random.default_rng(heads * tv)
    d = heads * dh
    q, k, v = rng.normal(0, 1, (1, heads, 1, dh)), rng.normal(0, 1, (1, heads, tv, dh)), rng.normal(0, 1, (1, heads, tv, dh))
    w, b, h = rng.normal(0, d ** -0.5, (d, d)), rng.normal(0, 0.1, d), rng.normal(0, 1, (1, d))
    Q, K, V, W, B = (_arr(a, dt) for a in (q, k, v, w, b))
    scale = dh ** -0.5

    def run(record):
        H = _arr(h, dt)
        Att, P = NDArray.empty((1, d), dt), NDArray.empty((1, d), dt)
        for arr in (Q, K, V, W, B, H):
            arr.sync_to_device()
        for arr in (Att, P):
            L.dbAllocateSpecialBuffer(arr.buffer.ptr)
        att4 = Att.view((1, heads, 1, dh), (d, dh, dh, 1))
        calls = [ex.bind_custom("dot_product_attention_v2", [Q, V, K], [att4], t_args=[scale, 0.0], b_args=[False, False]),
                 ex.bind_custom("xw_plus_b", [Att, W, B], [P], i_args=[0, 1]),
                 lambda: (L.execPairwiseTransform(None, Pairwise.Add, H.handle, P.handle, H.handle, None), N.check("execPairwiseTransform"))]
        if not record:
            for c in calls:
                c()
            return [[_bits(x).copy() for x in (Att, P, H)]], ""
        assert L.nd4jhipGraphBeginCapture() == 0, L.lastErrorMessage()
        for c in calls:
            c()
        g = L.nd4jhipGraphEndCapture()
        N.check("nd4jhipGraphEndCapture")
        assert g and L.nd4jhipGraphFusedOps(g) == 1 and L.nd4jhipGraphFusedApplied(g) == 1     # the Add rides in the projection
        assert L.nd4jhipGraphAudit(g) == 0, L.lastErrorMessage()
        outs, kern = [], ""
        try:
            for mode in (1, 0):
                L.nd4jhipSetGraphReplayMode(mode)
                H.assign_numpy(_arr(h, dt).to_numpy())
                Att.assign_numpy(np.zeros((1, d), np.uint16 if dt == BFLOAT16 else np.float16))
                assert L.nd4jhipGraphLaunch(g) == 0, L.lastErrorMessage()
                if mode == 1:
                    kern = L.nd4jhipLastGemmKernel().decode()
                outs.append([_bits(x).copy() for x in (Att, P, H)])
        finally:
            L.nd4jhipSetGraphReplayMode(0)
            L.nd4jhipGraphDestroy(g)
        return outs, kern

    (want,), _ = run(False)
    got, kern = run(True)
    assert "attn-merge" in kern, kern
    for outs in got:
        for name, g_, w_ in zip(("att", "p", "h"), outs, want):
            assert np.array_equal(g_, w_), (name, int((g_ != w_).sum()))
