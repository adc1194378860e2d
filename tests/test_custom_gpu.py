"""GPU parity tests of the declarable ops (matmul, softmax, layer_norm, dot_product_attention_v2, argmax and the
decoder glue ops), driven through OpContext + execCustomOp2 exactly as the Java executioner drives them.

Gates (north star): fp32 softmax / layer_norm |a-b| <= 1e-6 + 1e-5 |b|; fp32 mmul / attention <= 1e-4;
fp16 / bf16 <= 1e-2 against the fp32-accumulated oracle on the rounded inputs; argmax bit-exact.
"""
import math

import numpy as np
import pytest

from conftest import assert_close, materialize
from deeplearning4j_amd.ndarray import BFLOAT16, DOUBLE, FLOAT32, HALF, INT32, INT64, NDArray, bf16_bits_to_f32, f32_to_bf16_bits
from deeplearning4j_amd.nativeops import NativeOpsError

pytestmark = pytest.mark.gpu


def _pair(oracle, a, dtype):
    if dtype == BFLOAT16:
        bits = f32_to_bf16_bits(np.asarray(a, np.float32))
        return oracle.Arr(bits, oracle.BFLOAT16), NDArray.from_numpy(bits, BFLOAT16)
    npdt = {HALF: np.float16, FLOAT32: np.float32, DOUBLE: np.float64}[dtype]
    h = np.asarray(a).astype(npdt)
    return oracle.Arr(h), NDArray.from_numpy(h)


def _ozeros(oracle, shape, dtype):
    npdt = {HALF: np.float16, FLOAT32: np.float32, DOUBLE: np.float64, BFLOAT16: np.uint16}[dtype]
    return oracle.Arr(np.zeros(shape, npdt), dtype)


def _f(oa):
    return bf16_bits_to_f32(oa.a).astype(np.float64) if oa.dt == 17 else oa.a.astype(np.float64)


def _nd(spec, dtype=None):
    a = materialize(spec)
    return NDArray.from_numpy(np.ascontiguousarray(a) if spec["order"] != "f" else a, dtype, order=spec["order"] if a.ndim > 1 else "c")


# ---- the reference's own known-answer vectors ----------------------------------------------------------------------
def test_golden_matmul(ex, golden):
    cases = [c for c in golden if c["op"] == "matmul"]
    assert len(cases) >= 35
    for c in cases:
        x, y = _nd(c["inputs"][0]), _nd(c["inputs"][1])
        exp = materialize(c["expected"])
        outs = [_nd(c["initial_output"])] if "initial_output" in c else None
        z = ex.exec_custom("matmul", [x, y], outs, t_args=c["targs"], i_args=c["iargs"])[0]
        assert tuple(z.shape) == tuple(exp.shape), c["name"]
        if outs is None:
            # shape function: 'c' only when both inputs are 'c' (generic/blas/matmul.cpp:189-219)
            assert z.order == ("c" if x.order == "c" and y.order == "c" else "f"), c["name"]
        assert_close(z.to_numpy(), exp, 1e-6, 1e-9, c["name"])


def test_golden_softmax(ex, golden):
    cases = [c for c in golden if c["op"] == "softmax"]
    assert len(cases) == 12
    for c in cases:
        x = _nd(c["inputs"][0])
        z = ex.exec_custom("softmax", [x], i_args=c["iargs"])[0]
        assert_close(z.to_numpy(), materialize(c["expected"]), 1e-4, 1e-5, c["name"])


def test_golden_argmax(ex, golden):
    cases = [c for c in golden if c["op"] == "argmax"]
    for c in cases:
        x = _nd(c["inputs"][0])
        ins = [x]
        if len(c["inputs"]) > 1:   # axis array: the Java side passes integer axes
            ins.append(NDArray.from_numpy(materialize(c["inputs"][1]).astype(np.int64).ravel()))
        z = ex.exec_custom("argmax", ins, i_args=c["iargs"])[0]
        exp = materialize(c["expected"]).astype(np.int64)
        assert z.dtype == INT64 and np.array_equal(z.to_numpy(), exp), c["name"]


# ---- matmul ----------------------------------------------------------------------------------------------------------
@pytest.mark.parametrize("dtype,tol", [(FLOAT32, 1e-4), (HALF, 1e-2), (BFLOAT16, 1e-2), (DOUBLE, 1e-10)])
@pytest.mark.parametrize("M,N,K", [(64, 64, 64), (256, 256, 256), (130, 70, 50), (1, 768, 2304), (32, 768, 3072), (257, 129, 1024), (512, 384, 72)])
def test_matmul_vs_oracle(ex, oracle, dtype, tol, M, N, K):
    rng = np.random.default_rng(M + N + K)
    a = rng.normal(0, 1 / math.sqrt(K), (M, K))
    b = rng.normal(0, 1 / math.sqrt(K), (K, N))
    oa, da = _pair(oracle, a, dtype)
    ob, db = _pair(oracle, b, dtype)
    oz = _ozeros(oracle, (M, N), dtype)
    oracle.matmul(oa, ob, oz, accumulate=2 if dtype == DOUBLE else 1)
    z = ex.exec_custom("matmul", [da, db])[0]
    got = z.to_float() if dtype != DOUBLE else z.to_numpy()
    assert_close(got, _f(oz), tol, tol, "matmul %dx%dx%d dtype %d" % (M, N, K, dtype))
    # transposeB variant: same numbers from B stored as [N, K]
    obt, dbt = _pair(oracle, b.T.copy(), dtype)
    zt = ex.exec_custom("matmul", [da, dbt], i_args=[0, 1])[0]
    gt = zt.to_float() if dtype != DOUBLE else zt.to_numpy()
    assert_close(gt, _f(oz), tol, tol, "matmul transposeB")
    # transposeA
    oat, dat = _pair(oracle, a.T.copy(), dtype)
    za = ex.exec_custom("matmul", [dat, db], i_args=[1, 0])[0]
    ga = za.to_float() if dtype != DOUBLE else za.to_numpy()
    assert_close(ga, _f(oz), tol, tol, "matmul transposeA")


@pytest.mark.parametrize("dtype", [HALF, BFLOAT16])
@pytest.mark.parametrize("M,N,K", [(1, 2304, 768), (5, 768, 3072), (32, 3072, 768), (48, 200, 1024), (64, 64, 4096)])
def test_matmul_small_m_split_k(ex, oracle, dtype, M, N, K):
    """Skinny products take the split-K path (partial tiles + arrival tickets); run it repeatedly, so that tickets left
    over by one launch would show in the next, and with alpha/beta so the last-arriving block's epilogue is covered."""
    rng = np.random.default_rng(M * 7 + N + K)
    a = rng.normal(0, 1 / math.sqrt(K), (M, K))
    b = rng.normal(0, 1 / math.sqrt(K), (K, N))
    c0 = rng.normal(0, 1, (M, N))
    oa, da = _pair(oracle, a, dtype)
    ob, db = _pair(oracle, b, dtype)
    oz, dz = _pair(oracle, c0, dtype)
    oracle.matmul(oa, ob, oz, alpha=0.5, beta=2.0, accumulate=1)
    for rep in range(3):
        _, dz = _pair(oracle, c0, dtype)
        ex.exec_custom("matmul", [da, db], [dz], t_args=[0.5, 2.0])
        assert_close(dz.to_float(), _f(oz), 1e-2, 1e-2, "split-K repeat %d" % rep)
    # many launches back to back on one output, read once
    outs = [NDArray.empty((M, N), dtype) for _ in range(8)]
    for o in outs:
        ex.exec_custom("matmul", [da, db], [o])
    oz1 = _ozeros(oracle, (M, N), dtype)
    oracle.matmul(oa, ob, oz1, accumulate=1)
    for o in outs:
        assert_close(o.to_float(), _f(oz1), 1e-2, 1e-2, "split-K back to back")


@pytest.mark.parametrize("dtype,tol", [(FLOAT32, 1e-4), (BFLOAT16, 1e-2)])
def test_matmul_batched_alpha_beta_views(ex, oracle, dtype, tol):
    rng = np.random.default_rng(21)
    a = rng.normal(0, 0.2, (3, 2, 40, 24))
    b = rng.normal(0, 0.2, (3, 2, 24, 56))
    c0 = rng.normal(0, 1, (3, 2, 40, 56))
    oa, da = _pair(oracle, a, dtype)
    ob, db = _pair(oracle, b, dtype)
    oc, dc = _pair(oracle, c0, dtype)
    oracle.matmul(oa, ob, oc, alpha=0.5, beta=2.0, accumulate=1)
    ex.exec_custom("matmul", [da, db], [dc], t_args=[0.5, 2.0])
    assert_close(dc.to_float(), _f(oc), tol, tol, "batched alpha/beta")
    # permuted (strided) operands: x^T through a view instead of the transpose flag
    z = ex.exec_custom("matmul", [da.permute(0, 1, 3, 2), db], i_args=[1, 0])[0]
    oz = _ozeros(oracle, (3, 2, 40, 56), dtype)
    oracle.matmul(oa, ob, oz, accumulate=1)
    assert_close(z.to_float(), _f(oz), tol, tol, "permuted view + transX")


def test_matmul_shape_and_type_errors(ex):
    x = NDArray.from_numpy(np.zeros((3, 4), np.float32))
    y = NDArray.from_numpy(np.zeros((5, 3), np.float32))
    with pytest.raises(NativeOpsError, match="inconsistent shapes"):
        ex.exec_custom("matmul", [x, y])
    with pytest.raises(NativeOpsError, match="share one data type"):
        ex.exec_custom("matmul", [x, NDArray.from_numpy(np.zeros((4, 2), np.float64))], [NDArray.empty((3, 2), FLOAT32)])
    with pytest.raises(NativeOpsError, match="output array is wrong"):
        ex.exec_custom("matmul", [x, NDArray.from_numpy(np.zeros((4, 2), np.float32))], [NDArray.empty((3, 3), FLOAT32)])
    with pytest.raises(NativeOpsError, match="not registered"):
        ex.exec_custom("conv2d", [x])


def test_mmul_full_size_properties(ex):
    """4096^3 bf16 (BASELINE config 2): the oracle checks a sample of output elements in fp64; linearity and
    the transposeB identity hold for the whole result."""
    rng = np.random.default_rng(2002)
    n = 4096
    a = f32_to_bf16_bits(rng.normal(0, 1 / 64, (n, n)).astype(np.float32))
    b = f32_to_bf16_bits(rng.normal(0, 1 / 64, (n, n)).astype(np.float32))
    A, B = NDArray.from_numpy(a, BFLOAT16), NDArray.from_numpy(b, BFLOAT16)
    z = ex.exec_custom("matmul", [A, B])[0].to_float()
    af, bf = bf16_bits_to_f32(a).astype(np.float64), bf16_bits_to_f32(b).astype(np.float64)
    rows = rng.choice(n, 16, replace=False)
    cols = rng.choice(n, 16, replace=False)
    want = af[rows] @ bf[:, cols]
    assert_close(z[np.ix_(rows, cols)], want, 1e-2, 1e-2, "sampled elements")
    Bt = NDArray.from_numpy(np.ascontiguousarray(b.T), BFLOAT16)
    zt = ex.exec_custom("matmul", [A, Bt], i_args=[0, 1])[0].to_float()
    assert_close(zt, z, 1e-2, 1e-2, "transposeB agrees with plain B")


@pytest.mark.parametrize("dtype,tol", [(FLOAT32, 1e-4), (HALF, 1e-2), (BFLOAT16, 1e-2)])
@pytest.mark.parametrize("M,K,N", [(1, 768, 2304), (32, 3072, 768), (300, 256, 512), (7, 40, 24), (512, 512, 512)])
def test_xw_plus_b_vs_oracle(ex, oracle, dtype, tol, M, K, N):
    """z = x w + b; the oracle runs the reference's own two steps (mmul, then the bias row added to every row)."""
    rng = np.random.default_rng(M + K + N)
    x = rng.normal(0, 1 / math.sqrt(K), (M, K))
    w = rng.normal(0, 1, (K, N))
    b = rng.normal(0, 1, (N,))
    ox, dx = _pair(oracle, x, dtype)
    ow, dw = _pair(oracle, w, dtype)
    ob, db = _pair(oracle, b, dtype)
    oz = _ozeros(oracle, (M, N), dtype)
    oracle.matmul(ox, ow, oz, accumulate=1)
    oracle.add_row_vector(oz, ob, oz)
    z = ex.exec_custom("xw_plus_b", [dx, dw, db])[0]
    assert z.shape == (M, N)
    assert_close(z.to_float(), _f(oz), tol, tol, "xw_plus_b")
    # weights stored [N, K] (transpose flag 1) and a rank-3 x
    owt, dwt = _pair(oracle, w.T.copy(), dtype)
    zt = ex.exec_custom("xw_plus_b", [dx, dwt, db], i_args=[0, 1])[0]
    assert_close(zt.to_float(), _f(oz), tol, tol, "xw_plus_b, transposed weights")
    if M % 4 == 0:
        x3 = NDArray.from_numpy(np.asarray(ox.a).reshape(4, M // 4, K), dtype)
        z3 = ex.exec_custom("xw_plus_b", [x3, dw, db])[0]
        assert z3.shape == (4, M // 4, N)
        assert_close(z3.to_float().reshape(M, N), _f(oz), tol, tol, "xw_plus_b, rank-3 x")


@pytest.mark.parametrize("dtype", [BFLOAT16, HALF])
@pytest.mark.parametrize("M", [1, 2, 3, 4])
@pytest.mark.parametrize("K,N", [(768, 2304), (768, 768), (3072, 768), (768, 3072), (256, 288), (512, 1536), (320, 1536)])
def test_few_rows_times_row_major_weights(ex, oracle, dtype, M, K, N):
    """The decode-step shape: up to four rows of x against row-major weights (one strip kernel, no split-K partials),
    with and without the bias row, against the fp32-accumulating oracle."""
    rng = np.random.default_rng(M * 7 + K + N)
    x = rng.normal(0, 1, (M, K))
    w = rng.normal(0, 1 / math.sqrt(K), (K, N))
    b = rng.normal(0, 1, (N,))
    ox, dx = _pair(oracle, x, dtype)
    ow, dw = _pair(oracle, w, dtype)
    ob, db = _pair(oracle, b, dtype)
    oz = _ozeros(oracle, (M, N), dtype)
    oracle.matmul(ox, ow, oz, accumulate=1)
    z = ex.exec_custom("matmul", [dx, dw])[0]
    assert_close(z.to_float(), _f(oz), 1e-2, 1e-2, "few rows x row-major W")
    oracle.add_row_vector(oz, ob, oz)
    zb = ex.exec_custom("xw_plus_b", [dx, dw, db])[0]
    assert_close(zb.to_float(), _f(oz), 1e-2, 1e-2, "few rows x row-major W + bias")
    # the same rows as a strided view (row stride 2K) give the same bits
    wide = np.zeros((M, 2 * K), np.asarray(ox.a).dtype)
    wide[:, :K] = np.asarray(ox.a)
    xv = NDArray.from_numpy(wide, dtype).view((M, K), (2 * K, 1), 0)
    zv = ex.exec_custom("xw_plus_b", [xv, dw, db], outputs=[NDArray.empty((M, N), dtype)])[0]
    assert np.array_equal(zv.to_numpy(), zb.to_numpy())


@pytest.mark.parametrize("dtype", [BFLOAT16, HALF, FLOAT32])
@pytest.mark.parametrize("K,N", [(768, 2304), (768, 768), (3072, 768), (768, 3072), (768, 50257), (64, 5), (1024, 33), (8192, 7), (200, 64)])
def test_row_times_k_contiguous_weights(ex, oracle, dtype, K, N):
    """One row of x against [out, in] weights with the transpose flag (a decode step's projection and the tied output
    embedding): rows up to 12 wave passes long are held in registers, longer ones take the looping kernel."""
    rng = np.random.default_rng(K + N)
    x = rng.normal(0, 1, (1, K))
    wt = rng.normal(0, 1 / math.sqrt(K), (N, K))
    b = rng.normal(0, 1, (N,))
    ox, dx = _pair(oracle, x, dtype)
    ow, dw = _pair(oracle, wt, dtype)
    ob, db = _pair(oracle, b, dtype)
    oz = _ozeros(oracle, (1, N), dtype)
    oracle.matmul(ox, ow, oz, trans_y=True, accumulate=1)
    tol = 1e-4 if dtype == FLOAT32 else 1e-2
    z = ex.exec_custom("matmul", [dx, dw], i_args=[0, 1])[0]
    assert_close(z.to_float(), _f(oz), tol, tol, "row x W^T")
    oracle.add_row_vector(oz, ob, oz)
    zb = ex.exec_custom("xw_plus_b", [dx, dw, db], i_args=[0, 1])[0]
    assert_close(zb.to_float(), _f(oz), tol, tol, "row x W^T + bias")


@pytest.mark.parametrize("dtype", [BFLOAT16, HALF])
@pytest.mark.parametrize("M", [5, 16, 31, 32])
@pytest.mark.parametrize("K,N", [(768, 2304), (768, 768), (3072, 768), (768, 3072), (256, 32), (1024, 64), (4096, 96), (8192, 64)])
def test_up_to_32_rows_times_k_contiguous_weights(ex, oracle, dtype, M, K, N):
    """The batched decode-step shape: 5..32 rows of x against [out, in] weights with the transpose flag run as one
    launch (waves split K inside a block); with and without the bias row, and from a strided x view."""
    rng = np.random.default_rng(M + K + N)
    x = rng.normal(0, 1, (M, K))
    wt = rng.normal(0, 1 / math.sqrt(K), (N, K))
    b = rng.normal(0, 1, (N,))
    ox, dx = _pair(oracle, x, dtype)
    ow, dw = _pair(oracle, wt, dtype)
    ob, db = _pair(oracle, b, dtype)
    oz = _ozeros(oracle, (M, N), dtype)
    oracle.matmul(ox, ow, oz, trans_y=True, accumulate=1)
    z = ex.exec_custom("matmul", [dx, dw], i_args=[0, 1])[0]
    assert_close(z.to_float(), _f(oz), 1e-2, 1e-2, "rows x W^T")
    oracle.add_row_vector(oz, ob, oz)
    zb = ex.exec_custom("xw_plus_b", [dx, dw, db], i_args=[0, 1])[0]
    assert_close(zb.to_float(), _f(oz), 1e-2, 1e-2, "rows x W^T + bias")
    wide = np.zeros((M, 2 * K), np.asarray(ox.a).dtype)
    wide[:, :K] = np.asarray(ox.a)
    xv = NDArray.from_numpy(wide, dtype).view((M, K), (2 * K, 1), 0)
    zv = ex.exec_custom("xw_plus_b", [xv, dw, db], outputs=[NDArray.empty((M, N), dtype)], i_args=[0, 1])[0]
    assert np.array_equal(zv.to_numpy(), zb.to_numpy())


def test_xw_plus_b_errors(ex):
    x = NDArray.from_numpy(np.ones((4, 8), np.float32))
    w = NDArray.from_numpy(np.ones((9, 5), np.float32))
    b = NDArray.from_numpy(np.ones((5,), np.float32))
    with pytest.raises(NativeOpsError, match="inconsistent shapes"):
        ex.exec_custom("xw_plus_b", [x, w, b])
    w2 = NDArray.from_numpy(np.ones((8, 5), np.float32))
    b2 = NDArray.from_numpy(np.ones((6,), np.float32))
    with pytest.raises(NativeOpsError, match="bias"):
        ex.exec_custom("xw_plus_b", [x, w2, b2])


# ---- softmax ---------------------------------------------------------------------------------------------------------
@pytest.mark.parametrize("dtype,rtol,atol", [(FLOAT32, 1e-5, 1e-6), (BFLOAT16, 1e-2, 1e-4), (HALF, 1e-2, 1e-4), (DOUBLE, 1e-12, 1e-14)])
@pytest.mark.parametrize("shape,dim", [((4, 3, 8, 1024), 3), ((17, 33), 1), ((17, 33), 0), ((5, 6, 7), 1), ((3, 5000), 1), ((2, 20000), 1), ((6, 1000), -1),
                                       ((3, 50257), 1), ((2, 65536), 1), ((2, 100003), 1), ((1, 131077), 1),
                                       # rows that start off 16-byte boundaries: 16-bit types take a wave per row with the row in registers
                                       ((7, 1001), 1), ((5, 2047), 1), ((3, 4099), 1), ((9, 8191), 1), ((66, 17), 1), ((2, 3, 5, 1023), 3)])
def test_softmax_vs_oracle(ex, oracle, dtype, rtol, atol, shape, dim):
    rng = np.random.default_rng(abs(dim) + len(shape) + shape[-1])
    a = rng.normal(0, 2, shape)
    ox, dx = _pair(oracle, a, dtype)
    oz = _ozeros(oracle, shape, dtype)
    oracle.softmax(ox, oz, dim)
    z = ex.exec_custom("softmax", [dx], i_args=[dim])[0]
    got = z.to_float() if dtype != DOUBLE else z.to_numpy()
    assert_close(got, _f(oz), rtol, atol, "softmax %s dim %d dtype %d" % (shape, dim, dtype))
    assert_close(got.astype(np.float64).sum(dim), np.ones(np.delete(np.array(shape), dim)), 2e-2 if dtype in (HALF, BFLOAT16) else 1e-5, 0, "rows sum to one")


@pytest.mark.parametrize("dtype,rtol,atol", [(FLOAT32, 1e-5, 1e-6), (BFLOAT16, 1e-2, 1e-4)])
def test_softmax_permuted_view(ex, oracle, dtype, rtol, atol):
    # BASELINE config 3 layout at reduced batch: buffer [B, T, H, T] viewed through permute(0, 2, 1, 3), dense output
    rng = np.random.default_rng(3003)
    B, H, T = 2, 12, 256
    a = rng.normal(0, 2, (B, T, H, T))
    ox, dx = _pair(oracle, a, dtype)
    oxv = oracle.Arr(ox.a.transpose(0, 2, 1, 3), ox.dt)
    oz = _ozeros(oracle, (B, H, T, T), dtype)
    oracle.softmax(oxv, oz, 3)
    z = ex.exec_custom("softmax", [dx.permute(0, 2, 1, 3)], [NDArray.empty((B, H, T, T), dtype)], i_args=[3])[0]
    assert_close(z.to_float(), _f(oz), rtol, atol, "softmax on a permuted view")


def test_softmax_edge_semantics(ex, oracle):
    inf, nan = np.inf, np.nan
    rows = np.array([[0, inf, 1, -inf], [nan, 0, 0, 0], [-inf, -inf, -inf, -inf], [1e4, -1e4, 0, 5], [3, 3, 3, 3]], np.float32)
    rows = np.repeat(rows, 2, axis=0)
    want = oracle.softmax(rows, np.zeros_like(rows), 1)
    got = ex.exec_custom("softmax", [NDArray.from_numpy(rows)], i_args=[1])[0].to_numpy()
    assert_close(got, want, 1e-5, 1e-30, "inf/nan/clamp rows")
    # vector along its unit axis is all ones; rank-1 ignores the axis argument
    v = NDArray.from_numpy(np.array([[-1, 1, -2, 2, 3]], np.float32))
    assert np.array_equal(ex.exec_custom("softmax", [v], i_args=[0])[0].to_numpy(), np.ones((1, 5), np.float32))
    with pytest.raises(NativeOpsError, match="must be less than input array rank"):
        ex.exec_custom("softmax", [v], i_args=[2])


# ---- layer_norm ------------------------------------------------------------------------------------------------------
@pytest.mark.parametrize("dtype,rtol,atol", [(FLOAT32, 1e-5, 1e-5), (BFLOAT16, 1e-2, 1e-2), (HALF, 1e-2, 1e-2)])
@pytest.mark.parametrize("shape", [(4, 64, 768), (3, 5, 100), (7, 2048), (2, 3, 5000), (4099, 768), (4097, 40), (41, 101, 256), (3, 40000), (2, 20004),
                                   # row lengths that are not whole 16-byte vectors: a wave per row, element-aligned loads, the row in registers
                                   (37, 770), (5, 769), (9, 13), (3, 7, 1001), (6, 2047), (2, 4093)])
def test_layer_norm_last_axis(ex, oracle, dtype, rtol, atol, shape):
    rng = np.random.default_rng(shape[-1])
    C = shape[-1]
    ox, dx = _pair(oracle, rng.normal(0, 1, shape), dtype)
    og, dg = _pair(oracle, rng.normal(1, 0.02, C), dtype)
    ob, db = _pair(oracle, rng.normal(0, 0.02, C), dtype)
    oz = _ozeros(oracle, shape, dtype)
    axes = [len(shape) - 1]
    oracle.layer_norm(ox, og, ob, oz, axes, channels_first=False)
    z = ex.exec_custom("layer_norm", [dx, dg, db], i_args=axes, b_args=[False])[0]
    assert_close(z.to_float(), _f(oz), rtol, atol, "layer_norm %s" % (shape,))
    oz2 = _ozeros(oracle, shape, dtype)
    oracle.layer_norm(ox, og, None, oz2, axes, channels_first=False)
    z2 = ex.exec_custom("layer_norm", [dx, dg], i_args=axes, b_args=[False])[0]
    assert_close(z2.to_float(), _f(oz2), rtol, atol, "layer_norm without bias")


def test_layer_norm_channels_first_and_views(ex, oracle):
    rng = np.random.default_rng(31)
    x = rng.normal(0, 1, (3, 5, 4, 6)).astype(np.float32)
    g = rng.normal(1, 0.1, 5).astype(np.float32)
    b = rng.normal(0, 0.1, 5).astype(np.float32)
    want = oracle.layer_norm(x, g, b, np.zeros_like(x), [1, 2, 3], channels_first=True)
    z = ex.exec_custom("layer_norm", [NDArray.from_numpy(x), NDArray.from_numpy(g), NDArray.from_numpy(b)], i_args=[1, 2, 3])[0]   # BArg absent = channels first
    assert_close(z.to_numpy(), want, 1e-5, 1e-5, "NCHW over dims 1..3")
    x64 = x.astype(np.float64)
    closed = (x64 - x64.mean((1, 2, 3), keepdims=True)) / np.sqrt(x64.var((1, 2, 3), keepdims=True) + 1e-5) * g[None, :, None, None] + b[None, :, None, None]
    assert_close(z.to_numpy(), closed, 1e-5, 1e-5, "NCHW closed form")
    # strided rows: a sliced view along the row axis keeps unit stride inside rows
    X = NDArray.from_numpy(rng.normal(0, 1, (16, 10, 64)).astype(np.float32))
    g2 = rng.normal(1, 0.1, 64).astype(np.float32)
    xv = X.slice(1, 2, 9)
    want2 = oracle.layer_norm(X.to_numpy()[:, 2:9], g2, None, np.zeros((16, 7, 64), np.float32), [2], channels_first=False)
    z2 = ex.exec_custom("layer_norm", [xv, NDArray.from_numpy(g2)], [NDArray.empty((16, 7, 64), FLOAT32)], i_args=[2], b_args=[False])[0]
    assert_close(z2.to_numpy(), want2, 1e-5, 1e-5, "sliced view")
    with pytest.raises(NativeOpsError, match="wrong shape of gain"):
        ex.exec_custom("layer_norm", [X, NDArray.from_numpy(np.ones(7, np.float32))], i_args=[2], b_args=[False])


# ---- attention -------------------------------------------------------------------------------------------------------
@pytest.mark.parametrize("dtype,tol", [(FLOAT32, 1e-4), (HALF, 1e-2), (BFLOAT16, 1e-2)])
@pytest.mark.parametrize("causal", [False, True])
@pytest.mark.parametrize("B,Tq,Tv,D", [(3, 64, 64, 64), (2, 100, 100, 64), (2, 128, 256, 64), (1, 37, 91, 32), (2, 300, 72, 64), (1, 520, 200, 64),
                                      (2, 200, 200, 128), (1, 70, 330, 128), (2, 3, 200, 128),
                                      # a few queries against a long history: the streaming kernel cuts the key range into parts and merges them
                                      (12, 1, 640, 64), (1, 1, 1000, 128), (2, 1, 300, 64), (5, 4, 513, 64)])
def test_attention_vs_oracle(ex, oracle, dtype, tol, causal, B, Tq, Tv, D):
    # causal with Tq != Tv: key j is visible to query i iff j <= i (the lower-triangular mask of AttentionHelper.cpp:70-79)
    rng = np.random.default_rng(B * Tq + D)
    oq, dq = _pair(oracle, rng.normal(0, 1, (B, Tq, D)), dtype)
    ok, dk = _pair(oracle, rng.normal(0, 1, (B, Tv, D)), dtype)
    ov, dv = _pair(oracle, rng.normal(0, 1, (B, Tv, D)), dtype)
    oo, ow, ol = _ozeros(oracle, (B, Tq, D), dtype), _ozeros(oracle, (B, Tq, Tv), dtype), _ozeros(oracle, (B, Tq, Tv), dtype)
    scale = 1 / math.sqrt(D)
    oracle.attention_v2(oq, ov, ok, oo, ow, ol, scale=scale, causal=causal)
    # all three outputs (composition path)
    out, w, lg = ex.exec_custom("dot_product_attention_v2", [dq, dv, dk], t_args=[scale, 0.0], b_args=[causal, False])
    assert_close(out.to_float(), _f(oo), tol, tol, "out")
    assert_close(w.to_float(), _f(ow), tol, tol * 1e-2, "weights")
    keep = np.tril(np.ones((Tq, Tv), bool)) if causal else np.ones((Tq, Tv), bool)
    assert_close(lg.to_float()[:, keep], _f(ol)[:, keep], tol, tol, "logits")
    # output only (fused path where available): same numbers.  At D = 128 in bf16 the reference's own op-by-op composition
    # (every intermediate rounded to bf16) is 0.014 away from the exact result and the fused kernel 0.009: the two are
    # compared at 2.5 times the gate, and the kernel must not be further from the exact result than the composition is
    wide = 2.5 if (D == 128 and dtype == BFLOAT16) else 1.0
    out1 = ex.exec_custom("dot_product_attention_v2", [dq, dv, dk], [NDArray.empty((B, Tq, D), dtype)], t_args=[scale, 0.0], b_args=[causal, False])[0]
    assert_close(out1.to_float(), _f(oo), wide * tol, wide * tol, "out-only call")
    if D == 128:
        q64, k64, v64 = _f(oq), _f(ok), _f(ov)
        sc64 = np.einsum("bqd,bkd->bqk", q64, k64) * scale
        if causal:
            sc64 = np.where(np.tril(np.ones((Tq, Tv), bool)), sc64, -np.inf)
        p64 = np.exp(sc64 - sc64.max(-1, keepdims=True))
        truth = np.einsum("bqk,bkd->bqd", p64 / p64.sum(-1, keepdims=True), v64)
        assert np.abs(out1.to_float() - truth).max() <= 1.25 * np.abs(_f(oo) - truth).max() + 1e-3, "fused kernel against the exact result"


@pytest.mark.parametrize("dtype,tol", [(FLOAT32, 1e-4), (HALF, 1e-2), (BFLOAT16, 1e-2)])
@pytest.mark.parametrize("H,Tv,D", [(12, 640, 64), (12, 257, 64), (3, 2000, 128), (24, 513, 64), (1, 1100, 64)])
def test_attention_of_one_token_over_a_cut_up_history(ex, oracle, dtype, tol, H, Tv, D):
    """One query token, its heads as the inner batch level ([1, H, 1, D] against [1, H, Tv, D]): the streaming kernel cuts the
    key range into 2, 4 or 8 parts, a block each, and a second kernel merges the parts' records."""
    rng = np.random.default_rng(H * Tv + D)
    q, k, v = rng.normal(0, 1, (H, 1, D)), rng.normal(0, 1, (H, Tv, D)), rng.normal(0, 1, (H, Tv, D))
    oq, dq = _pair(oracle, q, dtype)
    ok, dk = _pair(oracle, k, dtype)
    ov, dv = _pair(oracle, v, dtype)
    oo = _ozeros(oracle, (H, 1, D), dtype)
    scale = 1 / math.sqrt(D)
    oracle.attention_v2(oq, ov, ok, oo, None, None, scale=scale, causal=False)
    q4, k4, v4 = dq.reshape(1, H, 1, D), dk.reshape(1, H, Tv, D), dv.reshape(1, H, Tv, D)
    out = ex.exec_custom("dot_product_attention_v2", [q4, v4, k4], [NDArray.empty((1, H, 1, D), dtype)], t_args=[scale, 0.0], b_args=[False, False])[0]
    wide = 2.5 if (D == 128 and dtype == BFLOAT16) else 1.0
    assert_close(out.to_float().reshape(H, 1, D), _f(oo), wide * tol, wide * tol, "one token, %d heads, %d keys" % (H, Tv))


@pytest.mark.parametrize("dtype,tol", [(HALF, 1e-2), (BFLOAT16, 1e-2)])
@pytest.mark.parametrize("causal", [False, True])
@pytest.mark.parametrize("scale", [0.125, 0.11])
def test_attention_scores_beyond_the_clip(ex, oracle, dtype, tol, causal, scale):
    """Scaled scores on both sides of the +-1e4 clip (AttentionHelper.cpp:340-352) in some key tiles and not in others:
    the fused kernel clips score by score only in tiles whose maximum calls for it, and must give what the oracle's
    clip of every score gives.  Rows differ in which keys tie at the clip, so a missed clip moves the output."""
    B, T, D = 2, 384, 64
    rng = np.random.default_rng(77)
    q = rng.normal(0, 1, (B, T, D))
    k = rng.normal(0, 1, (B, T, D))
    v = rng.normal(0, 1, (B, T, D))
    # a few long query / key pairs along one direction d: |q.k| * scale reaches 4e4 .. 6e4 there, of both signs; everything
    # else is orthogonal to d (a power of two in one coordinate, so exactly in every storage type) and keeps ordinary scores.
    # Key tile 0 (keys 0-63) is visible to every query under the causal mask, later tiles only to later queries.
    q[:, :, 0] = 0.0
    k[:, :, 0] = 0.0
    for b in range(B):
        for qi in (5, 130, 131, 260, 383):
            q[b, qi, 0] = 512.0
        # 140 and -144: products of 71,680 and -73,728, beyond the fp16 range (the reference's fp16 logits array holds +-inf
        # there, which scaling leaves and the clip turns into +-1e4) but inside the clip once scaled in fp32
        for kj, mag in ((3, 768.0), (40, 1024.0), (41, -1024.0), (100, 896.0), (150, 140.0), (151, -144.0), (200, -768.0), (300, 1024.0), (301, 640.0)):
            k[b, kj, 0] = mag
    oq, dq = _pair(oracle, q, dtype)
    ok, dk = _pair(oracle, k, dtype)
    ov, dv = _pair(oracle, v, dtype)
    oo, ow, ol = _ozeros(oracle, (B, T, D), dtype), _ozeros(oracle, (B, T, T), dtype), _ozeros(oracle, (B, T, T), dtype)
    oracle.attention_v2(oq, ov, ok, oo, ow, ol, scale=scale, causal=causal)
    lg = _f(ol)
    fin = lg[:, np.tril(np.ones((T, T), bool)) if causal else np.ones((T, T), bool)]   # the visible entries
    assert (np.abs(fin) >= 9.9e3).sum() >= 20 and (np.abs(fin) < 2e3).mean() > 0.9, "the case must have clipped and ordinary scores"
    out1 = ex.exec_custom("dot_product_attention_v2", [dq, dv, dk], [NDArray.empty((B, T, D), dtype)], t_args=[scale, 0.0], b_args=[causal, False])[0]
    assert_close(out1.to_float(), _f(oo), tol, tol, "output-only call")
    out3 = ex.exec_custom("dot_product_attention_v2", [dq, dv, dk], t_args=[scale, 0.0], b_args=[causal, False])[0]
    assert_close(out3.to_float(), _f(oo), tol, tol, "three-output call")
    if not causal:   # four query rows against the whole history: the streaming kernel of the decode steps
        oq4, dq4 = _pair(oracle, q[:, 4:8], dtype)
        oo4, ow4, ol4 = _ozeros(oracle, (B, 4, D), dtype), _ozeros(oracle, (B, 4, T), dtype), _ozeros(oracle, (B, 4, T), dtype)
        oracle.attention_v2(oq4, ov, ok, oo4, ow4, ol4, scale=scale, causal=False)
        out4 = ex.exec_custom("dot_product_attention_v2", [dq4, dv, dk], [NDArray.empty((B, 4, D), dtype)], t_args=[scale, 0.0], b_args=[False, False])[0]
        assert_close(out4.to_float(), _f(oo4), tol, tol, "four query rows")


@pytest.mark.parametrize("dtype,tol", [(FLOAT32, 1e-4), (HALF, 1e-2), (BFLOAT16, 1e-2)])
@pytest.mark.parametrize("causal", [False, True])
@pytest.mark.parametrize("B,Tq,Tv,D", [(3, 64, 64, 64), (2, 200, 200, 64), (2, 130, 300, 64), (2, 4, 150, 64), (1, 37, 91, 32), (2, 130, 300, 128),
                                      (2, 4, 150, 128)])
def test_attention_masks_vs_oracle(ex, oracle, dtype, tol, causal, B, Tq, Tv, D):
    """Query and value masks (inputs 3 and 4): all three outputs through the composition path, then the output-only call
    (fused prefill kernel, or the streaming decode kernel for a handful of query rows)."""
    rng = np.random.default_rng(B * Tq + D + Tv)
    oq, dq = _pair(oracle, rng.normal(0, 1, (B, Tq, D)), dtype)
    ok, dk = _pair(oracle, rng.normal(0, 1, (B, Tv, D)), dtype)
    ov, dv = _pair(oracle, rng.normal(0, 1, (B, Tv, D)), dtype)
    vm = (rng.random((B, Tv)) > 0.3).astype(np.float32)
    vm[:, 0] = 1                                           # key 0 stays: every query keeps a visible key
    vm[-1, Tv // 2:] = 0                                   # a padded tail
    qm = (rng.random((B, Tq)) > 0.3).astype(np.float32)
    ovm, dvm = _pair(oracle, vm, dtype)
    oqm, dqm = _pair(oracle, qm, dtype)
    oo, ow, ol = _ozeros(oracle, (B, Tq, D), dtype), _ozeros(oracle, (B, Tq, Tv), dtype), _ozeros(oracle, (B, Tq, Tv), dtype)
    scale = 1 / math.sqrt(D)
    oracle.attention_v2(oq, ov, ok, oo, ow, ol, scale=scale, causal=causal, q_mask=oqm, v_mask=ovm)
    out, w, lg = ex.exec_custom("dot_product_attention_v2", [dq, dv, dk, dqm, dvm], t_args=[scale, 0.0], b_args=[causal, False])
    assert_close(out.to_float(), _f(oo), tol, tol, "out")
    assert_close(w.to_float(), _f(ow), tol, tol * 1e-2, "weights")
    keep = (np.tril(np.ones((Tq, Tv), bool)) if causal else np.ones((Tq, Tv), bool))[None] & (vm != 0)[:, None, :]
    assert_close(lg.to_float()[keep], _f(ol)[keep], tol, tol, "visible logits")
    hidden = lg.to_float()[~keep]
    assert hidden.size == 0 or hidden.max() < -6.0e4       # hidden logits carry the penalty
    # output only, masks of other types: BOOL value mask, INT64 value mask as a strided view
    bvm = NDArray.from_numpy(vm != 0)
    out1 = ex.exec_custom("dot_product_attention_v2", [dq, dv, dk, dqm, bvm], [NDArray.empty((B, Tq, D), dtype)], t_args=[scale, 0.0], b_args=[causal, False])[0]
    assert_close(out1.to_float(), _f(oo), tol, tol, "out-only call, BOOL mask")
    ivm = NDArray.from_numpy(np.ascontiguousarray(vm.T).astype(np.int64)).permute(1, 0)
    out2 = ex.exec_custom("dot_product_attention_v2", [dq, dv, dk, dqm, ivm], [NDArray.empty((B, Tq, D), dtype)], t_args=[scale, 0.0], b_args=[causal, False])[0]
    assert np.array_equal(out2.to_numpy(), out1.to_numpy())


@pytest.mark.parametrize("dtype,tol", [(FLOAT32, 1e-4), (HALF, 1e-2), (BFLOAT16, 1e-2)])
def test_attention_padded_batch_identity_and_hidden_rows(ex, oracle, dtype, tol):
    """Masked trailing keys == truncated keys; a batch entry whose keys are all padded follows the reference's arithmetic
    (uniform-like weights over penalised logits for float / bfloat16, zero weights for half, whose penalty is -inf)."""
    rng = np.random.default_rng(8)
    B, Tq, Tv, D, cut = 3, 150, 256, 64, 170
    q, k, v = rng.normal(0, 1, (B, Tq, D)), rng.normal(0, 1, (B, Tv, D)), rng.normal(0, 1, (B, Tv, D))
    oq, dq = _pair(oracle, q, dtype)
    ok, dk = _pair(oracle, k, dtype)
    ov, dv = _pair(oracle, v, dtype)
    vm = np.ones((B, Tv), np.float32)
    vm[:, cut:] = 0
    _, dvm = _pair(oracle, vm, dtype)
    none = NDArray.empty((0,), dtype)                      # an absent query mask travels as an empty array
    masked = ex.exec_custom("dot_product_attention_v2", [dq, dv, dk, none, dvm], [NDArray.empty((B, Tq, D), dtype)], t_args=[0.125, 0.0], b_args=[False, False])[0].to_float()
    _, dk2 = _pair(oracle, k[:, :cut], dtype)
    _, dv2 = _pair(oracle, v[:, :cut], dtype)
    trunc = ex.exec_custom("dot_product_attention_v2", [dq, dv2, dk2], [NDArray.empty((B, Tq, D), dtype)], t_args=[0.125, 0.0], b_args=[False, False])[0].to_float()
    assert_close(masked, trunc, tol, tol, "masked tail against truncated keys")
    # batch entry 1 entirely padded, causal on top
    vm2 = np.ones((B, Tv), np.float32)
    vm2[1] = 0
    ovm2, dvm2 = _pair(oracle, vm2, dtype)
    oo = _ozeros(oracle, (B, Tq, D), dtype)
    oracle.attention_v2(oq, ov, ok, oo, scale=0.125, causal=True, v_mask=ovm2)
    got = ex.exec_custom("dot_product_attention_v2", [dq, dv, dk, none, dvm2], [NDArray.empty((B, Tq, D), dtype)], t_args=[0.125, 0.0], b_args=[True, False])[0].to_float()
    assert_close(got, _f(oo), tol, tol, "entirely padded batch entry")


def test_attention_rank4_and_default_keys(ex, oracle):
    rng = np.random.default_rng(41)
    B, H, T, D = 2, 3, 48, 64
    q = rng.normal(0, 1, (B, H, T, D)).astype(np.float32)
    v = rng.normal(0, 1, (B, H, T, D)).astype(np.float32)
    oo = np.zeros((B * H, T, D), np.float32)
    oracle.attention_v2(q.reshape(B * H, T, D), v.reshape(B * H, T, D), v.reshape(B * H, T, D), oo, scale=0.125, causal=True)
    out = ex.exec_custom("dot_product_attention_v2", [NDArray.from_numpy(q), NDArray.from_numpy(v)], [NDArray.empty((B, H, T, D), FLOAT32)],
                         t_args=[0.125], b_args=[True])[0]
    assert_close(out.to_numpy().reshape(B * H, T, D), oo, 1e-4, 1e-4, "rank 4, keys = values")


@pytest.mark.parametrize("dtype,tol", [(FLOAT32, 1e-4), (BFLOAT16, 1e-2), (HALF, 1e-2)])
@pytest.mark.parametrize("Tq,Tv,causal", [(40, 40, True), (1, 37, False), (5, 131, False)])
def test_attention_token_major_head_views(ex, oracle, dtype, tol, Tq, Tv, causal):
    """[batch, heads, T, 64] views of token-major buffers: the batch dims do not nest, key counts are ragged, the
    output is written through a strided view (the layout of a decoder's fused qkv buffer and its key/value cache)."""
    rng = np.random.default_rng(Tq * 1000 + Tv)
    B, H, D, M = 2, 3, 64, 160
    d = H * D
    qkv = rng.normal(0, 1, (B, Tq, 3 * d)).astype(np.float32)
    kc = rng.normal(0, 1, (B, M, d)).astype(np.float32)
    vc = rng.normal(0, 1, (B, M, d)).astype(np.float32)
    oqkv, dqkv = _pair(oracle, qkv, dtype)
    okc, dkc = _pair(oracle, kc, dtype)
    ovc, dvc = _pair(oracle, vc, dtype)
    want = _ozeros(oracle, (B, Tq, H, D), dtype)
    for b in range(B):
        q3 = oqkv.a[b].reshape(Tq, 3, H, D)[:, 0].transpose(1, 0, 2)
        k3 = okc.a[b, :Tv].reshape(Tv, H, D).transpose(1, 0, 2)
        v3 = ovc.a[b, :Tv].reshape(Tv, H, D).transpose(1, 0, 2)
        oracle.attention_v2(oracle.Arr(q3, oqkv.dt), oracle.Arr(v3, oqkv.dt), oracle.Arr(k3, oqkv.dt),
                            oracle.Arr(want.a[b].transpose(1, 0, 2), oqkv.dt), scale=0.125, causal=causal)
    q4 = dqkv.view((B, H, Tq, D), (Tq * 3 * d, D, 3 * d, 1), 0)
    k4 = dkc.view((B, H, Tv, D), (M * d, D, d, 1), 0)
    v4 = dvc.view((B, H, Tv, D), (M * d, D, d, 1), 0)
    att = NDArray.empty((B, Tq, d), dtype)
    o4 = att.view((B, H, Tq, D), (Tq * d, D, d, 1), 0)
    ex.exec_custom("dot_product_attention_v2", [q4, v4, k4], [o4], t_args=[0.125, 0.0], b_args=[causal, False])
    assert_close(att.to_float().reshape(B, Tq, H, D), _f(want), tol, tol, "token-major heads")


@pytest.mark.parametrize("dtype,tol", [(FLOAT32, 1e-4), (BFLOAT16, 1e-2)])
def test_matmul_batch_dims_that_do_not_nest(ex, oracle, dtype, tol):
    """x is a [B, H, T, D] view of a token-major buffer (strides of B and H do not fold), y is dense [B, H, D, N]."""
    rng = np.random.default_rng(73)
    B, H, T, D, Nn = 3, 4, 40, 64, 48
    xa = rng.normal(0, 1, (B, T, H * D)).astype(np.float32)
    ya = rng.normal(0, 0.2, (B, H, D, Nn)).astype(np.float32)
    ox, dx = _pair(oracle, xa, dtype)
    oy, dy = _pair(oracle, ya, dtype)
    want = _ozeros(oracle, (B, H, T, Nn), dtype)
    for b in range(B):
        for h in range(H):
            x2 = ox.a[b].reshape(T, H, D)[:, h]
            oracle.matmul(oracle.Arr(x2, ox.dt), oracle.Arr(oy.a[b, h], ox.dt), oracle.Arr(want.a[b, h], ox.dt))
    x4 = dx.view((B, H, T, D), (T * H * D, D, H * D, 1), 0)
    z = ex.exec_custom("matmul", [x4, dy])[0]
    assert z.shape == (B, H, T, Nn)
    assert_close(z.to_float(), _f(want), tol, tol, "two batch levels")


# ---- argmax + glue ops -----------------------------------------------------------------------------------------------
def test_argmax_logits_shape(ex, oracle):
    rng = np.random.default_rng(51)
    x = rng.normal(0, 1, (32, 50257)).astype(np.float32)
    x[3, [100, 40000]] = 9.0    # tie: the lower index wins
    z = ex.exec_custom("argmax", [NDArray.from_numpy(x)], i_args=[-1])[0]
    assert z.dtype == INT64 and z.shape == (32,)
    assert np.array_equal(z.to_numpy(), oracle.index_reduce(0, x, np.zeros(32, np.int64), [1]))
    assert z.to_numpy()[3] == 100
    zk = ex.exec_custom("argmax", [NDArray.from_numpy(x)], i_args=[1], b_args=[True], d_args=[INT32])[0]
    assert zk.shape == (32, 1) and zk.dtype == INT32
    zmin = ex.exec_custom("argmin", [NDArray.from_numpy(x)], i_args=[1])[0]
    assert np.array_equal(zmin.to_numpy(), np.argmin(x, 1))


def test_gather_add_concat(ex, oracle):
    rng = np.random.default_rng(61)
    table = rng.normal(0, 1, (1000, 96)).astype(np.float32)
    idx = rng.integers(0, 1000, (4, 7)).astype(np.int64)
    g = ex.exec_custom("gather", [NDArray.from_numpy(table), NDArray.from_numpy(idx)], i_args=[0])[0]
    assert g.shape == (4, 7, 96) and np.array_equal(g.to_numpy(), table[idx])
    bias = rng.normal(0, 1, 96).astype(np.float32)
    s = ex.exec_custom("add", [g, NDArray.from_numpy(bias)])[0]
    assert np.array_equal(s.to_numpy(), table[idx] + bias)
    m = ex.exec_custom("multiply", [g, NDArray.from_numpy(rng.normal(0, 1, (4, 1, 96)).astype(np.float32))])[0]
    assert m.shape == (4, 7, 96)
    a = rng.normal(0, 1, (2, 5, 8)).astype(np.float32)
    b = rng.normal(0, 1, (2, 3, 8)).astype(np.float32)
    c = ex.exec_custom("concat", [NDArray.from_numpy(a), NDArray.from_numpy(b)], i_args=[1])[0]
    assert np.array_equal(c.to_numpy(), np.concatenate([a, b], 1))


# ---- top_k ---------------------------------------------------------------------------------------------------------------
def _topk_cases():
    import json
    import os
    with open(os.path.join(os.path.dirname(__file__), "golden", "top_k_vectors.json")) as f:
        return json.load(f)["cases"]


@pytest.mark.parametrize("case", _topk_cases(), ids=lambda c: c["name"])
def test_golden_top_k(ex, case):
    order = case["order"]
    x = np.array(case["x"], np.float64).reshape(case["shape"], order=order.upper())
    dx = NDArray.from_numpy(x, DOUBLE, order=order)
    v, i = ex.exec_custom("top_k", [dx], i_args=[case["k"]], b_args=[case["sort"]])
    assert v.shape == tuple(case["zshape"]) and i.shape == tuple(case["zshape"]) and i.dtype == INT64
    assert np.array_equal(v.to_numpy(), np.array(case["v"], np.float64).reshape(case["zshape"], order=order.upper()))
    assert np.array_equal(i.to_numpy(), np.array(case["i"], np.int64).reshape(case["zshape"], order=order.upper()))


@pytest.mark.parametrize("shape,k", [((32, 50257), 40), ((3, 5, 129), 5), ((7, 64), 64), ((2, 4097), 1)])
@pytest.mark.parametrize("sort", [True, False])
def test_top_k_vs_oracle_distinct_values(ex, oracle, shape, k, sort):
    """Indices are bit-exact against the reference's algorithm wherever a row's values are pairwise different."""
    rng = np.random.default_rng(k + shape[-1])
    n = shape[-1]
    rows = int(np.prod(shape[:-1]))
    # every row a shuffled ramp: pairwise distinct floats (random normal draws of this length repeat values)
    x = np.stack([rng.permutation(n) for _ in range(rows)]).astype(np.float32).reshape(shape) * np.float32(0.25) - np.float32(100)
    ov = np.zeros(shape[:-1] + (k,), np.float32)
    oi = np.zeros(shape[:-1] + (k,), np.int64)
    oracle.top_k(x, ov, oi, k, sort)
    v, i = ex.exec_custom("top_k", [NDArray.from_numpy(x)], i_args=[k], b_args=[sort])
    assert np.array_equal(i.to_numpy(), oi)
    assert np.array_equal(v.to_numpy(), ov)


def test_top_k_types_views_ties_and_errors(ex, oracle):
    rng = np.random.default_rng(3)
    # bf16 values, int32 indices, k from a second input, permuted input view
    vals = rng.permutation(240).astype(np.float32).reshape(6, 40) - 100.0      # exact in bf16, pairwise distinct
    dx = NDArray.from_numpy(np.ascontiguousarray(vals.T), BFLOAT16).permute(1, 0)   # [6, 40] view with strides [1, 6]
    ox = oracle.Arr(f32_to_bf16_bits(vals), oracle.BFLOAT16)
    ov, oi = oracle.Arr(np.zeros((6, 4), np.uint16), oracle.BFLOAT16), np.zeros((6, 4), np.int64)
    oracle.top_k(ox, ov, oi, 4, True)
    kk = NDArray.from_numpy(np.array([4], np.int32))
    v, i = ex.exec_custom("top_k", [dx, kk], [NDArray.empty((6, 4), BFLOAT16), NDArray.empty((6, 4), INT32)])
    assert np.array_equal(i.to_numpy(), oi.astype(np.int32))
    assert np.array_equal(v.to_numpy(), ov.a)
    # k = 1: the first maximum wins, as in the reference
    t = np.array([[1, 9, 3, 9, 2], [5, 5, 5, 5, 5]], np.float32)
    ov1, oi1 = np.zeros((2, 1), np.float32), np.zeros((2, 1), np.int64)
    oracle.top_k(t, ov1, oi1, 1, True)
    v1, i1 = ex.exec_custom("top_k", [NDArray.from_numpy(t)], i_args=[1])
    assert np.array_equal(i1.to_numpy(), oi1) and list(i1.to_numpy().ravel()) == [1, 0]
    # k > 1 with repeated values: the k largest elements, ties to the lower index (the reference's loop differs here)
    v2, i2 = ex.exec_custom("top_k", [NDArray.from_numpy(t)], i_args=[3])
    assert np.array_equal(i2.to_numpy(), np.array([[1, 3, 2], [0, 1, 2]]))
    assert np.array_equal(v2.to_numpy(), np.array([[9, 9, 3], [5, 5, 5]], np.float32))
    # NaN sorts below every number
    tn = np.array([[np.nan, 2, 7, np.nan, 4]], np.float32)
    _, i3 = ex.exec_custom("top_k", [NDArray.from_numpy(tn)], i_args=[3])
    assert list(i3.to_numpy().ravel()) == [2, 4, 1]
    with pytest.raises(NativeOpsError, match="k should not be greater than last dimension"):
        ex.exec_custom("top_k", [NDArray.from_numpy(t)], [NDArray.empty((2, 6), FLOAT32), NDArray.empty((2, 6), INT64)], i_args=[6])
    with pytest.raises(NativeOpsError, match="k should be positive"):
        ex.exec_custom("top_k", [NDArray.from_numpy(t)], i_args=[0])

# ---- reduce_* custom ops -----------------------------------------------------------------------------------------------------
_REDUCE_OPS = [("reduce_sum", lambda x, ax, kd: x.sum(axis=ax, keepdims=kd)), ("reduce_max", lambda x, ax, kd: x.max(axis=ax, keepdims=kd)),
               ("reduce_min", lambda x, ax, kd: x.min(axis=ax, keepdims=kd)), ("reduce_prod", lambda x, ax, kd: x.prod(axis=ax, keepdims=kd)),
               ("reduce_mean", lambda x, ax, kd: x.mean(axis=ax, keepdims=kd)), ("reduce_norm1", lambda x, ax, kd: np.abs(x).sum(axis=ax, keepdims=kd)),
               ("reduce_norm2", lambda x, ax, kd: np.sqrt((x * x).sum(axis=ax, keepdims=kd))),
               ("reduce_norm_max", lambda x, ax, kd: np.abs(x).max(axis=ax, keepdims=kd)),
               ("reduce_sqnorm", lambda x, ax, kd: (x * x).sum(axis=ax, keepdims=kd))]


@pytest.mark.parametrize("name,ref", _REDUCE_OPS, ids=[n for n, _ in _REDUCE_OPS])
@pytest.mark.parametrize("shape,dims,keep", [((6, 40), [1], False), ((6, 40), [0], True), ((3, 5, 7), [0, 2], False), ((3, 5, 7), [-1], True),
                                             ((4, 9), [], False), ((33, 4096), [1], False)])
def test_reduce_custom_ops(ex, oracle, name, ref, shape, dims, keep):
    """generic/reduce/reduce_sum.cpp and siblings: dims from IArgs, keepDims from BArg 0, no dims = everything; the
    same kernels as the legacy reduce loops (whose oracle is pinned), checked here against fp64 numpy."""
    rng = np.random.default_rng(len(shape) + len(dims))
    x = rng.uniform(0.8, 1.2, shape) * rng.choice([-1.0, 1.0], shape) if name == "reduce_prod" and np.prod(shape) < 300 else rng.uniform(-1, 1, shape)
    if name == "reduce_prod":
        x = np.where(np.abs(x) < 0.5, 1.0, x)      # keeps long products away from underflow
    x = x.astype(np.float32)
    ax = tuple(dims) if dims else None
    want = ref(x.astype(np.float64), ax, keep)
    out = ex.exec_custom(name, [NDArray.from_numpy(x)], i_args=dims, b_args=[keep])[0]
    assert list(out.shape) == list(np.shape(want))
    assert_close(out.to_numpy(), want, 1e-5, 1e-5 * max(1.0, float(np.abs(want).max())), name)
    if dims:                                       # dims as a second input array give the same bits
        axes = NDArray.from_numpy(np.array(dims, dtype=np.int32))
        out2 = ex.exec_custom(name, [NDArray.from_numpy(x), axes], b_args=[keep])[0]
        assert np.array_equal(out2.to_numpy(), out.to_numpy())


@pytest.mark.parametrize("name,ddof_fn", [("reduce_variance", np.var), ("reduce_stdev", np.std)])
def test_reduce_variance_and_stdev_custom_ops(ex, name, ddof_fn):
    rng = np.random.default_rng(77)
    x = rng.normal(3, 2, (5, 300)).astype(np.float32)
    for keep, bias in ((False, False), (True, True)):
        out = ex.exec_custom(name, [NDArray.from_numpy(x)], i_args=[1], b_args=[keep, bias])[0]
        want = ddof_fn(x.astype(np.float64), axis=1, ddof=1 if bias else 0, keepdims=keep)
        assert list(out.shape) == list(want.shape)
        assert_close(out.to_numpy(), want, 1e-5, 1e-5, name)
    with pytest.raises(NativeOpsError, match="must be in range"):
        ex.exec_custom(name, [NDArray.from_numpy(x)], i_args=[2])

# ---- activation custom ops ---------------------------------------------------------------------------------------------------
def test_activation_custom_ops_match_their_legacy_ops(ex, oracle):
    """generic/nn/activations/*.cpp are one legacy transform or scalar op each: the custom op must give the legacy op's
    bits (same kernels), and the legacy ops are checked against the oracle elsewhere; tanh and relu also here."""
    from deeplearning4j_amd.executioner import Scalar, TransformSame, TransformStrict
    rng = np.random.default_rng(88)
    x = rng.normal(0, 2, (37, 129)).astype(np.float32)
    X = NDArray.from_numpy(x)
    S, T = TransformStrict, TransformSame
    for name, op in [("tanh", S.Tanh), ("sigmoid", S.Sigmoid), ("softplus", S.SoftPlus), ("softsign", S.SoftSign), ("hardsigmoid", S.HardSigmoid),
                     ("hardtanh", S.HardTanh), ("rationaltanh", S.RationalTanh), ("rectifiedtanh", S.RectifiedTanh), ("selu", S.SELU)]:
        got = ex.exec_custom(name, [X])[0].to_numpy()
        assert np.array_equal(got, ex.exec_transform_strict(op, X).to_numpy()), name
    assert np.array_equal(ex.exec_custom("cube", [X])[0].to_numpy(), ex.exec_transform_same(T.Cube, X).to_numpy())
    assert np.array_equal(ex.exec_custom("identity", [X])[0].to_numpy(), x)
    for name, op, targs, sc in [("relu", Scalar.RELU, [], 0.0), ("relu", Scalar.RELU, [0.5], 0.5), ("relu6", Scalar.RELU6, [0.0], 0.0),
                                ("lrelu", Scalar.LeakyRELU, [], 0.01), ("lrelu", Scalar.LeakyRELU, [0.2], 0.2), ("elu", Scalar.ELU, [], 1.0),
                                ("elu", Scalar.ELU, [0.7], 0.7)]:
        got = ex.exec_custom(name, [X], t_args=targs)[0].to_numpy()
        assert np.array_equal(got, ex.exec_scalar(op, X, np.float32(sc)).to_numpy()), (name, targs)
    want = np.zeros_like(x)
    oracle.transform_strict(S.Tanh, x, want)
    assert_close(ex.exec_custom("tanh", [X])[0].to_numpy(), want, 1e-5, 1e-6, "tanh")
    assert np.array_equal(ex.exec_custom("relu", [X])[0].to_numpy(), np.maximum(x, 0))
    # in place, bf16, and a type error
    B = NDArray.from_numpy(x, BFLOAT16)
    ref = ex.exec_transform_strict(S.Sigmoid, B).to_numpy()
    ex.exec_custom("sigmoid", [B], [B])
    assert np.array_equal(B.to_numpy(), ref)
    with pytest.raises(NativeOpsError, match="floating point type"):
        ex.exec_custom("tanh", [X], [NDArray.empty(x.shape, BFLOAT16)])

# ---- log_softmax -------------------------------------------------------------------------------------------------------------
import json as _json
import os as _os
_LSM = _json.load(open(_os.path.join(_os.path.dirname(__file__), "golden", "log_softmax_vectors.json")))["cases"]


@pytest.mark.parametrize("case", _LSM, ids=[c["name"].split()[-1] for c in _LSM])
def test_log_softmax_reference_vectors(ex, case):
    x = np.array(case["x"], np.float64).reshape(case["shape"])
    z = ex.exec_custom("log_softmax", [NDArray.from_numpy(x)], i_args=case["iargs"])[0].to_numpy()
    want = np.array(case["exp"], np.float64).reshape(case["shape"])
    assert z.shape == want.shape and np.allclose(z, want, rtol=2e-5, atol=case.get("tol", 1e-5))


@pytest.mark.parametrize("dtype,rtol,atol", [(FLOAT32, 1e-5, 1e-5), (DOUBLE, 1e-12, 1e-12), (BFLOAT16, 1e-2, 1e-2), (HALF, 1e-2, 1e-2)])
@pytest.mark.parametrize("shape,dim", [((7, 300), 1), ((5, 6, 33), 1), ((4, 5000), -1), ((3000, 3), 0), ((3, 50257), 1), ((2, 100003), 1)])
def test_log_softmax_vs_oracle(ex, oracle, dtype, rtol, atol, shape, dim):
    rng = np.random.default_rng(shape[0] + shape[-1])
    ox, dx = _pair(oracle, rng.normal(0, 2, shape), dtype)
    wide = np.float64 if dtype == DOUBLE else np.float32
    want = oracle.log_softmax(_f(ox).astype(wide), dim)
    i_args = [] if dim == -1 else [dim]
    z = ex.exec_custom("log_softmax", [dx], i_args=i_args)[0]
    assert_close(z.to_float(), want, rtol, atol, "log_softmax %s dim %d" % (shape, dim))
    # a term whose exponential underflows is -inf, as in the reference's exp / sum / log sequence
    if dtype == FLOAT32 and dim != 0:
        a = np.zeros(shape, np.float32)
        a[..., 0] = -200.0
        got = ex.exec_custom("log_softmax", [NDArray.from_numpy(a)])[0].to_numpy()
        assert np.isneginf(got[..., 0]).all() and np.isfinite(got[..., 1:]).all()

# ---- the rest of the broadcastable family --------------------------------------------------------------------------------------
def test_broadcastable_custom_ops_match_their_legacy_pairwise_ops(ex):
    """generic/broadcastable/*.cpp apply one legacy pairwise functor each under broadcasting: on equal shapes the custom op
    must give the legacy op's bits; under broadcasting, what the same op gives on the materialised operand."""
    from deeplearning4j_amd.executioner import Pairwise as P
    rng = np.random.default_rng(99)
    x = rng.uniform(0.5, 3, (6, 1, 33)).astype(np.float32) * rng.choice([-1, 1], (6, 1, 33)).astype(np.float32)
    y = rng.uniform(0.5, 3, (5, 33)).astype(np.float32)
    xb, yb = np.broadcast_to(x, (6, 5, 33)).copy(), np.broadcast_to(y, (6, 5, 33)).copy()
    X, Y, XB, YB = (NDArray.from_numpy(a) for a in (x, y, xb, yb))
    for name, op in [("maximum", P.MaxPairwise), ("minimum", P.MinPairwise), ("Pow", P.Pow), ("realdiv", P.Divide), ("reversedivide", P.ReverseDivide),
                     ("reversesubtract", P.ReverseSubtract), ("squaredsubtract", P.SquaredSubtract), ("floordiv", P.FloorDiv),
                     ("floormod", P.FloorMod), ("mod", P.Mod), ("reversemod", P.ReverseMod), ("truncatediv", P.TruncateDiv),
                     ("divide_no_nan", P.DivideNoNan), ("tf_atan2", P.Atan2), ("assign", P.CopyPws)]:
        want = ex.exec_pairwise(op, XB, YB).to_numpy()
        got = ex.exec_custom(name, [X, Y])[0]
        assert list(got.shape) == [6, 5, 33], name
        assert np.array_equal(got.to_numpy(), want, equal_nan=True), name
    assert np.array_equal(ex.exec_custom("maximum", [X, Y])[0].to_numpy(), np.maximum(xb, yb))
    assert_close(ex.exec_custom("Pow", [NDArray.from_numpy(np.abs(x)), Y])[0].to_numpy(), np.abs(xb).astype(np.float64) ** yb, 1e-5, 1e-6, "Pow")
    assert np.array_equal(ex.exec_custom("assign", [X, Y])[0].to_numpy(), yb)



# ---- two-parameter transforms ---------------------------------------------------------------------------------------------
def test_clipbyvalue_reference_vector_and_bounds_as_inputs(ex):
    """DeclarableOpsTests1.cpp:801-848: bounds as T arguments (ClipByValue1) and as two scalar inputs (ClipByValue2)."""
    x = np.full((5, 5), 4.0, np.float32)
    x.flat[0], x.flat[1] = -1.0, 2.0
    exp = np.full((5, 5), 3.0, np.float32)
    exp.flat[0], exp.flat[1] = 0.0, 2.0
    z = ex.exec_custom("clipbyvalue", [NDArray.from_numpy(x)], t_args=[0.0, 3.0])[0]
    assert np.array_equal(z.to_numpy(), exp)
    lo, hi = NDArray.from_numpy(np.zeros((1, 1), np.float32)), NDArray.from_numpy(np.full((1, 1), 3.0, np.float32))
    X = NDArray.from_numpy(x)
    ex.exec_custom("ClipByValue", [X, lo, hi], [X])      # in place, through the alias
    assert np.array_equal(X.to_numpy(), exp)
    with pytest.raises(NativeOpsError, match="left bound should be lesser than right"):
        ex.exec_custom("clipbyvalue", [NDArray.from_numpy(x)], t_args=[3.0, 0.0])


@pytest.mark.parametrize("dtype", [FLOAT32, DOUBLE, HALF, BFLOAT16])
def test_two_parameter_transforms_match_oracle(ex, oracle, dtype):
    """clipbyvalue and the legacy ClipByValue / Affine / ScaledTanh (extra parameters in device memory, array type)."""
    from oracle import oracle as onp
    rng = np.random.default_rng(77)
    x = rng.normal(0, 2, (6, 5, 33)).astype(np.float32)
    x[0, 0, :3] = [np.nan, np.inf, -np.inf]
    ox, dx = _pair(oracle, x, dtype)
    xr = _f(ox).astype(np.float64 if dtype == DOUBLE else np.float32)   # the values the device holds
    tol = {FLOAT32: 1e-5, DOUBLE: 1e-12, HALF: 1e-2, BFLOAT16: 1e-2}[dtype]
    view = dx.permute(2, 0, 1)                                           # strided input, dense output
    for lo, hi in [(-1.25, 0.5), (0.0, 3.0)]:
        want = onp.clip_by_value(xr, lo, hi)
        got = ex.exec_custom("clipbyvalue", [dx], t_args=[lo, hi])[0].to_float()
        assert np.array_equal(got, want, equal_nan=True), "clipbyvalue is exact"
        got = ex.exec_transform_same(19, dx, extra_args=[lo, hi]).to_float()
        assert np.array_equal(got, want, equal_nan=True), "legacy ClipByValue is exact"
        got = ex.exec_transform_same(19, view, extra_args=[lo, hi]).to_float()
        assert np.array_equal(got, want.transpose(2, 0, 1), equal_nan=True), "legacy ClipByValue, permuted view"
    fin = np.isfinite(xr)
    got = ex.exec_transform_strict(3, dx, extra_args=[2.5, -0.75]).to_float()
    assert_close(got[fin], onp.affine(xr.astype(np.float64), 2.5, -0.75)[fin], tol, tol, "Affine")
    # the dense array goes through the vector kernel, the permuted view through the element-wise one: same bits
    for op_num, extra in ((3, [2.5, -0.75]), (2, [1.7159, 0.6666]), (19, [2.0]), (25, [0.0, 1.0]), (25, [2.0, 4.0])):
        dense = ex.exec_transform_strict(op_num, dx, extra_args=extra).to_numpy()
        strided = ex.exec_transform_strict(op_num, view, extra_args=extra).to_numpy()
        assert np.array_equal(strided.view(np.uint8), dense.transpose(2, 0, 1).copy().view(np.uint8)), (op_num, extra)
    got = ex.exec_transform_strict(2, dx, extra_args=[1.7159, 0.6666]).to_float()
    # the parameters reach the kernel rounded to the array type
    a, b = (np.asarray(v, np.float64) for v in (1.7159, 0.6666))
    assert_close(got[fin], onp.scaled_tanh(xr.astype(np.float64), a, b)[fin], tol * 4, tol * 4, "ScaledTanh")
    with pytest.raises(NativeOpsError, match="needs two extra parameters"):
        ex.exec_transform_same(19, dx)
    # Stabilize (one parameter) and SetRange; k and the ranges are exact in every type
    got = ex.exec_transform_strict(19, dx, extra_args=[2.0]).to_float()
    assert_close(got[fin], onp.stabilize(xr, 2.0).astype(np.float64)[fin], tol, tol, "Stabilize")
    for lo, hi in [(0.0, 1.0), (2.0, 4.0)]:
        got = ex.exec_transform_strict(25, dx, extra_args=[lo, hi]).to_float()
        want = onp.set_range(xr, lo, hi).astype(np.float64)
        assert_close(got[fin], want[fin], tol, tol, "SetRange")


# ---- broadcastable ops: the reference's own vectors ------------------------------------------------------------------------
_BC = _json.load(open(_os.path.join(_os.path.dirname(__file__), "golden", "broadcastable_vectors.json")))


def _bc_array(shape, values, np_dt):
    if isinstance(values, dict):
        return np.full(shape, values["fill"], np_dt)
    return np.array(values, np_dt).reshape(shape)


@pytest.mark.parametrize("case", _BC["cases"], ids=[c["name"].split()[-1] for c in _BC["cases"]])
def test_broadcastable_reference_vectors(ex, case):
    """BroadcastableOpsTests.cpp: row / column / scalar / rank-extending broadcasts, empty operands, caller-supplied outputs."""
    np_dt, dt = (np.float64, DOUBLE) if case["dtype"] == "double" else (np.float32, FLOAT32)
    x = NDArray.from_numpy(_bc_array(case["x_shape"], case["x"], np_dt))
    y = NDArray.from_numpy(_bc_array(case["y_shape"], case["y"], np_dt))
    exp = _bc_array(case["exp_shape"], case["exp"], np_dt)
    got = ex.exec_custom(case["op"], [x, y])[0]                       # output sized by the op's shape function
    assert list(got.shape) == case["exp_shape"]
    if exp.size:
        assert np.array_equal(got.to_numpy(), exp)
    z = NDArray.from_numpy(np.full(case["exp_shape"], 119, np_dt))     # output supplied by the caller
    ex.exec_custom(case["op"], [x, y], [z])
    if exp.size:
        assert np.array_equal(z.to_numpy(), exp)


@pytest.mark.parametrize("case", _BC["shape_cases"], ids=[c["name"].split()[-1] for c in _BC["shape_cases"]])
def test_broadcastable_reference_shape_function(ex, case):
    x, y = NDArray.empty(case["x_shape"], FLOAT32), NDArray.empty(case["y_shape"], FLOAT32)
    shapes = ex.calculate_output_shapes(_BC["shape_op"], [x, y])
    si = shapes[0]
    assert [int(s) for s in si[1:1 + int(si[0])]] == case["exp_shape"]


# ---- cast, stack, unstack ----------------------------------------------------------------------------------------------------
def test_cast_reference_cases(ex):
    """DeclarableOpsTests1.cpp:1543-1556 (5x5 linspace float -> half via IArg 3), DeclarableOpsTests16.cpp:158-166 (empty bool ->
    int64 via IArg 10); the D argument names the type as well."""
    x = np.arange(1, 26, dtype=np.float32).reshape(5, 5)
    z = ex.exec_custom("cast", [NDArray.from_numpy(x)], i_args=[3])[0]
    assert z.dtype == HALF and np.array_equal(z.to_numpy(), x.astype(np.float16))
    from deeplearning4j_amd.ndarray import BOOL
    e = ex.exec_custom("cast", [NDArray.empty((1, 0, 2), BOOL)], i_args=[10])[0]
    assert e.dtype == INT64 and list(e.shape) == [1, 0, 2]
    rng = np.random.default_rng(3)
    v = (rng.normal(0, 40, (7, 9)).astype(np.float32))
    for dt, npdt in [(DOUBLE, np.float64), (INT32, np.int32), (INT64, np.int64), (HALF, np.float16)]:
        got = ex.exec_custom("Cast", [NDArray.from_numpy(v)], d_args=[dt])[0]
        assert got.dtype == dt and np.array_equal(got.to_numpy(), v.astype(npdt)), dt     # numpy truncates toward zero as C++ does
    b = ex.exec_custom("cast", [NDArray.from_numpy(v)], d_args=[BFLOAT16])[0]
    assert np.array_equal(b.to_numpy(), f32_to_bf16_bits(v))
    back = ex.exec_custom("cast", [NDArray.from_numpy(v.astype(np.int32))], d_args=[FLOAT32])[0]
    assert np.array_equal(back.to_numpy(), v.astype(np.int32).astype(np.float32))


def test_stack_reference_vectors(ex):
    """DeclarableOpsTests14.cpp:1728-1800 (Stack_1..3), :1935-1955 (Stack_11), :2113-2135 (Stack_21: stack == reshaped concat)."""
    a = np.arange(1, 13, dtype=np.float32).reshape(3, 4)
    b = np.array([13, 14, 16, 16, 17, 18, 19, 20, 21, 22, 23, 24], np.float32).reshape(3, 4)
    A, B = NDArray.from_numpy(a), NDArray.from_numpy(b)
    z = ex.exec_custom("stack", [A, B], i_args=[0])[0]
    assert list(z.shape) == [2, 3, 4] and np.array_equal(z.to_numpy().ravel(), np.concatenate([a.ravel(), b.ravel()]))
    z = ex.exec_custom("stack", [A, B], i_args=[1])[0]
    exp = np.array([1, 2, 3, 4, 13, 14, 16, 16, 5, 6, 7, 8, 17, 18, 19, 20, 9, 10, 11, 12, 21, 22, 23, 24], np.float32).reshape(3, 2, 4)
    assert list(z.shape) == [3, 2, 4] and np.array_equal(z.to_numpy(), exp)
    z = ex.exec_custom("pack", [NDArray.from_numpy(a.reshape(1, 12)), NDArray.from_numpy(b.reshape(1, 12))], i_args=[0])[0]
    assert list(z.shape) == [2, 1, 12] and np.array_equal(z.to_numpy().ravel(), np.concatenate([a.ravel(), b.ravel()]))
    one = NDArray.from_numpy(np.array([1.0], np.float32))
    z = ex.exec_custom("stack", [one, one, one])[0]
    assert list(z.shape) == [3, 1] and np.array_equal(z.to_numpy().ravel(), [1, 1, 1])
    z = ex.exec_custom("stack", [one, one, one], i_args=[1])[0]
    assert list(z.shape) == [1, 3]
    x1, x2 = np.arange(0, 6, dtype=np.float32).reshape(3, 2), np.arange(6, 12, dtype=np.float32).reshape(3, 2)
    st = ex.exec_custom("stack", [NDArray.from_numpy(x1), NDArray.from_numpy(x2)], i_args=[0])[0]
    cc = ex.exec_custom("concat", [NDArray.from_numpy(x1), NDArray.from_numpy(x2)], i_args=[0])[0]
    assert np.array_equal(st.to_numpy(), cc.to_numpy().reshape(2, 3, 2))
    # last axis, strided inputs, negative axis; numpy.stack is the same function
    rng = np.random.default_rng(8)
    big = rng.normal(0, 1, (5, 6, 7)).astype(np.float32)
    BIG = NDArray.from_numpy(big)
    views = [BIG.permute(2, 0, 1), BIG.permute(2, 0, 1)]
    z = ex.exec_custom("stack", views, i_args=[-1])[0]
    assert np.array_equal(z.to_numpy(), np.stack([big.transpose(2, 0, 1)] * 2, axis=-1))
    with pytest.raises(NativeOpsError, match="shapes of all input arrays must be the same"):
        ex.exec_custom("stack", [A, one])


def test_unstack_reference_cases(ex):
    """DeclarableOpsTests9.cpp:833-866: a 5x5 array gives 5 rows; a vector of 5 gives 5 scalars 1..5."""
    x = np.arange(1, 26, dtype=np.float64).reshape(5, 5)
    outs = ex.exec_custom("unstack", [NDArray.from_numpy(x)], i_args=[0])
    assert len(outs) == 5 and all(list(o.shape) == [5] for o in outs)
    assert all(np.array_equal(o.to_numpy(), x[i]) for i, o in enumerate(outs))
    outs = ex.exec_custom("unstack", [NDArray.from_numpy(x)], i_args=[1])
    assert all(np.array_equal(o.to_numpy(), x[:, i]) for i, o in enumerate(outs))
    outs = ex.exec_custom("unstack", [NDArray.from_numpy(np.arange(1, 6, dtype=np.float64))], i_args=[0])
    assert len(outs) == 5 and all(list(o.shape) == [] for o in outs)
    assert [float(o.to_numpy()) for o in outs] == [1, 2, 3, 4, 5]
    rng = np.random.default_rng(9)
    v = rng.normal(0, 1, (3, 4, 5)).astype(np.float32)
    outs = ex.exec_custom("unpack", [NDArray.from_numpy(v)], i_args=[-2])
    assert len(outs) == 4 and all(np.array_equal(o.to_numpy(), v[:, i]) for i, o in enumerate(outs))
    with pytest.raises(NativeOpsError, match="Unstack dimension should be lower then rank"):
        ex.exec_custom("unstack", [NDArray.from_numpy(v)], i_args=[3])


def test_biasadd_reference_vectors(ex):
    """DeclarableOpsTests4.cpp:692-741 (biasadd_1..3: NHWC, NCHW, rank 2) and :795-808 (double input, float bias and output)."""
    b2 = NDArray.from_numpy(np.array([1.0, 2.0]))
    z = ex.exec_custom("biasadd", [NDArray.from_numpy(np.zeros((2, 3, 3, 2))), b2])[0]
    assert np.array_equal(z.to_numpy(), np.tile([1.0, 2.0], 18).reshape(2, 3, 3, 2))
    z = ex.exec_custom("biasadd", [NDArray.from_numpy(np.zeros((2, 2, 3, 3))), b2], b_args=[True])[0]
    assert np.array_equal(z.to_numpy(), np.tile(np.repeat([1.0, 2.0], 9), 2).reshape(2, 2, 3, 3))
    row = NDArray.from_numpy(np.array([1.0, 2.0, 3.0]))
    z = ex.exec_custom("bias_add", [NDArray.from_numpy(np.zeros((2, 3))), row], b_args=[True])[0]
    assert np.array_equal(z.to_numpy(), [[1, 2, 3], [1, 2, 3]])
    zf = NDArray.empty((2, 3), FLOAT32)
    ex.exec_custom("biasadd", [NDArray.from_numpy(np.zeros((2, 3))), NDArray.from_numpy(np.array([1, 2, 3], np.float32))], [zf], b_args=[True])
    assert np.array_equal(zf.to_numpy(), np.array([[1, 2, 3], [1, 2, 3]], np.float32))
    rng = np.random.default_rng(12)
    x = rng.normal(0, 1, (3, 5, 4, 6)).astype(np.float32)
    b = rng.normal(0, 1, 5).astype(np.float32)
    z = ex.exec_custom("biasadd", [NDArray.from_numpy(x), NDArray.from_numpy(b)], b_args=[True])[0]
    assert np.array_equal(z.to_numpy(), x + b[None, :, None, None])
    with pytest.raises(NativeOpsError, match="not suitable for broadcast operation along channel dimension"):
        ex.exec_custom("biasadd", [NDArray.from_numpy(x), NDArray.from_numpy(b)])


def test_comparison_ops_reference_vectors(ex):
    """BroadcastableOpsTests.cpp:505-517 (broadcast_equals_1), :646-700 (broadcast_bool_1..3), :629-644 (broadcast_bool_empty_2)."""
    from deeplearning4j_amd.ndarray import BOOL
    x = NDArray.from_numpy(np.array([[1, 2, 3, 4]], np.float64))
    y = NDArray.from_numpy(np.array([[0, 0, 0, 0], [1, 2, 3, 4], [1, 2, 3, 4]], np.float64))
    z = ex.exec_custom("equals", [x, y])[0]
    assert z.dtype == BOOL and np.array_equal(z.to_numpy().astype(bool), [[False] * 4, [True] * 4, [True] * 4])
    a, b = NDArray.from_numpy(np.full((3, 1, 2), 4, np.float32)), NDArray.from_numpy(np.full((2, 2), 2, np.float32))
    z = ex.exec_custom("greater", [a, b])[0]
    assert list(z.shape) == [3, 2, 2] and z.to_numpy().astype(bool).all()
    z = ex.exec_custom("equals", [NDArray.from_numpy(np.full((3, 1, 2), 1, np.float32)), b])[0]
    assert list(z.shape) == [3, 2, 2] and not z.to_numpy().astype(bool).any()
    z = ex.exec_custom("less", [NDArray.from_numpy(np.array(0, np.int32)), NDArray.from_numpy(np.array([2, 1, 2], np.int32))])[0]
    assert list(z.shape) == [3] and z.to_numpy().astype(bool).all()
    e = ex.exec_custom("greater", [NDArray.empty((0, 4), DOUBLE), NDArray.from_numpy(np.array([[1, 2, 3, 4]], np.float64))])[0]
    assert e.dtype == BOOL and list(e.shape) == [0, 4]
    # every comparison against numpy, NaN included, integers beyond the float mantissa
    rng = np.random.default_rng(21)
    u = rng.integers(-3, 4, (5, 1, 17)).astype(np.float32)
    v = rng.integers(-3, 4, (6, 17)).astype(np.float32)
    u[0, 0, 0] = np.nan
    for name, fn in [("equals", np.equal), ("equal", np.equal), ("not_equals", np.not_equal), ("greater", np.greater),
                     ("greater_equal", np.greater_equal), ("less", np.less), ("less_equal", np.less_equal)]:
        got = ex.exec_custom(name, [NDArray.from_numpy(u), NDArray.from_numpy(v)])[0].to_numpy().astype(bool)
        assert np.array_equal(got, fn(u, v)), name
        for dt in (HALF, BFLOAT16):
            got = ex.exec_custom(name, [NDArray.from_numpy(u, dt), NDArray.from_numpy(v, dt)])[0].to_numpy().astype(bool)
            assert np.array_equal(got, fn(u, v)), (name, dt)
    big = np.array([16777217, 16777216, -16777217], np.int64)
    got = ex.exec_custom("greater", [NDArray.from_numpy(big), NDArray.from_numpy(np.array(16777216, np.int64))])[0].to_numpy().astype(bool)
    assert np.array_equal(got, [True, False, False])


def test_tile_and_slice_reference_vectors(ex):
    """DeclarableOpsTests3.cpp:36-60 (Test_Tile_1/2: a 2x3 array tiled 2x2), DeclarableOpsTests9.cpp:736-750 ({1,6} tiled {2,1}),
    IndexingTests.cpp:90-160 (SimpleSlice_1..4)."""
    x = np.array([[1, 2, 3], [4, 5, 6]], np.float32)
    want = np.tile(x, (2, 2))
    z = ex.exec_custom("tile", [NDArray.from_numpy(x), NDArray.from_numpy(np.array([[2, 2]], np.int32))])[0]
    assert list(z.shape) == [4, 6] and np.array_equal(z.to_numpy(), want)
    z = ex.exec_custom("tile", [NDArray.from_numpy(x)], i_args=[2, 2])[0]
    assert np.array_equal(z.to_numpy(), want)
    row = np.array([[1, 2, 3, 4, 5, 6]], np.float64)
    z = ex.exec_custom("tile", [NDArray.from_numpy(row), NDArray.from_numpy(np.array([[2, 1]], np.int32))])[0]
    assert list(z.shape) == [2, 6] and np.array_equal(z.to_numpy(), np.array([[1, 2, 3, 4, 5, 6]] * 2, np.float64))
    rng = np.random.default_rng(14)
    v = rng.normal(0, 1, (3, 4, 5)).astype(np.float32)
    z = ex.exec_custom("tile", [NDArray.from_numpy(v).permute(1, 2, 0)], i_args=[2, 1, 3])[0]
    assert np.array_equal(z.to_numpy(), np.tile(v.transpose(1, 2, 0), (2, 1, 3)))
    with pytest.raises(NativeOpsError, match="reps can't contain 0s"):
        ex.exec_custom("tile", [NDArray.from_numpy(x)], i_args=[2, 0])

    inp = np.array([1, 1, 1, 2, 2, 2, 3, 3, 3, 4, 4, 4, 5, 5, 5, 6, 6, 6], np.float32).reshape(3, 2, 3)
    z = ex.exec_custom("slice", [NDArray.from_numpy(inp)], i_args=[1, 0, 0, 1, 1, 3])[0]
    assert list(z.shape) == [1, 1, 3] and np.array_equal(z.to_numpy().ravel(), [3, 3, 3])
    z = ex.exec_custom("slice", [NDArray.from_numpy(inp)], i_args=[1, 0, 0, 1, 2, 3])[0]
    assert list(z.shape) == [1, 2, 3] and np.array_equal(z.to_numpy().ravel(), [3, 3, 3, 4, 4, 4])
    z = ex.exec_custom("slice", [NDArray.from_numpy(inp)], i_args=[1, 0, 0, 2, 1, 3])[0]
    assert list(z.shape) == [2, 1, 3] and np.array_equal(z.to_numpy().ravel(), [3, 3, 3, 5, 5, 5])
    start, size = NDArray.from_numpy(np.array([1.0, 0.0, 0.0])), NDArray.from_numpy(np.array([2.0, 1.0, 3.0]))
    z = ex.exec_custom("slice", [NDArray.from_numpy(inp.astype(np.float64)), start, size])[0]
    assert list(z.shape) == [2, 1, 3] and np.array_equal(z.to_numpy().ravel(), [3, 3, 3, 5, 5, 5])
    z = ex.exec_custom("slice", [NDArray.from_numpy(v)], i_args=[1, 2, 0, -1, 1, -1])[0]
    assert np.array_equal(z.to_numpy(), v[1:, 2:3, :])
    with pytest.raises(NativeOpsError, match="out of bounds for dimension 1"):
        ex.exec_custom("slice", [NDArray.from_numpy(v)], i_args=[0, 2, 0, 1, 3, 1])


def test_zeros_as_and_ones_as(ex):
    """generic/tensor/zeros_as.cpp:30-60, ones_as.cpp: the input's shape, the type of DArg 0 when given."""
    x = NDArray.from_numpy(np.arange(12, dtype=np.float32).reshape(3, 4))
    for name in ("zeros_as", "zeroslike", "zeros_like"):
        z = ex.exec_custom(name, [x])[0]
        assert z.dtype == FLOAT32 and list(z.shape) == [3, 4] and not z.to_numpy().any()
    o = ex.exec_custom("ones_as", [x], d_args=[DOUBLE])[0]
    assert o.dtype == DOUBLE and np.array_equal(o.to_numpy(), np.ones((3, 4)))
    h = ex.exec_custom("ones_as", [x], d_args=[BFLOAT16])[0]
    assert np.array_equal(h.to_float(), np.ones((3, 4), np.float32))
    e = ex.exec_custom("zeros_as", [NDArray.empty((2, 0, 3), FLOAT32)])[0]
    assert list(e.shape) == [2, 0, 3]
