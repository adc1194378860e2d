"""Every matmul kernel instantiation the dispatcher can pick for BASELINE config 2 (and the sizes around it), checked at
its real shape.

Each case asserts which kernel ran (`nd4jhipLastGemmKernel`), so that a change of the dispatch rules cannot silently
leave a kernel untested, then checks
  * 16 whole rows and 16 whole columns of the result against an fp64 product of the (rounded) inputs -- every tile row
    and every tile column of the launch grid is crossed;
  * whole-result identities: transposeB == plain B, transposeA == plain A, and fp16 == bf16 within the 16-bit gate.
Gates (north star): fp32 1e-4, fp16 / bf16 1e-2.  Flag combinations follow the reference's matmul tests
(libnd4j/tests_cpu/layers_tests/DeclarableOpsTests14.cpp:601-1260: transX / transY, c order).
"""
import math

import numpy as np
import pytest

from conftest import assert_close
from deeplearning4j_amd.ndarray import BFLOAT16, FLOAT32, HALF, NDArray, bf16_bits_to_f32, f32_to_bf16_bits

pytestmark = pytest.mark.gpu

TOL = {FLOAT32: 1e-4, HALF: 1e-2, BFLOAT16: 1e-2}


def _device(a, dtype):
    """(device array, fp64 view of the values it holds)"""
    a = np.ascontiguousarray(a, dtype=np.float32)
    if dtype == BFLOAT16:
        bits = f32_to_bf16_bits(a)
        return NDArray.from_numpy(bits, BFLOAT16), bf16_bits_to_f32(bits).astype(np.float64)
    if dtype == HALF:
        h = a.astype(np.float16)
        return NDArray.from_numpy(h), h.astype(np.float64)
    return NDArray.from_numpy(a), a.astype(np.float64)


def _last_kernel(ex):
    return ex.L.nd4jhipLastGemmKernel().decode()


def _run(ex, A, B, i_args, expect_kernel):
    z = ex.exec_custom("matmul", [A, B], i_args=i_args)[0]
    name = _last_kernel(ex)
    assert name.startswith(expect_kernel), "shape reached %s, the test means to check %s" % (name, expect_kernel)
    return z.to_float()


def _check_rows_cols(z, a64, b64, tol, rng, what):
    M, N = z.shape
    rows = rng.choice(M, min(16, M), replace=False)
    cols = rng.choice(N, min(16, N), replace=False)
    assert_close(z[rows], a64[rows] @ b64, tol, tol, what + ": sampled rows")
    assert_close(z[:, cols], a64 @ b64[:, cols], tol, tol, what + ": sampled columns")


# (dtype, M, N, K, kernel for plain B, kernel for transposeB, kernel for transposeA or None)
CASES = [
    # BASELINE config 2 at 4096^3
    (FLOAT32, 4096, 4096, 4096, "gemm_mfma32q<f32,128x128,akc=1,bkc=0,pd=4,bk=16>", "gemm_mfma32q<f32,128x128,akc=1,bkc=1,pd=4,bk=16>", "gemm_mfma32q<f32,128x128,akc=0,bkc=0,pd=4,bk=16>"),
    (HALF, 4096, 4096, 4096, "gemm_mfma16r<f16,256x256,akc=1,bkc=0>", "gemm_mfma16d<f16,256x256,akc=1,bkc=1>", "gemm_mfma16d<f16,256x256,akc=0,bkc=0>"),
    (BFLOAT16, 4096, 4096, 4096, "gemm_mfma16r<bf16,256x256,akc=1,bkc=0>", "gemm_mfma16d<bf16,256x256,akc=1,bkc=1>", "gemm_mfma16d<bf16,256x256,akc=0,bkc=0>"),
    # the ring kernel at its shortest K (the prologue alone fills the rings) and at a K that ends in the middle of both rings;
    # a K that is a multiple of 64 only stays on the two-stage direct kernel
    (BFLOAT16, 4096, 4096, 128, "gemm_mfma16r<bf16,256x256,akc=1,bkc=0>", "gemm_mfma16d<bf16,256x256,akc=1,bkc=1>", None),
    (HALF, 4096, 4096, 640, "gemm_mfma16r<f16,256x256,akc=1,bkc=0>", "gemm_mfma16d<f16,256x256,akc=1,bkc=1>", None),
    (BFLOAT16, 4096, 4096, 1152, "gemm_mfma16r<bf16,256x256,akc=1,bkc=0>", "gemm_mfma16d<bf16,256x256,akc=1,bkc=1>", None),
    (BFLOAT16, 4096, 4096, 192, "gemm_mfma16d<bf16,256x256,akc=1,bkc=0>", "gemm_mfma16d<bf16,256x256,akc=1,bkc=1>", None),
    # BASELINE config 2 at 1024^3
    (FLOAT32, 1024, 1024, 1024, "gemm_mfma32q<f32,64x64,akc=1,bkc=0,pd=4,bk=32>", "gemm_mfma32q<f32,64x64,akc=1,bkc=1,pd=4,bk=32>", "gemm_mfma32q<f32,64x64,akc=0,bkc=0,pd=4,bk=32>"),
    (HALF, 1024, 1024, 1024, "gemm_mfma16s<f16,64x64,akc=1,bkc=0,stages=8>", "gemm_mfma16s<f16,64x64,akc=1,bkc=1,stages=8>", "gemm_mfma16s<f16,64x64,akc=0,bkc=0,stages=8>"),
    (BFLOAT16, 1024, 1024, 1024, "gemm_mfma16s<bf16,64x64,akc=1,bkc=0,stages=8>", "gemm_mfma16s<bf16,64x64,akc=1,bkc=1,stages=8>", "gemm_mfma16s<bf16,64x64,akc=0,bkc=0,stages=8>"),
    # the 128 x 128 configuration (2048-class sizes), whole tiles
    (BFLOAT16, 2048, 2048, 2048, "gemm_mfma16s<bf16,128x128,akc=1,bkc=0,stages=4>", "gemm_mfma16s<bf16,128x128,akc=1,bkc=1,stages=4>", "gemm_mfma16s<bf16,128x128,akc=0,bkc=0,stages=4>"),
    (HALF, 2048, 2048, 1024, "gemm_mfma16s<f16,128x128,akc=1,bkc=0,stages=4>", "gemm_mfma16s<f16,128x128,akc=1,bkc=1,stages=4>", None),
    # a K of whole K-tiles that is not a multiple of four of them stays on the register-staged kernel
    (HALF, 2048, 2048, 320, "gemm_mfma16f<f16,128x128,akc=1,bkc=0>", "gemm_mfma16f<f16,128x128,akc=1,bkc=1>", "gemm_mfma16f<f16,128x128,akc=0,bkc=0>"),
    # ragged edges on the large tiles (bounds-handling kernel)
    (BFLOAT16, 3600, 3704, 72, "gemm_mfma16p<bf16,256x256,akc=1,bkc=0>", "gemm_mfma16p<bf16,256x256,akc=1,bkc=1>", "gemm_mfma16p<bf16,256x256,akc=0,bkc=0>"),
    # ... from K = 128 on the direct-load kernels take them, also with a K that ends inside a K-tile
    (BFLOAT16, 3600, 3704, 1000, "gemm_mfma16r<bf16,256x256,akc=1,bkc=0,edge,ktail>", "gemm_mfma16d<bf16,256x256,akc=1,bkc=1,edge,ktail>", "gemm_mfma16d<bf16,256x256,akc=0,bkc=0,edge,ktail>"),
    # ragged edges with aligned rows and a K of whole K-tiles: the direct-load kernels' edge instantiations (clamped loads,
    # bounds-checked store) -- a last tile row of 16 rows and a last tile column of 120, of 8 (one column group) and of 1
    (BFLOAT16, 3600, 3704, 1024, "gemm_mfma16r<bf16,256x256,akc=1,bkc=0,edge>", "gemm_mfma16d<bf16,256x256,akc=1,bkc=1,edge>", "gemm_mfma16d<bf16,256x256,akc=0,bkc=0,edge>"),
    (HALF, 3599, 3592, 192, "gemm_mfma16d<f16,256x256,akc=1,bkc=0,edge>", "gemm_mfma16d<f16,256x256,akc=1,bkc=1,edge>", None),
    (BFLOAT16, 3601, 3585, 256, "gemm_mfma16r<bf16,256x256,akc=1,bkc=0,edge,unaligned>", "gemm_mfma16d<bf16,256x256,akc=1,bkc=1,edge>", None),
    (BFLOAT16, 2000, 2000, 2048, "gemm_mfma16s<bf16,128x128,akc=1,bkc=0,stages=4,edge>", "gemm_mfma16s<bf16,128x128,akc=1,bkc=1,stages=4,edge>", "gemm_mfma16s<bf16,128x128,akc=0,bkc=0,stages=4,edge>"),
    (HALF, 1000, 1000, 1024, "gemm_mfma16s<f16,64x64,akc=1,bkc=0,stages=8,edge>", "gemm_mfma16s<f16,64x64,akc=1,bkc=1,stages=8,edge>", "gemm_mfma16s<f16,64x64,akc=0,bkc=0,stages=8,edge>"),
    (BFLOAT16, 500, 2304, 768, "gemm_mfma16s<bf16,64x64,akc=1,bkc=0,stages=4,edge>", "gemm_mfma16s<bf16,64x64,akc=1,bkc=1,stages=4,edge>", None),
    # ... and with a K that is not a whole number of K-tiles (from 128 on: the ring kernel with the page of zeros; below: the
    # bounds-handling kernel)
    (HALF, 1800, 1800, 520, "gemm_mfma16s<f16,128x128,akc=1,bkc=0,stages=4,edge,ktail>", "gemm_mfma16s<f16,128x128,akc=1,bkc=1,stages=4,edge,ktail>", None),
    (BFLOAT16, 1104, 904, 1000, "gemm_mfma16s<bf16,64x64,akc=1,bkc=0,stages=4,edge,ktail>", "gemm_mfma16s<bf16,64x64,akc=1,bkc=1,stages=4,edge,ktail>", "gemm_mfma16s<bf16,64x64,akc=0,bkc=0,stages=4,edge,ktail>"),
    (HALF, 1800, 1800, 72, "gemm_mfma16p<f16,128x128,akc=1,bkc=0>", "gemm_mfma16p<f16,128x128,akc=1,bkc=1>", None),
    (BFLOAT16, 1104, 904, 104, "gemm_mfma16p<bf16,64x64,akc=1,bkc=0>", "gemm_mfma16p<bf16,64x64,akc=1,bkc=1>", None),
    # K a multiple of 256 but not of 512: the four-stage ring; more tiles than CUs (two blocks on a CU): four stages as well;
    # the shortest K the ring takes
    (BFLOAT16, 1024, 1024, 768, "gemm_mfma16s<bf16,64x64,akc=1,bkc=0,stages=4>", "gemm_mfma16s<bf16,64x64,akc=1,bkc=1,stages=4>", "gemm_mfma16s<bf16,64x64,akc=0,bkc=0,stages=4>"),
    (HALF, 512, 2304, 1024, "gemm_mfma16s<f16,64x64,akc=1,bkc=0,stages=4>", "gemm_mfma16s<f16,64x64,akc=1,bkc=1,stages=4>", None),
    (BFLOAT16, 1024, 1024, 512, "gemm_mfma16s<bf16,64x64,akc=1,bkc=0,stages=8>", "gemm_mfma16s<bf16,64x64,akc=1,bkc=1,stages=8>", None),
    (FLOAT32, 1024, 1024, 384, "gemm_mfma32q<f32,64x64,akc=1,bkc=0,pd=4,bk=32>", "gemm_mfma32q<f32,64x64,akc=1,bkc=1,pd=4,bk=32>", None),
    (FLOAT32, 2048, 2048, 640, "gemm_mfma32q<f32,128x128,akc=1,bkc=0,pd=4,bk=16>", "gemm_mfma32q<f32,128x128,akc=1,bkc=1,pd=4,bk=16>", None),
    # few 64 x 64 tiles: up to K = 2048 one block per tile on the ring kernel, beyond that split-K with its finishing launch
    (BFLOAT16, 512, 512, 512, "gemm_mfma16s<bf16,64x64,akc=1,bkc=0,stages=8>", "gemm_mfma16s<bf16,64x64,akc=1,bkc=1,stages=8>", None),
    (HALF, 512, 768, 2048, "gemm_mfma16s<f16,64x64,akc=1,bkc=0,stages=8>", "gemm_mfma16s<f16,64x64,akc=1,bkc=1,stages=8>", None),
    (BFLOAT16, 256, 256, 4096, "gemm_mfma16s<bf16,64x64,akc=1,bkc=0,stages=4,split>+splitk_finish", "gemm_mfma16s<bf16,64x64,akc=1,bkc=1,stages=4,split>+splitk_finish", "gemm_mfma16s<bf16,64x64,akc=0,bkc=0,stages=4,split>+splitk_finish"),
    (HALF, 250, 250, 4104, "gemm_mfma16<f16,64x64,akc=1,bkc=0>+splitk_finish", "gemm_mfma16s<f16,64x64,akc=1,bkc=1,stages=", None),
    # row lengths that are not multiples of 8 (rows start off 16-byte boundaries, the last vector of a row is partial): the
    # bounds-handling kernels read element-aligned vectors -- a batched decode step's logits against the row-major
    # [768, 50257] embedding, a prefill's, and a product with nothing aligned in any layout
    (BFLOAT16, 32, 50257, 768, "gemm_mfma16p<bf16,32x128,akc=1,bkc=0>", "gemm_mfma16p<bf16,32x128,akc=1,bkc=1>", None),
    (BFLOAT16, 1024, 50257, 768, "gemm_mfma16r<bf16,256x256,akc=1,bkc=0,edge,unaligned>", "gemm_mfma16d<bf16,256x256,akc=1,bkc=1,edge>", None),
    (HALF, 1000, 1003, 515, "gemm_mfma16p<f16,64x64,akc=1,bkc=0>", "gemm_mfma16p<f16,64x64,akc=1,bkc=1>", "gemm_mfma16p<f16,64x64,akc=0,bkc=0>"),
    (BFLOAT16, 2001, 1999, 1003, "gemm_mfma16p<bf16,128x128,akc=1,bkc=0>", "gemm_mfma16p<bf16,128x128,akc=1,bkc=1>", "gemm_mfma16p<bf16,128x128,akc=0,bkc=0>"),
    (HALF, 20, 4097, 2051, "gemm_mfma16<f16,32x128,akc=1,bkc=0>+splitk_finish", "gemm_mfma16<f16,32x128,akc=1,bkc=1>+splitk_finish", None),
    # the same for fp32 (row lengths that are not multiples of 4)
    (FLOAT32, 1000, 1003, 515, "gemm_mfma32<f32,64x64,akc=1,bkc=0>", "gemm_mfma32<f32,64x64,akc=1,bkc=1>", "gemm_mfma32<f32,64x64,akc=0,bkc=0>"),
    (FLOAT32, 257, 50257, 770, "gemm_mfma32<f32,128x128,akc=1,bkc=0>", "gemm_mfma32<f32,128x128,akc=1,bkc=1>", None),
    # fp32 ragged with aligned rows and a K of whole rounds: the edge instantiation of the deep-pipeline kernel
    (FLOAT32, 1000, 1000, 1024, "gemm_mfma32q<f32,64x64,akc=1,bkc=0,pd=4,bk=32,edge>", "gemm_mfma32q<f32,64x64,akc=1,bkc=1,pd=4,bk=32,edge>", "gemm_mfma32q<f32,64x64,akc=0,bkc=0,pd=4,bk=32,edge>"),
    (FLOAT32, 2004, 2000, 512, "gemm_mfma32q<f32,128x128,akc=1,bkc=0,pd=4,bk=16,edge>", "gemm_mfma32q<f32,128x128,akc=1,bkc=1,pd=4,bk=16,edge>", "gemm_mfma32q<f32,128x128,akc=0,bkc=0,pd=4,bk=16,edge>"),
    # fp32 ragged
    (FLOAT32, 1100, 900, 1000, "gemm_mfma32q<f32,64x64,akc=1,bkc=0,pd=4,bk=32,edge,ktail>", "gemm_mfma32q<f32,64x64,akc=1,bkc=1,pd=4,bk=32,edge,ktail>", None),
    (FLOAT32, 2100, 2052, 520, "gemm_mfma32q<f32,128x128,akc=1,bkc=0,pd=4,bk=16,edge,ktail>", "gemm_mfma32q<f32,128x128,akc=1,bkc=1,pd=4,bk=16,edge,ktail>", "gemm_mfma32q<f32,128x128,akc=0,bkc=0,pd=4,bk=16,edge,ktail>"),
    (FLOAT32, 1100, 900, 200, "gemm_mfma32<f32,64x64,akc=1,bkc=0>", "gemm_mfma32<f32,64x64,akc=1,bkc=1>", None),
    (FLOAT32, 2100, 2052, 136, "gemm_mfma32<f32,128x128,akc=1,bkc=0>", "gemm_mfma32<f32,128x128,akc=1,bkc=1>", "gemm_mfma32<f32,128x128,akc=0,bkc=0>"),
]


@pytest.mark.parametrize("dtype,M,N,K,kern_plain,kern_tb,kern_ta", CASES,
                         ids=["%s-%dx%dx%d" % ({FLOAT32: "f32", HALF: "f16", BFLOAT16: "bf16"}[c[0]], c[1], c[2], c[3]) for c in CASES])
def test_matmul_kernel_at_real_shape(ex, dtype, M, N, K, kern_plain, kern_tb, kern_ta):
    rng = np.random.default_rng(2002 + M + 3 * N + 7 * K + dtype)
    tol = TOL[dtype]
    a = rng.normal(0, 1 / math.sqrt(K), (M, K)).astype(np.float32)
    b = rng.normal(0, 1 / math.sqrt(K), (K, N)).astype(np.float32)
    A, a64 = _device(a, dtype)
    B, b64 = _device(b, dtype)
    z = _run(ex, A, B, [0, 0], kern_plain)
    _check_rows_cols(z, a64, b64, tol, rng, "plain")
    Bt, _ = _device(b.T, dtype)
    zt = _run(ex, A, Bt, [0, 1], kern_tb)
    _check_rows_cols(zt, a64, b64, tol, rng, "transposeB")
    assert_close(zt, z, tol, tol, "transposeB agrees with plain B over the whole result")
    if kern_ta:
        At, _ = _device(a.T, dtype)
        za = _run(ex, At, B, [1, 0], kern_ta)
        _check_rows_cols(za, a64, b64, tol, rng, "transposeA")
        assert_close(za, z, tol, tol, "transposeA agrees with plain A over the whole result")


@pytest.mark.parametrize("dtype,M,N,K", [(BFLOAT16, 3600, 3705, 256), (HALF, 3599, 3591, 128), (BFLOAT16, 3585, 3704, 384),
                                         (BFLOAT16, 499, 2312, 768), (HALF, 1921, 1928, 512), (FLOAT32, 999, 1004, 256), (FLOAT32, 1925, 1924, 384),
                                         (BFLOAT16, 3600, 3705, 200)],
                         ids=["bf16-rows-off-by-one", "f16-seven-columns-left", "bf16-aligned-ragged", "bf16-64x64-tiles", "f16-128x128-tiles",
                              "f32-64x64-tiles", "f32-128x128-tiles", "bf16-rows-off-by-one-k200"])
def test_ragged_product_on_the_direct_load_kernels_whole_result(ex, dtype, M, N, K):
    _whole_result(ex, dtype, M, N, K, False)


@pytest.mark.parametrize("tb", [False, True], ids=["plain", "transposeB"])
@pytest.mark.parametrize("dtype,M,N,K", [(BFLOAT16, 1000, 1000, 1000), (HALF, 1024, 1024, 520), (BFLOAT16, 2000, 2000, 1000), (HALF, 512, 512, 1992),
                                         (BFLOAT16, 1920, 2048, 968), (BFLOAT16, 3700, 3704, 1000), (HALF, 4096, 3840, 136),
                                         (FLOAT32, 1000, 1000, 1000), (FLOAT32, 1920, 2048, 268), (BFLOAT16, 1000, 1000, 136), (HALF, 2000, 1800, 328),
                                         (BFLOAT16, 504, 504, 200)],
                         ids=["bf16-1000", "f16-whole-tiles-k520", "bf16-128x128-tiles", "f16-few-tiles", "bf16-k968", "bf16-256x256-tiles", "f16-256x256-k136",
                              "f32-1000", "f32-128x128-k268", "bf16-k136", "f16-128x128-k328", "bf16-few-tiles-k200"])
def test_k_tail_on_the_direct_load_kernels_whole_result(ex, dtype, M, N, K, tb):
    """A K that is not a whole number of K-tiles on the ring kernel: the lanes beyond K read a page of zeros.  Every element of
    the result, with operands whose neighbours in memory (the next row, which a load past K would bring in) are large."""
    _whole_result(ex, dtype, M, N, K, tb, expect=",ktail")


@pytest.mark.parametrize("tb", [False, True], ids=["plain", "transposeB"])
@pytest.mark.parametrize("dtype,M,N,K", [(BFLOAT16, 512, 768, 3072), (HALF, 504, 496, 4008), (BFLOAT16, 72, 768, 3072), (HALF, 256, 320, 2200)],
                         ids=["bf16-mlp-down", "f16-ragged", "bf16-72-rows", "f16-k2200"])
def test_split_k_on_the_direct_load_ring_whole_result(ex, dtype, M, N, K, tb):
    """Few 64 x 64 tiles and a long K: split-K on the ring kernel (every block a range of K-tiles, zeros beyond its range and
    beyond K), partial tiles added up by the finishing launch.  Every element of the result."""
    _whole_result(ex, dtype, M, N, K, tb, expect=",split>+splitk_finish")


def test_split_k_on_the_ring_batched_with_alpha_beta(ex):
    """Three batch entries of few tiles and a long K: every entry's splits park their tiles under the entry's own index, and the
    finishing launch applies alpha and beta."""
    rng = np.random.default_rng(31)
    batch, M, N, K = 3, 136, 128, 4104
    a = rng.normal(0, 1 / math.sqrt(K), (batch, M, K)).astype(np.float32)
    b = rng.normal(0, 1 / math.sqrt(K), (batch, K, N)).astype(np.float32)
    c0 = rng.normal(0, 1, (batch, M, N)).astype(np.float32)
    A, a64 = _device(a, BFLOAT16)
    B, b64 = _device(b, BFLOAT16)
    C, c64 = _device(c0, BFLOAT16)
    ex.exec_custom("matmul", [A, B], [C], t_args=[0.5, 2.0])
    assert ",split>+splitk_finish" in _last_kernel(ex), _last_kernel(ex)
    got = C.to_float()
    for bi in range(batch):
        assert_close(got[bi], 0.5 * (a64[bi] @ b64[bi]) + 2.0 * c64[bi], 1e-2, 2e-2, "batch %d" % bi)


def _whole_result(ex, dtype, M, N, K, tb, expect=",edge"):
    """The edge instantiations of the direct-load kernels, every element of the result: a row-major B with rows of 3705
    (every row starts 2 bytes further off a 16-byte boundary; one column is left for the bounds-handling kernel), of 3591
    (seven columns left), and an aligned B with a ragged last tile row and column."""
    rng = np.random.default_rng(M + N + K)
    a = rng.normal(0, 1 / math.sqrt(K), (M, K)).astype(np.float32)
    b = rng.normal(0, 1 / math.sqrt(K), (K, N)).astype(np.float32)
    A, a64 = _device(a, dtype)
    B, b64 = _device(b, dtype)
    if tb:
        B, _ = _device(b.T, dtype)
    z = ex.exec_custom("matmul", [A, B], i_args=[0, 1 if tb else 0])[0].to_float()
    name = _last_kernel(ex)
    assert expect in name, name
    assert ("unaligned" in name) == (dtype != FLOAT32 and N % 8 != 0 and not tb), name
    assert_close(z, a64 @ b64, TOL[dtype], TOL[dtype], "whole result")
    if dtype != FLOAT32 and M % 8 == 0:
        # the same product with A handed over transposed ([K, M], the transposeA flag): the kernels that keep A's k-rows in LDS
        At, _ = _device(a.T, dtype)
        zt = ex.exec_custom("matmul", [At, B], i_args=[1, 1 if tb else 0])[0].to_float()
        name = _last_kernel(ex)
        assert expect in name and "akc=0" in name, name
        assert_close(zt, a64 @ b64, TOL[dtype], TOL[dtype], "whole result, transposed A")


@pytest.mark.parametrize("n", [1024, 4096])
def test_fp16_and_bf16_agree(ex, n):
    """Inputs exactly representable in both 16-bit types (multiples of 1/8 in [-2, 2]): fp16 and bf16 kernels multiply
    the same numbers, so their results differ only by the final rounding."""
    rng = np.random.default_rng(n)
    a = (rng.integers(-16, 17, (n, n)) / 8.0).astype(np.float32) / math.sqrt(n)
    b = (rng.integers(-16, 17, (n, n)) / 8.0).astype(np.float32)
    # a / sqrt(n) stays exact in both types for n a power of four
    Ah, a64 = _device(a, HALF)
    Bh, b64 = _device(b, HALF)
    Ab, a64b = _device(a, BFLOAT16)
    Bb, b64b = _device(b, BFLOAT16)
    assert np.array_equal(a64, a64b) and np.array_equal(b64, b64b)
    zh = ex.exec_custom("matmul", [Ah, Bh])[0].to_float()
    kh = _last_kernel(ex)
    zb = ex.exec_custom("matmul", [Ab, Bb])[0].to_float()
    kb = _last_kernel(ex)
    assert "<f16," in kh and "<bf16," in kb and kh.split("<")[0] == kb.split("<")[0]
    assert_close(zh, zb, 1e-2, 1e-2, "fp16 result against bf16 result")
    rows = rng.choice(n, 8, replace=False)
    assert_close(zh[rows], a64[rows] @ b64, 1e-2, 1e-2, "fp16 sampled rows")


def test_alpha_beta_on_the_ring_kernel(ex):
    """C = alpha A B + beta C through the 256 x 256 ring kernel (its epilogue reads C), batched."""
    rng = np.random.default_rng(19)
    M, N, K = 512, 768, 512
    # a 256-tile launch needs at least 192 tiles: batch the problem
    batch = 32
    a = rng.normal(0, 1 / math.sqrt(K), (batch, M, K)).astype(np.float32)
    b = rng.normal(0, 1 / math.sqrt(K), (batch, K, N)).astype(np.float32)
    c0 = rng.normal(0, 1, (batch, M, N)).astype(np.float32)
    A, a64 = _device(a, BFLOAT16)
    B, b64 = _device(b, BFLOAT16)
    C, c64 = _device(c0, BFLOAT16)
    ex.exec_custom("matmul", [A, B], [C], t_args=[0.5, 2.0])
    assert _last_kernel(ex).startswith("gemm_mfma16r<bf16,256x256,akc=1,bkc=0>"), _last_kernel(ex)
    got = C.to_float()
    for bi in (0, 13, 31):
        assert_close(got[bi], 0.5 * (a64[bi] @ b64[bi]) + 2.0 * c64[bi], 1e-2, 2e-2, "batch %d" % bi)
    # the same through the two-stage direct kernel (transposed B)
    Bt, _ = _device(np.ascontiguousarray(np.swapaxes(b, 1, 2)), BFLOAT16)
    C2, _ = _device(c0, BFLOAT16)
    ex.exec_custom("matmul", [A, Bt], [C2], t_args=[0.5, 2.0], i_args=[0, 1])
    assert _last_kernel(ex).startswith("gemm_mfma16d<bf16,256x256,akc=1,bkc=1>"), _last_kernel(ex)
    assert np.array_equal(C2.to_float(), got), "transposed B gives the same bits (same products, same order)"


@pytest.mark.parametrize("dtype", [BFLOAT16, FLOAT32], ids=["bf16", "f32"])
def test_alpha_beta_batched_ragged_on_the_edge_kernels(ex, dtype):
    """C = alpha A B + beta C, batched, with M, N and K all off the tile sizes: the edge instantiations read C back in their
    bounds-checked epilogue, and every batch entry clamps against its own operand.  Then the same product with A and B as
    pitched views (rows longer than the extent that is multiplied)."""
    rng = np.random.default_rng(29)
    batch, M, N, K = 5, 1000, 1096, 1000
    tol = TOL[dtype]
    a = rng.normal(0, 1 / math.sqrt(K), (batch, M, K)).astype(np.float32)
    b = rng.normal(0, 1 / math.sqrt(K), (batch, K, N)).astype(np.float32)
    c0 = rng.normal(0, 1, (batch, M, N)).astype(np.float32)
    A, a64 = _device(a, dtype)
    B, b64 = _device(b, dtype)
    C, c64 = _device(c0, dtype)
    ex.exec_custom("matmul", [A, B], [C], t_args=[0.5, 2.0])
    assert ",edge,ktail" in _last_kernel(ex), _last_kernel(ex)
    got = C.to_float()
    for bi in range(batch):
        assert_close(got[bi], 0.5 * (a64[bi] @ b64[bi]) + 2.0 * c64[bi], tol, 2 * tol, "batch %d" % bi)
    # pitched views: A inside a [M, K + 24] array, B inside a [K, N + 40] array, one batch entry
    wideA = rng.normal(0, 1 / math.sqrt(K), (M, K + 24)).astype(np.float32)
    wideB = rng.normal(0, 1 / math.sqrt(K), (K, N + 40)).astype(np.float32)
    WA, wa64 = _device(wideA, dtype)
    WB, wb64 = _device(wideB, dtype)
    z = ex.exec_custom("matmul", [WA.slice(1, 8, 8 + K), WB.slice(1, 16, 16 + N)])[0].to_float()
    assert ",edge,ktail" in _last_kernel(ex), _last_kernel(ex)
    assert_close(z, wa64[:, 8:8 + K] @ wb64[:, 16:16 + N], tol, tol, "pitched views")


def test_bias_row_on_the_large_kernels(ex):
    """xw_plus_b at a shape that lands on the 256 x 256 kernels: the bias row is added in their epilogue."""
    rng = np.random.default_rng(23)
    M, K, N = 4096, 512, 4096
    x = rng.normal(0, 1 / math.sqrt(K), (M, K)).astype(np.float32)
    w = rng.normal(0, 1, (K, N)).astype(np.float32)
    bias = rng.normal(0, 1, (N,)).astype(np.float32)
    X, x64 = _device(x, BFLOAT16)
    W, w64 = _device(w, BFLOAT16)
    Bv, b64 = _device(bias, BFLOAT16)
    z = ex.exec_custom("xw_plus_b", [X, W, Bv])[0].to_float()
    assert _last_kernel(ex).startswith("gemm_mfma16r<bf16,256x256,akc=1,bkc=0>"), _last_kernel(ex)
    rows = rng.choice(M, 16, replace=False)
    assert_close(z[rows], x64[rows] @ w64 + b64, 1e-2, 1e-2, "sampled rows")
    Wt, _ = _device(np.ascontiguousarray(w.T), BFLOAT16)
    zt = ex.exec_custom("xw_plus_b", [X, Wt, Bv], i_args=[0, 1])[0].to_float()
    assert _last_kernel(ex).startswith("gemm_mfma16d<bf16,256x256,akc=1,bkc=1>"), _last_kernel(ex)
    assert np.array_equal(zt, z)


def test_small_tile_ring_and_register_staged_kernel_give_the_same_bits(tmp_path):
    """The 64 x 64 direct-load ring (gemm_mfma16s) and the register-staged kernel it replaced by default (gemm_mfma16q, kept
    for operands the ring does not take) add the same products in the same order: identical results, with a pitched A and
    with alpha / beta / bias as well."""
    import os, subprocess, sys
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    child = r"""
import sys, math, numpy as np
sys.path.insert(0, %r)
from deeplearning4j_amd.executioner import Executioner
from deeplearning4j_amd.ndarray import NDArray, BFLOAT16, HALF, f32_to_bf16_bits
ex = Executioner()
rng = np.random.default_rng(77)
out, names = {}, []
for n, (dt, M, N, K) in enumerate([(BFLOAT16, 1024, 1024, 1024), (HALF, 1024, 1024, 768), (BFLOAT16, 1024, 1024, 512)]):
    conv = (lambda v: f32_to_bf16_bits(v.astype(np.float32))) if dt == BFLOAT16 else (lambda v: v.astype(np.float16))
    a = rng.normal(0, 1 / math.sqrt(K), (M, K + 8)); b = rng.normal(0, 1, (K, N)); c = rng.normal(0, 1, (M, N))
    A = NDArray.from_numpy(conv(a), dt).slice(1, 0, K)                  # pitched rows
    B, Bt = NDArray.from_numpy(conv(b), dt), NDArray.from_numpy(conv(np.ascontiguousarray(b.T)), dt)
    for tag, ops, ia in (("plain", [A, B], [0, 0]), ("tb", [A, Bt], [0, 1])):
        Z = NDArray.from_numpy(conv(c), dt)
        ex.exec_custom("matmul", ops, [Z], t_args=[0.5, 2.0], i_args=ia)
        out["%%d_%%s" %% (n, tag)] = Z.to_numpy(); names.append(ex.L.nd4jhipLastGemmKernel().decode())
np.savez(sys.argv[1], names=np.array(names), **out)
"""
    res = []
    for ring in (1, 0):
        path = str(tmp_path / ("ring%d.npz" % ring))
        r = subprocess.run([sys.executable, "-c", child % root, path], env=dict(os.environ, ND4JHIP_GEMM_SMALL_RING=str(ring)),
                           capture_output=True, text=True, timeout=300)
        assert r.returncode == 0, r.stderr[-2000:]
        res.append(np.load(path))
    one, two = res
    assert all("gemm_mfma16s" in str(s_) for s_ in one["names"]), list(one["names"])
    assert all("gemm_mfma16q" in str(s_) for s_ in two["names"]), list(two["names"])
    for key in one.files:
        if key != "names":
            assert np.array_equal(one[key], two[key]), key


@pytest.mark.parametrize("dtype", [HALF, BFLOAT16])
def test_matmul_on_views_without_a_unit_stride(ex, dtype):
    """Operands whose elements are two apart along both axes (every second row and column of a larger array) and a
    result written into such a view: no vector loader takes them, the element-gathering tile kernel does."""
    rng = np.random.default_rng(99 + dtype)
    M, N, K = 300, 260, 200
    a = rng.normal(0, 1 / math.sqrt(K), (2 * M, 2 * K)).astype(np.float32)
    b = rng.normal(0, 1 / math.sqrt(K), (2 * K, 2 * N)).astype(np.float32)
    A, a64 = _device(a, dtype)
    B, b64 = _device(b, dtype)
    Av = A.view((M, K), (4 * K, 2))
    Bv = B.view((K, N), (4 * N, 2))
    z = ex.exec_custom("matmul", [Av, Bv])[0]
    assert _last_kernel(ex).startswith("gemm_mfma16u<%s,128x128,arf=0,brf=1>" % ("f16" if dtype == HALF else "bf16")), _last_kernel(ex)
    assert_close(z.to_float(), a64[::2, ::2] @ b64[::2, ::2], TOL[dtype], TOL[dtype], "every second row and column")
    # transposed views of the same operands: the smaller stride now runs along the rows of A and along k of B
    At, Bt = Av.permute(1, 0), Bv.permute(1, 0)
    zt = ex.exec_custom("matmul", [At, Bt], i_args=[1, 1])[0]
    assert _last_kernel(ex).startswith("gemm_mfma16u<"), _last_kernel(ex)
    assert_close(zt.to_float(), a64[::2, ::2] @ b64[::2, ::2], TOL[dtype], TOL[dtype], "transposed views, both flags")
