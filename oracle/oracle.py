"""ctypes binding of the CPU oracle (libnd4j_oracle.so) -- test infrastructure only.

Arrays cross the boundary as numpy arrays plus a shapeInfo descriptor built from the numpy
view itself (shape, element strides, dtype, order), so strided/permuted numpy views exercise
the same shapeInfo walk the reference performs.  bf16 arrays are numpy uint16 arrays tagged
with dtype code BFLOAT16; fp16 uses numpy float16.
"""
import ctypes
import os
import subprocess

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "libnd4j_oracle.so")

BOOL, HALF, FLOAT32, DOUBLE, INT32, INT64, BFLOAT16 = 1, 3, 5, 6, 9, 10, 17
_NP2DT = {np.dtype(np.float16): HALF, np.dtype(np.float32): FLOAT32, np.dtype(np.float64): DOUBLE,
          np.dtype(np.int32): INT32, np.dtype(np.int64): INT64, np.dtype(np.bool_): BOOL}
DT_FLAG = {HALF: 4096, BFLOAT16: 2048, FLOAT32: 8192, DOUBLE: 16384, INT32: 131072, INT64: 262144, BOOL: 524288}
DT_NP = {HALF: np.float16, BFLOAT16: np.uint16, FLOAT32: np.float32, DOUBLE: np.float64, INT32: np.int32,
         INT64: np.int64, BOOL: np.bool_}


def build(force=False):
    """Compile the oracle with the Makefile next to this file."""
    if force or not os.path.exists(LIB_PATH):
        subprocess.check_call(["make", "-C", HERE, "-B" if force else "-s", "libnd4j_oracle.so"])
    return LIB_PATH


_lib = None


def lib():
    global _lib
    if _lib is None:
        build()
        L = ctypes.CDLL(LIB_PATH)
        vp, i64p, i32, i64, dbl = ctypes.c_void_p, ctypes.POINTER(ctypes.c_int64), ctypes.c_int, ctypes.c_int64, ctypes.c_double
        L.orc_hash.restype = i64
        L.orc_hash.argtypes = [ctypes.c_char_p]
        L.orc_offset.restype = i64
        L.orc_offset.argtypes = [i64p, i64]
        L.orc_length.restype = i64
        L.orc_length.argtypes = [i64p]
        L.orc_tad.restype = i64
        L.orc_tad.argtypes = [i64p, i64p, i32, i64p, i64p]
        L.orc_f32_to_bf16.restype = ctypes.c_uint16
        L.orc_f32_to_bf16.argtypes = [ctypes.c_float]
        L.orc_f32_to_f16.restype = ctypes.c_uint16
        L.orc_f32_to_f16.argtypes = [ctypes.c_float]
        L.orc_f16_to_f32.restype = ctypes.c_float
        L.orc_f16_to_f32.argtypes = [ctypes.c_uint16]
        L.orc_pairwise.argtypes = [i32, vp, i64p, vp, i64p, vp, i64p]
        L.orc_transform_strict.argtypes = [i32, vp, i64p, vp, i64p]
        L.orc_transform_float.argtypes = [i32, vp, i64p, vp, i64p]
        L.orc_transform_same.argtypes = [i32, vp, i64p, vp, i64p]
        L.orc_transform_bool.argtypes = [i32, vp, i64p, vp, i64p]
        L.orc_summary_stats.argtypes = [i32, vp, i64p, vp, i64p, i64p, i32, i32]
        L.orc_reduce_count.argtypes = [i32, vp, i64p, vp, i64p, i64p, i32]
        L.orc_reduce3.argtypes = [i32, vp, i64p, vp, i64p, vp, i64p, i64p, i32]
        L.orc_scalar.argtypes = [i32, vp, i64p, dbl, vp, i64p]
        L.orc_broadcast.argtypes = [i32, vp, i64p, vp, i64p, vp, i64p, i64p, i32]
        for f in (L.orc_reduce_same, L.orc_reduce_float, L.orc_index_reduce):
            f.argtypes = [i32, vp, i64p, vp, i64p, i64p, i32]
        L.orc_softmax.argtypes = [vp, i64p, vp, i64p, i32, i32]
        L.orc_top_k.argtypes = [vp, i64p, vp, i64p, vp, i64p, i64, i32]
        L.orc_layer_norm.argtypes = [vp, i64p, vp, i64p, vp, i64p, vp, i64p, i64p, i32, i32]
        L.orc_matmul.argtypes = [vp, i64p, vp, i64p, vp, i64p, i32, i32, i32, dbl, dbl, i32]
        L.orc_attention_v2.argtypes = [vp, i64p, vp, i64p, vp, i64p, vp, i64p, vp, i64p, vp, i64p, dbl, i32, vp, i64p, vp, i64p]
        L.orc_add_row_vector.argtypes = [vp, i64p, vp, i64p, vp, i64p]
        L.orc_set_threads.argtypes = [i32]
        L.orc_get_threads.restype = i32
        _lib = L
    return _lib


def f32_to_bf16(a):
    """RNE float32 -> bf16 bit patterns (uint16), NaN -> 0x7FC0 (types/bfloat16.h:186-213)."""
    a = np.ascontiguousarray(a, dtype=np.float32)
    u = a.view(np.uint32).astype(np.uint64)
    lsb = (u >> 16) & 1
    r = ((u + 0x7FFF + lsb) >> 16).astype(np.uint16)
    r[np.isnan(a)] = 0x7FC0
    return r


def bf16_to_f32(h):
    return (np.asarray(h, dtype=np.uint16).astype(np.uint32) << 16).view(np.float32)


def shape_info(a, dtype=None, order=None):
    """Reference descriptor int64[2*rank+4] for a numpy view (helpers/shape.h:76-104)."""
    dt = dtype if dtype is not None else _NP2DT[a.dtype]
    r = a.ndim
    if r == 0:
        return np.array([0, 0, 1, DT_FLAG[dt], 1, 99], dtype=np.int64)
    strides = [s // a.itemsize for s in a.strides]
    if order is None:
        order = 'c' if a.flags['C_CONTIGUOUS'] or not a.flags['F_CONTIGUOUS'] else 'f'
    dense = a.flags['C_CONTIGUOUS'] or a.flags['F_CONTIGUOUS']
    return np.array([r, *a.shape, *strides, DT_FLAG[dt], 1 if dense else 0, ord(order)], dtype=np.int64)


def _p(a):
    return ctypes.c_void_p(a.ctypes.data) if a is not None else None


def _s(si):
    return si.ctypes.data_as(ctypes.POINTER(ctypes.c_int64)) if si is not None else None


class Arr:
    """numpy view + dtype code (bf16 lives in uint16 storage)."""

    def __init__(self, a, dtype=None):
        self.a = a
        self.dt = dtype if dtype is not None else _NP2DT[a.dtype]
        self.si = shape_info(a, self.dt)


def _arr(a):
    return a if isinstance(a, Arr) else Arr(a)


def _check(rc, what):
    if rc != 0:
        raise ValueError("oracle %s: unsupported arguments (code %d)" % (what, rc))


def _dims(dims):
    d = np.asarray([] if dims is None else dims, dtype=np.int64).reshape(-1)
    return d, len(d)


def hash_name(name):
    return lib().orc_hash(name.encode())


def offset(si, i):
    return lib().orc_offset(_s(si), i)


def tad(a, dims):
    a = _arr(a)
    d, n = _dims(dims)
    tsi = np.zeros(2 * max(a.a.ndim, 1) + 4, dtype=np.int64)
    cnt = lib().orc_tad(_s(a.si), _s(d), n, _s(tsi), None)
    offs = np.zeros(max(cnt, 1), dtype=np.int64)
    lib().orc_tad(_s(a.si), _s(d), n, _s(tsi), _s(offs))
    rank = int(tsi[0])
    return tsi[: (6 if rank == 0 else 2 * rank + 4)], offs[:cnt]


def pairwise(op, x, y, z):
    x, y, z = _arr(x), _arr(y), _arr(z)
    _check(lib().orc_pairwise(op, _p(x.a), _s(x.si), _p(y.a), _s(y.si), _p(z.a), _s(z.si)), "pairwise")
    return z.a


def transform_strict(op, x, z):
    x, z = _arr(x), _arr(z)
    _check(lib().orc_transform_strict(op, _p(x.a), _s(x.si), _p(z.a), _s(z.si)), "transform_strict")
    return z.a


def transform_float(op, x, z):
    x, z = _arr(x), _arr(z)
    _check(lib().orc_transform_float(op, _p(x.a), _s(x.si), _p(z.a), _s(z.si)), "transform_float")
    return z.a


def transform_same(op, x, z):
    x, z = _arr(x), _arr(z)
    _check(lib().orc_transform_same(op, _p(x.a), _s(x.si), _p(z.a), _s(z.si)), "transform_same")
    return z.a


def scalar(op, x, value, z):
    x, z = _arr(x), _arr(z)
    _check(lib().orc_scalar(op, _p(x.a), _s(x.si), float(value), _p(z.a), _s(z.si)), "scalar")
    return z.a


def broadcast(op, x, y, z, dims):
    x, y, z = _arr(x), _arr(y), _arr(z)
    d, n = _dims(dims)
    _check(lib().orc_broadcast(op, _p(x.a), _s(x.si), _p(y.a), _s(y.si), _p(z.a), _s(z.si), _s(d), n), "broadcast")
    return z.a


def transform_bool(op, x, z):
    x, z = _arr(x), _arr(z)
    _check(lib().orc_transform_bool(op, _p(x.a), _s(x.si), _p(z.a), _s(z.si)), "transform_bool")
    return z.a


def summary_stats(op, x, z, dims=None, bias_corrected=False):
    x, z = _arr(x), _arr(z)
    d, n = _dims(dims)
    _check(lib().orc_summary_stats(op, _p(x.a), _s(x.si), _p(z.a), _s(z.si), _s(d), n, int(bias_corrected)), "summary_stats")
    return z.a


def reduce3(op, x, y, z, dims=None):
    x, y, z = _arr(x), _arr(y), _arr(z)
    d, n = _dims(dims)
    _check(lib().orc_reduce3(op, _p(x.a), _s(x.si), _p(y.a), _s(y.si), _p(z.a), _s(z.si), _s(d), n), "reduce3")
    return z.a


def reduce_long(op, x, z, dims=None):
    x, z = _arr(x), _arr(z)
    d, n = _dims(dims)
    _check(lib().orc_reduce_count(op, _p(x.a), _s(x.si), _p(z.a), _s(z.si), _s(d), n), "reduce_long")
    return z.a


def reduce_bool(op, x, z, dims=None):
    x, z = _arr(x), _arr(z)
    d, n = _dims(dims)
    _check(lib().orc_reduce_count(10 + op, _p(x.a), _s(x.si), _p(z.a), _s(z.si), _s(d), n), "reduce_bool")
    return z.a


def _reduce(fn, name, op, x, z, dims):
    x, z = _arr(x), _arr(z)
    d, n = _dims(dims)
    _check(fn(op, _p(x.a), _s(x.si), _p(z.a), _s(z.si), _s(d), n), name)
    return z.a


def reduce_same(op, x, z, dims=None):
    return _reduce(lib().orc_reduce_same, "reduce_same", op, x, z, dims)


def reduce_float(op, x, z, dims=None):
    return _reduce(lib().orc_reduce_float, "reduce_float", op, x, z, dims)


def reduce_of_empty(table, op, x_dtype, z_dtype):
    """What every element of Z holds after a reduction of an EMPTY X: the op's starting value
    (loops/cpu/reduce/reduce_same.hpp:47,166-176; reduce_float.hpp:103-106,243-251; reduce_long.hpp:50-53,212-217;
    reduce_bool.hpp:45-48; indexreduce.hpp:106-113 with ops/op_macros_index_reduce.h:46-51 and ops.h:2079-2085,2123-2129).
    table: "same", "float", "long", "bool", "index".  Starting values: Sum / ASum 0, Prod 1 (ops.h:2363-2364,1170), Max / Min
    -+infOrMax<X> (ops.h:2365-2368) where infOrMax is infinity for float and double only and the largest finite value for
    every other type, float16 (65504) and bfloat16 included (array/DataTypeUtils.h:588-617); Mean nanOrZero<Z>, NaN for float
    and double only (reduce_float.hpp:244-246, DataTypeUtils.h:619-636); every other ReduceFloat op 0; counts 0; Any 0, All 1
    (ops.h:1200-1215), the other ReduceBool ops 0; IndexMax / IndexMin ... index 0, FirstIndex / LastIndex -1.
    AMax / AMin (ops.h:1225-1243) and the summary statistics start from x[0], which does not exist: None.
    x_dtype / z_dtype: numpy dtypes, or the strings "bfloat16" / "float16"."""
    xk, zk = str(x_dtype), str(z_dtype)

    def largest(kind):
        if kind in ("float32", "float64"):
            return np.inf
        if kind == "float16":
            return 65504.0
        if kind == "bfloat16":
            return float(bf16_to_f32(np.array([0x7F7F], np.uint16))[0])
        if kind == "bool":
            return 1
        return np.iinfo(np.dtype(kind)).max

    if table == "same":
        if op in (0, 4):
            return 0
        if op == 3:
            return 1
        if op == 1:
            return -largest(xk)
        if op == 2:
            return largest(xk)
        return None
    if table == "float":
        if op == 0:
            return np.nan if zk in ("float32", "float64") else 0.0
        return 0.0
    if table == "long":
        return 0
    if table == "bool":
        return 1 if op == 1 else 0
    if table == "index":
        return -1 if op in (4, 5) else 0
    raise ValueError(table)


def matmul_int(x, y, z=None, alpha=1.0, beta=0.0):
    """matmul of integer arrays: the reference's plain loop in the arrays' own type (helpers/cpu/MmulHelper.cpp:35-110:
    val += A * B in T3, then alphaZ * val (+ betaZ * C) with alpha and beta cast to T3).  numpy's integer matmul wraps
    around the same way; 32-bit arrays are widened first and narrowed at the end, which gives the same residues."""
    x, y = np.asarray(x), np.asarray(y)
    assert x.dtype == y.dtype and x.dtype in (np.int32, np.int64)
    with np.errstate(over="ignore"):
        v = np.matmul(x.astype(np.int64), y.astype(np.int64))
        out = np.int64(int(alpha)) * v
        if beta:
            out = out + np.int64(int(beta)) * np.asarray(z).astype(np.int64)
    return out.astype(x.dtype)


def index_reduce(op, x, z, dims=None):
    return _reduce(lib().orc_index_reduce, "index_reduce", op, x, z, dims)


def top_k(x, values, indices, k, need_sort=True):
    x, values, indices = _arr(x), _arr(values), _arr(indices)
    _check(lib().orc_top_k(_p(x.a), _s(x.si), _p(values.a), _s(values.si), _p(indices.a), _s(indices.si), int(k), int(need_sort)), "top_k")
    return values.a, indices.a


def softmax(x, z, dim=-1, literal_half=False):
    x, z = _arr(x), _arr(z)
    _check(lib().orc_softmax(_p(x.a), _s(x.si), _p(z.a), _s(z.si), dim, int(literal_half)), "softmax")
    return z.a


def layer_norm(x, gain, bias, z, axes, channels_first=True):
    x, gain, z = _arr(x), _arr(gain), _arr(z)
    bias = _arr(bias) if bias is not None else None
    d, n = _dims(axes)
    _check(lib().orc_layer_norm(_p(x.a), _s(x.si), _p(gain.a), _s(gain.si), _p(bias.a) if bias else None,
                                _s(bias.si) if bias else None, _p(z.a), _s(z.si), _s(d), n, int(channels_first)),
           "layer_norm")
    return z.a


def matmul(x, y, z, trans_x=False, trans_y=False, trans_z=False, alpha=1.0, beta=0.0, accumulate=1):
    x, y, z = _arr(x), _arr(y), _arr(z)
    _check(lib().orc_matmul(_p(x.a), _s(x.si), _p(y.a), _s(y.si), _p(z.a), _s(z.si), int(trans_x), int(trans_y),
                            int(trans_z), alpha, beta, accumulate), "matmul")
    return z.a


def attention_v2(q, v, k, out, weights=None, logits=None, scale=1.0, causal=False, q_mask=None, v_mask=None):
    q, v, k, out = _arr(q), _arr(v), _arr(k), _arr(out)
    w = _arr(weights) if weights is not None else None
    lg = _arr(logits) if logits is not None else None
    qm = _arr(q_mask) if q_mask is not None else None
    vm = _arr(v_mask) if v_mask is not None else None
    _check(lib().orc_attention_v2(_p(q.a), _s(q.si), _p(v.a), _s(v.si), _p(k.a), _s(k.si), _p(out.a), _s(out.si),
                                  _p(w.a) if w else None, _s(w.si) if w else None, _p(lg.a) if lg else None,
                                  _s(lg.si) if lg else None, scale, int(causal), _p(qm.a) if qm else None, _s(qm.si) if qm else None,
                                  _p(vm.a) if vm else None, _s(vm.si) if vm else None), "attention_v2")
    return out.a


def add_row_vector(x, row, z):
    x, row, z = _arr(x), _arr(row), _arr(z)
    _check(lib().orc_add_row_vector(_p(x.a), _s(x.si), _p(row.a), _s(row.si), _p(z.a), _s(z.si)), "add_row_vector")
    return z.a


def set_threads(n):
    lib().orc_set_threads(n)


def get_threads():
    return lib().orc_get_threads()


# ---- shape ops: numpy restatements (index work, bit-exact) ------------------------------------------------------------
def permute(x, perm=None):
    """permute / transpose (generic/shape/permute.cpp:35-63, transpose.cpp:33-77): dense copy of the permuted view;
    no permutation = reversed axes."""
    return np.ascontiguousarray(np.transpose(x, perm if perm else None))


def reshape(x, shape, order="c"):
    """reshape (generic/shape/reshape.cpp:33-71): the element sequence in `order` is kept; one -1 is inferred."""
    return np.reshape(x, shape, order=order.upper())


def squeeze(x, axes=None):
    """squeeze (generic/shape/squeeze.cpp:32-78): unit axes dropped -- all of them, or the listed ones that are unit."""
    if x.ndim == 0 or (x.ndim == 1 and x.size == 1):
        return x.reshape(())
    axes = [a + x.ndim if a < 0 else a for a in (axes or [])]
    keep = [s for d, s in enumerate(x.shape) if not (s == 1 and (not axes or d in axes))]
    return x.reshape(keep)


def expand_dims(x, axis):
    """expand_dims (generic/shape/expand_dims.cpp:32-50,56-98)."""
    if x.size == 1 and x.ndim <= 1:
        return x.reshape((1,) if x.ndim < 1 else (1, 1))
    return np.expand_dims(x, axis + x.ndim + 1 if axis < 0 else axis)


def split(x, num_splits, axis=0):
    """split (generic/transforms/split.cpp:32-72): equal parts along the axis."""
    return [np.ascontiguousarray(p) for p in np.split(x, num_splits, axis=axis)]


def strided_slice(x, begin, end, strides, begin_mask=0, ellipsis_mask=0, end_mask=0, new_axis_mask=0, shrink_axis_mask=0):
    """strided_slice (generic/tensor/strided_slice.cpp:135-370): every written index becomes one numpy index term --
    Ellipsis, a new axis, an integer (shrink) or a slice whose masked ends are left open -- and numpy's own slicing rules
    (the ones the op's canonical/clamp arithmetic encodes) do the rest."""
    idx = []
    for i in range(len(strides)):
        bit = 1 << i
        if ellipsis_mask & bit:
            idx.append(Ellipsis)
        elif new_axis_mask & bit:
            idx.append(np.newaxis)
        elif shrink_axis_mask & bit:
            idx.append(int(begin[i]))
        else:
            idx.append(slice(None if begin_mask & bit else int(begin[i]), None if end_mask & bit else int(end[i]), int(strides[i])))
    return np.ascontiguousarray(np.asarray(x)[tuple(idx)])


# ---- gradient ops: numpy restatements of the reference's array-op compositions ------------------------------------------
# Arrays are float32 or float64 numpy arrays; every intermediate keeps the array dtype, as the reference's
# temporaries do.  16-bit inputs are widened by the caller and the result rounded once.
def softmax_bp(grad_o, softmaxed, dim=-1):
    """softmax_bp (generic/nn/softmax.cpp:53-95): gradI = s * (gradO - sum_dim(s * gradO))."""
    s = softmaxed
    summed = np.sum(s * grad_o, axis=dim, keepdims=True, dtype=s.dtype)
    return s * (grad_o - summed)


def standardize(x, axes):
    """standardize (generic/transforms/standardize.cpp:34-78): (x - mean) / sqrt(population variance + 1e-5)."""
    axes = tuple(int(a) for a in axes)
    mean = np.mean(x, axis=axes, keepdims=True, dtype=x.dtype)
    var = np.var(x.astype(np.float64), axis=axes, keepdims=True).astype(x.dtype)   # Welford in double, stored as T
    return (x - mean) / np.sqrt(var + x.dtype.type(1e-5))


def standardize_bp(x, eps, axes):
    """standardize_bp (standardize.cpp:84-154) with reduce_mean_bp (gradO / N spread over the group) and
    reduce_stdev_bp (generic/reduce/reduceStDev.cpp:109-177: gradO * divide_no_nan(x - mean, stdev * N)); the
    standard deviation carries no epsilon here; NaN results become 0."""
    axes = tuple(int(a) for a in axes)
    n = 1
    for a in axes:
        n *= x.shape[a]
    T = x.dtype.type
    with np.errstate(all="ignore"):
        mean = np.mean(x, axis=axes, keepdims=True, dtype=x.dtype)
        stdev = np.std(x.astype(np.float64), axis=axes, keepdims=True).astype(x.dtype)
        out = eps / stdev
        dldu_sum = -np.sum(out, axis=axes, keepdims=True, dtype=x.dtype)
        out = out + dldu_sum / T(n)
        tmp = (mean - x) * eps / (stdev * stdev)
        dlds_sum = np.sum(tmp, axis=axes, keepdims=True, dtype=x.dtype)
        denom = np.broadcast_to(stdev * T(n), x.shape)
        ratio = np.where(denom == 0, T(0), (x - mean) / np.where(denom == 0, T(1), denom))
        out = out + ratio * dlds_sum
    return np.where(np.isnan(out), T(0), out).astype(x.dtype)


def layer_norm_bp(x, gain, eps, axes, channels_first=True, with_bias=True):
    """layer_norm_bp (generic/nn/layer_norm.cpp:85-157): returns (dLdx, dLdg, dLdb or None)."""
    dim_c = 1 if channels_first else x.ndim - 1
    others = tuple(d for d in range(x.ndim) if d != dim_c)
    dldb = np.sum(eps, axis=others, dtype=x.dtype) if with_bias else None
    dldg = np.sum(standardize(x, axes) * eps, axis=others, dtype=x.dtype)
    bshape = [1] * x.ndim
    bshape[dim_c] = x.shape[dim_c]
    dldx = standardize_bp(x, eps * gain.reshape(bshape), axes)
    return dldx, dldg, dldb


def matmul_bp(x, y, eps, trans_x=False, trans_y=False, trans_z=False, alpha=1.0, beta=0.0):
    """matmul_bp (generic/blas/matmul.cpp:239-332), non-scalar eps: dLdx = matmul(eps, y; transZ, !transY, transX),
    dLdy = matmul(x, eps; !transX, transZ, transY); each through the matmul restatement above."""
    dldx = np.zeros_like(x)
    dldy = np.zeros_like(y)
    matmul(eps, y, dldx, bool(trans_z), not trans_y, bool(trans_x), alpha, beta)
    matmul(x, eps, dldy, not trans_x, bool(trans_z), bool(trans_y), alpha, beta)
    return dldx, dldy


def clip_by_value(x, left, right):
    """clipbyvalue / legacy ClipByValue (helpers/cpu/clip.cpp:211-219, ops/ops.h:412-415): the upper bound is tested first,
    comparisons against the bounds as given, NaN passes through."""
    x = np.asarray(x)
    return np.where(x > right, np.asarray(right, x.dtype), np.where(x < left, np.asarray(left, x.dtype), x)).astype(x.dtype)


def affine(x, a, b):
    """legacy Affine (ops/ops.h:453): a * x + b in the array type."""
    x = np.asarray(x)
    return (x.dtype.type(a) * x + x.dtype.type(b)).astype(x.dtype)


def scaled_tanh(x, a, b):
    """legacy ScaledTanh (ops/ops.h:1088-1090): a * tanh(b * x) in the array type."""
    x = np.asarray(x)
    return (x.dtype.type(a) * np.tanh(x.dtype.type(b) * x)).astype(x.dtype)


def stabilize(x, k):
    """legacy Stabilize (ops/ops.h:458-468, system/common.h:164-165): where x * k leaves +-3.79297773665 the value becomes
    that cutoff divided by k."""
    x = np.asarray(x)
    t = x.dtype.type
    cut = t(np.float32(3.79297773665))
    with np.errstate(invalid="ignore"):
        return np.where(x * t(k) > cut, cut / t(k), np.where(x * t(k) < -cut, -cut / t(k), x)).astype(x.dtype)


def set_range(x, lo, hi):
    """legacy SetRange (ops/ops.h:427-438): values inside [lo, hi] stay; others become floor(v * (hi - lo)) + lo, with
    v = sigmoid(x) when the range is [0, 1] and v = x otherwise."""
    x = np.asarray(x)
    t = x.dtype.type
    lo, hi = t(lo), t(hi)
    with np.errstate(over="ignore", invalid="ignore"):
        v = t(1) / (t(1) + np.exp(-x)) if (lo == 0 and hi == 1) else x
        return np.where((x >= lo) & (x <= hi), x, np.floor(v * (hi - lo)) + lo).astype(x.dtype)


def log_softmax(x, dim=-1):
    """log_softmax (generic/nn/logSoftmax.cpp:34-49 -> helpers/cpu/activations.cpp:100-145,236-256): max, exp(x - max), sum,
    divide, log -- in that order, in the array type (so a term that underflows in exp comes out as -inf).  A vector
    ([n], [1, n] or [n, 1]) is normalised whole unless `dim` names its unit axis, which gives zeros."""
    x = np.asarray(x)
    if dim < 0:
        dim += max(x.ndim, 1)
    is_vector = x.ndim == 1 or (x.ndim == 2 and 1 in x.shape)
    with np.errstate(divide="ignore"):
        if x.ndim == 0:
            return np.zeros_like(x)
        if is_vector:
            if x.ndim == 1 or x.shape[dim] != 1:
                e = np.exp(x - x.max())
                return np.log(e / e.sum(dtype=x.dtype))
            return np.zeros_like(x)
        e = np.exp(x - x.max(axis=dim, keepdims=True))
        return np.log(e / e.sum(axis=dim, keepdims=True, dtype=x.dtype))


# ---- ops built on a match condition read from the extra parameters (numpy restatements) -----------------------------------
def _in_type(a, like):
    """Round a float64 value / array through the dtype of `like` (comparisons run in the array's own type)."""
    return np.asarray(a).astype(like.dtype)


def match_mask(x, compare, eps, mode):
    """MatchConditionBool (ops/ops.h:1800-1845): the sixteen modes of Conditions.ConditionMode, evaluated in x's type."""
    x = np.asarray(x)
    c, e = _in_type(compare, x), _in_type(eps, x)
    with np.errstate(invalid="ignore"):
        diff = np.abs((x - c).astype(x.dtype))
        inf, nan = np.isinf(x) if x.dtype.kind == "f" else np.zeros(x.shape, bool), np.isnan(x) if x.dtype.kind == "f" else np.zeros(x.shape, bool)
        table = {0: lambda: diff <= e, 1: lambda: diff > e, 2: lambda: x < c, 3: lambda: x > c, 4: lambda: x <= c, 5: lambda: x >= c,
                 6: lambda: np.abs(x) < c, 7: lambda: np.abs(x) > c, 8: lambda: inf, 9: lambda: nan, 10: lambda: x == c, 11: lambda: x != c,
                 12: lambda: np.abs(x) >= c, 13: lambda: np.abs(x) <= c, 14: lambda: ~(inf | nan), 15: lambda: inf | nan}
        return np.asarray(table[int(mode)](), dtype=bool)


def compare_and_set_transform(x, compare, set_value, eps, mode):
    """TransformSame 13 (ops.h:845-940): z = cond(x) ? set : x."""
    x = np.asarray(x)
    return np.where(match_mask(x, compare, eps, mode), _in_type(set_value, x), x)


def compare_and_set(x, y, compare, eps, mode):
    """Pairwise 12 / Scalar 33 (ops.h:719-840): the SECOND operand is tested and taken: z = cond(y) ? y : x."""
    x = np.asarray(x)
    y = np.broadcast_to(np.asarray(y, dtype=x.dtype), x.shape)
    return np.where(match_mask(y, compare, eps, mode), y, x)


def compare_and_replace(x, y, compare, eps, mode):
    """Pairwise 13 (ops.h:593-715): z = cond(x) ? y : x."""
    x = np.asarray(x)
    return np.where(match_mask(x, compare, eps, mode), np.asarray(y, dtype=x.dtype), x)


def _along(x, dims):
    x = np.asarray(x)
    if dims is None or len(dims) == 0:
        return x.reshape(1, -1), ()
    dims = sorted(d + x.ndim if d < 0 else d for d in dims)
    keep = [d for d in range(x.ndim) if d not in dims]
    t = np.transpose(x, keep + dims)
    out_shape = tuple(x.shape[d] for d in keep)
    return t.reshape(int(np.prod(out_shape)) if out_shape else 1, -1), out_shape


def match_count(x, compare, eps, mode, dims=None):
    """ReduceLong 2 MatchCondition (ops.h:2430-2500): how many elements of each sub-array meet the condition."""
    rows, shape = _along(x, dims)
    return match_mask(rows, compare, eps, mode).sum(1).astype(np.int64).reshape(shape)


def first_last_index(x, compare, eps, mode, dims=None, last=False):
    """IndexReduce 4 / 5 (ops.h:2061-2150): position (row-major inside the sub-array) of the first / last element that meets
    the condition, -1 when none does."""
    rows, shape = _along(x, dims)
    m = match_mask(rows, compare, eps, mode)
    n = m.shape[1]
    idx = np.where(m.any(1), (n - 1 - m[:, ::-1].argmax(1)) if last else m.argmax(1), -1)
    return idx.astype(np.int64).reshape(shape)


def norm_p(x, p, dims=None):
    """ReduceFloat 6 NormP (ops.h:1280-1286): (sum |x|^p)^(1/p)."""
    rows, shape = _along(np.asarray(x, dtype=np.float64), dims)
    return ((np.abs(rows) ** p).sum(1) ** (1.0 / p)).reshape(shape)


def equals_with_eps(x, y, eps, dims=None):
    """Reduce3 4 EqualsWithEps (op_macros_special.h:449-480, templatemath.h:115): 1 when |x - y| <= eps for every pair."""
    rx, shape = _along(np.asarray(x, dtype=np.float64), dims)
    ry, _ = _along(np.asarray(y, dtype=np.float64), dims)
    return (np.abs(rx - ry) <= eps).all(1).astype(np.float64).reshape(shape)


# ---- the remaining pairwise / scalar ops (numpy restatements, arithmetic in the array's type) --------------------------------
def relative_error(x, y):
    """sd_re (math/templatemath.h:1144-1153): |x - y| / (|x| + |y|), 0 where both are 0.  Pairwise 24 RelativeError."""
    x = np.asarray(x)
    y = np.asarray(y, dtype=x.dtype)
    with np.errstate(invalid="ignore", divide="ignore"):
        r = (np.abs(x - y) / (np.abs(x) + np.abs(y))).astype(x.dtype)
    return np.where((x == 0) & (y == 0), x.dtype.type(0), r)


def binary_relative_error(x, y, threshold):
    """Pairwise 25 (ops/ops.h:2218-2270): 1 where the relative error exceeds the threshold."""
    x = np.asarray(x)
    return (relative_error(x, y) > _in_type(threshold, x)).astype(x.dtype)


def binary_min_abs_relative_error(x, y, rel, absolute):
    """Pairwise 26 (ops/ops.h:2274-2340): 1 where the relative error exceeds `rel` and |x - y| is not below `absolute`."""
    x = np.asarray(x)
    y = np.asarray(y, dtype=x.dtype)
    return ((relative_error(x, y) > _in_type(rel, x)) & ~(np.abs(x - y) < _in_type(absolute, x))).astype(x.dtype)


def axpy(x, y, alpha):
    """Pairwise 10 (ops/ops.h:328-333): alpha * x + y."""
    x = np.asarray(x)
    return (_in_type(alpha, x) * x + np.asarray(y, dtype=x.dtype)).astype(x.dtype)


def pow_derivative(x, y):
    """Pairwise 31 / Scalar 32 (ops/ops.h:82-87): y * x^(y - 1)."""
    x = np.asarray(x)
    y = np.broadcast_to(np.asarray(y, dtype=x.dtype), x.shape)
    with np.errstate(all="ignore"):
        return (y * np.power(x, y - x.dtype.type(1))).astype(x.dtype)


def log_poisson_loss(x, y, full=False):
    """Pairwise 32 / 33 (ops/ops.h:2389-2394, 1494-1502): exp(y) - x y, `full` adds Stirling's x log x - x + log(2 pi x) / 2."""
    x = np.asarray(x)
    y = np.asarray(y, dtype=x.dtype)
    with np.errstate(all="ignore"):
        r = np.exp(y) - x * y
        if full:
            r = r + (x * np.log(x) - x + x.dtype.type(0.5) * np.log(x.dtype.type(2.0 * np.pi) * x))
    return r.astype(x.dtype)


def igamma(a, x, complement=False):
    """sd_igamma / sd_igammac (math/templatemath.h:963-991): the regularised lower incomplete gamma function summed as
    x^a e^-x / Gamma(a) * sum_i x^i / (a (a+1) .. (a+i)), the series cut off once the running denominator passes 1e12;
    0 where a <= 1e-6.  Evaluated in the array's type (float for float32, double for float64)."""
    import math
    a = np.asarray(a)
    dt = a.dtype.type
    x = np.broadcast_to(np.asarray(x, dtype=a.dtype), a.shape)
    out = np.zeros(a.shape, a.dtype)
    for idx in np.ndindex(a.shape):
        av, xv = dt(a[idx]), dt(x[idx])
        if av <= dt(0.000001):
            r = dt(0)
        else:
            with np.errstate(all="ignore"):
                aim = dt(np.power(xv, av) / (np.exp(xv) * dt(math.gamma(float(av)))))
                s, denom, xi, i = dt(0), dt(1), dt(1), 0
                while dt(1) / denom > dt(1.0e-12) and i < 4096:
                    denom = dt(denom * dt(av + dt(i)))
                    s = dt(s + xi / denom)
                    xi = dt(xi * xv)
                    i += 1
                r = dt(aim * s)
        out[idx] = dt(1) - r if complement else r
    return out


# ---- the bool tables: pairwise / scalar / broadcast ops with a BOOL result (numpy restatements) -------------------------------
def bool_table(op, x, y, params=None, bf16=False):
    """z = op(x, y, extraParams) for the members of BROADCAST_BOOL_OPS / SCALAR_BOOL_OPS / PAIRWISE_BOOL_OPS
    (loops/legacy_ops.h:30-32, 74-76, 117-119); every loop of the three families calls the functor's three-argument form
    (loops/cpu/pairwise_bool.cpp:73-143, scalar_bool.cpp:77-138, broadcasting_bool.hpp:91-325).  x and y are numpy arrays
    of one dtype and one shape (see operand_along / scalars_along for the operand shapes of the other families); with
    bf16=True they are float32 arrays holding bfloat16 values and differences are rounded to bfloat16.
    0 EqualTo, 1 GreaterThan, 2 LessThan, 4 GreaterThanOrEqual, 6 NotEqualTo, 11 LessThanOrEqual: ops.h:181-186 (x OP y).
    3 Epsilon (ops.h:1755-1790): |x - y| <= params[0] when parameters are given, else (also) |x - y| <= X(1e-5); all true for BOOL.
    7 And / 8 Or / 9 Xor (ops.h:1051-1063, 1896-1925): with parameters on "differs from params[0]", without on bool(x), bool(y).
    10 Not (ops.h:1927-1932): the three-argument form is x != y."""
    x, y = np.asarray(x), np.asarray(y)
    assert x.dtype == y.dtype and x.shape == y.shape
    op = int(op)
    with np.errstate(invalid="ignore", over="ignore"):
        if op in (0, 1, 2, 4, 6, 10, 11):
            return {0: x == y, 1: x > y, 2: x < y, 4: x >= y, 6: x != y, 10: x != y, 11: x <= y}[op]
        if op == 3:
            if x.dtype == np.bool_:
                # X = bool: the difference and both tolerances are held as bool, static_cast<bool>(1e-5) is true, and
                # "absDiff <= true" holds for either value of absDiff: every pair matches
                return np.ones(x.shape, np.bool_)
            if bf16:
                diff = bf16_to_f32(f32_to_bf16((x - y).astype(np.float32)))
                tol = bf16_to_f32(f32_to_bf16(np.array([1e-5], np.float32)))[0]
            else:
                diff = (x - y).astype(x.dtype)
                tol = np.array(1e-5).astype(x.dtype)          # static_cast<X>(1e-5): 0 for the integer types
            ad = np.abs(diff)
            hit = ad <= tol
            if params is not None:
                p0 = np.float32(params[0]) if bf16 else np.array(params[0]).astype(x.dtype)
                hit = hit | (ad <= p0)
            return hit
        if params is not None:
            c = np.float32(params[0]) if bf16 else np.array(params[0]).astype(x.dtype)
            a, b = x != c, y != c
            if op == 9:                                       # exactly one of the two equals the parameter
                a, b = x == c, y == c
                return a != b
        else:
            a, b = x != 0, y != 0                             # static_cast<bool>: NaN counts as true
            if op == 9:
                return a != b
        return {7: a & b, 8: a | b}[op]


def operand_along(y, x_shape, dims):
    """The second operand of the broadcast loops seen with x's shape: y's non-unit dims line up with `dims` of x
    (loops/cpu/broadcasting_bool.hpp:60-120: one sub-array of x along `dims` per pass, y walked alongside it)."""
    y = np.asarray(y)
    dims = sorted(d + len(x_shape) if d < 0 else d for d in dims)
    yshape = [s for s in y.shape if s != 1]
    full = [1] * len(x_shape)
    it = iter(yshape)
    for d in dims:
        if x_shape[d] != 1:
            full[d] = next(it)
    return np.broadcast_to(y.reshape(full), x_shape)


def scalars_along(s, x_shape, dims):
    """One scalar per sub-array of x along `dims`, the sub-arrays numbered in c order over x's other dims
    (loops/cpu/scalar.hpp:37-80, scalar_bool.cpp:37-80), seen with x's shape."""
    s = np.asarray(s).reshape(-1)
    dims = sorted(d + len(x_shape) if d < 0 else d for d in dims)
    other = [d for d in range(len(x_shape)) if d not in dims]
    full = [x_shape[d] if d in other else 1 for d in range(len(x_shape))]
    assert s.size == int(np.prod([x_shape[d] for d in other])) if other else s.size == 1
    return np.broadcast_to(s.reshape(full), x_shape)


def reduce3_all(op, x, y, dims):
    """execReduce3All (loops/cpu/reduce3.hpp execAll; legacy/NativeOps.h:208): z[i][j] = reduce3(op, x's sub-array i, y's
    sub-array j), the sub-arrays taken along `dims` and numbered in c order over the other dims.  The pairing is restated
    here; each pair goes through the oracle's reduce3."""
    x, y = np.asarray(x), np.asarray(y)
    dims = sorted(d + x.ndim if d < 0 else d for d in dims)
    other = [d for d in range(x.ndim) if d not in dims]
    xt = np.transpose(x, other + dims).reshape((-1,) + tuple(x.shape[d] for d in dims))
    yt = np.transpose(y, other + dims).reshape((-1,) + tuple(y.shape[d] for d in dims))
    z = np.zeros((xt.shape[0], yt.shape[0]), x.dtype)
    for i in range(xt.shape[0]):
        for j in range(yt.shape[0]):
            z[i, j] = reduce3(op, np.ascontiguousarray(xt[i]), np.ascontiguousarray(yt[j]), np.zeros((), x.dtype))
    return z
