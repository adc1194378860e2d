"""Host-side op executioner: the stand-in for the Java `NativeOpExecutioner` / `CudaExecutioner`.

Follows the call protocol of
nd4j/nd4j-backends/nd4j-backend-impls/nd4j-cpu-backend-common/src/main/java/org/nd4j/linalg/cpu/nativecpu/ops/NativeOpExecutioner.java:
  * legacy ops: allocate z when it is not given (:676), pass array handles, poll lastErrorCode() after
    the call (:194, :440, :715);
  * index accumulations produce INT64 (:157); reduce "same" keeps the input type, reduce "float" of a
    float input keeps it too (:304-305);
  * custom ops: build an OpContext, ask calculateOutputShapes2 for the output shapes when outputs are
    not supplied, push arrays and T/I/B/D arguments, call execCustomOp2 and turn a non-zero status into
    an exception carrying lastErrorMessage() (:1001-1091).
"""
import ctypes

import numpy as np

from . import nativeops as N
from .ndarray import BOOL, DOUBLE, FLOAT32, HALF, BFLOAT16, INT32, INT64, NDArray  # noqa: F401


# opNum tables: libnd4j/include/loops/legacy_ops.h
class Pairwise:
    Add, CopyPws, Divide, Multiply, Pow, ReverseSubtract, Subtract, MaxPairwise, MinPairwise, Copy2 = 0, 1, 2, 3, 4, 5, 6, 7, 8, 9
    ReverseDivide, Remainder, FMod, Atan2, TruncateDiv, FloorDiv, FloorMod, SquaredSubtract = 11, 14, 15, 16, 17, 18, 19, 20
    ReverseMod, SafeDivide, Mod, LogicalOr, LogicalXor, LogicalNot, LogicalAnd = 21, 22, 23, 27, 28, 29, 30
    AMaxPairwise, AMinPairwise, TruncateMod, ReplaceNans, DivideNoNan = 34, 35, 36, 37, 38
    CompareAndSet, CompareAndReplace = 12, 13   # extraArgs [compare, set, eps, mode]
    Axpy, RelativeError, BinaryRelativeError, BinaryMinimumAbsoluteRelativeError = 10, 24, 25, 26   # extraArgs [alpha] / - / [threshold] / [relative, absolute]
    PowDerivative, LogPoissonLoss, LogPoissonLossFull, IGamma, IGammac = 31, 32, 33, 39, 40


class TransformStrict:
    Cosine, Exp, Log, Sigmoid, Sin, SoftPlus, Tanh, Swish, Erf, GELU, PreciseGELU = 22, 23, 24, 26, 27, 28, 29, 43, 45, 53, 55
    TanhDerivative, SigmoidDerivative, SoftSignDerivative, TanDerivative, SELUDerivative = 4, 6, 7, 8, 9
    RationalTanhDerivative, RectifiedTanhDerivative, SwishDerivative, ACoshDerivative, ASinhDerivative = 11, 12, 13, 14, 15
    SinhDerivative, LogSigmoidDerivative, SpecialDerivative, CubeDerivative = 16, 17, 18, 21
    HardTanhDerivative, HardSigmoidDerivative, StabilizeFP16 = 5, 10, 20   # the first two return their input (ops/ops.h:222-226)
    ACos, ASin, ATan, HardTanh, SoftSign, HardSigmoid, RationalTanh, RectifiedTanh, Sinh, Cosh, Tan, SELU = 30, 31, 32, 33, 34, 36, 37, 38, 39, 40, 41, 42
    Log1p, ACosh, ASinh, Rint, LogSigmoid, Erfc, Expm1, ATanh, GELUDerivative, PreciseGELUDerivative, Mish, MishDerivative = 44, 46, 47, 48, 49, 50, 51, 52, 54, 56, 57, 58


class TransformFloat:
    Sqrt, RSqrt = 1, 3


class TransformSame:
    Abs, Ones, Neg, Round, TimesOneMinus, Cube, OneMinus, Reciprocal, Square, Identity, Ceiling, Floor, Copy = 0, 2, 3, 4, 5, 6, 7, 11, 12, 15, 17, 18, 21
    CompareAndSetTransform = 13   # extraArgs [compare, set, eps, mode]
    Sign = 1   # as the reference computes it: 1 for every non-zero number, -1 for 0 and NaN (ops/ops.h:217-219)


class ReduceSame:
    Sum, Max, Min, Prod, ASum, AMax, AMin = 0, 1, 2, 3, 4, 5, 6


class ReduceFloat:
    Mean, AMean, Norm1, Norm2, NormMax, NormFrobenius, SquaredNorm, Entropy, LogEntropy, ShannonEntropy = 0, 1, 2, 3, 4, 5, 7, 8, 9, 10
    NormP = 6   # extraArgs [p]


class IndexReduce:
    IndexMax, IndexMin, IndexAbsoluteMax, IndexAbsoluteMin = 0, 1, 2, 3
    FirstIndex, LastIndex = 4, 5   # extraArgs [compare, eps, mode]


class TransformBool:
    IsInf, IsNan, IsFinite, IsInfOrNan, IsPositive, Not, IsNegative = 1, 2, 3, 4, 6, 7, 8
    MatchConditionBool = 5   # extraArgs [compare, eps, mode]


class SummaryStats:
    Variance, StandardDeviation = 0, 1


class Reduce3:
    ManhattanDistance, EuclideanDistance, CosineSimilarity, Dot, CosineDistance, JaccardDistance, SimpleHammingDistance = 0, 1, 2, 3, 5, 6, 7
    EqualsWithEps = 4   # extraArgs [-, -, eps]


class ReduceLong:
    CountNonZero, CountZero = 0, 1
    MatchCondition = 2   # extraArgs [compare, eps, mode]


class ReduceBool:
    Any, All, IsFinite, IsInfOrNan, IsNan, IsInf, IsPositive, IsNegative = 0, 1, 2, 3, 4, 5, 6, 7   # 2-7: true when any element is


class BoolOp:
    """The bool tables of the pairwise / scalar / broadcast families (loops/legacy_ops.h:30-32, 74-76, 117-119)."""
    EqualTo, GreaterThan, LessThan, Epsilon, GreaterThanOrEqual, MatchCondition, NotEqualTo, And, Or, Xor, Not, LessThanOrEqual = range(12)


class Scalar:
    Add, Subtract, Multiply, Divide, ReverseDivide, ReverseSubtract, MaxPairwise, ELU, ELUDerivative = 0, 1, 2, 3, 4, 5, 6, 7, 8
    MinPairwise, CopyPws, Mod, ReverseMod, Remainder, FMod, TruncateDiv, FloorDiv, FloorMod, SquaredSubtract = 13, 14, 15, 16, 17, 18, 19, 20, 21, 22
    SafeDivide, AMaxPairwise, AMinPairwise, Atan2, LogicalOr, LogicalXor, LogicalNot, LogicalAnd, Pow = 23, 24, 25, 26, 27, 28, 29, 30, 31
    SXELogitsSmoother, LeakyRELU, LeakyRELUDerivative, ReplaceNans, LogX, RELU, RELU6, Step, LstmClip = 34, 35, 36, 37, 38, 39, 40, 41, 42
    TruncateMod, SquaredReverseSubtract, ReversePow, DivideNoNan, RELUDerivative = 43, 44, 45, 46, 49
    CompareAndSet = 33   # extraArgs [compare, set, eps, mode]
    PowDerivative, IGamma, IGammac = 32, 47, 48


class Broadcast:
    Add, Subtract, Multiply, Divide, ReverseDivide, ReverseSubtract, CopyPws, Pow = 0, 1, 2, 3, 4, 5, 6, 7
    MinPairwise, MaxPairwise, AMinPairwise, AMaxPairwise, SquaredSubtract, FloorMod, FloorDiv, ReverseMod = 13, 14, 15, 16, 17, 18, 19, 20
    SafeDivide, Mod, TruncateDiv, Atan2, LogicalOr, LogicalXor, LogicalNot, LogicalAnd, DivideNoNan = 21, 22, 23, 26, 27, 28, 29, 30, 31
    IGamma, IGammac, PowDerivative = 32, 33, 34


_FLOAT_TYPES = (HALF, FLOAT32, DOUBLE, BFLOAT16)


def _reduced_shape(shape, dims, keep_dims):
    if dims is None or len(dims) == 0:
        return [1] * len(shape) if keep_dims else []
    r = len(shape)
    dims = sorted(d + r if d < 0 else d for d in dims)
    out = []
    for i, s in enumerate(shape):
        if i in dims:
            if keep_dims:
                out.append(1)
        else:
            out.append(s)
    return out


_DIMS_CACHE = {}


def _dims_array(dims):
    """INT64 host array holding the dimensions (cached: the same few tuples recur on every call)."""
    key = tuple(int(d) for d in dims)
    arr = _DIMS_CACHE.get(key)
    if arr is None:
        arr = NDArray.from_numpy(np.asarray(key, dtype=np.int64))
        _DIMS_CACHE[key] = arr
    return arr


class OpContext:
    """graph::Context wrapper (the Java side's CpuOpContext / CudaOpContext)."""

    def __init__(self):
        self.ptr = N.load().createGraphContext(1)
        self._keep = []

    def set_inputs(self, arrays):
        L = N.load()
        arr = (ctypes.c_void_p * len(arrays))(*[a.handle for a in arrays])
        L.setGraphContextInputArraysArr(self.ptr, len(arrays), arr)
        N.check("setGraphContextInputArraysArr")
        self._keep.append(list(arrays))

    def set_outputs(self, arrays):
        L = N.load()
        for i, a in enumerate(arrays):
            if a is not None:
                L.setGraphContextOutputArray(self.ptr, i, a.handle)
        N.check("setGraphContextOutputArray")
        self._keep.append(list(arrays))

    def set_args(self, t_args=(), i_args=(), b_args=(), d_args=()):
        L = N.load()
        if len(t_args):
            L.setGraphContextTArguments(self.ptr, (ctypes.c_double * len(t_args))(*[float(t) for t in t_args]), len(t_args))
        if len(i_args):
            L.setGraphContextIArguments(self.ptr, (ctypes.c_longlong * len(i_args))(*[int(i) for i in i_args]), len(i_args))
        if len(b_args):
            L.setGraphContextBArguments(self.ptr, (ctypes.c_bool * len(b_args))(*[bool(b) for b in b_args]), len(b_args))
        if len(d_args):
            L.setGraphContextDArguments(self.ptr, (ctypes.c_int * len(d_args))(*[int(d) for d in d_args]), len(d_args))

    def close(self):
        if self.ptr:
            N.load().deleteGraphContext(self.ptr)
            self.ptr = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


class Executioner:
    def __init__(self):
        self.L = N.load()
        self.L.initializeDevicesAndFunctions()
        N.check("initializeDevicesAndFunctions")
        self._hashes = {}
        for item in self.L.getAllCustomOps().decode().split(";"):
            if item:
                parts = item.split(":")
                self._hashes[parts[0]] = int(parts[1])

    # ---- legacy ops ----
    def _extra_params(self, extra_args, dtype):
        """extraArgs of a legacy op as the native side gets them: a buffer of the array's own type, device pointer
        (the Java executioners convert with `op.extraArgsDataBuff(dtype)` and pass the allocator's pointer)."""
        if extra_args is None:
            return None, None
        holder = NDArray.from_numpy(np.asarray(extra_args, np.float64 if dtype == DOUBLE else np.float32), dtype)
        holder.sync_to_device()
        return holder, self.L.dbSpecialBuffer(holder.buffer.ptr)

    def exec_transform_strict(self, op_num, x, z=None, extra_args=None):
        z = z if z is not None else NDArray.empty(x.shape, x.dtype)
        holder, extra = self._extra_params(extra_args, x.dtype)
        self.L.execTransformStrict(None, op_num, x.handle, extra, z.handle)
        N.check("execTransformStrict")
        return z

    def exec_transform_float(self, op_num, x, z=None):
        # the result of a float transform or reduction of an integer / bool array takes the default floating point type, as
        # Op.resultType() gives it on the Java side
        z = z if z is not None else NDArray.empty(x.shape, x.dtype if x.dtype in _FLOAT_TYPES else FLOAT32)
        self.L.execTransformFloat(None, op_num, x.handle, None, z.handle)
        N.check("execTransformFloat")
        return z

    def exec_transform_same(self, op_num, x, z=None, extra_args=None):
        z = z if z is not None else NDArray.empty(x.shape, x.dtype)
        holder, extra = self._extra_params(extra_args, x.dtype)
        self.L.execTransformSame(None, op_num, x.handle, extra, z.handle)
        N.check("execTransformSame")
        return z

    def exec_assign(self, x, z):
        self.L.execTransformAny(None, 0, x.handle, None, z.handle)
        N.check("execTransformAny")
        return z

    def exec_pairwise(self, op_num, x, y, z=None, extra_args=None):
        z = z if z is not None else NDArray.empty(x.shape, x.dtype)
        holder, extra = self._extra_params(extra_args, z.dtype)
        self.L.execPairwiseTransform(None, op_num, x.handle, y.handle, z.handle, extra)
        N.check("execPairwiseTransform")
        return z

    def exec_scalar(self, op_num, x, scalar, z=None, extra_args=None):
        z = z if z is not None else NDArray.empty(x.shape, x.dtype)
        s = scalar if isinstance(scalar, NDArray) else NDArray.scalar(scalar, x.dtype)
        holder, extra = self._extra_params(extra_args, z.dtype)
        self.L.execScalar(None, op_num, x.handle, z.handle, s.handle, extra)
        N.check("execScalar")
        return z

    def exec_broadcast(self, op_num, x, y, dims, z=None):
        z = z if z is not None else NDArray.empty(x.shape, x.dtype)
        d = _dims_array(dims)
        self.L.execBroadcast(None, op_num, x.handle, y.handle, z.handle, None, d.handle)
        N.check("execBroadcast")
        return z

    # ---- the bool tables (loops/legacy_ops.h:30-32, 74-76, 117-119): operands of one type, BOOL result ----
    def exec_pairwise_bool(self, op_num, x, y, z=None, extra_args=None):
        z = z if z is not None else NDArray.empty(x.shape, BOOL)
        holder, extra = self._extra_params(extra_args, x.dtype)
        self.L.execPairwiseTransformBool(None, op_num, x.handle, y.handle, extra, z.handle)
        N.check("execPairwiseTransformBool")
        return z

    def exec_scalar_bool(self, op_num, x, scalar, z=None, extra_args=None):
        z = z if z is not None else NDArray.empty(x.shape, BOOL)
        s = scalar if isinstance(scalar, NDArray) else NDArray.scalar(scalar, x.dtype)
        holder, extra = self._extra_params(extra_args, x.dtype)
        self.L.execScalarBool(None, op_num, x.handle, z.handle, s.handle, extra)
        N.check("execScalarBool")
        return z

    def exec_broadcast_bool(self, op_num, x, y, dims, z=None, extra_args=None):
        z = z if z is not None else NDArray.empty(x.shape, BOOL)
        d = _dims_array(dims)
        holder, extra = self._extra_params(extra_args, x.dtype)
        self.L.execBroadcastBool(None, op_num, x.handle, y.handle, z.handle, extra, d.handle)
        N.check("execBroadcastBool")
        return z

    def exec_scalar_bool_tad(self, op_num, x, scalars, dims, z=None, extra_args=None):
        """One scalar per sub-array of x along `dims`."""
        z = z if z is not None else NDArray.empty(x.shape, BOOL)
        d = _dims_array(dims)
        holder, extra = self._extra_params(extra_args, x.dtype)
        self.L.execScalarBoolTad(None, op_num, x.handle, z.handle, scalars.handle, extra, d.handle)
        N.check("execScalarBoolTad")
        return z

    def exec_scalar_tad(self, op_num, x, scalars, dims, z=None):
        """execScalar with one scalar per sub-array of x along `dims`."""
        z = z if z is not None else NDArray.empty(x.shape, x.dtype)
        d = _dims_array(dims)
        self.L.execScalarTad(None, op_num, x.handle, z.handle, scalars.handle, None, d.handle)
        N.check("execScalarTad")
        return z

    def _reduce(self, scalar_fn, dim_fn, name, op_num, x, dims, keep_dims, z, zdtype, extra_args=None, extra_dtype=None):
        if z is None:
            z = NDArray.empty(_reduced_shape(x.shape, dims, keep_dims), zdtype)
        holder, extra = self._extra_params(extra_args, extra_dtype if extra_dtype is not None else x.dtype)
        if dims is None or len(dims) == 0:
            scalar_fn(None, op_num, x.handle, extra, z.handle)
        else:
            d = _dims_array(dims)
            dim_fn(None, op_num, x.handle, extra, z.handle, d.handle)
        N.check(name)
        return z

    def exec_reduce_same(self, op_num, x, dims=None, keep_dims=False, z=None):
        return self._reduce(self.L.execReduceSame, self.L.execReduceSame2, "execReduceSame", op_num, x, dims, keep_dims, z, x.dtype)

    def exec_reduce_float(self, op_num, x, dims=None, keep_dims=False, z=None, extra_args=None):
        """extra_args reach the native side in Z's type (NormP's exponent)."""
        zdt = z.dtype if z is not None else (x.dtype if x.dtype in _FLOAT_TYPES else FLOAT32)
        return self._reduce(self.L.execReduceFloat, self.L.execReduceFloat2, "execReduceFloat", op_num, x, dims, keep_dims, z, zdt, extra_args, zdt)

    def exec_index_reduce(self, op_num, x, dims=None, keep_dims=False, z=None, extra_args=None):
        return self._reduce(self.L.execIndexReduceScalar, self.L.execIndexReduce, "execIndexReduce", op_num, x, dims, keep_dims, z, INT64, extra_args)

    def exec_transform_bool(self, op_num, x, z=None, extra_args=None):
        if z is None:
            z = NDArray.empty(x.shape, BOOL)
        holder, extra = self._extra_params(extra_args, x.dtype)
        self.L.execTransformBool(None, op_num, x.handle, extra, z.handle)
        N.check("execTransformBool")
        return z

    def exec_summary_stats(self, op_num, x, dims=None, bias_corrected=False, keep_dims=False, z=None):
        if z is None:
            z = NDArray.empty(_reduced_shape(x.shape, dims, keep_dims), x.dtype)
        if dims is None or len(dims) == 0:
            self.L.execSummaryStatsScalar(None, op_num, x.handle, None, z.handle, bool(bias_corrected))
        else:
            self.L.execSummaryStatsTad(None, op_num, x.handle, None, z.handle, _dims_array(dims).handle, bool(bias_corrected))
        N.check("execSummaryStats")
        return z

    def exec_reduce3(self, op_num, x, y, dims=None, keep_dims=False, z=None, extra_args=None):
        if z is None:
            z = NDArray.empty(_reduced_shape(x.shape, dims, keep_dims), x.dtype)
        holder, extra = self._extra_params(extra_args, z.dtype)
        if dims is None or len(dims) == 0:
            self.L.execReduce3Scalar(None, op_num, x.handle, extra, y.handle, z.handle)
        else:
            self.L.execReduce3Tad(None, op_num, x.handle, extra, y.handle, z.handle, _dims_array(dims).handle)
        N.check("execReduce3")
        return z

    def exec_reduce3_all(self, op_num, x, y, dims, z=None, extra_args=None):
        """Every sub-array of x along `dims` against every sub-array of y along them: z [sub-arrays of x, sub-arrays of y]."""
        if z is None:
            nd = [d + len(x.shape) if d < 0 else d for d in dims]
            nx = int(np.prod([s for i, s in enumerate(x.shape) if i not in nd]))
            ny = int(np.prod([s for i, s in enumerate(y.shape) if i not in nd]))
            z = NDArray.empty((nx, ny), x.dtype)
        holder, extra = self._extra_params(extra_args, z.dtype)
        self.L.execReduce3All(None, op_num, x.handle, y.handle, z.handle, _dims_array(dims).handle, extra)
        N.check("execReduce3All")
        return z

    def _reduce_dims_only(self, fn, name, op_num, x, dims, keep_dims, z, zdtype, extra_args=None):
        if z is None:
            z = NDArray.empty(_reduced_shape(x.shape, dims, keep_dims), zdtype)
        d = _dims_array(dims if dims else list(range(len(x.shape))))
        holder, extra = self._extra_params(extra_args, x.dtype)
        fn(None, op_num, x.handle, extra, z.handle, d.handle)
        N.check(name)
        return z

    def exec_reduce_long(self, op_num, x, dims=None, keep_dims=False, z=None, extra_args=None):
        return self._reduce_dims_only(self.L.execReduceLong, "execReduceLong", op_num, x, dims, keep_dims, z, INT64, extra_args)

    def exec_reduce_bool(self, op_num, x, dims=None, keep_dims=False, z=None):
        return self._reduce_dims_only(self.L.execReduceBool, "execReduceBool", op_num, x, dims, keep_dims, z, BOOL)

    # ---- custom ops ----
    def op_hash(self, name):
        if name not in self._hashes:
            raise N.NativeOpsError("custom op '%s' is not registered in nd4j-hip" % name)
        return self._hashes[name]

    def calculate_output_shapes(self, name, inputs, t_args=(), i_args=(), b_args=(), d_args=()):
        ctx = OpContext()
        try:
            ctx.set_inputs(inputs)
            ctx.set_args(t_args, i_args, b_args, d_args)
            sl = self.L.calculateOutputShapes2(None, self.op_hash(name), ctx.ptr)
            N.check("calculateOutputShapes2")
            out = []
            for i in range(self.L.getShapeListSize(sl)):
                p = self.L.getShape(sl, i)
                rank = p[0]
                n = 6 if rank == 0 else 2 * rank + 4
                out.append(np.array([p[j] for j in range(n)], dtype=np.int64))
            self.L.deleteShapeList(sl)
            return out
        finally:
            ctx.close()

    def exec_custom(self, name, inputs, outputs=None, t_args=(), i_args=(), b_args=(), d_args=(), n_outputs=None):
        """Returns the list of output arrays.  `outputs=None` sizes them with calculateOutputShapes2;
        `n_outputs` limits how many of the reported outputs are materialised."""
        from .ndarray import dtype_of_extra
        if outputs is None:
            shapes = self.calculate_output_shapes(name, inputs, t_args, i_args, b_args, d_args)
            if n_outputs is not None:
                shapes = shapes[:n_outputs]
            outputs = []
            for si in shapes:
                rank = int(si[0])
                extra = int(si[3] if rank == 0 else si[2 * rank + 1])
                dt = dtype_of_extra(extra)
                order = chr(int(si[-1]))
                outputs.append(NDArray.empty([int(s) for s in si[1:1 + rank]], dt, order))
        ctx = OpContext()
        try:
            ctx.set_inputs(inputs)
            ctx.set_outputs(outputs)
            ctx.set_args(t_args, i_args, b_args, d_args)
            status = self.L.execCustomOp2(None, self.op_hash(name), ctx.ptr)
            if status != 0:
                raise N.NativeOpsError("Op [%s] execution failed: %s" % (name, self.L.lastErrorMessage().decode(errors="replace")))
        finally:
            ctx.close()
        return outputs

    def bind_custom(self, name, inputs, outputs, t_args=(), i_args=(), b_args=(), d_args=()):
        """Build the OpContext once and return a zero-argument callable that runs execCustomOp2 on it.
        For loops that execute the same op on the same arrays many times (benchmarks, decode steps)."""
        ctx = OpContext()
        ctx.set_inputs(inputs)
        ctx.set_outputs(outputs)
        ctx.set_args(t_args, i_args, b_args, d_args)
        h = self.op_hash(name)
        run = self.L.execCustomOp2

        def call():
            if run(None, h, ctx.ptr) != 0:
                raise N.NativeOpsError("Op [%s] execution failed: %s" % (name, self.L.lastErrorMessage().decode(errors="replace")))
        call.ctx = ctx
        return call

    def synchronize(self):
        self.L.streamSynchronize(None)
        N.check("streamSynchronize")
