"""Host-side mirror of the slice of `hyle::compute` that the tensor hot path uses, over the
C ABI of libhyle_hip.so.

Names, argument meaning and error behaviour follow the reference so that tests read like the
reference's own provider tests:

    context  = Context.create(device=0)                         # include/hyle/compute/device.h:124-140
    prepared = prepare(context, Binary(BinaryKind.kAdd), a, b)  # include/hyle/compute/prepared_operation.h:313-317
    run      = prepared.create_invocation(workspace)            # ...prepared_operation.h:144-291
    run.submit(stream, inputs, outputs)                         # enqueue only; never blocks

Errors surface as StatusError carrying the reference's StatusCode; `is_unimplemented()` is the
clean decline a route table moves past (src/compute/operation.cc:1259-1266).  There is no CPU
fallback anywhere in this module: without the built library it cannot be imported.
"""
from __future__ import annotations

import ctypes as C
import enum
from dataclasses import dataclass, field
from typing import Optional, Sequence

from . import capi


# ---- status ---------------------------------------------------------------------------
class StatusCode(enum.IntEnum):  # include/hyle/error/status.h:18-38
    kOk = 0
    kCancelled = 1
    kInvalidArgument = 3
    kResourceExhausted = 8
    kFailedPrecondition = 9
    kOutOfRange = 11
    kUnimplemented = 12
    kInternal = 13
    kUnavailable = 14


class StatusError(RuntimeError):
    def __init__(self, code: int, message: str):
        super().__init__(f"{capi.status_name(code)}: {message}")
        self.code = StatusCode(code)
        self.message = message

    def is_unimplemented(self) -> bool:
        return self.code == StatusCode.kUnimplemented

    def is_invalid_argument(self) -> bool:
        return self.code == StatusCode.kInvalidArgument

    def is_out_of_range(self) -> bool:
        return self.code == StatusCode.kOutOfRange

    def is_failed_precondition(self) -> bool:
        return self.code == StatusCode.kFailedPrecondition


def _check(code: int) -> None:
    if code != capi.OK:
        raise StatusError(code, capi.last_error())


# ---- descriptors ------------------------------------------------------------------------
class GgufQuantizedType(enum.IntEnum):  # include/hyle/compute/low_precision.h:36-41 (the decoded ones)
    kQ4K = 1
    kQ6K = 3
    kQ8_0 = 4


GGUF_BLOCKS = {GgufQuantizedType.kQ4K: (256, 144), GgufQuantizedType.kQ6K: (256, 210),
               GgufQuantizedType.kQ8_0: (32, 34)}


class DataType(enum.IntEnum):  # include/hyle/compute/tensor_desc.h:17-34
    kUnknown = 0
    kBool = 1
    kFloat8E4M3FN = 2
    kFloat8E5M2 = 3
    kFloat16 = 4
    kBFloat16 = 5
    kFloat32 = 6
    kFloat64 = 7
    kInt8 = 8
    kUInt8 = 9
    kInt16 = 10
    kUInt16 = 11
    kInt32 = 12
    kUInt32 = 13
    kInt64 = 14
    kUInt64 = 15


_SIZES = {DataType.kBool: 1, DataType.kFloat8E4M3FN: 1, DataType.kFloat8E5M2: 1, DataType.kInt8: 1, DataType.kUInt8: 1,
          DataType.kFloat16: 2, DataType.kBFloat16: 2, DataType.kInt16: 2, DataType.kUInt16: 2,
          DataType.kFloat32: 4, DataType.kInt32: 4, DataType.kUInt32: 4,
          DataType.kFloat64: 8, DataType.kInt64: 8, DataType.kUInt64: 8}


def data_type_size(dtype: DataType) -> int:
    return _SIZES.get(DataType(dtype), 0)


@dataclass(frozen=True)
class TensorDesc:
    """Logical dims + byte strides (include/hyle/compute/tensor_desc.h:141-225)."""
    data_type: DataType
    dimensions: tuple
    byte_strides: tuple
    blocked: bool = False
    block_axis: int = 0
    elements_per_block: int = 1
    bytes_per_block: int = 0

    @staticmethod
    def dense(data_type: DataType, dimensions: Sequence[int]) -> "TensorDesc":
        dims = tuple(int(d) for d in dimensions)
        if len(dims) > capi.MAX_RANK:
            raise StatusError(capi.INVALID_ARGUMENT, "tensor shape rank exceeds kMaxTensorRank")
        if any(d < 0 for d in dims):
            raise StatusError(capi.INVALID_ARGUMENT, "tensor shape dimension is negative")
        if 0 in dims:  # src/compute_ops/tensor_desc.cc:219-222
            return TensorDesc(DataType(data_type), dims, tuple(0 for _ in dims))
        strides, step = [], data_type_size(data_type)
        for d in reversed(dims):
            strides.append(step)
            step *= d
        return TensorDesc(DataType(data_type), dims, tuple(reversed(strides)))

    @staticmethod
    def strided_bytes(data_type: DataType, dimensions: Sequence[int], byte_strides: Sequence[int]) -> "TensorDesc":
        if len(dimensions) != len(byte_strides):
            raise StatusError(capi.INVALID_ARGUMENT, "stride count differs from rank")
        return TensorDesc(DataType(data_type), tuple(int(d) for d in dimensions),
                          tuple(int(s) for s in byte_strides))

    @staticmethod
    def gguf_q8_0_weight(logical_type: DataType, k: int, n: int, row_stride: Optional[int] = None) -> "TensorDesc":
        """gguf_weight_description(kQ8_0, type, k, n): logical [K, N], physical rows of K/32
        34-byte blocks (src/compute_ops/low_precision.cc:269-297)."""
        if k <= 0 or n <= 0 or k % 32 != 0:
            raise StatusError(capi.INVALID_ARGUMENT, "GGUF weight dimensions do not contain complete K blocks")
        stride = (k // 32) * 34 if row_stride is None else int(row_stride)
        return TensorDesc(DataType(logical_type), (k, n), (34, stride), blocked=True, block_axis=0,
                          elements_per_block=32, bytes_per_block=34)

    @staticmethod
    def gguf_weight(kind: "GgufQuantizedType", logical_type: DataType, k: int, n: int,
                    row_stride: Optional[int] = None) -> "TensorDesc":
        """gguf_weight_description(type, logical_type, k, n) (include/hyle/compute/low_precision.h:181-186)
        for the block formats this provider decodes: logical [K, N], physical rows of native K blocks
        (geometry: src/compute_ops/low_precision.cc:22-29)."""
        per_block, block_bytes = GGUF_BLOCKS[GgufQuantizedType(kind)]
        if k <= 0 or n <= 0 or k % per_block != 0:
            raise StatusError(capi.INVALID_ARGUMENT, "GGUF weight dimensions do not contain complete K blocks")
        stride = (k // per_block) * block_bytes if row_stride is None else int(row_stride)
        return TensorDesc(DataType(logical_type), (k, n), (block_bytes, stride), blocked=True, block_axis=0,
                          elements_per_block=per_block, bytes_per_block=block_bytes)

    @property
    def rank(self) -> int:
        return len(self.dimensions)

    def element_count(self) -> int:
        n = 1
        for d in self.dimensions:
            n *= d
        return n

    def is_plain(self) -> bool:
        return not self.blocked

    def is_dense(self) -> bool:
        return (not self.blocked) and self == TensorDesc.dense(self.data_type, self.dimensions)

    def required_bytes(self) -> int:  # src/compute_ops/tensor_desc.cc:494-540
        if 0 in self.dimensions:
            return 0
        last = 0
        for axis, (d, s) in enumerate(zip(self.dimensions, self.byte_strides)):
            units = d // self.elements_per_block if (self.blocked and axis == self.block_axis) else d
            last += (units - 1) * s
        return last + (self.bytes_per_block if self.blocked else data_type_size(self.data_type))

    def to_c(self) -> capi.TensorDescC:
        c = capi.TensorDescC()
        c.dtype, c.rank = int(self.data_type), len(self.dimensions)
        c.storage = 1 if self.blocked else 0
        c.block_axis = self.block_axis
        c.elements_per_block, c.bytes_per_block = self.elements_per_block, self.bytes_per_block
        for i, (d, s) in enumerate(zip(self.dimensions, self.byte_strides)):
            c.dims[i], c.byte_strides[i] = d, s
        return c

    @staticmethod
    def from_c(c: capi.TensorDescC) -> "TensorDesc":
        dims = tuple(int(c.dims[i]) for i in range(c.rank))
        strides = tuple(int(c.byte_strides[i]) for i in range(c.rank))
        if c.storage == 1:
            return TensorDesc(DataType(c.dtype), dims, strides, True, c.block_axis,
                              c.elements_per_block, c.bytes_per_block)
        return TensorDesc(DataType(c.dtype), dims, strides)


# ---- operations (include/hyle/compute/operation.h) -----------------------------------------
class OperationKind(enum.IntEnum):
    kCopy = 2
    kFill = 3
    kCast = 4
    kUnary = 5
    kBinary = 6
    kSelect = 7
    kReduce = 8
    kRmsNorm = 9
    kLayerNorm = 10
    kGatedActivation = 12
    kGather = 13
    kConcat = 15
    kRoPE = 16
    kSoftmax = 18
    kTopK = 19
    kBinaryChain = 0x100
    kQ8_0DequantSumSquares = 0x101
    kGgufMatVec = 0x102
    kRandomBits = 0x103
    kCategorical = 0x104


class UnaryKind(enum.IntEnum):
    kAbs = 0
    kNeg = 1
    kExp = 2
    kLog = 3
    kSqrt = 4
    kRsqrt = 5
    kTanh = 6
    kSigmoid = 7
    kRelu = 8
    kGelu = 9
    kGeluTanh = 10
    kSilu = 11
    kSoftplus = 12


class BinaryKind(enum.IntEnum):
    kAdd = 0
    kSubtract = 1
    kMultiply = 2
    kDivide = 3
    kMinimum = 4
    kMaximum = 5


class ReductionKind(enum.IntEnum):
    kSum = 0
    kMean = 1
    kMinimum = 2
    kMaximum = 3


class GatedActivationKind(enum.IntEnum):
    kSilu = 0
    kGelu = 1
    kGeluTanh = 2


class GatedInputKind(enum.IntEnum):
    kPackedHalves = 0
    kSeparate = 1


class SoftmaxKind(enum.IntEnum):
    kSoftmax = 0
    kLogSoftmax = 1


class MaskKind(enum.IntEnum):
    kNone = 0
    kAdditive = 1
    kBoolean = 2


@dataclass(frozen=True)
class Copy:
    """Materialise any plain tensor (dense or strided) as a dense tensor of the same type."""


@dataclass(frozen=True)
class ScalarValue:
    """Exact scalar payload of Fill (include/hyle/compute/operation.h:187-230): a type and the
    element's bit pattern."""
    data_type: DataType = DataType.kUnknown
    bits: int = 0

    @staticmethod
    def of(data_type: DataType, value) -> "ScalarValue":
        """The pattern the reference's typed constructors store; float16 / bfloat16 patterns
        (from_bits there) are the nearest-even narrowing of `value`."""
        import numpy as np
        if data_type == DataType.kBool:
            return ScalarValue(data_type, 1 if value else 0)
        if data_type == DataType.kFloat32:
            return ScalarValue(data_type, int(np.array(value, np.float32).view(np.uint32)))
        if data_type == DataType.kFloat16:
            return ScalarValue(data_type, int(np.array(value, np.float16).view(np.uint16)))
        if data_type == DataType.kFloat64:
            return ScalarValue(data_type, int(np.array(value, np.float64).view(np.uint64)))
        if data_type in (DataType.kFloat8E4M3FN, DataType.kFloat8E5M2):
            raise StatusError(capi.INVALID_ARGUMENT, "8-bit float scalars are given by their bits (from_bits)")
        if data_type == DataType.kBFloat16:
            word = int(np.array(value, np.float32).view(np.uint32))
            if (word & 0x7FFFFFFF) > 0x7F800000:
                return ScalarValue(data_type, (word >> 16) | 0x40)
            return ScalarValue(data_type, ((word + 0x7FFF + ((word >> 16) & 1)) >> 16) & 0xFFFF)
        size = data_type_size(data_type)
        if size == 0:
            raise StatusError(capi.INVALID_ARGUMENT, "Fill requires a valid shape and exactly typed scalar")
        return ScalarValue(data_type, int(value) & ((1 << (8 * size)) - 1))

    @staticmethod
    def from_bits(data_type: DataType, bits: int) -> "ScalarValue":
        return ScalarValue(data_type, bits)


@dataclass(frozen=True)
class Fill:
    """No inputs: a dense tensor of `output_shape` whose every element is `value`."""
    output_shape: tuple = ()
    output_type: DataType = DataType.kUnknown
    value: ScalarValue = ScalarValue()


@dataclass(frozen=True)
class Select:
    """Inputs (condition Bool, first, second) broadcast together; first where the condition holds."""


@dataclass(frozen=True)
class Concat:
    """1..4 inputs of one type and rank joined along `axis`.  A wider Concat is issued in groups of
    four into one output: `total` is then the output's extent on the axis and `start` the place
    where this group begins."""
    axis: int = 0
    total: int = 0
    start: int = 0


class IndexBoundsPolicy(enum.IntEnum):  # include/hyle/compute/operation.h:102-105
    kChecked = 0
    kUnchecked = 1


@dataclass(frozen=True)
class Gather:
    """Inputs (source, Int32 / Int64 indices): the source with `axis` replaced by the shape of the
    indices (include/hyle/compute/operation.h:367-370).  With checked bounds an index outside the
    axis leaves the output untouched and `OperationInvocation.wait` raises OutOfRange."""
    axis: int = 0
    bounds: IndexBoundsPolicy = IndexBoundsPolicy.kChecked


@dataclass(frozen=True)
class Cast:
    output_type: DataType = DataType.kUnknown


@dataclass(frozen=True)
class Unary:
    kind: UnaryKind = UnaryKind.kAbs


@dataclass(frozen=True)
class Binary:
    kind: BinaryKind = BinaryKind.kAdd


@dataclass(frozen=True)
class BinaryChain:
    """out = (in0 first in1) second in2 with the intermediate rounded to storage."""
    first: BinaryKind = BinaryKind.kAdd
    second: BinaryKind = BinaryKind.kMultiply


@dataclass(frozen=True)
class Axes:
    """include/hyle/compute/operation.h:232-247: every axis, or an explicit list whose entries
    may count from the end.  Duplicates are refused when the output is inferred."""
    values: tuple = ()
    all_axes: bool = True

    @staticmethod
    def all() -> "Axes":
        return Axes()

    @staticmethod
    def from_(axes) -> "Axes":  # Axes::from (src/compute_ops/operation.cc:768-789)
        axes = tuple(int(a) for a in axes)
        if not axes:
            raise StatusError(StatusCode.kInvalidArgument, "explicit axis list cannot be empty")
        if len(axes) > capi.MAX_RANK:
            raise StatusError(StatusCode.kInvalidArgument, "axis list exceeds kMaxTensorRank")
        if any(a < -capi.MAX_RANK or a >= capi.MAX_RANK for a in axes):
            raise StatusError(StatusCode.kOutOfRange, "axis cannot address a supported tensor rank")
        return Axes(axes, False)

    def is_all(self) -> bool:
        return self.all_axes


@dataclass(frozen=True)
class Reduce:
    kind: ReductionKind = ReductionKind.kSum
    axes: Axes = Axes()
    keep_dimensions: bool = False
    accumulation_type: DataType = DataType.kUnknown


@dataclass(frozen=True)
class RmsNorm:
    epsilon: float = 1.0e-5
    accumulation_type: DataType = DataType.kFloat32


@dataclass(frozen=True)
class LayerNorm:
    epsilon: float = 1.0e-5
    accumulation_type: DataType = DataType.kFloat32


@dataclass(frozen=True)
class GatedActivation:
    activation: GatedActivationKind = GatedActivationKind.kSilu
    inputs: GatedInputKind = GatedInputKind.kPackedHalves


@dataclass(frozen=True)
class Softmax:
    axis: int = -1
    scale: float = 1.0
    kind: SoftmaxKind = SoftmaxKind.kSoftmax
    mask: MaskKind = MaskKind.kNone
    accumulation_type: DataType = DataType.kFloat32


@dataclass(frozen=True)
class TopK:
    count: int = 1
    axis: int = -1
    largest: bool = True
    sorted: bool = True
    stable: bool = True


@dataclass(frozen=True)
class Q8_0DequantSumSquares:
    pass


@dataclass(frozen=True)
class GgufDequantSumSquares(Q8_0DequantSumSquares):
    """The same operation under its general name: Q8_0, Q4_K or Q6_K weights, told apart by the
    block geometry of the input descriptor."""


class ActivationArithmetic(enum.IntEnum):
    """How GgufMatVec treats the activations: kExact multiplies exactly decoded weights by them in
    f32; kGgmlQ8 first quantises them to ggml's 8-bit blocks and takes integer block dot products,
    which is what the reference's ggml CPU route computes."""
    kExact = 0
    kGgmlQ8 = 1


@dataclass(frozen=True)
class GgufMatVec:
    """MatMul(activations, GGUF weight) for a few activation rows: inputs (weight [K, N], x [K] or
    [M, K]); output [N] or [M, N] of x's type."""
    activations: ActivationArithmetic = ActivationArithmetic.kExact


class RopeLayout(enum.IntEnum):  # include/hyle/compute/operation.h:112-115
    kInterleaved = 0
    kHalfSplit = 1


@dataclass(frozen=True)
class RoPE:
    """Inputs (data, Int32 / Int64 positions, F32 frequencies): the first `rotary_dimensions`
    elements of every row rotated pair by pair through frequency * position
    (include/hyle/compute/operation.h:388-392)."""
    rotary_dimensions: int = 0
    sequence_axis: int = -2
    layout: RopeLayout = RopeLayout.kInterleaved


@dataclass(frozen=True)
class RandomBits:
    """sampling_ops::RandomBits (include/hyle/compute/sampling_ops.h:12-35): input U32 [R, 4]
    identities (key low / high, draw low / high); output U32 [R, word_count] Philox4x32-10 words."""
    word_count: int = 4


@dataclass(frozen=True)
class Categorical:
    """sampling_ops::Categorical (include/hyle/compute/sampling_ops.h:37-66): inputs (log-weights
    [R, V], U32 [R, 4] identities); outputs I32 [R] indices and, when asked, F32 [R] normalised log
    probabilities.  A row without valid mass fails `OperationInvocation.wait` with InvalidArgument."""
    return_log_probability: bool = False


def _op_desc(operation, inputs: Sequence[TensorDesc]) -> capi.OpDescC:
    c = capi.OpDescC()
    c.abi_version = capi.ABI_VERSION
    c.scale, c.largest = 1.0, 1
    if isinstance(operation, Copy):
        c.op = OperationKind.kCopy
    elif isinstance(operation, Cast):
        c.op, c.kind = OperationKind.kCast, int(operation.output_type)
    elif isinstance(operation, Fill):
        # the scalar's type travels as the output type: they must agree (operation.cc:1263-1275)
        shape = tuple(operation.output_shape)
        if (operation.value.data_type != operation.output_type or len(shape) > capi.MAX_RANK
                or any(d < 0 for d in shape) or inputs):
            raise StatusError(capi.INVALID_ARGUMENT, "Fill requires a valid shape and exactly typed scalar")
        c.op, c.kind, c.count = OperationKind.kFill, int(operation.output_type), operation.value.bits
        c.inputs[0].rank = len(shape)
        for i, d in enumerate(shape):
            c.inputs[0].dims[i] = d
    elif isinstance(operation, Select):
        c.op = OperationKind.kSelect
    elif isinstance(operation, Concat):
        c.op, c.axis, c.kind, c.count = OperationKind.kConcat, operation.axis, operation.total, operation.start
    elif isinstance(operation, Gather):
        c.op, c.axis, c.kind2 = OperationKind.kGather, operation.axis, int(operation.bounds)
    elif isinstance(operation, Unary):
        c.op, c.kind = OperationKind.kUnary, int(operation.kind)
    elif isinstance(operation, Binary):
        c.op, c.kind = OperationKind.kBinary, int(operation.kind)
    elif isinstance(operation, BinaryChain):
        c.op, c.kind, c.kind2 = OperationKind.kBinaryChain, int(operation.first), int(operation.second)
    elif isinstance(operation, Reduce):
        c.op, c.kind = OperationKind.kReduce, int(operation.kind)
        c.axes_count = 0 if operation.axes.is_all() else len(operation.axes.values)
        for i, axis in enumerate(operation.axes.values):
            c.axes[i] = axis
        c.keep_dimensions, c.accumulation = int(operation.keep_dimensions), int(operation.accumulation_type)
    elif isinstance(operation, RmsNorm):
        c.op, c.epsilon, c.accumulation = OperationKind.kRmsNorm, operation.epsilon, int(operation.accumulation_type)
    elif isinstance(operation, LayerNorm):
        c.op, c.epsilon, c.accumulation = OperationKind.kLayerNorm, operation.epsilon, int(operation.accumulation_type)
    elif isinstance(operation, GatedActivation):
        c.op, c.kind, c.kind2 = OperationKind.kGatedActivation, int(operation.activation), int(operation.inputs)
    elif isinstance(operation, Softmax):
        c.op, c.axis, c.scale = OperationKind.kSoftmax, operation.axis, operation.scale
        c.kind2, c.mask, c.accumulation = int(operation.kind), int(operation.mask), int(operation.accumulation_type)
    elif isinstance(operation, TopK):
        c.op, c.count, c.axis, c.largest = OperationKind.kTopK, operation.count, operation.axis, int(operation.largest)
    elif isinstance(operation, Q8_0DequantSumSquares):
        c.op = OperationKind.kQ8_0DequantSumSquares
    elif isinstance(operation, GgufMatVec):
        c.op, c.kind2 = OperationKind.kGgufMatVec, int(operation.activations)
    elif isinstance(operation, RoPE):
        if operation.rotary_dimensions < 0:
            raise StatusError(capi.INVALID_ARGUMENT, "RoPE rotary dimension must be positive, even and fit the last axis")
        c.op, c.count, c.axis, c.kind2 = OperationKind.kRoPE, operation.rotary_dimensions, operation.sequence_axis, int(operation.layout)
    elif isinstance(operation, RandomBits):
        if operation.word_count < 0:
            raise StatusError(capi.INVALID_ARGUMENT, "RandomBits word count is negative")
        c.op, c.count = OperationKind.kRandomBits, operation.word_count
    elif isinstance(operation, Categorical):
        c.op, c.kind2 = OperationKind.kCategorical, 1 if operation.return_log_probability else 0
    else:
        raise StatusError(capi.UNIMPLEMENTED, f"operation {type(operation).__name__} is not served by this provider")
    if len(inputs) > capi.MAX_INPUTS:
        raise StatusError(capi.INVALID_ARGUMENT, "operation input count does not match its typed contract")
    c.input_count = len(inputs)
    for i, desc in enumerate(inputs):
        c.inputs[i] = desc.to_c()
    return c


def infer_output_descriptions(operation, inputs: Sequence[TensorDesc]) -> list:
    """src/compute_ops/operation.cc:1214-1704 for the operations of this provider."""
    req = _op_desc(operation, inputs)
    outs = (capi.TensorDescC * capi.MAX_OUTPUTS)()
    count = C.c_uint32(0)
    _check(capi.load().hyle_hip_infer_outputs(C.byref(req), outs, C.byref(count)))
    return [TensorDesc.from_c(outs[i]) for i in range(count.value)]


# ---- context / prepare / submit ----------------------------------------------------------
class Context:
    """One HIP device bound to the provider (ProviderVTable::create_context)."""

    def __init__(self, handle: Optional[int], device: int):
        self._handle, self.device = handle, device

    @staticmethod
    def create(device: int = 0) -> "Context":
        handle = C.c_void_p()
        _check(capi.load().hyle_hip_context_create(device, C.byref(handle)))
        return Context(handle.value, device)

    @staticmethod
    def planning_only() -> "Context":
        """No device: plans can be built and inspected (cold path), never launched."""
        capi.load()
        return Context(None, -1)

    @property
    def compute_units(self) -> int:
        return capi.load().hyle_hip_context_compute_units(self._handle)

    def close(self) -> None:
        if self._handle:
            capi.load().hyle_hip_context_destroy(self._handle)
            self._handle = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


@dataclass(frozen=True)
class WorkspaceRequirement:
    size: int = 0
    alignment: int = 1


class PreparedOperation:
    def __init__(self, context: Context, handle: int, inputs: Sequence[TensorDesc]):
        self._context, self._handle, self._inputs = context, handle, list(inputs)
        lib = capi.load()
        outs = (capi.TensorDescC * capi.MAX_OUTPUTS)()
        count = C.c_uint32(0)
        _check(lib.hyle_hip_plan_outputs(handle, outs, C.byref(count)))
        self._outputs = [TensorDesc.from_c(outs[i]) for i in range(count.value)]
        size, align = C.c_size_t(0), C.c_size_t(1)
        _check(lib.hyle_hip_plan_workspace(handle, C.byref(size), C.byref(align)))
        self._workspace = WorkspaceRequirement(size.value, align.value)

    def output_descriptions(self) -> list:
        return list(self._outputs)

    def output_description(self) -> TensorDesc:
        return self._outputs[0]

    def workspace_requirement(self) -> WorkspaceRequirement:
        return self._workspace

    def alias_support(self, output_index: int, input_index: int) -> bool:
        return bool(capi.load().hyle_hip_plan_alias_support(self._handle, output_index, input_index))

    def dispatch_count(self) -> int:
        return capi.load().hyle_hip_plan_dispatch_count(self._handle)

    def route_name(self) -> str:
        return capi.load().hyle_hip_plan_route_name(self._handle).decode()

    def create_invocation(self, workspace: int = 0, workspace_size: int = 0) -> "OperationInvocation":
        """`workspace` is a device address the caller owns for the invocation's lifetime."""
        if self._workspace.size and (not workspace or workspace_size < self._workspace.size):
            raise StatusError(capi.INVALID_ARGUMENT, "workspace is smaller than the plan requires")
        return OperationInvocation(self, workspace, workspace_size)

    def create_invocation_without_workspace(self) -> "OperationInvocation":
        """An invocation for `submit_without_workspace` only."""
        return OperationInvocation(self, 0, 0)

    def close(self) -> None:
        if self._handle:
            capi.load().hyle_hip_plan_destroy(self._handle)
            self._handle = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


class OperationInvocation:
    def __init__(self, prepared: PreparedOperation, workspace: int, workspace_size: int):
        self._prepared, self._workspace, self._workspace_size = prepared, workspace, workspace_size
        self._in = (C.c_void_p * capi.MAX_INPUTS)()
        self._out = (C.c_void_p * capi.MAX_OUTPUTS)()

    def submit(self, stream: int, inputs: Sequence[int], outputs: Sequence[int]) -> None:
        """Enqueue on HIP stream handle `stream` (0 = default stream) and return at once.
        `inputs` / `outputs` are device addresses."""
        for i, p in enumerate(inputs):
            self._in[i] = p
        for i, p in enumerate(outputs):
            self._out[i] = p
        _check(capi.load().hyle_hip_plan_launch(
            self._prepared._handle, self._in, len(inputs), self._out, len(outputs),
            self._workspace, self._workspace_size, stream))

    def wait(self, stream: int, static_scratch: bool = False) -> None:
        """Completion::wait for launches whose kernels can refuse their input (checked Gather):
        waits for `stream` and raises StatusError(OutOfRange) when the device said so.  Plans
        without a device verdict return at once."""
        _check(capi.load().hyle_hip_plan_device_status(
            self._prepared._handle, None if static_scratch else self._workspace, stream))

    def submit_without_workspace(self, stream: int, inputs: Sequence[int], outputs: Sequence[int]) -> None:
        """The same launch through hyle_hip_plan_launch_static: the route's workspace is the
        library's per-device scratch array, nothing is allocated.  Calls that may overlap on
        one device race on that array."""
        for i, p in enumerate(inputs):
            self._in[i] = p
        for i, p in enumerate(outputs):
            self._out[i] = p
        _check(capi.load().hyle_hip_plan_launch_static(
            self._prepared._handle, self._in, len(inputs), self._out, len(outputs), stream))


def launch_variants() -> list:
    """Labels of every kernel launch shape compiled into the library (diagnostics)."""
    lib = capi.load()
    return [lib.hyle_hip_variant_label(i).decode() for i in range(lib.hyle_hip_variant_count())]


def last_launch_variant() -> str:
    """Label(s) of the dispatches this thread's last submit enqueued, joined by ' + '."""
    return capi.load().hyle_hip_last_launch_variant().decode()


def prepare(context: Context, operation, *inputs: TensorDesc,
            outputs: Optional[Sequence[TensorDesc]] = None) -> PreparedOperation:
    """hyle::compute::prepare(context, operation, input descriptors...)."""
    req = _op_desc(operation, inputs)
    handle = C.c_void_p()
    if outputs is None:
        outs, count = None, 0
    else:
        outs = (capi.TensorDescC * capi.MAX_OUTPUTS)()
        for i, d in enumerate(outputs):
            outs[i] = d.to_c()
        count = len(outputs)
    _check(capi.load().hyle_hip_plan_create(context._handle, C.byref(req), outs, count, C.byref(handle)))
    return PreparedOperation(context, handle.value, inputs)
