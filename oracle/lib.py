"""ctypes binding of oracle/libhyle_oracle.so over numpy arrays.

Test infrastructure only.  Narrow floats travel as uint16 bit patterns.
"""
from __future__ import annotations

import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "libhyle_oracle.so")

F32, F16, BF16 = 0, 1, 2
BOOL, I32 = 3, 4  # Cast only
ADD, SUBTRACT, MULTIPLY, DIVIDE, MINIMUM, MAXIMUM = range(6)
SUM, MEAN, MIN, MAX = range(4)
MASK_NONE, MASK_ADDITIVE, MASK_BOOLEAN = range(3)

RAW1, RAW2, RAW4, RAW8 = 10, 11, 12, 13  # storage words for the operations that only move bits

_NP = {F32: np.float32, F16: np.uint16, BF16: np.uint16, BOOL: np.uint8, I32: np.int32,
       RAW1: np.uint8, RAW2: np.uint16, RAW4: np.uint32, RAW8: np.uint64}


def build() -> None:
    """Compile the checker (and oracle/_ref when the reference tree exists)."""
    subprocess.run(["make", "-C", _HERE, "--no-print-directory"], check=True)


def _load() -> C.CDLL:
    if not os.path.exists(_SO):
        build()
    return C.CDLL(_SO)


_lib = _load()

_vp = C.c_void_p
_sz = C.c_size_t
_i64p = C.POINTER(C.c_int64)


def _sig(name, restype, *argtypes):
    fn = getattr(_lib, name)
    fn.restype = restype
    fn.argtypes = list(argtypes)
    return fn


_f16_to_f32 = _sig("hyle_oracle_f16_to_f32", C.c_float, C.c_uint16)
_f32_to_f16 = _sig("hyle_oracle_f32_to_f16", C.c_uint16, C.c_float)
_bf16_to_f32 = _sig("hyle_oracle_bf16_to_f32", C.c_float, C.c_uint16)
_f32_to_bf16 = _sig("hyle_oracle_f32_to_bf16", C.c_uint16, C.c_float)
_to_f32 = _sig("hyle_oracle_convert_to_f32", None, C.c_int, _vp, _vp, _sz)
_from_f32 = _sig("hyle_oracle_convert_from_f32", None, C.c_int, _vp, _vp, _sz)
_bshape = _sig("hyle_oracle_broadcast_shape", C.c_int, _i64p, C.c_int, _i64p, C.c_int, _i64p)
_boff = _sig("hyle_oracle_broadcast_byte_offset", _sz, _i64p, _i64p, C.c_int, _i64p, C.c_int, _sz)
_loff = _sig("hyle_oracle_logical_byte_offset", _sz, _i64p, _i64p, C.c_int, _sz)
_bscalar = _sig("hyle_oracle_binary_scalar", C.c_float, C.c_int, C.c_float, C.c_float)
_binary = _sig("hyle_oracle_binary", None, C.c_int, C.c_int, _vp, _i64p, _i64p, C.c_int,
               _vp, _i64p, _i64p, C.c_int, _vp, _i64p, C.c_int)
_chain = _sig("hyle_oracle_binary_chain", None, C.c_int, C.c_int, C.c_int,
              _vp, _i64p, _i64p, C.c_int, _vp, _i64p, _i64p, C.c_int,
              _vp, _i64p, _i64p, C.c_int, _vp, _i64p, C.c_int)
_sigmoid = _sig("hyle_oracle_sigmoid", C.c_float, C.c_float)
_silu1 = _sig("hyle_oracle_silu", C.c_float, C.c_float)
_silu = _sig("hyle_oracle_silu_rows", None, C.c_int, _vp, _vp, _sz)
_swiglu = _sig("hyle_oracle_swiglu", None, C.c_int, _vp, _vp, _vp, _sz)
_unary = _sig("hyle_oracle_unary", None, C.c_int, C.c_int, _vp, _vp, _sz)
_unary1 = _sig("hyle_oracle_unary_scalar", C.c_float, C.c_int, C.c_float)
_gated = _sig("hyle_oracle_gated", None, C.c_int, C.c_int, _vp, _vp, _vp, _sz)
_swiglu_packed = _sig("hyle_oracle_swiglu_packed", None, C.c_int, _vp, _vp, _sz, _sz)
_rms = _sig("hyle_oracle_rms_norm", None, C.c_int, C.c_int, _vp, _vp, _vp, _sz, _sz, C.c_float)
_rms_native = _sig("hyle_oracle_rms_norm_native", None, C.c_int, C.c_int, _vp, _vp, _vp, _sz, _sz, C.c_float)
_layer = _sig("hyle_oracle_layer_norm", None, C.c_int, C.c_int, _vp, _vp, _vp, _vp, _sz, _sz, C.c_float)
_softmax_row = _sig("hyle_oracle_softmax_f32_row", None, _vp, _vp, _sz)
_softmax = _sig("hyle_oracle_softmax", None, C.c_int, _vp, _vp, _i64p, C.c_int, C.c_float,
                C.c_int, _vp, _i64p, _i64p, C.c_int)
_log_softmax = _sig("hyle_oracle_log_softmax", None, C.c_int, _vp, _vp, _i64p, C.c_int, C.c_float,
                    C.c_int, _vp, _i64p, _i64p, C.c_int)
_log_softmax_row = _sig("hyle_oracle_log_softmax_f32_row", None, _vp, _vp, _sz)
_log_softmax_floor_row = _sig("hyle_oracle_log_softmax_floor_f32_row", None, _vp, _vp, _sz)
_reduce = _sig("hyle_oracle_reduce_last_axis", None, C.c_int, C.c_int, _vp, _vp, _sz, _sz)
_iom = _sig("hyle_oracle_index_of_max_f32", _sz, _vp, _sz)
_topk1 = _sig("hyle_oracle_topk1_f32", None, _vp, _sz, _sz, _vp, _vp)
_q8_bf16 = _sig("hyle_oracle_q8_0_dequant_bf16", None, _vp, _sz, _sz, _sz, _vp, _vp, _vp)
_q8_f32 = _sig("hyle_oracle_q8_0_dequant_f32", None, _vp, _sz, _sz, _sz, _vp)
_reduce_axes = _sig("hyle_oracle_reduce", None, C.c_int, C.c_int, _vp, C.c_int, _i64p, _i64p, C.c_uint32, _vp)
_topk = _sig("hyle_oracle_topk", None, C.c_int, _vp, C.c_int, _i64p, _i64p, C.c_int, _sz, C.c_int, _vp, _vp)
_k_quant = _sig("hyle_oracle_k_quant_dequant", None, C.c_int, _vp, _sz, _sz, _sz, _vp, _vp, _vp)
_matvec = _sig("hyle_oracle_gguf_matvec", None, C.c_int, _vp, _sz, _sz, _sz, _vp, _sz, _vp, _vp)
_fill = _sig("hyle_oracle_fill", None, C.c_size_t, C.c_uint64, C.c_size_t, _vp)
_select = _sig("hyle_oracle_select", None, C.c_size_t, _vp, _i64p, _i64p, C.c_int, _vp, _i64p, _i64p, C.c_int,
               _vp, _i64p, _i64p, C.c_int, _i64p, C.c_int, _vp)
_gather = _sig("hyle_oracle_gather", C.c_int, C.c_size_t, _vp, _i64p, _i64p, C.c_int, C.c_int, _vp, C.c_int, _i64p, _i64p,
               C.c_int, C.c_int, _vp)
_rope = _sig("hyle_oracle_rope", None, C.c_int, _vp, _i64p, C.c_int, C.c_int, _vp, C.c_int, C.c_int, _vp, C.c_int, C.c_int64,
             C.c_int, _vp)
_u32p = C.POINTER(C.c_uint32)
_philox = _sig("hyle_oracle_philox_block", None, _vp, C.c_uint64, _vp)
_random_bits = _sig("hyle_oracle_random_bits", None, _vp, C.c_size_t, C.c_size_t, _vp)
_uniform = _sig("hyle_oracle_categorical_uniform", C.c_double, _vp)
_categorical = _sig("hyle_oracle_categorical", C.c_int, C.c_int, _vp, _vp, C.c_size_t, C.c_size_t, _vp, _vp)
_concat = _sig("hyle_oracle_concat_part", None, C.c_size_t, _vp, _i64p, _i64p, C.c_int, C.c_int, C.c_int64, _i64p, _vp)
_cast = _sig("hyle_oracle_cast", C.c_int, C.c_int, C.c_int, _vp, _i64p, _i64p, C.c_int, _vp)


def _ptr(a: np.ndarray | None):
    return None if a is None else a.ctypes.data_as(_vp)


def _i64(values):
    arr = (C.c_int64 * max(len(values), 1))(*[int(v) for v in values])
    return arr


def _c(a: np.ndarray, dtype=None) -> np.ndarray:
    a = np.ascontiguousarray(a)
    if dtype is not None and a.dtype != np.dtype(dtype):
        raise TypeError(f"expected {np.dtype(dtype)}, got {a.dtype}")
    return a


def np_dtype(type_id: int):
    return _NP[type_id]


def itemsize(type_id: int) -> int:
    return 4 if type_id == F32 else 2


def dense_strides(dims, type_id) -> list[int]:
    strides, step = [], itemsize(type_id)
    for d in reversed(list(dims)):
        strides.append(step)
        step *= int(d)
    return list(reversed(strides))


# ---- codecs ---------------------------------------------------------------
def f16_to_f32(bits: int) -> float:
    return _f16_to_f32(int(bits))


def f32_to_f16(x: float) -> int:
    return _f32_to_f16(np.float32(x).item() if not isinstance(x, float) else x)


def bf16_to_f32(bits: int) -> float:
    return _bf16_to_f32(int(bits))


def f32_bits_to_bf16(bits32: int) -> int:
    """Round one f32 given as its bit pattern (keeps NaN payloads intact)."""
    src = np.array([bits32], dtype=np.uint32).view(np.float32)
    return int(from_f32(BF16, src)[0])


def to_f32(type_id: int, a: np.ndarray) -> np.ndarray:
    a = _c(a, _NP[type_id])
    out = np.empty(a.shape, np.float32)
    _to_f32(type_id, _ptr(a), _ptr(out), a.size)
    return out


def from_f32(type_id: int, a: np.ndarray) -> np.ndarray:
    a = _c(a, np.float32)
    out = np.empty(a.shape, _NP[type_id])
    _from_f32(type_id, _ptr(a), _ptr(out), a.size)
    return out


# ---- shapes ---------------------------------------------------------------
def broadcast_shape(left, right):
    out = (C.c_int64 * 8)()
    rank = _bshape(_i64(left), len(left), _i64(right), len(right), out)
    if rank < 0:
        return None
    return [int(out[i]) for i in range(rank)]


def broadcast_byte_offset(in_dims, in_strides, out_dims, linear: int) -> int:
    return _boff(_i64(in_dims), _i64(in_strides), len(in_dims), _i64(out_dims), len(out_dims), linear)


def logical_byte_offset(dims, strides, linear: int) -> int:
    return _loff(_i64(dims), _i64(strides), len(dims), linear)


# ---- elementwise ----------------------------------------------------------
def binary_scalar(kind: int, left: float, right: float) -> float:
    return _bscalar(kind, left, right)


def binary(kind, type_id, left, right, left_strides=None, right_strides=None):
    """Broadcasting Binary.  Arrays carry the logical dims; strides default to
    dense.  A custom stride list (bytes) reads `left`/`right` as raw storage."""
    left, right = _c(left, _NP[type_id]), _c(right, _NP[type_id])
    ld, rd = list(left.shape), list(right.shape)
    od = broadcast_shape(ld, rd)
    if od is None:
        raise ValueError("shapes do not broadcast")
    ls = left_strides or dense_strides(ld, type_id)
    rs = right_strides or dense_strides(rd, type_id)
    out = np.empty(od, _NP[type_id])
    _binary(kind, type_id, _ptr(left), _i64(ld), _i64(ls), len(ld), _ptr(right), _i64(rd),
            _i64(rs), len(rd), _ptr(out), _i64(od), len(od))
    return out


def binary_raw(kind, type_id, left, ld, ls, right, rd, rs, od):
    """Binary over raw storage buffers with explicit dims / byte strides."""
    out = np.empty(od, _NP[type_id])
    _binary(kind, type_id, _ptr(left), _i64(ld), _i64(ls), len(ld), _ptr(right), _i64(rd),
            _i64(rs), len(rd), _ptr(out), _i64(od), len(od))
    return out


def binary_chain(kind0, kind1, type_id, a, b, c):
    a, b, c = (_c(x, _NP[type_id]) for x in (a, b, c))
    ad, bd, cd = list(a.shape), list(b.shape), list(c.shape)
    od = broadcast_shape(broadcast_shape(ad, bd), cd)
    out = np.empty(od, _NP[type_id])
    _chain(kind0, kind1, type_id,
           _ptr(a), _i64(ad), _i64(dense_strides(ad, type_id)), len(ad),
           _ptr(b), _i64(bd), _i64(dense_strides(bd, type_id)), len(bd),
           _ptr(c), _i64(cd), _i64(dense_strides(cd, type_id)), len(cd),
           _ptr(out), _i64(od), len(od))
    return out


def sigmoid(x: float) -> float:
    return _sigmoid(x)


def silu_scalar(x: float) -> float:
    return _silu1(x)


def silu(type_id, src):
    src = _c(src, _NP[type_id])
    out = np.empty_like(src)
    _silu(type_id, _ptr(src), _ptr(out), src.size)
    return out


def swiglu(type_id, gate, value):
    gate, value = _c(gate, _NP[type_id]), _c(value, _NP[type_id])
    assert gate.shape == value.shape
    out = np.empty_like(gate)
    _swiglu(type_id, _ptr(gate), _ptr(value), _ptr(out), gate.size)
    return out


def unary(kind: int, type_id: int, src):
    src = _c(src, _NP[type_id])
    out = np.empty_like(src)
    _unary(int(kind), type_id, _ptr(src), _ptr(out), src.size)
    return out


def gated(activation: int, type_id: int, gate, value):
    gate, value = _c(gate, _NP[type_id]), _c(value, _NP[type_id])
    out = np.empty_like(gate)
    _gated(int(activation), type_id, _ptr(gate), _ptr(value), _ptr(out), gate.size)
    return out


def swiglu_packed(type_id, packed):
    packed = _c(packed, _NP[type_id])
    hidden = packed.shape[-1] // 2
    rows = packed.size // (2 * hidden) if hidden else 0
    out = np.empty(packed.shape[:-1] + (hidden,), _NP[type_id])
    _swiglu_packed(type_id, _ptr(packed), _ptr(out), rows, hidden)
    return out


# ---- normalisation --------------------------------------------------------
def rms_norm(type_id, src, weight, epsilon, weight_type=None, native=False):
    src = _c(src, _NP[type_id])
    weight_type = type_id if weight_type is None else weight_type
    if weight is not None:
        weight = _c(weight, _NP[weight_type])
    hidden = src.shape[-1]
    rows = src.size // hidden if hidden else 0
    out = np.empty_like(src)
    fn = _rms_native if native else _rms
    fn(type_id, weight_type, _ptr(src), _ptr(weight), _ptr(out), rows, hidden, float(epsilon))
    return out


def layer_norm(type_id, src, scale, bias, epsilon, param_type=None):
    src = _c(src, _NP[type_id])
    param_type = type_id if param_type is None else param_type
    if scale is None and bias is not None:
        raise ValueError("LayerNorm takes a bias only together with a scale")
    scale = None if scale is None else _c(scale, _NP[param_type])
    bias = None if bias is None else _c(bias, _NP[param_type])
    hidden = src.shape[-1]
    rows = src.size // hidden if hidden else 0
    out = np.empty_like(src)
    _layer(type_id, param_type, _ptr(src), _ptr(scale), _ptr(bias), _ptr(out), rows, hidden, float(epsilon))
    return out


# ---- softmax / reductions -------------------------------------------------
def softmax_f32_row(src):
    src = _c(src, np.float32)
    out = np.empty_like(src)
    _softmax_row(_ptr(src), _ptr(out), src.size)
    return out


def softmax_bool_f32_rows(src, mask, threads=1):
    """Row softmax of dense f32 [rows, cols] under a Boolean mask [mask_rows, cols] (row r uses
    mask row r % mask_rows), rows fanned out over `threads` host threads (the C loop releases
    the interpreter lock)."""
    from concurrent.futures import ThreadPoolExecutor
    src = _c(src, np.float32)
    mask = _c(mask, np.uint8)
    rows, cols = src.shape
    out = np.empty_like(src)
    fn = _lib.hyle_oracle_rows_softmax_bool_f32
    fn.restype = None
    fn.argtypes = [C.c_void_p, C.c_void_p, C.c_void_p, C.c_size_t, C.c_size_t, C.c_size_t, C.c_size_t]
    threads = max(1, min(threads, rows))
    edges = [rows * t // threads for t in range(threads + 1)]
    with ThreadPoolExecutor(max_workers=threads) as pool:
        list(pool.map(lambda t: fn(_ptr(src), _ptr(mask), _ptr(out), cols, mask.shape[0], edges[t], edges[t + 1]),
                      range(threads)))
    return out


def log_softmax_f32_row(src):
    src = _c(src, np.float32)
    out = np.empty_like(src)
    _log_softmax_row(_ptr(src), _ptr(out), src.size)
    return out


def log_softmax_floor_f32_row(src):
    """The scalar floor's own form of LogSoftmax (double sum, one log, one shift)."""
    src = _c(src, np.float32)
    out = np.empty_like(src)
    _log_softmax_floor_row(_ptr(src), _ptr(out), src.size)
    return out


def softmax(type_id, src, scale=1.0, mask_kind=MASK_NONE, mask=None, mask_strides=None, log=False):
    src = _c(src, _NP[type_id])
    out = np.empty_like(src)
    md, ms = [], []
    if mask_kind != MASK_NONE:
        mask = np.ascontiguousarray(mask)
        md = list(mask.shape)
        ms = mask_strides or _byte_strides(md, mask.itemsize)
    (_log_softmax if log else _softmax)(type_id, _ptr(src), _ptr(out), _i64(src.shape), src.ndim, float(scale),
                                        mask_kind, _ptr(mask), _i64(md), _i64(ms), len(md))
    return out


def _byte_strides(dims, width):
    strides, step = [], width
    for d in reversed(list(dims)):
        strides.append(step)
        step *= int(d)
    return list(reversed(strides))


def reduce_last_axis(kind, type_id, src):
    src = _c(src, _NP[type_id])
    width = src.shape[-1]
    rows = int(np.prod(src.shape[:-1], dtype=np.int64))
    out = np.empty(src.shape[:-1], _NP[type_id])
    _reduce(kind, type_id, _ptr(src), _ptr(out), rows, width)
    return out


def reduce(kind, type_id, storage, dims, axes=None, byte_strides=None, keep_dimensions=False):
    """Reduce the axes `axes` (None = all; entries may be negative) of the plain tensor held in
    `storage` (read as bytes) with logical `dims` and `byte_strides` (dense when omitted)."""
    dims = [int(d) for d in dims]
    rank = len(dims)
    if byte_strides is None:
        byte_strides = _byte_strides(dims, np.dtype(_NP[type_id]).itemsize)
    selected = range(rank) if axes is None else [a + rank if a < 0 else a for a in axes]
    mask = 0
    for a in selected:
        mask |= 1 << a
    shape = [1 if (mask >> a) & 1 else dims[a] for a in range(rank)]
    if not keep_dimensions:
        shape = [dims[a] for a in range(rank) if not (mask >> a) & 1]
    raw = np.ascontiguousarray(storage).view(np.uint8).reshape(-1)
    out = np.empty(shape, _NP[type_id])
    _reduce_axes(kind, type_id, _ptr(raw), rank, _i64(dims), _i64(byte_strides), mask, _ptr(out))
    return out


def index_of_max(data) -> int:
    data = _c(data, np.float32)
    return int(_iom(_ptr(data), data.size))


def topk1(data):
    data = _c(data, np.float32)
    width = data.shape[-1]
    rows = int(np.prod(data.shape[:-1], dtype=np.int64))
    values = np.empty(data.shape[:-1], np.float32)
    indices = np.empty(data.shape[:-1], np.int32)
    _topk1(_ptr(data), rows, width, _ptr(values), _ptr(indices))
    return values, indices


def topk(type_id, storage, dims, count, axis=-1, largest=True, byte_strides=None):
    """TopK(count) along `axis` of the plain tensor held in `storage` (read as bytes) with logical
    `dims` and `byte_strides` (dense when omitted): (values as stored bits, int32 indices)."""
    dims = [int(d) for d in dims]
    axis = axis + len(dims) if axis < 0 else axis
    if byte_strides is None:
        byte_strides = _byte_strides(dims, np.dtype(_NP[type_id]).itemsize)
    shape = list(dims)
    shape[axis] = int(count)
    raw = np.ascontiguousarray(storage).view(np.uint8).reshape(-1)
    values, indices = np.empty(shape, _NP[type_id]), np.empty(shape, np.int32)
    _topk(type_id, _ptr(raw), len(dims), _i64(dims), _i64(byte_strides), axis, int(count), int(bool(largest)),
          _ptr(values), _ptr(indices))
    return values, indices


# ---- Q8_0 -----------------------------------------------------------------
def q8_0_dequant_bf16(blocks: np.ndarray, rows: int, k: int, row_stride: int | None = None):
    blocks = _c(blocks, np.uint8)
    row_stride = (k // 32) * 34 if row_stride is None else row_stride
    out = np.empty((rows, k), np.uint16)
    sumsq = np.empty(rows, np.float32)
    sumsq_rounded = np.empty(rows, np.float32)
    _q8_bf16(_ptr(blocks), rows, k, row_stride, _ptr(out), _ptr(sumsq), _ptr(sumsq_rounded))
    return out, sumsq, sumsq_rounded


Q4_K, Q6_K = 0, 1
K_QUANT_BLOCK_BYTES = {Q4_K: 144, Q6_K: 210}


def k_quant_dequant(kind: int, blocks: np.ndarray, rows: int, k: int, row_stride: int | None = None):
    """GGUF Q4_K / Q6_K rows -> (f32 [rows, k], bf16 bits [rows, k], f32 sums of squares [rows])."""
    blocks = _c(blocks, np.uint8)
    row_stride = (k // 256) * K_QUANT_BLOCK_BYTES[kind] if row_stride is None else row_stride
    wide, narrow = np.empty((rows, k), np.float32), np.empty((rows, k), np.uint16)
    sumsq = np.empty(rows, np.float32)
    _k_quant(kind, _ptr(blocks), rows, k, row_stride, _ptr(wide), _ptr(narrow), _ptr(sumsq))
    return wide, narrow, sumsq


Q8_0 = 2
GGUF_BLOCK = {Q4_K: (256, 144), Q6_K: (256, 210), Q8_0: (32, 34)}


def gguf_matvec(kind: int, blocks: np.ndarray, rows: int, k: int, x: np.ndarray, row_stride: int | None = None):
    """(float64 [m, rows] products of exactly decoded rows with x [m, k] f32, float64 sums of |w x|)."""
    blocks = _c(blocks, np.uint8)
    x = _c(np.atleast_2d(x), np.float32)
    per_block, block_bytes = GGUF_BLOCK[kind]
    row_stride = (k // per_block) * block_bytes if row_stride is None else row_stride
    out = np.empty((x.shape[0], rows), np.float64)
    magnitude = np.empty_like(out)
    _matvec(kind, _ptr(blocks), rows, k, row_stride, _ptr(x), x.shape[0], _ptr(out), _ptr(magnitude))
    return out, magnitude


def quantize_q8_0(x: np.ndarray):
    """ggml's Q8_0 activation blocks (AVX form): (int8 codes [k], f32 scales [k / 32], each an f16 value)."""
    x = _c(x, np.float32).reshape(-1)
    codes, scales = np.empty(x.size, np.int8), np.empty(x.size // 32, np.float32)
    fn = _lib.hyle_oracle_quantize_q8_0
    fn.restype, fn.argtypes = None, [_vp, _sz, _vp, _vp]
    fn(_ptr(x), x.size, _ptr(codes), _ptr(scales))
    return codes, scales


def quantize_q8_k(x: np.ndarray):
    """ggml's Q8_K activation blocks: (int8 codes [k], f32 scales [k / 256])."""
    x = _c(x, np.float32).reshape(-1)
    codes, scales = np.empty(x.size, np.int8), np.empty(x.size // 256, np.float32)
    fn = _lib.hyle_oracle_quantize_q8_k
    fn.restype, fn.argtypes = None, [_vp, _sz, _vp, _vp]
    fn(_ptr(x), x.size, _ptr(codes), _ptr(scales))
    return codes, scales


def gguf_matvec_q8(kind: int, blocks: np.ndarray, rows: int, k: int, x: np.ndarray, row_stride: int | None = None):
    """MatMul with 8-bit activation blocks, as the reference's ggml CPU route computes it:
    (float64 centre [m, rows], float64 bound [m, rows] the reference's tests accept around it)."""
    blocks = _c(blocks, np.uint8)
    x = _c(np.atleast_2d(x), np.float32)
    per_block, block_bytes = GGUF_BLOCK[kind]
    row_stride = (k // per_block) * block_bytes if row_stride is None else row_stride
    centre = np.empty((x.shape[0], rows), np.float64)
    bound = np.empty_like(centre)
    fn = _lib.hyle_oracle_gguf_matvec_q8
    fn.restype, fn.argtypes = None, [C.c_int, _vp, _sz, _sz, _sz, _vp, _sz, _vp, _vp]
    fn(kind, _ptr(blocks), rows, k, row_stride, _ptr(x), x.shape[0], _ptr(centre), _ptr(bound))
    return centre, bound


def q8_0_dequant_f32(blocks: np.ndarray, rows: int, k: int, row_stride: int | None = None):
    blocks = _c(blocks, np.uint8)
    row_stride = (k // 32) * 34 if row_stride is None else row_stride
    out = np.empty((rows, k), np.float32)
    _q8_f32(_ptr(blocks), rows, k, row_stride, _ptr(out))
    return out


# ---- Cast / Copy ------------------------------------------------------------
def cast(src_type: int, dst_type: int, storage: np.ndarray, dims, byte_strides=None) -> np.ndarray:
    """Cast a plain tensor held in `storage` (any dtype, read as bytes) with logical `dims` and
    `byte_strides` (dense when omitted) to a dense array of dst_type's storage dtype."""
    dims = [int(d) for d in dims]
    if byte_strides is None:
        step, byte_strides = np.dtype(_NP[src_type]).itemsize, []
        for d in reversed(dims):
            byte_strides.append(step)
            step *= d
        byte_strides = list(reversed(byte_strides))
    raw = np.ascontiguousarray(storage).view(np.uint8).reshape(-1)
    out = np.empty(dims, _NP[dst_type])
    if _cast(src_type, dst_type, _ptr(raw), _i64(dims), _i64(byte_strides), len(dims), _ptr(out)) != 0:
        raise ValueError("the reference does not define this Cast pair")
    return out


# ---- Fill / Select ----------------------------------------------------------
def fill(type_id: int, dims, bits: int) -> np.ndarray:
    """A dense array of `dims` whose every element has the bit pattern `bits`."""
    out = np.empty([int(d) for d in dims], _NP[type_id])
    _fill(out.dtype.itemsize, int(bits), out.size, _ptr(out))
    return out


def select(type_id: int, condition, first, second) -> np.ndarray:
    """Select over operands given as (storage, dims, byte_strides) triples (byte_strides None =
    dense); the condition's elements are single bytes.  Returns the dense result."""
    def operand(triple, width):
        storage, dims, strides = triple
        dims = [int(d) for d in dims]
        if strides is None:
            strides = _byte_strides(dims, width)
        return np.ascontiguousarray(storage).view(np.uint8).reshape(-1), dims, [int(x) for x in strides]
    width = np.dtype(_NP[type_id]).itemsize
    c, a, b = operand(condition, 1), operand(first, width), operand(second, width)
    shape = broadcast_shape(c[1], broadcast_shape(a[1], b[1]))
    out = np.empty(shape, _NP[type_id])
    _select(width, _ptr(c[0]), _i64(c[1]), _i64(c[2]), len(c[1]), _ptr(a[0]), _i64(a[1]), _i64(a[2]), len(a[1]),
            _ptr(b[0]), _i64(b[1]), _i64(b[2]), len(b[1]), _i64(shape), len(shape), _ptr(out))
    return out


# ---- Concat ---------------------------------------------------------------
def concat(type_id: int, parts, axis: int, total: int = 0, start: int = 0, into: np.ndarray | None = None) -> np.ndarray:
    """Concat of `parts` = (storage, dims, byte_strides or None) along `axis`.  `total` / `start`
    place the group inside a wider output (`into`, written in place) as the C ABI's grouped form
    does; by default the output is exactly the parts joined."""
    width = np.dtype(_NP[type_id]).itemsize
    first = [int(d) for d in parts[0][1]]
    axis = axis + len(first) if axis < 0 else axis
    extent = sum(int(p[1][axis]) for p in parts)
    shape = list(first)
    shape[axis] = total if total else extent
    out = into if into is not None else np.zeros(shape, _NP[type_id])
    at = start
    for storage, dims, strides in parts:
        dims = [int(d) for d in dims]
        if strides is None:
            strides = _byte_strides(dims, width)
        raw = np.ascontiguousarray(storage).view(np.uint8).reshape(-1)
        if int(np.prod(dims)) != 0:
            _concat(width, _ptr(raw), _i64(dims), _i64([int(x) for x in strides]), len(dims), axis, at, _i64(shape), _ptr(out))
        at += dims[axis]
    return out


# ---- Gather ---------------------------------------------------------------
def gather(source: np.ndarray, dims, strides, axis: int, indices: np.ndarray, index_dims, index_strides,
           checked: bool = True, into: np.ndarray | None = None, width: int | None = None, wide: bool | None = None):
    """Gather along `axis`.  `source` / `indices` are the storage, described by dims and byte
    strides (None = dense).  The element width and the index width (`wide` = Int64) come from the
    arrays' dtypes unless given, as they must be for raw byte storage.  Returns (status, output):
    status 1 means an index was refused and the output (`into`, or zeros) was left as it was."""
    width = source.dtype.itemsize if width is None else width
    wide = indices.dtype.itemsize == 8 if wide is None else wide
    dims = [int(d) for d in dims]
    index_dims = [int(d) for d in index_dims]
    axis = axis + len(dims) if axis < 0 else axis
    strides = _byte_strides(dims, width) if strides is None else [int(x) for x in strides]
    index_strides = _byte_strides(index_dims, 8 if wide else 4) if index_strides is None else [int(x) for x in index_strides]
    shape = dims[:axis] + index_dims + dims[axis + 1:]
    out = into if into is not None else np.zeros(shape, source.dtype)
    raw = np.ascontiguousarray(source).view(np.uint8).reshape(-1)
    ids = np.ascontiguousarray(indices).view(np.uint8).reshape(-1)
    status = _gather(width, _ptr(raw), _i64(dims), _i64(strides), len(dims), axis, _ptr(ids), 1 if wide else 0,
                     _i64(index_dims), _i64(index_strides), len(index_dims), 1 if checked else 0, _ptr(out))
    return status, out


# ---- Sampling -------------------------------------------------------------
def philox_block(identity, index: int) -> np.ndarray:
    """Words 4 * index .. 4 * index + 3 of the stream of `identity` = (key low, key high, draw low, draw high)."""
    ident = np.ascontiguousarray(identity, np.uint32)
    out = np.empty(4, np.uint32)
    _philox(_ptr(ident), int(index), _ptr(out))
    return out


def random_bits(identities: np.ndarray, word_count: int) -> np.ndarray:
    ident = np.ascontiguousarray(identities, np.uint32).reshape(-1, 4)
    out = np.empty((ident.shape[0], word_count), np.uint32)
    _random_bits(_ptr(ident), ident.shape[0], word_count, _ptr(out))
    return out


def categorical_uniform(identity) -> float:
    return float(_uniform(_ptr(np.ascontiguousarray(identity, np.uint32))))


def categorical(type_id: int, logits: np.ndarray, identities: np.ndarray, scored: bool = False):
    """(status, indices, scores or None); status 1: a row without valid mass, nothing written."""
    logits = _c(logits, _NP[type_id])
    rows, width = logits.shape
    ident = np.ascontiguousarray(identities, np.uint32).reshape(rows, 4)
    indices = np.full(rows, -1, np.int32)
    scores = np.full(rows, np.nan, np.float32) if scored else None
    status = _categorical(type_id, _ptr(logits), _ptr(ident), rows, width, _ptr(indices), _ptr(scores))
    return status, indices, scores


# ---- RoPE -----------------------------------------------------------------
def rope(type_id: int, data: np.ndarray, positions: np.ndarray, frequencies: np.ndarray, rotary: int,
         sequence_axis: int = -2, half_split: bool = False) -> np.ndarray:
    """RoPE over dense `data` (storage dtype of type_id); positions int32 / int64 of rank 1 or the
    data's leading dimensions through the sequence axis; frequencies float32 [rotary / 2] or [S, rotary / 2]."""
    data = _c(data, _NP[type_id])
    positions = np.ascontiguousarray(positions)
    frequencies = np.ascontiguousarray(frequencies, np.float32)
    axis = sequence_axis + data.ndim if sequence_axis < 0 else sequence_axis
    out = np.empty_like(data)
    _rope(type_id, _ptr(data), _i64(data.shape), data.ndim, axis, _ptr(positions), 1 if positions.dtype.itemsize == 8 else 0,
          1 if positions.ndim > 1 else 0, _ptr(frequencies), 1 if frequencies.ndim == 2 else 0, int(rotary),
          1 if half_split else 0, _ptr(out))
    return out
