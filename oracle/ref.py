"""ctypes binding of oracle/_ref/libhyle_ref_scalar.so: the reference's own
scalar semantic floor, compiled from its sources by oracle/Makefile.

Test infrastructure only; used to validate oracle/hyle_oracle.c bit for bit.
`available()` is False where the library was never built (no reference tree).
"""
from __future__ import annotations

import ctypes as C
import os

import numpy as np

_SO = os.path.join(os.path.dirname(os.path.abspath(__file__)), "_ref", "libhyle_ref_scalar.so")
_lib = C.CDLL(_SO) if os.path.exists(_SO) else None

_vp, _sz = C.c_void_p, C.c_size_t


def available() -> bool:
    return _lib is not None


def _fn(name, restype, *argtypes):
    fn = getattr(_lib, name)
    fn.restype, fn.argtypes = restype, list(argtypes)
    return fn


def _p(a):
    return None if a is None else a.ctypes.data_as(_vp)


def f16_to_f32(bits: np.ndarray) -> np.ndarray:
    bits = np.ascontiguousarray(bits, np.uint16)
    out = np.empty(bits.shape, np.float32)
    _fn("ref_f16_to_f32_n", None, _vp, _vp, _sz)(_p(bits), _p(out), bits.size)
    return out


def f32_to_f16(values: np.ndarray) -> np.ndarray:
    values = np.ascontiguousarray(values, np.float32)
    out = np.empty(values.shape, np.uint16)
    _fn("ref_f32_to_f16_n", None, _vp, _vp, _sz)(_p(values), _p(out), values.size)
    return out


def f32_to_bf16(values: np.ndarray) -> np.ndarray:
    values = np.ascontiguousarray(values, np.float32)
    out = np.empty(values.shape, np.uint16)
    _fn("ref_f32_to_bf16_n", None, _vp, _vp, _sz)(_p(values), _p(out), values.size)
    return out


_SUFFIX = {0: "f32", 1: "f16", 2: "bf16"}


def silu(type_id: int, src: np.ndarray) -> np.ndarray:
    src = np.ascontiguousarray(src)
    out = np.empty_like(src)
    _fn(f"ref_silu_{_SUFFIX[type_id]}", None, _vp, _vp, _sz)(_p(src), _p(out), src.size)
    return out


def swiglu(type_id: int, gate: np.ndarray, value: np.ndarray) -> np.ndarray:
    gate, value = np.ascontiguousarray(gate), np.ascontiguousarray(value)
    out = np.empty_like(gate)
    _fn(f"ref_swiglu_{_SUFFIX[type_id]}", None, _vp, _vp, _vp, _sz)(
        _p(gate), _p(value), _p(out), gate.size)
    return out


def rms_norm_row(type_id: int, src: np.ndarray, weight, epsilon: float) -> np.ndarray:
    src = np.ascontiguousarray(src)
    weight = None if weight is None else np.ascontiguousarray(weight)
    out = np.empty_like(src)
    _fn(f"ref_rms_norm_{_SUFFIX[type_id]}", None, _vp, _vp, _vp, _sz, C.c_float)(
        _p(src), _p(weight), _p(out), src.size, float(epsilon))
    return out


def activation(name: str, type_id: int, src: np.ndarray) -> np.ndarray:
    """name: gelu, gelu_tanh (f32/f16/bf16), sigmoid, relu (f32)."""
    src = np.ascontiguousarray(src)
    out = np.empty_like(src)
    _fn(f"ref_{name}_{_SUFFIX[type_id]}", None, _vp, _vp, _sz)(_p(src), _p(out), src.size)
    return out


def gated(name: str, type_id: int, gate: np.ndarray, value: np.ndarray) -> np.ndarray:
    """name: geglu, geglu_tanh (f32/bf16)."""
    gate, value = np.ascontiguousarray(gate), np.ascontiguousarray(value)
    out = np.empty_like(gate)
    _fn(f"ref_{name}_{_SUFFIX[type_id]}", None, _vp, _vp, _vp, _sz)(_p(gate), _p(value), _p(out), gate.size)
    return out


def layer_norm_row(type_id: int, src: np.ndarray, scale, bias, epsilon: float) -> np.ndarray:
    src = np.ascontiguousarray(src)
    scale = None if scale is None else np.ascontiguousarray(scale)
    bias = None if bias is None else np.ascontiguousarray(bias)
    out = np.empty_like(src)
    _fn(f"ref_layer_norm_{_SUFFIX[type_id]}", None, _vp, _vp, _vp, _vp, _sz, C.c_float)(
        _p(src), _p(scale), _p(bias), _p(out), src.size, float(epsilon))
    return out


def softmax_f32(src: np.ndarray) -> np.ndarray:
    src = np.ascontiguousarray(src, np.float32)
    out = np.empty_like(src)
    _fn("ref_softmax_f32", None, _vp, _vp, _sz)(_p(src), _p(out), src.size)
    return out


def log_softmax_f32(src: np.ndarray) -> np.ndarray:
    src = np.ascontiguousarray(src, np.float32)
    out = np.empty_like(src)
    _fn("ref_log_softmax_f32", None, _vp, _vp, _sz)(_p(src), _p(out), src.size)
    return out
