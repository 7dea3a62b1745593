"""Shared plumbing of the GPU parity tests: torch owns device buffers, every result comes
from libhyle_hip.so through its C ABI, and the checker is the CPU oracle."""
from __future__ import annotations

import functools
import sys

import numpy as np
import torch

from hyle_amd import compute as hc
from hyle_amd import torch_io as tio
from oracle import lib as orc

DEVICE = "cuda:0"

TYPES = {
    "f32": (hc.DataType.kFloat32, orc.F32, torch.float32),
    "bf16": (hc.DataType.kBFloat16, orc.BF16, torch.bfloat16),
    "f16": (hc.DataType.kFloat16, orc.F16, torch.float16),
}


def note(message: str) -> None:
    """Name the case before its GPU step, flushed, so a lost box still tells which one ran."""
    print(f"[gpu-case] {message}", file=sys.stderr, flush=True)


@functools.lru_cache(maxsize=1)
def context() -> hc.Context:
    if not torch.cuda.is_available():
        raise RuntimeError("GPU tests selected but no HIP device is visible")
    return hc.Context.create(0)


def to_device(array: np.ndarray, tag: str) -> torch.Tensor:
    """numpy (float32, or uint16 bit patterns for narrow types) -> device tensor."""
    array = np.ascontiguousarray(array)
    if tag == "f32":
        return torch.from_numpy(array).to(DEVICE)
    torch_dtype = TYPES[tag][2]
    return torch.from_numpy(array.view(np.int16)).to(DEVICE).view(torch_dtype)


def to_host(tensor: torch.Tensor) -> np.ndarray:
    """device tensor -> numpy float32 / uint16 bit patterns / integer arrays."""
    if tensor.dtype in (torch.bfloat16, torch.float16):
        return tensor.contiguous().view(torch.int16).cpu().numpy().view(np.uint16)
    return tensor.contiguous().cpu().numpy()


def host_values(array: np.ndarray, tag: str) -> np.ndarray:
    """float32 values -> storage representation of `tag` (through the oracle's codec)."""
    array = np.ascontiguousarray(array, np.float32)
    return array if tag == "f32" else orc.from_f32(TYPES[tag][1], array)


# Labels of the kernel launch shapes the tests of this session launched (hyle_hip_last_launch_variant
# after every submit): tests/test_zy_launch_shape_coverage.py holds them against the list of shapes
# compiled into the library.
LAUNCHED = set()


def _noting(submit):
    @functools.wraps(submit)
    def noted(self, *args, **kwargs):
        submit(self, *args, **kwargs)
        chosen = hc.last_launch_variant()
        if chosen:
            LAUNCHED.update(chosen.split(" + "))
    return noted


# every launch a GPU test makes goes through one of these two, whichever helper it uses
hc.OperationInvocation.submit = _noting(hc.OperationInvocation.submit)
hc.OperationInvocation.submit_without_workspace = _noting(hc.OperationInvocation.submit_without_workspace)


def run(operation, *tensors, descs=None, outputs=None):
    return tio.run(context(), operation, *tensors, descs=descs, outputs=outputs)


# ---- comparisons ----------------------------------------------------------------------------
def ordered16(bits: np.ndarray) -> np.ndarray:
    """Sign-magnitude 16-bit float patterns -> integers ordered like the values (+-0 -> 0)."""
    bits = bits.astype(np.int32)
    return np.where(bits & 0x8000, -(bits & 0x7FFF), bits)


def assert_bits_equal(got: np.ndarray, want: np.ndarray, nan_payload_free: bool = True) -> None:
    """Bit-exact, except that any NaN matches any NaN when nan_payload_free."""
    got, want = np.asarray(got), np.asarray(want)
    assert got.shape == want.shape, (got.shape, want.shape)
    if got.dtype == np.float32:
        gb, wb = got.view(np.uint32), want.view(np.uint32)
        g_nan, w_nan = np.isnan(got), np.isnan(want)
    else:
        gb, wb = got, want
        g_nan = w_nan = None
    if nan_payload_free and g_nan is not None:
        assert np.array_equal(g_nan, w_nan)
        bad = (gb != wb) & ~w_nan
    else:
        bad = gb != wb
    if bad.any():
        at = np.argwhere(bad)[0]
        raise AssertionError(f"{int(bad.sum())} mismatches, first at {tuple(at)}: "
                             f"got {gb[tuple(at)]:#x} want {wb[tuple(at)]:#x}")


def narrow_is_nan(bits: np.ndarray, tag: str) -> np.ndarray:
    bits = bits.astype(np.uint32) & 0x7FFF
    return bits > (0x7F80 if tag == "bf16" else 0x7C00)


def assert_narrow_ulp(got: np.ndarray, want: np.ndarray, tag: str, ulps: int = 1) -> int:
    """Narrow float bit patterns within `ulps` units in the last place; NaN matches NaN; where
    both are zeros they must be the same zero (+0 and -0 are zero units apart but not equal).
    Returns how many elements differ at all."""
    g_nan, w_nan = narrow_is_nan(got, tag), narrow_is_nan(want, tag)
    assert np.array_equal(g_nan, w_nan), "NaN positions differ"
    zeros = ((got & 0x7FFF) == 0) & ((want & 0x7FFF) == 0) & (got != want)
    if zeros.any():
        at = tuple(np.argwhere(zeros)[0])
        raise AssertionError(f"{int(zeros.sum())} zeros of the wrong sign, first at {at}: "
                             f"got {got[at]:#06x} want {want[at]:#06x}")
    diff = np.abs(ordered16(got) - ordered16(want))
    diff[w_nan] = 0
    worst = int(diff.max()) if diff.size else 0
    if worst > ulps:
        at = tuple(np.argwhere(diff == worst)[0])
        raise AssertionError(f"max {worst} ulp at {at}: got {got[at]:#06x} want {want[at]:#06x}")
    return int((diff != 0).sum())


def assert_close_f32(got: np.ndarray, want: np.ndarray, rel: float, abs_floor: float = 0.0) -> None:
    """|got - want| <= rel * |want| + abs_floor; NaN/inf must match exactly."""
    got, want = np.asarray(got, np.float32), np.asarray(want, np.float32)
    assert got.shape == want.shape
    w_nan = np.isnan(want)
    assert np.array_equal(np.isnan(got), w_nan), "NaN positions differ"
    w_inf = np.isinf(want)
    assert np.array_equal(got[w_inf], want[w_inf]), "infinities differ"
    ok = ~(w_nan | w_inf)
    g, w = got[ok].astype(np.float64), want[ok].astype(np.float64)
    err = np.abs(g - w)
    limit = rel * np.abs(w) + abs_floor
    if (err > limit).any():
        i = int(np.argmax(err - limit))
        raise AssertionError(f"got {g[i]!r} want {w[i]!r} (err {err[i]:.3e} > {limit[i]:.3e})")
