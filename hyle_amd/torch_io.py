"""Plumbing between torch tensors (device memory, streams) and hyle_amd.compute.

torch only owns the buffers and the stream here; every result is produced by the HIP
kernels of libhyle_hip.so through the C ABI.
"""
from __future__ import annotations

from typing import Optional, Sequence

import torch

from . import compute as hc

_TO_HYLE = {torch.float32: hc.DataType.kFloat32, torch.float16: hc.DataType.kFloat16,
            torch.bfloat16: hc.DataType.kBFloat16, torch.bool: hc.DataType.kBool,
            torch.uint8: hc.DataType.kUInt8, torch.int8: hc.DataType.kInt8,
            torch.int32: hc.DataType.kInt32, torch.float64: hc.DataType.kFloat64,
            torch.int16: hc.DataType.kInt16, torch.int64: hc.DataType.kInt64,
            torch.uint16: hc.DataType.kUInt16, torch.uint32: hc.DataType.kUInt32,
            torch.uint64: hc.DataType.kUInt64, torch.float8_e4m3fn: hc.DataType.kFloat8E4M3FN,
            torch.float8_e5m2: hc.DataType.kFloat8E5M2}
_TO_TORCH = {v: k for k, v in _TO_HYLE.items()}


def desc_of(tensor: torch.Tensor) -> hc.TensorDesc:
    """TensorDesc of a torch tensor: logical dims + byte strides (0 on expanded axes)."""
    dtype, shape = _TO_HYLE[tensor.dtype], tuple(tensor.shape)
    dense = hc.TensorDesc.dense(dtype, shape)
    if 0 in shape:
        return dense
    size = tensor.element_size()
    # torch leaves the stride of an extent-1 axis arbitrary; the descriptor wants the canonical one
    strides = tuple(c if d == 1 else s * size
                    for d, s, c in zip(shape, tensor.stride(), dense.byte_strides))
    return hc.TensorDesc.strided_bytes(dtype, shape, strides)


def empty_like_desc(desc: hc.TensorDesc, device) -> torch.Tensor:
    return torch.empty(desc.dimensions, dtype=_TO_TORCH[desc.data_type], device=device)


def current_stream_handle(device=None) -> int:
    return torch.cuda.current_stream(device).cuda_stream


class Bound:
    """A prepared operation with its workspace, ready to be submitted repeatedly."""

    def __init__(self, context: hc.Context, operation, input_descs: Sequence[hc.TensorDesc], device="cuda:0"):
        self.prepared = hc.prepare(context, operation, *input_descs)
        req = self.prepared.workspace_requirement()
        self.workspace: Optional[torch.Tensor] = None
        if req.size:
            self.workspace = torch.empty(req.size, dtype=torch.uint8, device=device)  # 512-byte aligned
        ptr = self.workspace.data_ptr() if self.workspace is not None else 0
        self.invocation = self.prepared.create_invocation(ptr, req.size)
        self.device = device

    def outputs(self) -> list:
        return [empty_like_desc(d, self.device) for d in self.prepared.output_descriptions()]

    def submit(self, inputs: Sequence[torch.Tensor], outputs: Sequence[torch.Tensor], stream: Optional[int] = None):
        handle = current_stream_handle() if stream is None else stream
        self.invocation.submit(handle, [t.data_ptr() for t in inputs], [t.data_ptr() for t in outputs])


def run(context: hc.Context, operation, *inputs: torch.Tensor, outputs: Optional[Sequence[torch.Tensor]] = None,
        descs: Optional[Sequence[hc.TensorDesc]] = None):
    """prepare + create_invocation + submit on torch's current stream; returns the outputs."""
    descs = list(descs) if descs is not None else [desc_of(t) for t in inputs]
    bound = Bound(context, operation, descs, device=inputs[0].device if inputs else "cuda:0")
    outs = list(outputs) if outputs is not None else bound.outputs()
    bound.submit(inputs, outs)
    # the workspace must outlive the enqueued kernels
    torch.cuda.current_stream().synchronize()
    bound.invocation.wait(current_stream_handle())  # the device's verdict, where the route has one
    return outs
