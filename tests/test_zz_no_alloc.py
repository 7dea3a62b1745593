"""hyle_hip_plan_launch_static: the launch for callers that cannot allocate.  The workspace of the
two-dispatch routes is the library's per-device scratch array; results must equal those of
hyle_hip_plan_launch with a caller-owned workspace bit for bit, also on a second call with a
smaller input that finds the first call's contents in the array."""
from __future__ import annotations

import numpy as np
import pytest
import torch

from hyle_amd import capi
from hyle_amd import compute as hc
from hyle_amd import torch_io as tio

from gpu_support import DEVICE, context, note

pytestmark = pytest.mark.gpu

F32 = hc.DataType.kFloat32


def _both_ways(operation, x: torch.Tensor):
    """Outputs of the caller-workspace launch and of the static-scratch launch."""
    bound = tio.Bound(context(), operation, [tio.desc_of(x)], device=x.device)
    assert bound.prepared.workspace_requirement().size > 0, "the case must be a route that uses a workspace"
    assert bound.prepared.workspace_requirement().size <= capi.load().hyle_hip_static_scratch_bytes()
    stream = tio.current_stream_handle()
    wanted = bound.outputs()
    bound.submit([x], wanted)
    got = bound.outputs()
    for t in got:
        t.fill_(-7)  # stale contents must be overwritten
    invocation = bound.prepared.create_invocation_without_workspace()
    invocation.submit_without_workspace(stream, [x.data_ptr()], [t.data_ptr() for t in got])
    torch.cuda.current_stream().synchronize()
    return wanted, got


def _assert_same(wanted, got):
    for w, g in zip(wanted, got):
        assert w.shape == g.shape and w.dtype == g.dtype
        wb, gb = (t.contiguous().reshape(-1).view(torch.uint8).cpu().numpy() for t in (w, g))
        assert np.array_equal(wb, gb), "static-scratch launch differs from the workspace launch"


@pytest.mark.parametrize("operation,first,second", [
    (lambda: hc.TopK(count=64), (64, 40000), (8, 36000)),
    (lambda: hc.TopK(), (64, 151936), (4, 3000)),
    (lambda: hc.Reduce(hc.ReductionKind.kMaximum, hc.Axes.all(), accumulation_type=F32), (4096, 4096), (1024, 2048)),
], ids=["topk64", "argmax", "reduce-max-all"])
def test_static_scratch_launch_matches_workspace_launch_twice(operation, first, second):
    rng = np.random.default_rng(11)
    for shape in (first, second):  # the second, smaller call meets the first call's leftovers
        note(f"launch_static {operation().__class__.__name__} {shape}")
        x = torch.from_numpy(rng.standard_normal(shape, dtype=np.float32)).to(DEVICE)
        wanted, got = _both_ways(operation(), x)
        _assert_same(wanted, got)
        if isinstance(operation(), hc.TopK):
            values, indices = got
            order = torch.sort(x, dim=-1, descending=True, stable=True)
            k = values.shape[-1]
            assert torch.equal(values, order.values[:, :k])
            assert torch.equal(indices.long(), order.indices[:, :k])


def test_static_scratch_launch_refuses_plans_beyond_the_array():
    big = hc.prepare(context(), hc.TopK(count=1024), hc.TensorDesc.dense(F32, [4096, 65536]))
    limit = capi.load().hyle_hip_static_scratch_bytes()
    assert big.workspace_requirement().size > limit
    invocation = big.create_invocation_without_workspace()
    with pytest.raises(hc.StatusError) as refused:
        invocation.submit_without_workspace(tio.current_stream_handle(), [256], [256, 256])
    assert refused.value.code == capi.RESOURCE_EXHAUSTED
    assert "workspace" in str(refused.value)


def test_static_scratch_launch_serves_routes_without_workspace():
    x = torch.from_numpy(np.random.default_rng(3).standard_normal((64, 256), dtype=np.float32)).to(DEVICE)
    bound = tio.Bound(context(), hc.Unary(hc.UnaryKind.kRelu), [tio.desc_of(x)], device=x.device)
    assert bound.prepared.workspace_requirement().size == 0
    (out,) = bound.outputs()
    bound.prepared.create_invocation_without_workspace().submit_without_workspace(
        tio.current_stream_handle(), [x.data_ptr()], [out.data_ptr()])
    torch.cuda.current_stream().synchronize()
    assert torch.equal(out, torch.relu(x))
