"""The launches are capture-compatible (ProviderRuntimeProperties::capture_compatible,
include/hyle/compute/provider.h:136-139): a captured HIP graph of the hot-path kernels replays
to the same bits as eager submission, replay after replay, with eager work in between."""
from __future__ import annotations

import numpy as np
import pytest
import torch

from hyle_amd import compute as hc
from hyle_amd import torch_io as tio
from hyle_amd import workloads as wl

from gpu_support import DEVICE, context, note, to_device, to_host

pytestmark = pytest.mark.gpu


def test_captured_step_replays_bit_identically():
    ctx = context()
    x, w = wl.config2(rows=512)
    gate, up = wl.config3_swiglu(rows=64)
    logits = wl.config4_argmax(rows=8)
    s, mask = wl.config4_softmax(heads=2, seq=256)
    blocks = wl.config5(rows=128)
    dx, dw = to_device(x, "bf16"), to_device(w, "bf16")
    dg, du = to_device(gate, "bf16"), to_device(up, "bf16")
    dl = to_device(logits, "f32")
    ds = to_device(s, "f32")
    dm = torch.from_numpy(mask).to(DEVICE).view(torch.bool)
    db = torch.from_numpy(blocks).to(DEVICE)

    ops = [
        (tio.Bound(ctx, hc.RmsNorm(1e-6), [tio.desc_of(dx), tio.desc_of(dw)]), [dx, dw]),
        (tio.Bound(ctx, hc.GatedActivation(hc.GatedActivationKind.kSilu, hc.GatedInputKind.kSeparate),
                   [tio.desc_of(dg), tio.desc_of(du)]), [dg, du]),
        (tio.Bound(ctx, hc.TopK(), [tio.desc_of(dl)]), [dl]),
        (tio.Bound(ctx, hc.Softmax(mask=hc.MaskKind.kBoolean), [tio.desc_of(ds), tio.desc_of(dm)]), [ds, dm]),
        (tio.Bound(ctx, hc.Q8_0DequantSumSquares(), [hc.TensorDesc.gguf_q8_0_weight(hc.DataType.kBFloat16, 2048, 128)]),
         [db]),
    ]
    note("eager pass of rmsnorm, swiglu, argmax, softmax, q8_0")
    eager_outs = []
    for bound, inputs in ops:
        outs = bound.outputs()
        bound.submit(inputs, outs)
        eager_outs.append(outs)
    torch.cuda.synchronize()
    want = [[to_host(t).copy() for t in outs] for outs in eager_outs]

    note("capture the same five launches into one HIP graph")
    graph_outs = [bound.outputs() for bound, _ in ops]
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        stream = torch.cuda.current_stream().cuda_stream
        for (bound, inputs), outs in zip(ops, graph_outs):
            bound.submit(inputs, outs, stream=stream)
    for replay in range(3):
        note(f"graph replay {replay}")
        for outs in graph_outs:
            for t in outs:
                t.zero_()
        # unrelated eager work and a synchronisation between replays
        scratch = torch.randn(1 << 20, device=DEVICE).sum().item()
        assert np.isfinite(scratch)
        graph.replay()
        torch.cuda.synchronize()
        for outs, expected in zip(graph_outs, want):
            for t, e in zip(outs, expected):
                got = to_host(t)
                assert np.array_equal(got.view(np.uint8), e.view(np.uint8))


def test_captured_two_dispatch_routes_replay_bit_identically():
    """The routes that pass partial results through the caller's workspace (Reduce over few long
    rows or over columns, TopK by selection and by sorted tiles, Gather with checked indices), plus
    Cast, LayerNorm, LogSoftmax, the K-quant decoder, Concat, Select, Categorical and RandomBits:
    captured once, replayed three times, same bits as eager."""
    ctx = context()
    rng = np.random.default_rng(1600)
    f32 = hc.DataType.kFloat32
    long_rows = to_device(rng.normal(0, 1, (2, 300000)).astype(np.float32), "f32")
    columns = to_device(rng.normal(0, 1, (70000, 8)).astype(np.float32), "f32")
    logits = to_device(rng.normal(0, 3, (4, 40000)).astype(np.float32), "f32")
    hidden = to_device(rng.normal(0, 1, (64, 2048)).astype(np.float32), "f32")
    raw = torch.randint(0, 256, (32, 8 * 144), dtype=torch.uint8)
    raw.view(32, 8, 144)[:, :, 1] &= 0x3B
    raw.view(32, 8, 144)[:, :, 3] &= 0x3B
    weights = raw.to(DEVICE)
    table = to_device(rng.normal(0, 1, (5000, 256)).astype(np.float32), "f32")
    ids = torch.from_numpy(rng.integers(0, 5000, 3000).astype(np.int32)).to(DEVICE)
    flags = torch.from_numpy(rng.integers(0, 2, (64, 2048)).astype(np.uint8)).to(DEVICE).view(torch.bool)
    keys = torch.from_numpy(rng.integers(0, 1 << 31, (4, 4)).astype(np.int32)).to(DEVICE)
    key_desc = hc.TensorDesc.dense(hc.DataType.kUInt32, [4, 4])
    ops = [
        (hc.Reduce(hc.ReductionKind.kSum, hc.Axes.from_([-1])), [long_rows], None),
        (hc.Reduce(hc.ReductionKind.kMaximum, hc.Axes.from_([0])), [columns], None),
        (hc.TopK(count=16), [logits], None),
        (hc.TopK(count=300, largest=False), [logits], None),
        (hc.Cast(hc.DataType.kBFloat16), [hidden], None),
        (hc.LayerNorm(1e-5), [hidden], None),
        (hc.Softmax(kind=hc.SoftmaxKind.kLogSoftmax), [hidden], None),
        (hc.GgufDequantSumSquares(), [weights],
         [hc.TensorDesc.gguf_weight(hc.GgufQuantizedType.kQ4K, hc.DataType.kBFloat16, 2048, 32)]),
        (hc.Gather(0), [table, ids], None),   # checked: the flags of the first dispatch live in the workspace
        (hc.Concat(-1), [hidden, hidden], None),
        (hc.Select(), [flags, hidden, torch.zeros((), device=DEVICE)], None),
        (hc.Categorical(True), [logits, keys], [tio.desc_of(logits), key_desc]),   # tile records and the status word
        (hc.RandomBits(33), [keys], [key_desc]),
    ]
    bounds = [(tio.Bound(ctx, op, descs or [tio.desc_of(t) for t in inputs]), inputs) for op, inputs, descs in ops]
    routes = [b.prepared.route_name() for b, _ in bounds]
    assert routes[:4] == ["reduce-row-tiles", "reduce-column-segments", "topk-select-tiles", "topk-sorted-tiles"]
    note("eager pass of " + ", ".join(routes))
    eager_outs = []
    for bound, inputs in bounds:
        outs = bound.outputs()
        bound.submit(inputs, outs)
        eager_outs.append(outs)
    torch.cuda.synchronize()
    want = [[to_host(t).copy() for t in outs] for outs in eager_outs]

    note("capture the same launches into one HIP graph")
    graph_outs = [bound.outputs() for bound, _ in bounds]
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        stream = torch.cuda.current_stream().cuda_stream
        for (bound, inputs), outs in zip(bounds, graph_outs):
            bound.submit(inputs, outs, stream=stream)
    for replay in range(3):
        note(f"graph replay {replay} of the two-dispatch routes")
        for outs in graph_outs:
            for t in outs:
                t.zero_()
        for bound, _ in bounds:                      # stale partial results must not matter
            if bound.workspace is not None:
                bound.workspace.fill_(0xFF if replay % 2 else 0)
        scratch = torch.randn(1 << 20, device=DEVICE).sum().item()
        assert np.isfinite(scratch)
        graph.replay()
        torch.cuda.synchronize()
        for bound, _ in bounds:                      # the device's verdict (checked Gather): accepted
            bound.invocation.wait(tio.current_stream_handle())
        for outs, expected in zip(graph_outs, want):
            for t, e in zip(outs, expected):
                got = to_host(t)
                assert np.array_equal(got.view(np.uint8), e.view(np.uint8))
