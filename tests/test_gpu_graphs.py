"""HIP-graph capture of the decode path (restates tests/core/test_graphs.py of the reference for hipGraph): every
launcher only enqueues kernels, so a dense step and a whole MoE layer (router GEMV, device-side top-k, routed expert
GEMVs, SwiGLU, combine) can be captured once and replayed.  Each graph is replayed several times with eager work and
synchronisations in between, on new inputs copied into the captured buffers, and every replay must equal the eager
result bit for bit."""
from __future__ import annotations

import numpy as np
import pytest
import torch

from moe_exact import moe_layer_exact
from orin_qwen_lossless_amd import synth
from test_gpu_kernels import tbf16
from test_gpu_roundtrip import enc

pytestmark = pytest.mark.gpu
NIB, HP = 1, 3


def capture(fn):
    """Warm up on a side stream (lazy initialisation must not happen under capture), then capture fn()."""
    s = torch.cuda.Stream()
    s.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(s):
        fn()
    torch.cuda.current_stream().wait_stream(s)
    torch.cuda.synchronize()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g):
        out = fn()
    return g, out


@pytest.mark.parametrize("T", [1, 2, 4])
def test_dense_step_graph(ops, T):
    K = 2048
    head = enc(ops, synth.weights(16 * 64, K, 61), HP, 16, False, True)   # wave64 GEMV
    qkv = enc(ops, synth.weights(512, K, 62), HP, 8, False, False)         # reference-layout GEMV
    small = enc(ops, synth.weights(512, K, 63), NIB)                       # NIBBLE GEMV
    x = tbf16(synth.activations(T, K, 64))

    def step():
        a = ops.mmv(x, qkv)
        b = ops.mmv(x, small)
        c = ops.linear(x, head)
        return a, b, c

    g, outs = capture(step)
    for rep in range(4):
        x.copy_(tbf16(synth.activations(T, K, 70 + rep)))
        eager = [t.clone() for t in step()]
        torch.cuda.synchronize()
        for t in outs:
            t.zero_()  # eager work between replays; a replay has to rewrite everything
        g.replay()
        torch.cuda.synchronize()
        for got, want in zip(outs, eager):
            assert torch.equal(got, want), rep


@pytest.mark.parametrize("T", [1, 4])
def test_moe_layer_graph(ops, T):
    E, k, K, N = 16, 4, 2048, 512
    # router matrix: E rows would not fill a unit; keep it a NIBBLE matrix of 64 rows and use the first E logits
    router = enc(ops, synth.weights(64, K, 81), NIB)
    gate = enc(ops, synth.weights(E * N, K, 82), HP, 8, True)
    up = enc(ops, synth.weights(E * N, K, 83), HP, 8, True)
    down = enc(ops, synth.weights(E * K, N, 84), HP, 16, False, True)
    x = tbf16(synth.activations(T, K, 85))

    def layer():
        logits = ops.mmv(x, router)[:, :E].contiguous()
        wts, ids = ops.router_topk(logits, k)
        return ops.moe_experts(x, gate, up, down, wts, ids, E), ids

    g, (out, ids) = capture(layer)
    seen = set()
    for rep in range(4):
        x.copy_(tbf16(synth.activations(T, K, 90 + rep)))
        want, want_ids = layer()
        want, want_ids = want.clone(), want_ids.clone()
        torch.cuda.synchronize()
        out.zero_()
        g.replay()
        torch.cuda.synchronize()
        assert torch.equal(ids, want_ids), rep
        assert torch.equal(out, want), rep
        seen.add(tuple(np.sort(ids.cpu().numpy(), axis=None).tolist()))
    assert len(seen) > 1  # the routing changed between replays: it is computed inside the graph
    ref = moe_layer_exact(ops, x, gate, up, down, *ops.router_topk(ops.mmv(x, router)[:, :E].contiguous(), k), E)
    scale = float(ref.float().abs().max())
    assert float((out.float() - ref.float()).abs().max()) <= 2e-2 * scale


@pytest.mark.parametrize("layout,E,T", [("units", 8, 64), ("tiles", 8, 300), ("tiles", 8, 64), ("tiles", 40, 12)])
def test_batched_moe_graph(ops, layout, E, T):
    # routing lists, fused gate/up + SwiGLU and down run as batched kernels inside the graph: 4- and 16-row wave64 units
    # (decode -> LDS tile -> MFMA) and the tile layout in its three shapes (128-token passes at 300 tokens, 32-token
    # passes at 64, K split over wavefronts at 12 tokens of 40 experts); the routing changes from replay to replay
    k, K, N = 2, 2048, 512
    r_gu, r_dn = (4, 16) if layout == "units" else (32, 32)
    gate = enc(ops, synth.weights(E * N, K, 101), HP, r_gu, False, True)
    up = enc(ops, synth.weights(E * N, K, 102), HP, r_gu, False, True)
    down = enc(ops, synth.weights(E * K, N, 103), HP, r_dn, False, True)
    assert ops.mm_ids_supported(gate, up) and ops.mm_ids_supported(down)
    x = tbf16(synth.activations(T, K, 104))
    logits = torch.randn((T, E), generator=torch.Generator().manual_seed(1)).cuda()

    def layer():
        wts, ids = ops.router_topk(logits, k)
        return ops.moe_experts(x, gate, up, down, wts, ids, E)

    g, out = capture(layer)
    for rep in range(3):
        x.copy_(tbf16(synth.activations(T, K, 110 + rep)))
        logits.copy_(torch.randn((T, E), generator=torch.Generator().manual_seed(2 + rep)))
        want = layer().clone()
        torch.cuda.synchronize()
        out.zero_()
        g.replay()
        torch.cuda.synchronize()
        assert torch.equal(out, want), rep
