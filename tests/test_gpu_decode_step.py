"""The 40-layer decode step (the full decode-step weight stream: per layer qkv, o, router, top-8 of 256 experts + the
shared one, glue; the reference's engines own this composition and replay it as a CUDA graph, tests/core/test_graphs.py)
captured as one HIP graph at 1 and 4 tokens on seeded weights of the benchmark's generator: every replay on new
activations equals the eager step bit for bit, every one of the 40 layers is checked against an FP64 evaluation on the
exact weights that rounds where the step rounds (BF16 between the launches), and the final hidden state against the
same 40 layers evaluated in FP64 from the first input on, within the BF16 roundings of the residual stream."""
from __future__ import annotations

import pytest
import torch

pytestmark = pytest.mark.gpu

N_LAYERS, N_SETS = 40, 8


@pytest.fixture(scope="module")
def sets40(ops):
    from orin_qwen_lossless_amd import decode_step as D, synth

    seed = [5000]

    def gen(rows, k):
        seed[0] += 1
        return synth.weights_torch(rows, k, seed[0], "cuda")

    sets, raw, _ = D.make_layer_sets(ops, gen, N_SETS, True)
    return sets, raw


def rn(t):
    return t.float().to(torch.bfloat16).double()


def rms(t):
    return t * torch.rsqrt((t * t).mean(-1, keepdim=True) + 1e-6)


def layer_fp64(D, r, h, x1, ids, hidden_bf16):
    """One layer in FP64 on the exact weights r (BF16 tensors), rounding to BF16 where the step does, with the experts
    `ids` [T, 9] the step chose.  h, x1: FP64 values of BF16 numbers.  Returns (x1', h', logits, weights)."""
    T = h.shape[0]
    q = rn(x1 @ r["qkv"].double().t())
    o = rn(q[:, :D.ATT] @ r["o"].double().t())
    s = h + o
    h2, x2 = rn(s), rn(rms(s))
    logits = x2 @ r["router"].double().t()
    p = torch.softmax(logits, -1)
    wts = torch.ones((T, D.TOPK + 1), dtype=torch.float64, device=h.device)
    sel = p.gather(1, ids[:, :D.TOPK].long())
    wts[:, :D.TOPK] = sel / sel.sum(-1, keepdim=True)
    comb = torch.zeros_like(h)
    for t in range(T):
        for k in range(D.TOPK + 1):
            e = int(ids[t, k])
            g = r["gate"][e * D.N_MID:(e + 1) * D.N_MID].double() @ x2[t]
            u = r["up"][e * D.N_MID:(e + 1) * D.N_MID].double() @ x2[t]
            hid = g / (1.0 + torch.exp(-g)) * u
            hid = rn(hid) if hidden_bf16 else hid.float().double()  # the batched kernels hand BF16 to the down product
            comb[t] += wts[t, k] * (r["down"][e * D.K_MODEL:(e + 1) * D.K_MODEL].double() @ hid)
    s2 = h2 + comb
    return rn(rms(s2)), rn(s2), logits, wts


@pytest.mark.parametrize("T", [1, 4])
def test_forty_layer_decode_step_as_one_graph(ops, sets40, T):
    from orin_qwen_lossless_amd import decode_step as D, synth

    sets, raw = sets40
    step = D.Bf16nStep(ops, sets, None, N_LAYERS, T)
    hs = [synth.activations_torch(T, D.K_MODEL, 5100 + i, "cuda") for i in range(3)]
    hbuf = hs[0].clone()
    graph, out = D.capture(step, hbuf)
    for rep in (1, 2):  # two replays on changed input, each against the eager step
        hbuf.copy_(hs[rep])
        want = step(hbuf).clone()
        torch.cuda.synchronize()
        out.zero_()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out, want), rep
    # the same step launch by launch (what the graph holds), every layer's input, routing and output kept
    batched = ops.moe_experts_batched(T, D.TOPK + 1, sets[0]["gate"], sets[0]["up"], sets[0]["down"], D.EA)
    h = hs[2]
    x1 = ops.add_rmsnorm(h)
    h_ref, x1_ref = h.double(), rn(rms(h.double()))   # the free-running FP64 evaluation
    assert bool(((x1.double() - x1_ref).abs() <= 2.0 ** -8 * x1_ref.abs()).all())
    for i in range(N_LAYERS):
        w, r = sets[i % N_SETS], raw[i % N_SETS]
        x1n, hn = step.layer(w, h, x1)
        wts, ids = (t.clone() for t in step.routing)
        assert bool((ids[:, D.TOPK] == D.E).all()) and bool((wts[:, D.TOPK] == 1.0).all())
        assert all(len(set(ids[t, :D.TOPK].tolist())) == D.TOPK and int(ids[t, :D.TOPK].max()) < D.E for t in range(T))
        # this layer alone, from the step's own input: tight
        xe, he, logits, wref = layer_fp64(D, r, h.double(), x1.double(), ids, batched)
        kth = torch.topk(logits, D.TOPK, dim=-1).values[:, -1:]
        chosen = logits.gather(1, ids[:, :D.TOPK].long())
        assert bool((chosen >= kth - 1e-2 * logits.abs().max()).all()), i   # the step's experts are a top-8 of the FP64 logits
        assert bool(((wts.double() - wref).abs() <= 2e-2 * wref + 1e-4).all()), i
        scale = float(he.abs().max())
        assert bool(((hn.double() - he).abs() <= 2.0 ** -6 * he.abs() + 2e-3 * scale).all()), i
        assert bool(((x1n.double() - xe).abs() <= 2.0 ** -6 * xe.abs() + 2e-3 * float(xe.abs().max())).all()), i
        # the FP64 evaluation goes its own way from the first input on, with the experts the step chose
        x1_ref, h_ref, _, _ = layer_fp64(D, r, h_ref, x1_ref, ids, batched)
        h, x1 = hn, x1n
    assert torch.equal(x1, out)  # hs[2] was the last replay's input: the graph's output is this chain's
    # final state after 40 layers: the roundings of the residual stream (BF16, 2^-9 relative per element and launch
    # boundary) add up along the layers; the deviation stays a small fraction of the state's size
    err = (h.double() - h_ref).norm() / h_ref.norm()
    assert float(err) <= 0.02, float(err)
    errx = (x1.double() - x1_ref).norm() / x1_ref.norm()
    assert float(errx) <= 0.02, float(errx)
