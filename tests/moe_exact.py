"""Test helper: one MoE layer's routed experts evaluated on the exactly decoded weights, for comparison with the fused
kernels.  Plays the part of the reference's moe_experts_reference (engines/vllm/vllm_bf16n/ops.py:274-287); it lives with
the tests because nothing in the product uses it."""
from __future__ import annotations

import torch


def moe_layer_exact(ops, x, gate, up, down, topk_weights, topk_ids, n_experts):
    """x [T, K] BF16; gate / up / down: encoded expert stacks; topk_ids / topk_weights [T, k].  Returns [T, H] BF16:
    sum over a token's slots of weight * down_e(silu(gate_e x) * (up_e x)), FP32 arithmetic on dequantised weights, no
    rounding of the hidden activations."""
    n_tok, k = topk_ids.shape
    n_mid = gate.meta.rows // n_experts
    n_out = down.meta.rows // n_experts
    flat_ids = topk_ids.reshape(-1).long()
    flat_w = topk_weights.reshape(-1).float()
    order = torch.argsort(flat_ids, stable=True)              # pairs grouped by expert, token order inside a group
    counts = torch.bincount(flat_ids, minlength=n_experts).tolist()
    acc = torch.zeros((n_tok, n_out), dtype=torch.float32, device=x.device)
    start = 0
    for e, c in enumerate(counts):
        if c == 0:
            continue
        pairs = order[start: start + c]
        start += c
        tokens = torch.div(pairs, k, rounding_mode="floor")
        xe = x.index_select(0, tokens).float()
        w_gate = ops.dequant(gate, e * n_mid, n_mid).float()
        w_up = ops.dequant(up, e * n_mid, n_mid).float()
        w_down = ops.dequant(down, e * n_out, n_out).float()
        hidden = torch.nn.functional.silu(xe @ w_gate.t()) * (xe @ w_up.t())
        acc.index_add_(0, tokens, (hidden @ w_down.t()) * flat_w[pairs].unsqueeze(1))
    return acc.to(torch.bfloat16)
