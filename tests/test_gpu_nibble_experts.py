"""Experts in the 4-bit code (NIBBLE, rows of all experts stacked) through the batched matrix-core kernel
(bf16n_mm_ids -> k_nib_mm_ids): the fused gate / up + SwiGLU product and the down product against FP64 products of the
exact weights, at every pass length (32 / 64 / 128 tokens), with ragged passes, an expert that every token uses,
experts without tokens, escaped weights, and row groups that do not fill the last slab.  The reference's batched kernel
(core/src/kernels.cuh:1162-1505) does not take this format; the operator's contract is the same."""
from __future__ import annotations

import numpy as np
import pytest
import torch

from orin_qwen_lossless_amd import synth

pytestmark = pytest.mark.gpu


def nib(ops, w):
    bits = w.cpu().view(torch.int16).numpy().view(np.uint16)
    plane, aux, fmt, _ = ops.encode_bits(bits, 1, 0)
    assert fmt == 1
    ta = torch.from_numpy(aux)
    return ops.upload(torch.from_numpy(plane), ta, ops.parse_header(ta), "cuda")


def silu64(v):
    return v / (1.0 + torch.exp(-v))


@pytest.mark.parametrize("E,N,K,T,topk,popular", [
    (16, 64, 512, 5, 4, False),      # 32-token passes, a short matrix: two row groups of gate / up, one slab
    (16, 96, 1024, 40, 4, True),     # an expert with 40 tokens: two passes of 32; 3 row groups
    (8, 512, 2048, 300, 4, False),   # 150 pairs per expert: passes of 128, the last ragged; the down product too
    (32, 160, 512, 600, 2, False),   # 37 pairs per expert: passes of 64; 5 row groups: the last slab is not full
    (16, 512, 512, 9, 4, False),     # gate / up and down, 32-token passes
    (64, 64, 512, 3, 2, False),      # most experts without tokens
])
def test_batched_products_of_experts_in_the_4_bit_code(ops, E, N, K, T, topk, popular):
    g = torch.Generator(device="cuda").manual_seed(E * 1000 + T)
    wg = synth.weights_torch(E * N, K, 11 + T, "cuda")
    wu = synth.weights_torch(E * N, K, 12 + T, "cuda")
    wd = synth.weights_torch(E * K, N, 13 + T, "cuda") if N % 512 == 0 else None  # (the down product has K = N)
    for w in (wg, wu, wd):  # exponents outside a row's window: escape records in some rows of some experts
        if w is not None:
            w.view(torch.int16)[::7, ::53] = 0x4500
    gate, up, down = nib(ops, wg), nib(ops, wu), nib(ops, wd) if wd is not None else None
    assert ops.mm_ids_supported(gate, up) and (down is None or ops.mm_ids_supported(down))
    x = torch.randn((T, K), generator=g, device="cuda").to(torch.bfloat16)
    logits = torch.randn((T, E), generator=g, device="cuda")
    if popular:
        logits[:, 3] = 50.0
    _, ids = ops.router_topk(logits, topk)
    src1, dst, bounds = ops.mm_ids_route(ids, E, False)
    a = ops.moe_mm_ids(x, ids, gate, E, up=up, out_dtype=torch.float32, routes=(src1, dst, bounds))
    a16 = ops.moe_mm_ids(x, ids, gate, E, up=up, out_dtype=torch.bfloat16, routes=(src1, dst, bounds))
    assert torch.equal(a16, a.to(torch.bfloat16))  # BF16 out: the one rounding of the FP32 result
    ys = ops.moe_mm_ids(a16, ids, down, E, routes=(dst, dst, bounds)) if down is not None else None
    g_only = ops.moe_mm_ids(x, ids, gate, E, out_dtype=torch.float32, routes=(src1, dst, bounds))
    # the fused product is the SwiGLU of the two plain products of the same kernel (the same accumulators), whatever the
    # size of the sums: only the exponential differs (the kernel's fast one)
    u_only = ops.moe_mm_ids(x, ids, up, E, out_dtype=torch.float32, routes=(src1, dst, bounds))
    fused_from_plain = u_only * (g_only / (1 + torch.exp(-g_only)))
    assert torch.all((a - fused_from_plain).abs() <= 2e-5 * fused_from_plain.abs() + 1e-30)
    xd = x.double()
    for e in range(E):
        tok, slot = torch.nonzero(ids == e, as_tuple=True)
        if tok.numel() == 0:
            continue
        we_g, we_u = wg[e * N:(e + 1) * N].double(), wu[e * N:(e + 1) * N].double()
        we_d = wd[e * K:(e + 1) * K].double() if wd is not None else None
        xe = xd[tok]                                  # [n, K]
        gg, uu = xe @ we_g.T, xe @ we_u.T
        want = uu * silu64(gg)
        got = a[tok, slot].double()
        assert torch.all((got - want).abs() <= 1e-3 * want.abs() + 1e-5), e
        bound = xe.abs() @ we_g.abs().T
        assert torch.all((g_only[tok, slot].double() - gg).abs() <= 1e-5 * bound), e
        if down is not None:
            hh = a16[tok, slot].double()
            err = (ys[tok, slot].double() - hh @ we_d.T).abs()
            assert torch.all(err <= 1e-5 * (hh.abs() @ we_d.abs().T) + 1e-30), e
    # the per-pair GEMV columns of the same matrices agree within the products' bound
    if T <= 8:
        y_gemv = ops.mmv_glu2(x, gate, up, ids, N)
        assert torch.all((y_gemv - a).abs() <= 1e-3 * a.abs() + 1e-5)
    # equivariance: the tokens in another order give the same rows, bit for bit (a token's sums never meet another's)
    perm = torch.randperm(T, generator=g, device="cuda")
    ids_p = ids[perm].contiguous()
    r_p = ops.mm_ids_route(ids_p, E, False)
    a_p = ops.moe_mm_ids(x[perm].contiguous(), ids_p, gate, E, up=up, out_dtype=torch.float32, routes=r_p)
    assert torch.equal(a_p, a[perm])


@pytest.mark.parametrize("T", [2, 30])
def test_moe_experts_on_the_4_bit_code_in_both_token_regimes(ops, T):
    """moe_experts with the expert stacks in the 4-bit code: expert GEMVs for few tokens, the batched kernel beyond, against
    the layer evaluated on the exactly decoded weights."""
    from moe_exact import moe_layer_exact

    E, k, K, N = 16, 2, 1024, 512
    gate, up = nib(ops, synth.weights_torch(E * N, K, 61, "cuda")), nib(ops, synth.weights_torch(E * N, K, 62, "cuda"))
    down = nib(ops, synth.weights_torch(E * K, N, 63, "cuda"))
    g = torch.Generator(device="cuda").manual_seed(T)
    x = torch.randn((T, K), generator=g, device="cuda").to(torch.bfloat16)
    wts, ids = ops.router_topk(torch.randn((T, E), generator=g, device="cuda"), k)
    assert ops.moe_experts_batched(T, k, gate, up, down, E) == (T == 30)
    got = ops.moe_experts(x, gate, up, down, wts, ids, E).float()
    ref = moe_layer_exact(ops, x, gate, up, down, wts, ids, E).float()
    assert torch.all((got - ref).abs() <= 2e-2 * ref.abs() + 2e-2 * ref.abs().max())


def test_batched_kernel_limits_of_the_4_bit_code(ops):
    """More than 1,024 experts, or rows per expert that are no multiple of 32: a clear error, no launch."""
    w = nib(ops, synth.weights_torch(2048 * 32, 512, 71, "cuda"))
    x = torch.zeros((4, 512), dtype=torch.bfloat16, device="cuda")
    ids = torch.zeros((4, 1), dtype=torch.int32, device="cuda")
    with pytest.raises(ValueError, match="at most 1024 experts"):
        ops.moe_mm_ids(x, ids, w, 2048)
    with pytest.raises(ValueError, match="multiples of 32"):
        ops.moe_mm_ids(x, ids, w, 4096)
    assert ops.moe_mm_ids(x, ids, w, 1024).shape == (4, 1, 64)


def test_which_token_counts_take_the_batched_kernels(ops):
    """moe_experts_batched for 256 experts with nine slots per token: the tiles leave the expert GEMVs above 0.14 routed
    pairs per expert (35.8: 3 tokens), the 4-bit code above 0.5 (14 tokens: its GEMV has no decode chain), other layouts
    with a batched kernel above 0.7 (19 tokens)."""
    E, rows = 256, 32

    def enc(K, fmt, R, w64):
        plane, aux, _, _ = ops.encode_bits(synth.weights(E * rows, K, 91 + K), fmt, R, False, wave64=w64)
        ta = torch.from_numpy(aux)
        return ops.upload(torch.from_numpy(plane), ta, ops.parse_header(ta), "cuda")

    for fmt, R, w64, last_gemv in ((3, 32, True, 3), (1, 0, False, 14), (3, 4, True, 19)):
        gate_up, down = enc(2048, fmt, R, w64), enc(512, fmt, R, w64)
        assert ops.mm_ids_supported(gate_up, gate_up) and ops.mm_ids_supported(down)
        got = [T for T in range(1, 40) if not ops.moe_experts_batched(T, 9, gate_up, gate_up, down, E)]
        assert got == list(range(1, last_gemv + 1)), (fmt, R, got)


def test_a_call_whose_unit_list_would_not_fit_is_refused(ops):
    """The batched kernel lists (expert, pass) units in LDS, 2048 at most: a call with more (experts + routed pairs / 128
    with the longest passes) is refused on the host instead of leaving the last experts uncomputed; the largest call
    that fits is computed, the last expert included."""
    E, N, K, topk = 257, 32, 512, 9
    w = synth.weights_torch(E * N, K, 77, "cuda")
    gate = nib(ops, w)
    T_fit = (2048 - E) * 128 // topk          # experts + pairs / 128 == 2048 at most
    T_over = T_fit + 128
    for T in (T_over, T_fit):
        x = synth.activations_torch(T, K, 78, "cuda")
        # every token names the last expert (a shared expert stacked behind the routed ones) and eight others in turn
        base = (torch.arange(T, device="cuda", dtype=torch.int32)[:, None] * 8 + torch.arange(8, device="cuda", dtype=torch.int32)[None, :]) % (E - 1)
        ids = torch.cat([base, torch.full((T, 1), E - 1, device="cuda", dtype=torch.int32)], 1).contiguous()
        if T == T_over:
            with pytest.raises(ValueError, match="too many routed pairs"):
                ops.moe_mm_ids(x, ids, gate, E)
            continue
        y = ops.moe_mm_ids(x, ids, gate, E)
        last = w[(E - 1) * N:].float()
        for t in (0, T // 2, T - 1):   # the stacked expert's rows of the first, a middle and the last token
            want = last.double() @ x[t].double()
            bound = last.double().abs() @ x[t].double().abs()
            assert torch.all((y[t, topk - 1].double() - want).abs() <= 1e-5 * bound), t
