"""Batched MoE prefill (mm_ids) on the GPU: restates the reference's batched-kernel tests
(tests/core/test_kernels.py:248-360: results against the exact dequantised weights in FP64 within 1e-5 * sum|w x|,
BF16 output = RNE of the FP32 output, token tiles of 127 / 128 / 129, experts without tokens, the 8 / 9 token switch of
moe_experts).  One-hot activations make the product an exact copy of the weights: a transposed operand, a wrong tile row
or a wrong accumulator lane fails that test bit for bit."""
from __future__ import annotations

import numpy as np
import pytest
import torch

from moe_exact import moe_layer_exact
from orin_qwen_lossless_amd import synth
from test_gpu_kernels import rne_bf16, tbf16
from test_gpu_roundtrip import bits, enc

pytestmark = pytest.mark.gpu
HP = 3

# (K, rows per expert, R, chunk_major, wave64): gate / up in reference chunk-major units and in wave64 units; down in
# reference row-major units and in wave64 units
SHAPES = [(2048, 128, 8, True, False), (2048, 128, 8, False, True), (2048, 128, 4, False, True), (2048, 128, 2, False, True),
          (512, 256, 16, False, False), (512, 256, 16, False, True), (512, 256, 8, False, True), (512, 256, 4, False, True)]


def routing(T: int, k: int, E: int, counts: dict[int, int], seed: int) -> np.ndarray:
    """ids [T, k] without repeats inside a token; expert e gets exactly counts[e] pairs, the rest goes to the other
    experts at random."""
    rng = np.random.default_rng(seed)
    ids = -np.ones((T, k), dtype=np.int64)
    slots = [(t, s) for t in range(T) for s in range(k)]
    rng.shuffle(slots)
    fixed = set(counts)
    for e, n in counts.items():
        got = 0
        for (t, s) in slots:
            if got == n:
                break
            if ids[t, s] < 0 and e not in ids[t]:
                ids[t, s] = e
                got += 1
        assert got == n
    free = [e for e in range(E) if e not in fixed]
    for t in range(T):
        for s in range(k):
            if ids[t, s] < 0:
                cand = [e for e in free if e not in ids[t]]
                ids[t, s] = cand[rng.integers(len(cand))]
    return ids.astype(np.int32)


def reference(wf: np.ndarray, xf: np.ndarray, ids: np.ndarray, N: int, per_slot: bool):
    """FP64 products with the exact weights and sum |w x| per output."""
    T, k = ids.shape
    y = np.zeros((T, k, N))
    s = np.zeros((T, k, N))
    w64 = wf.astype(np.float64)
    for t in range(T):
        for i in range(k):
            xv = (xf[t, i] if per_slot else xf[t]).astype(np.float64)
            we = w64[ids[t, i] * N: (ids[t, i] + 1) * N]
            y[t, i] = we @ xv
            s[t, i] = np.abs(we) @ np.abs(xv)
    return y, s


@pytest.mark.parametrize("K,N,R,cm,w64", SHAPES)
def test_mm_ids_against_exact_weights(ops, K, N, R, cm, w64):
    E, k, T = 6, 2, 260
    wb = synth.weights(E * N, K, 11 + K + R)
    w = enc(ops, wb, HP, R, cm, w64)
    assert ops.mm_ids_supported(w)
    wf = synth.bf16_bits_to_f32(wb)
    # tiles of 129 / 128 / 127 tokens and an expert without tokens
    ids = routing(T, k, E, {0: 129, 1: 128, 2: 127, 3: 0}, 5)
    per_slot = K == 512  # down takes one activation row per (token, slot)
    xb = synth.activations(T * (k if per_slot else 1), K, 3).reshape((T, k, K) if per_slot else (T, K))
    xf = synth.bf16_bits_to_f32(xb)
    got = ops.moe_mm_ids(tbf16(xb), torch.from_numpy(ids).cuda(), w, E).cpu().numpy()
    y, s = reference(wf, xf, ids, N, per_slot)
    assert np.all(np.abs(got - y) <= 1e-5 * s + 1e-30)
    assert np.all(np.abs(got - y) <= 1e-3 * np.abs(y) + 1e-5)
    # BF16 output is the round-to-nearest-even of the FP32 output
    got16 = ops.moe_mm_ids(tbf16(xb), torch.from_numpy(ids).cuda(), w, E, out_dtype=torch.bfloat16)
    assert np.array_equal(bits(got16), rne_bf16(got))
    # int64 ids give the same lists
    got64 = ops.moe_mm_ids(tbf16(xb), torch.from_numpy(ids.astype(np.int64)).cuda(), w, E).cpu().numpy()
    assert np.array_equal(got64, got)


@pytest.mark.parametrize("K,N,R,cm,w64", SHAPES)
def test_mm_ids_one_hot_is_exact(ops, K, N, R, cm, w64):
    # x = 2^-3 at one column: the output is the weight column scaled by a power of two, exactly
    E, k, T = 4, 2, 70
    wb = synth.weights(E * N, K, 21 + K)
    w = enc(ops, wb, HP, R, cm, w64)
    wf = synth.bf16_bits_to_f32(wb)
    ids = routing(T, k, E, {}, 9)
    per_slot = K == 512
    shape = (T, k, K) if per_slot else (T, K)
    xf = np.zeros(shape, dtype=np.float32)
    cols = np.random.default_rng(2).integers(0, K, size=shape[:-1])
    np.put_along_axis(xf, cols[..., None], 0.125, axis=-1)
    got = ops.moe_mm_ids(torch.from_numpy(xf).cuda().to(torch.bfloat16), torch.from_numpy(ids).cuda(), w, E).cpu().numpy()
    for t in range(T):
        for i in range(k):
            c = cols[t, i] if per_slot else cols[t]
            assert np.array_equal(got[t, i], wf[ids[t, i] * N: (ids[t, i] + 1) * N, c] * np.float32(0.125)), (t, i)


@pytest.mark.parametrize("cm,w64", [(True, False), (False, True)])
def test_mm_ids_fused_gate_up_swiglu(ops, cm, w64):
    K, N, E, k, T = 2048, 128, 5, 3, 150
    gb, ub = synth.weights(E * N, K, 31), synth.weights(E * N, K, 32)
    g, u = enc(ops, gb, HP, 8, cm, w64), enc(ops, ub, HP, 8, cm, w64)
    assert ops.mm_ids_supported(g, u)
    ids = routing(T, k, E, {4: 0}, 6)
    xb = synth.activations(T, K, 8)
    xt, it = tbf16(xb), torch.from_numpy(ids).cuda()
    fused = ops.moe_mm_ids(xt, it, g, E, up=u).cpu().numpy()
    yg = ops.moe_mm_ids(xt, it, g, E).cpu().numpy()
    yu = ops.moe_mm_ids(xt, it, u, E).cpu().numpy()
    want = (yu.astype(np.float64) * (yg.astype(np.float64) / (1.0 + np.exp(-yg.astype(np.float64)))))
    assert np.all(np.abs(fused - want) <= 2e-6 * np.abs(want) + 1e-12)
    # against FP64 with the exact weights
    xf = synth.bf16_bits_to_f32(xb)
    y1, _ = reference(synth.bf16_bits_to_f32(gb), xf, ids, N, False)
    y2, _ = reference(synth.bf16_bits_to_f32(ub), xf, ids, N, False)
    ref = y2 * (y1 / (1.0 + np.exp(-y1)))
    assert np.all(np.abs(fused - ref) <= 1e-3 * np.abs(ref) + 1e-5)
    # BF16 output rounds only the final result
    f16 = ops.moe_mm_ids(xt, it, g, E, up=u, out_dtype=torch.bfloat16)
    assert np.array_equal(bits(f16), rne_bf16(fused))


def test_mm_ids_contract(ops):
    wb = synth.weights(4 * 128, 2048, 41)
    rm = enc(ops, wb, HP, 8, False)          # row-major K = 2048: no batched kernel
    assert not ops.mm_ids_supported(rm)
    ids = torch.zeros((9, 1), dtype=torch.int32, device="cuda")
    x = torch.zeros((9, 2048), dtype=torch.bfloat16, device="cuda")
    with pytest.raises(ValueError, match="no batched kernel"):
        ops.moe_mm_ids(x, ids, rm, 4)
    cm = enc(ops, wb, HP, 8, True)
    with pytest.raises(ValueError, match="BF16 activations"):
        ops.moe_mm_ids(x.float(), ids, cm, 4)
    nib = enc(ops, wb, 1)                    # the 4-bit code has a batched kernel of its own (rows per expert: groups of 32)
    assert ops.mm_ids_supported(nib)
    with pytest.raises(ValueError, match="multiples of 32"):
        ops.moe_mm_ids(x, ids, nib, 32)


@pytest.mark.parametrize("cm,w64", [(True, False), (False, True)])
@pytest.mark.parametrize("T", [8, 9, 40])
def test_moe_experts_switches_to_batched_kernels(ops, T, cm, w64):
    # up to 8 tokens: expert GEMVs; more: fused gate/up + SwiGLU (BF16) then down, both against the exact-weight reference
    E, k, Kd, N = 8, 2, 2048, 512
    gate = enc(ops, synth.weights(E * N, Kd, 51), HP, 8, cm, w64)
    up = enc(ops, synth.weights(E * N, Kd, 52), HP, 8, cm, w64)
    assert ops.mm_ids_supported(gate, up)
    down = enc(ops, synth.weights(E * Kd, N, 53), HP, 16, False, True)
    ids = torch.from_numpy(routing(T, k, E, {}, T)).cuda()
    wts = torch.softmax(torch.randn((T, k), generator=torch.Generator().manual_seed(T)), dim=-1).cuda()
    x = tbf16(synth.activations(T, Kd, 54))
    got = ops.moe_experts(x, gate, up, down, wts, ids, E).float().cpu().numpy()
    ref = moe_layer_exact(ops, x, gate, up, down, wts, ids, E).float().cpu().numpy()
    scale = np.abs(ref).max()
    assert np.all(np.abs(got - ref) <= 2e-2 * np.abs(ref) + 2e-2 * scale)


def sweep_cases(n: int):
    rng = np.random.default_rng(4242)
    layouts = [(2048, 8, True, False), (2048, 8, False, True), (2048, 4, False, True), (2048, 2, False, True),
               (512, 16, False, False), (512, 16, False, True), (512, 8, False, True), (512, 4, False, True)]
    out = []
    for i in range(n):
        K, R, cm, w64 = layouts[i % len(layouts)]
        E = int(rng.integers(2, 10))
        N = 64 * int(rng.integers(1, 4))
        k = int(rng.integers(1, min(E, 4) + 1))
        T = int(rng.integers(9, 300))
        out.append((K, R, cm, w64, E, N, k, T, bool(rng.integers(2)), int(rng.integers(1 << 30))))
    return out


def tile_sweep_cases(n: int):
    rng = np.random.default_rng(2424)
    out = []
    for i in range(n):
        K = [2048, 512, 1024, 4096, 1536][i % 5]
        E = int(rng.integers(2, 10))
        out.append((K, 32, False, True, E, 32 * int(rng.integers(1, 20)), int(rng.integers(1, min(E, 4) + 1)), int(rng.integers(9, 300)),
                    bool(rng.integers(2)), int(rng.integers(1 << 30))))
    return out


@pytest.mark.parametrize("K,R,cm,w64,E,N,k,T,fused,seed", sweep_cases(24) + tile_sweep_cases(20))
def test_mm_ids_seeded_sweep(ops, K, R, cm, w64, E, N, k, T, fused, seed):
    rng = np.random.default_rng(seed)
    wb = synth.weights(E * N, K, seed)
    w = enc(ops, wb, HP, R, cm, w64)
    ids = np.stack([rng.permutation(E)[:k] for _ in range(T)]).astype(np.int32)
    per_slot = K == 512
    xb = synth.activations(T * (k if per_slot else 1), K, seed + 1).reshape((T, k, K) if per_slot else (T, K))
    xf = synth.bf16_bits_to_f32(xb)
    it = torch.from_numpy(ids).cuda()
    y, s = reference(synth.bf16_bits_to_f32(wb), xf, ids, N, per_slot)
    got = ops.moe_mm_ids(tbf16(xb), it, w, E).cpu().numpy()
    assert np.all(np.abs(got - y) <= 1e-5 * s + 1e-30)
    if fused and (K == 2048 or R == 32) and not per_slot:
        ub = synth.weights(E * N, K, seed + 2)
        u = enc(ops, ub, HP, R, cm, w64)
        yu, _ = reference(synth.bf16_bits_to_f32(ub), xf, ids, N, False)
        ref = yu * (y / (1.0 + np.exp(-y)))
        f = ops.moe_mm_ids(tbf16(xb), it, w, E, up=u).cpu().numpy()
        assert np.all(np.abs(f - ref) <= 1e-3 * np.abs(ref) + 1e-5)
        # the decode-side fused kernel agrees with the batched one on the first tokens (different summation orders)
        if ops.glu2_supported(w, u):
            g8 = ops.mmv_glu2(tbf16(xb[:8]), w, u, it[:8].contiguous(), N).cpu().numpy()
            assert np.all(np.abs(g8 - f[:8]) <= 1e-3 * np.abs(ref[:8]) + 1e-5)
