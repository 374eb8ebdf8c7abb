"""Seeded sweep over shapes, unit sizes, layouts, batch sizes and expert routing: every case decodes bit-exactly and its
products stay within the FP64 bound of the exact weights (|err| <= 1e-5 * sum|w x|) and within 1e-3 relative of them.
The cases are drawn once from a fixed seed, so a failure names a reproducible configuration."""
from __future__ import annotations

import numpy as np
import pytest
import torch

from orin_qwen_lossless_amd import synth
from test_gpu_kernels import tbf16
from test_gpu_roundtrip import bits, enc

pytestmark = pytest.mark.gpu
NIB, HUF, HP = 1, 2, 3


def cases(n: int):
    rng = np.random.default_rng(20240607)
    out = []
    while len(out) < n:
        K = int(rng.choice([512, 1024, 1536, 2048, 2560, 4096]))
        fmt = int(rng.choice([NIB, HUF, HP, HP, HP]))
        R = 0 if fmt == NIB else int(rng.choice([1, 2, 4, 8, 16]))
        cm = bool(fmt == HP and K > 512 and R >= 4 and rng.random() < 0.3)
        C = K // 512
        w64 = bool(fmt == HP and not cm and C in (1, 2, 4, 8) and (R * C // 2) % (4 if C == 8 else 2) == 0 and (R * C) % 2 == 0
                   and rng.random() < 0.6)
        units = int(rng.integers(1, 40))
        E = int(rng.choice([1, 1, 3, 5]))
        rows_per = units * max(R, 1)
        T = int(rng.integers(1, 9))
        out.append((K, fmt, R, cm, w64, rows_per, E, T, int(rng.integers(1 << 30))))
    return out


def tile_cases(n: int):
    """The tile form of the wave64 layout (R = 32): any K, row groups per matrix, experts, batch."""
    rng = np.random.default_rng(31337)
    out = []
    for _ in range(n):
        K = int(rng.choice([512, 1024, 1536, 2048, 2560, 3072, 3584, 4096]))
        out.append((K, HP, 32, False, True, 32 * int(rng.integers(1, 12)), int(rng.choice([1, 1, 3, 5])), int(rng.integers(1, 9)),
                    int(rng.integers(1 << 30))))
    return out


@pytest.mark.parametrize("K,fmt,R,cm,w64,rows_per,E,T,seed", cases(120) + tile_cases(40))
def test_random_configuration(ops, K, fmt, R, cm, w64, rows_per, E, T, seed):
    rows = rows_per * E
    wb = synth.model_like(rows, K, seed) if seed % 3 == 0 else synth.weights(rows, K, seed)
    w = enc(ops, wb, fmt, R, cm, w64)
    assert np.array_equal(bits(ops.dequant(w)), wb)
    rng = np.random.default_rng(seed + 7)
    # a row range of whole units decodes to the same bits as the slice
    unit = max(R, 1)
    u0 = int(rng.integers(0, rows // unit))
    un = int(rng.integers(1, rows // unit - u0 + 1))
    assert np.array_equal(bits(ops.dequant(w, u0 * unit, un * unit)), wb[u0 * unit: (u0 + un) * unit])
    if fmt == NIB or (fmt == HP and not cm):
        # row gather with a base row that is not unit-aligned; BF16 and FP32 outputs are the exact weights
        row0 = int(rng.integers(0, rows))
        idn = rng.integers(0, rows - row0, size=5)
        for idt in (torch.int32, torch.int64):
            ids = torch.from_numpy(idn).to(idt).cuda()
            assert np.array_equal(bits(ops.get_rows(ids, w, torch.bfloat16, row0)), wb[row0 + idn])
        got32 = ops.get_rows(torch.from_numpy(idn).to(torch.int32).cuda(), w, torch.float32, row0).cpu().numpy()
        assert np.array_equal(got32.view(np.uint32), synth.bf16_bits_to_f32(wb[row0 + idn]).view(np.uint32))
    xb = synth.activations(T, K, seed + 1)
    xf = synth.bf16_bits_to_f32(xb).astype(np.float64)
    wf = synth.bf16_bits_to_f32(wb).astype(np.float64)
    finite_rows = np.isfinite(wf).all(axis=1) & (np.abs(wf).max(axis=1) < 1e30)
    if E == 1:
        y = ops.mmv(tbf16(xb), w).cpu().numpy().astype(np.float64)
        with np.errstate(invalid="ignore", over="ignore"):
            ref, bound = xf @ wf.T, np.abs(xf) @ np.abs(wf).T
        ok = finite_rows[None, :]
    else:
        k = min(2, E)
        rng = np.random.default_rng(seed)
        ids = np.stack([rng.permutation(E)[:k] for _ in range(T)]).astype(np.int32)
        y = ops.mmv(tbf16(xb), w, torch.from_numpy(ids).cuda(), rows_per).cpu().numpy().astype(np.float64)
        we = wf.reshape(E, rows_per, K)[ids]                      # [T, k, rows_per, K]
        ref = np.einsum("tkrc,tc->tkr", we, xf)
        bound = np.einsum("tkrc,tc->tkr", np.abs(we), np.abs(xf))
        ok = finite_rows.reshape(E, rows_per)[ids]
    with np.errstate(invalid="ignore", over="ignore"):
        err = np.abs(y - ref)
    assert np.all(err[np.broadcast_to(ok, err.shape)] <= (1e-5 * bound + 1e-30)[np.broadcast_to(ok, err.shape)])
    assert np.all(err[np.broadcast_to(ok, err.shape)] <= (1e-3 * np.abs(ref) + 1e-5)[np.broadcast_to(ok, err.shape)])


def batched_cases(n: int):
    """Batched products on the tile layout: K, rows per expert, experts, top-k and tokens drawn so that all shapes of the
    kernel come up (K split over wavefronts for few active experts, 32-token passes, 128-token passes)."""
    rng = np.random.default_rng(424242)
    out = []
    for _ in range(n):
        K = int(rng.choice([512, 1024, 1536, 2048, 3072, 4096]))
        N = 32 * int(rng.integers(1, 18))
        E = int(rng.choice([1, 2, 7, 16, 40]))
        k = int(rng.integers(1, min(E, 4) + 1))
        T = int(rng.choice([1, 2, 5, 17, 33, 70, 150, 300]))
        out.append((K, N, E, k, T, bool(rng.random() < 0.4), bool(rng.random() < 0.3), int(rng.integers(1 << 30))))
    return out


@pytest.mark.parametrize("K,N,E,k,T,glu,per_slot,seed", batched_cases(48))
def test_random_batched_products_on_tiles(ops, K, N, E, k, T, glu, per_slot, seed):
    from conftest import GEMV_REL
    from test_gpu_mm_ids import reference

    rng = np.random.default_rng(seed)
    wb = synth.weights(E * N, K, seed)
    w = enc(ops, wb, HP, 32, False, True)
    ids = np.stack([rng.permutation(E)[:k] for _ in range(T)]).astype(np.int32)
    if E > 2 and T > 40:
        ids[:, 0] = np.where(rng.random(T) < 0.6, 0, ids[:, 0])       # one busy expert: several passes
        for t in range(T):                                            # no repeats inside a token
            if k > 1 and ids[t, 0] in ids[t, 1:]:
                ids[t, 0] = next(e for e in range(E) if e not in ids[t, 1:])
    per_slot = per_slot and not glu
    xb = synth.activations(T * (k if per_slot else 1), K, seed + 1).reshape((T, k, K) if per_slot else (T, K))
    xf = synth.bf16_bits_to_f32(xb)
    xt, it = tbf16(xb), torch.from_numpy(ids).cuda()
    y, s = reference(synth.bf16_bits_to_f32(wb), xf, ids, N, per_slot)
    if not glu:
        got = ops.moe_mm_ids(xt, it, w, E).cpu().numpy()
        assert np.all(np.abs(got - y) <= GEMV_REL * s + 1e-30)
        assert np.all(np.abs(got - y) <= 1e-3 * np.abs(y) + 1e-5)
        got16 = ops.moe_mm_ids(xt, it, w, E, out_dtype=torch.bfloat16)
        assert np.array_equal(bits(got16), synth.f32_to_bf16_bits(got))
    else:
        ub = synth.weights(E * N, K, seed + 2)
        u = enc(ops, ub, HP, 32, False, True)
        fused = ops.moe_mm_ids(xt, it, w, E, up=u).cpu().numpy()
        y2, s2 = reference(synth.bf16_bits_to_f32(ub), xf, ids, N, False)
        sg = 1.0 / (1.0 + np.exp(-y))
        ref = y2 * y * sg
        # first-order bound of silu(g) * u under |dg| <= eps sum|w x| (gate) and |du| <= eps sum|w x| (up), plus one rounding
        dsilu = np.abs(sg * (1.0 + y * (1.0 - sg)))
        tol = GEMV_REL * (np.abs(y2) * dsilu * s + np.abs(y * sg) * s2) * 1.5 + 2.0 ** -22 * np.abs(ref) + 1e-12
        assert np.all(np.abs(fused - ref) <= tol)
