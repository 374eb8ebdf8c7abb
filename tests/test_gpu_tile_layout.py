"""The tile form of the wave64 layout (R = 32: 32-row x 256-column units in matrix-core operand order) on the GPU:
bit-exact dequant and row gather against the source bits and the oracle decoder, GEMV / fused gate-up GEMV against the
oracle (1e-3 relative, 1e-5 absolute floor; FP64 bound 1e-5 * sum|w x|), one-hot activations bit for bit, and the batched
MoE kernel against FP64 products with the exact weights (reference tests/core/test_kernels.py:248-360)."""
from __future__ import annotations

import numpy as np
import pytest
import torch

from conftest import GEMV_REL
from moe_exact import moe_layer_exact
from orin_qwen_lossless_amd import synth
from test_gpu_kernels import check_gemv, rne_bf16, tbf16
from test_gpu_mm_ids import reference, routing
from test_gpu_roundtrip import bits, enc

pytestmark = pytest.mark.gpu
HP = 3


@pytest.mark.parametrize("K", [512, 1024, 1536, 2048, 4096])
def test_dequant_and_get_rows_are_bit_exact(ops, oracle, K):
    rows = 32 * 5
    wb = synth.model_like(rows, K, K + 1)
    plane, aux, _, R = ops.encode_bits(wb, HP, 32, False, wave64=True)
    assert R == 32 and np.array_equal(oracle.decode(plane, aux), wb)
    w = enc(ops, wb, HP, 32, False, True)
    assert np.array_equal(bits(ops.dequant(w)), wb)
    assert np.array_equal(bits(ops.dequant(w, 64, 96)), wb[64:160])
    assert ops.roundtrip_equal(w, tbf16(wb))
    ids = np.array([0, 31, 32, 159, 77, 77, 5], dtype=np.int32)
    got = ops.get_rows(torch.from_numpy(ids).cuda(), w)
    assert np.array_equal(bits(got), wb[ids])
    got32 = ops.get_rows(torch.from_numpy(ids).cuda(), w, out_dtype=torch.float32).cpu().numpy()
    assert np.array_equal(got32.view(np.uint32), wb[ids].astype(np.uint32) << 16)
    with pytest.raises(ValueError, match="whole units"):
        ops.dequant(w, 16, 32)


@pytest.mark.parametrize("K", [512, 1024, 1536, 2048, 2560, 4096])
def test_gemv_dense(ops, oracle, K):
    rows = 32 * 7
    wb = synth.weights(rows, K, K + 32)
    w = enc(ops, wb, HP, 32, False, True)
    xb = synth.activations(3, K, 7)
    xf = synth.bf16_bits_to_f32(xb)
    y_bf = ops.mmv(tbf16(xb), w).cpu().numpy()
    y_f32 = ops.mmv(torch.from_numpy(xf).cuda(), w).cpu().numpy()
    check_gemv(oracle, y_bf, wb, xf)
    check_gemv(oracle, y_f32, wb, xf)
    y16 = ops.mmv(tbf16(xb), w, out_dtype=torch.bfloat16)
    assert np.array_equal(bits(y16), rne_bf16(y_bf))
    y1 = np.stack([ops.mmv(tbf16(xb[t: t + 1]), w).cpu().numpy()[0] for t in range(3)])
    assert np.array_equal(y1, y_bf)


def test_one_hot_activations_give_exact_weights(ops):
    K, rows = 2048, 64
    wb = synth.model_like(rows, K, 3)
    wb[(wb & 0x7F80) == 0x7F80] = 0x3F80
    w = enc(ops, wb, HP, 32, False, True)
    for k, scale in ((0, 1.0), (3, -2.0), (517, 0.5), (2047, 4.0), (24, 1.0), (1000, 2.0)):
        x = np.zeros((1, K), dtype=np.float32)
        x[0, k] = scale
        want = synth.bf16_bits_to_f32(wb[:, k]) * np.float32(scale)
        for xt in (torch.from_numpy(x).cuda(), torch.from_numpy(x).cuda().to(torch.bfloat16)):
            got = ops.mmv(xt, w).cpu().numpy()[0]
            nz = np.abs(want) >= np.float32(2.0 ** -126)
            assert np.array_equal(got[nz], want[nz]), (k, scale)


@pytest.mark.parametrize("K,N", [(2048, 64), (512, 128), (4096, 32)])
def test_routed_gemv_and_fused_gate_up(ops, oracle, K, N):
    E, T, k = 6, 3, 2
    gb, ub = synth.weights(E * N, K, 61 + K), synth.weights(E * N, K, 62 + K)
    g, u = enc(ops, gb, HP, 32, False, True), enc(ops, ub, HP, 32, False, True)
    assert ops.glu2_supported(g, u)
    ids = np.array([[0, 5], [3, 1], [5, 2]], dtype=np.int32)
    xb = synth.activations(T, K, 9)
    xf = synth.bf16_bits_to_f32(xb)
    it = torch.from_numpy(ids).cuda()
    yg = ops.mmv(tbf16(xb), g, ids=it, rows_per_matrix=N).cpu().numpy()
    yu = ops.mmv(torch.from_numpy(xf).cuda(), u, ids=it, rows_per_matrix=N).cpu().numpy()
    for t in range(T):
        for i in range(k):
            e = ids[t, i]
            check_gemv(oracle, yg[t, i][None], gb[e * N:(e + 1) * N], xf[t][None])
            check_gemv(oracle, yu[t, i][None], ub[e * N:(e + 1) * N], xf[t][None])
    for xt in (tbf16(xb), torch.from_numpy(xf).cuda()):
        fused = ops.mmv_glu2(xt, g, u, ids=it, rows_per_matrix=N).cpu().numpy()
        # the fused launch may split K over the wavefronts differently from the plain one (FP32 reassociation)
        want = yu.astype(np.float64) * (yg.astype(np.float64) / (1.0 + np.exp(-yg.astype(np.float64))))
        assert np.all(np.abs(fused - want) <= 1e-5 * np.abs(want) + 1e-6)
    dense = ops.mmv_glu2(tbf16(xb), g, u).cpu().numpy()   # all experts as one dense matrix
    u0 = ops.mmv(tbf16(xb), u).cpu().numpy().astype(np.float64)
    g0 = ops.mmv(tbf16(xb), g).cpu().numpy().astype(np.float64)
    want0 = u0 * (g0 / (1.0 + np.exp(-g0)))
    assert np.all(np.abs(dense - want0) <= 2e-6 * np.abs(want0) + 1e-12)


# (K, rows per expert): gate / up and down shapes, row counts that fill a work item, half of one, and an odd group count
MM_SHAPES = [(2048, 128), (2048, 512), (512, 256), (512, 544), (1024, 96), (4096, 32)]


@pytest.mark.parametrize("K,N", MM_SHAPES)
def test_mm_ids_against_exact_weights(ops, K, N):
    E, k, T = 6, 2, 260
    wb = synth.weights(E * N, K, 11 + K + N)
    w = enc(ops, wb, HP, 32, False, True)
    assert ops.mm_ids_supported(w)
    wf = synth.bf16_bits_to_f32(wb)
    ids = routing(T, k, E, {0: 129, 1: 128, 2: 127, 3: 0}, 5)
    per_slot = K == 512
    xb = synth.activations(T * (k if per_slot else 1), K, 3).reshape((T, k, K) if per_slot else (T, K))
    xf = synth.bf16_bits_to_f32(xb)
    got = ops.moe_mm_ids(tbf16(xb), torch.from_numpy(ids).cuda(), w, E).cpu().numpy()
    y, s = reference(wf, xf, ids, N, per_slot)
    assert np.all(np.abs(got - y) <= GEMV_REL * s + 1e-30)
    assert np.all(np.abs(got - y) <= 1e-3 * np.abs(y) + 1e-5)
    got16 = ops.moe_mm_ids(tbf16(xb), torch.from_numpy(ids).cuda(), w, E, out_dtype=torch.bfloat16)
    assert np.array_equal(bits(got16), rne_bf16(got))


@pytest.mark.parametrize("K,N", MM_SHAPES)
def test_mm_ids_few_tokens_per_expert(ops, K, N):
    # up to 16 routed pairs per expert the kernel runs passes of 32 tokens, here (few experts) with K split over the
    # wavefronts of an item: experts with none, one, 32, 33 and 70 tokens (one to three passes), against FP64 products
    # of the exact weights; the same tokens inside a larger call (passes of 128 tokens, another summation order) agree
    # within the bound
    E, k, T = 12, 2, 90
    wb = synth.weights(E * N, K, 41 + K + N)
    w = enc(ops, wb, HP, 32, False, True)
    wf = synth.bf16_bits_to_f32(wb)
    ids = routing(T, k, E, {0: 70, 1: 33, 2: 32, 3: 1, 4: 0}, 15)
    per_slot = K == 512
    xb = synth.activations(T * (k if per_slot else 1), K, 4).reshape((T, k, K) if per_slot else (T, K))
    xf = synth.bf16_bits_to_f32(xb)
    got = ops.moe_mm_ids(tbf16(xb), torch.from_numpy(ids).cuda(), w, E).cpu().numpy()
    y, s = reference(wf, xf, ids, N, per_slot)
    assert np.all(np.abs(got - y) <= GEMV_REL * s + 1e-30)
    assert np.all(np.abs(got - y) <= 1e-3 * np.abs(y) + 1e-5)
    got16 = ops.moe_mm_ids(tbf16(xb), torch.from_numpy(ids).cuda(), w, E, out_dtype=torch.bfloat16)
    assert np.array_equal(bits(got16), rne_bf16(got))
    more = 8 * E                                    # the same tokens followed by others: more than 16 pairs per expert
    ids2 = np.concatenate([ids, routing(more, k, E, {}, 16)])
    xb2 = np.concatenate([xb, synth.activations(more * (k if per_slot else 1), K, 5).reshape((more,) + xb.shape[1:])])
    got2 = ops.moe_mm_ids(tbf16(xb2), torch.from_numpy(ids2).cuda(), w, E).cpu().numpy()
    assert np.all(np.abs(got2[:T] - got) <= 2 * GEMV_REL * s + 1e-30)


def test_mm_ids_more_experts_than_a_block_lists(ops):
    # above 1024 experts the blocks do not list the active ones (and K is not split): every expert's items are visited
    E, k, T, K, N = 1500, 2, 40, 512, 32
    wb = synth.weights(E * N, K, 77)
    w = enc(ops, wb, HP, 32, False, True)
    rng = np.random.default_rng(8)
    ids = np.stack([rng.permutation(E)[:k] for _ in range(T)]).astype(np.int32)
    ids[:, 0] = np.where(np.arange(T) % 2 == 0, 1499, ids[:, 0])     # the last expert takes half of the tokens
    xb = synth.activations(T, K, 9)
    got = ops.moe_mm_ids(tbf16(xb), torch.from_numpy(ids).cuda(), w, E).cpu().numpy()
    y, s = reference(synth.bf16_bits_to_f32(wb), synth.bf16_bits_to_f32(xb), ids, N, False)
    assert np.all(np.abs(got - y) <= GEMV_REL * s + 1e-30)


@pytest.mark.parametrize("K,N", [(2048, 128), (2048, 512), (1024, 96)])
def test_mm_ids_fused_gate_up_few_tokens_per_expert(ops, K, N):
    E, k, T = 10, 2, 70
    gb, ub = synth.weights(E * N, K, 51), synth.weights(E * N, K, 52)
    g, u = enc(ops, gb, HP, 32, False, True), enc(ops, ub, HP, 32, False, True)
    ids = routing(T, k, E, {0: 40, 1: 0}, 7)
    xb = synth.activations(T, K, 9)
    xt, it = tbf16(xb), torch.from_numpy(ids).cuda()
    fused = ops.moe_mm_ids(xt, it, g, E, up=u).cpu().numpy()
    xf = synth.bf16_bits_to_f32(xb)
    y1, _ = reference(synth.bf16_bits_to_f32(gb), xf, ids, N, False)
    y2, _ = reference(synth.bf16_bits_to_f32(ub), xf, ids, N, False)
    ref = y2 * (y1 / (1.0 + np.exp(-y1)))
    assert np.all(np.abs(fused - ref) <= 1e-3 * np.abs(ref) + 1e-5)
    more = 9 * E
    ids2 = np.concatenate([ids, routing(more, k, E, {}, 17)])
    xb2 = np.concatenate([xb, synth.activations(more, K, 6)])
    fused2 = ops.moe_mm_ids(tbf16(xb2), torch.from_numpy(ids2).cuda(), g, E, up=u).cpu().numpy()
    assert np.all(np.abs(fused2[:T] - fused) <= 1e-4 * np.abs(fused) + 1e-6)


@pytest.mark.parametrize("K,N", MM_SHAPES)
def test_mm_ids_one_hot_is_exact(ops, K, N):
    E, k, T = 4, 2, 70
    wb = synth.weights(E * N, K, 21 + K)
    w = enc(ops, wb, HP, 32, False, True)
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


@pytest.mark.parametrize("K,N", [(2048, 128), (2048, 512), (1024, 96)])
def test_mm_ids_fused_gate_up_swiglu(ops, K, N):
    E, k, T = 5, 3, 150
    gb, ub = synth.weights(E * N, K, 31), synth.weights(E * N, K, 32)
    g, u = enc(ops, gb, HP, 32, False, True), enc(ops, ub, HP, 32, False, True)
    assert ops.mm_ids_supported(g, u)
    ids = routing(T, k, E, {4: 0}, 6)
    xb = synth.activations(T, K, 8)
    xt, it = tbf16(xb), torch.from_numpy(ids).cuda()
    fused = ops.moe_mm_ids(xt, it, g, E, up=u).cpu().numpy()
    yg = ops.moe_mm_ids(xt, it, g, E).cpu().numpy()
    yu = ops.moe_mm_ids(xt, it, u, E).cpu().numpy()
    want = (yu.astype(np.float64) * (yg.astype(np.float64) / (1.0 + np.exp(-yg.astype(np.float64)))))
    assert np.all(np.abs(fused - want) <= 2e-6 * np.abs(want) + 1e-12)
    xf = synth.bf16_bits_to_f32(xb)
    y1, _ = reference(synth.bf16_bits_to_f32(gb), xf, ids, N, False)
    y2, _ = reference(synth.bf16_bits_to_f32(ub), xf, ids, N, False)
    ref = y2 * (y1 / (1.0 + np.exp(-y1)))
    assert np.all(np.abs(fused - ref) <= 1e-3 * np.abs(ref) + 1e-5)
    f16 = ops.moe_mm_ids(xt, it, g, E, up=u, out_dtype=torch.bfloat16)
    assert np.array_equal(bits(f16), rne_bf16(fused))


@pytest.mark.parametrize("T", [3, 8, 9, 40])
def test_moe_experts_in_both_token_regimes(ops, T):
    E, k, Kd, N = 8, 2, 2048, 512
    gate = enc(ops, synth.weights(E * N, Kd, 51), HP, 32, False, True)
    up = enc(ops, synth.weights(E * N, Kd, 52), HP, 32, False, True)
    down = enc(ops, synth.weights(E * Kd, N, 53), HP, 32, False, True)
    ids = torch.from_numpy(routing(T, k, E, {}, T)).cuda()
    wts = torch.softmax(torch.randn((T, k), generator=torch.Generator().manual_seed(T)), dim=-1).cuda()
    x = tbf16(synth.activations(T, Kd, 54))
    got = ops.moe_experts(x, gate, up, down, wts, ids, E).float().cpu().numpy()
    ref = moe_layer_exact(ops, x, gate, up, down, wts, ids, E).float().cpu().numpy()
    scale = np.abs(ref).max()
    assert np.all(np.abs(got - ref) <= 2e-2 * np.abs(ref) + 2e-2 * scale)


@pytest.mark.parametrize("T", [7, 8, 9, 30])
def test_moe_experts_path_switch_by_routed_pairs_per_expert(ops, T, monkeypatch):
    # 240 experts, top-4: expert GEMVs up to 0.14 * 240 = 33.6 routed pairs (8 tokens), the batched kernels above; both
    # within tolerance
    E, k, Kd, N = 240, 4, 512, 512
    gate = enc(ops, synth.weights(E * N, Kd, 81), HP, 32, False, True)
    up = enc(ops, synth.weights(E * N, Kd, 82), HP, 32, False, True)
    down = enc(ops, synth.weights(E * Kd, N, 83), HP, 32, False, True)
    batched_calls = []
    real = ops.moe_mm_ids
    monkeypatch.setattr(ops, "moe_mm_ids", lambda *a, **kw: (batched_calls.append(1), real(*a, **kw))[1])
    rng = np.random.default_rng(T)
    ids = torch.from_numpy(np.stack([rng.permutation(E)[:k] for _ in range(T)]).astype(np.int32)).cuda()
    wts = torch.softmax(torch.randn((T, k), generator=torch.Generator().manual_seed(T)), dim=-1).cuda()
    x = tbf16(synth.activations(T, Kd, 84))
    got = ops.moe_experts(x, gate, up, down, wts, ids, E).float().cpu().numpy()
    assert len(batched_calls) == (0 if T <= 8 else 2)
    ref = moe_layer_exact(ops, x, gate, up, down, wts, ids, E).float().cpu().numpy()
    scale = np.abs(ref).max()
    assert np.all(np.abs(got - ref) <= 2e-2 * np.abs(ref) + 2e-2 * scale)


@pytest.mark.parametrize("T,n", [(1, 2048), (4, 2048), (3, 1000), (2, 5120), (1, 4104)])
def test_add_rmsnorm_glue(ops, T, n):
    """The decode step's glue launch: the FP32 sum of its addends (BF16 rows in argument order, then the weighted sum
    over expert slots with moe_combine's fmaf chain) rounded once to BF16, and its RMS norm against FP64."""
    rng = np.random.default_rng(n + T)
    mk = lambda s=1.0: torch.from_numpy((rng.standard_normal((T, n)) * s).astype(np.float32)).cuda().to(torch.bfloat16)  # noqa: E731
    a, b, c = mk(), mk(0.3), mk(3.0)
    gamma = torch.from_numpy((1 + 0.1 * rng.standard_normal(n)).astype(np.float32)).cuda().to(torch.bfloat16)
    ys = torch.from_numpy(rng.standard_normal((T, 9, n)).astype(np.float32)).cuda()
    wts = torch.softmax(torch.from_numpy(rng.standard_normal((T, 9)).astype(np.float32)).cuda(), -1)
    for bb, cc, yy, gg in ((None, None, None, None), (b, None, None, None), (b, c, None, None), (b, c, ys, gamma),
                           (None, None, ys, None), (None, c, None, gamma)):
        for w in (wts, wts.to(torch.bfloat16)):
            y, ysum = ops.add_rmsnorm(a, bb, cc, ys=yy, topk_weights=w if yy is not None else None, gamma=gg, eps=1e-6, want_sum=True)
            s32 = a.float()
            for t in (bb, cc):
                s32 = s32 + t.float() if t is not None else s32
            if yy is not None:
                s32 = s32 + ops.moe_combine(yy, w, torch.float32)
            assert torch.equal(ysum, s32.to(torch.bfloat16))
            s64 = s32.double()
            ref = s64 * torch.rsqrt((s64 * s64).mean(-1, keepdim=True) + 1e-6) * (gg.double() if gg is not None else 1.0)
            assert torch.all((y.double() - ref).abs() <= 2.0 ** -8 * ref.abs() + 1e-30)
            assert torch.equal(ops.add_rmsnorm(a, bb, cc, ys=yy, topk_weights=w if yy is not None else None, gamma=gg, eps=1e-6), y)
    with pytest.raises(ValueError):
        ops.add_rmsnorm(a, ys=ys, topk_weights=wts[:, :4].contiguous())


def test_router_topk_into_wider_rows(ops):
    """The router's top-k written into the first k columns of wider rows: the other columns (a stacked shared expert's
    id and weight) stay as the caller set them, and the k columns equal the dense call's."""
    lg = torch.randn((5, 256), generator=torch.Generator().manual_seed(3)).cuda()
    wts, ids = torch.full((5, 9), 1.0, device="cuda"), torch.full((5, 9), 256, dtype=torch.int32, device="cuda")
    w2, i2 = ops.router_topk(lg, 8, out=(wts, ids))
    dw, di = ops.router_topk(lg, 8)
    assert w2 is wts and i2 is ids
    assert torch.equal(ids[:, :8], di) and torch.equal(wts[:, :8], dw)
    assert bool((ids[:, 8] == 256).all()) and bool((wts[:, 8] == 1.0).all())
    with pytest.raises(ValueError):
        ops.router_topk(lg, 8, out=(wts[:, :4].contiguous(), ids[:, :4].contiguous()))


@pytest.mark.parametrize("T,E,k,extra", [(1, 256, 8, 1), (4, 256, 8, 1), (16, 256, 8, 1), (7, 64, 4, 0), (16, 1000, 64, 0),
                                         (3, 300, 8, 3), (17, 256, 8, 1)])
def test_router_topk_and_routing_lists_in_one_launch(ops, oracle, T, E, k, extra, monkeypatch):
    """router_topk_routes against router_topk followed by mm_ids_route, and the lists against the oracle's: bit for
    bit, with stacked always-on experts in the columns behind the k routed ones, logits with ties, a token that names an
    expert twice (the last slot counts) and, above 16 tokens, the two-launch form it falls back to."""
    monkeypatch.setattr(ops, "TOPK_ROUTE_ONE_LAUNCH_TOKENS", 16)  # every size the kernel takes
    g = torch.Generator().manual_seed(T * 1000 + E)
    lg = torch.randn((T, E), generator=g).cuda()
    lg[:, : E // 4] = lg[:, : E // 4].round()  # ties
    n_listed, n_slots = E + extra, k + extra

    def rows():
        wts = torch.full((T, n_slots), 1.0, device="cuda")
        ids = torch.full((T, n_slots), 0, dtype=torch.int32, device="cuda")
        for j in range(extra):
            ids[:, k + j] = E + j
        if extra >= 3:
            ids[:, k + 2] = E + 1  # slot k + 2 names the expert of slot k + 1 again
        return wts, ids

    def listed(ids, bounds):
        """positions of the lists that hold entries (a token naming an expert twice leaves a gap behind its list)"""
        ids, bounds = ids.cpu().numpy(), bounds.cpu().numpy()
        pos = [bounds[e] + j for e in range(n_listed) for j in range(int((ids == e).any(axis=1).sum()))]
        return torch.tensor(pos, dtype=torch.long, device="cuda")

    w1, i1, (s1, d1, b1) = ops.router_topk_routes(lg, k, n_listed, out=rows())
    w2, i2 = ops.router_topk(lg, k, out=rows())
    s2, d2, b2 = ops.mm_ids_route(i2, n_listed, False)
    assert torch.equal(i1, i2) and torch.equal(w1, w2)
    at = listed(i2, b2)
    assert len(at) == T * (n_slots - (extra >= 3))
    assert torch.equal(b1, b2) and torch.equal(s1[at], s2[at]) and torch.equal(d1[at], d2[at])
    os1, od, ob = oracle.route(i2.cpu().numpy(), n_listed, nchannels_y=1, sis1=1)
    assert np.array_equal(ob, b1.cpu().numpy()) and np.array_equal(od[at.cpu().numpy()], d1[at].cpu().numpy())
    assert np.array_equal(os1[at.cpu().numpy()], s1[at].cpu().numpy())
    if extra == 0:  # dense rows of k
        w3, i3, (s3, d3, b3) = ops.router_topk_routes(lg, k, n_listed)
        assert torch.equal(i3, i2) and torch.equal(b3, b2) and torch.equal(d3, d2)
    # a second call with other logits
    lg2 = torch.randn((T, E), generator=g).cuda()
    _, i4, (s4, d4, b4) = ops.router_topk_routes(lg2, k, n_listed, out=rows())
    s5, d5, b5 = ops.mm_ids_route(i4, n_listed, False)
    at = listed(i4, b5)
    assert torch.equal(b4, b5) and torch.equal(d4[at], d5[at]) and torch.equal(s4[at], s5[at])


@pytest.mark.parametrize("T,E,k,extra,N,K", [(1, 256, 8, 1, 512, 2048), (3, 256, 8, 1, 512, 2048), (2, 40, 4, 0, 64, 512),
                                              (1, 64, 6, 2, 96, 1024)])
def test_gate_up_gemv_that_selects_its_experts(ops, T, E, k, extra, N, K):
    """bf16n_mmv_glu2_topk: the routed gate / up GEMV with the router's softmax + top-k in its prologue writes the ids
    and weights that bf16n_router_topk_strided writes and the products that bf16n_mmv_glu2 writes with those ids, bit
    for bit; the columns of the id rows from k on (experts every token uses) are read and left alone; ties and NaN
    logits select as the stand-alone kernel does."""
    EA = E + extra
    gate = enc(ops, synth.weights(EA * N, K, 801), HP, 32, False, True)
    up = enc(ops, synth.weights(EA * N, K, 802), HP, 32, False, True)
    assert ops.topk_in_gemv_supported(gate, up, E, k)
    x = tbf16(synth.activations(T, K, 803))
    lg = torch.randn((T, E), generator=torch.Generator().manual_seed(4)).cuda()
    lg[0, 5] = lg[0, 9] = lg[0].max() + 1.0     # a tie at the top: the lower index first
    lg[T - 1, 3] = float("nan")                  # NaN counts as -inf
    n = k + extra

    def rows():
        wts = torch.full((T, n), 1.0, device="cuda")
        ids = torch.full((T, n), -7, dtype=torch.int32, device="cuda")
        for j in range(extra):
            ids[:, k + j] = E + j
        return wts, ids

    w_ref, i_ref = ops.router_topk(lg, k, out=rows())
    y_ref = ops.mmv_glu2(x, gate, up, i_ref, N)
    w_f, i_f = rows()
    y_f = ops.mmv_glu2_topk(x, gate, up, lg, k, N, (w_f, i_f))
    assert torch.equal(i_f, i_ref) and torch.equal(w_f, w_ref)
    assert int(i_f[0, 0]) == 5 and int(i_f[0, 1]) == 9 and 3 not in i_f[T - 1, :k].tolist()
    assert torch.equal(y_f, y_ref)
    y16 = ops.mmv_glu2_topk(x, gate, up, lg, k, N, rows(), out_dtype=torch.bfloat16)
    assert torch.equal(y16, ops.mmv_glu2(x, gate, up, i_ref, N, out_dtype=torch.bfloat16))
    # without renormalisation the weights are the softmax values themselves
    w_n, i_n = rows()
    ops.mmv_glu2_topk(x, gate, up, lg, k, N, (w_n, i_n), renorm=False)
    w_s, _ = ops.router_topk(lg, k, renorm=False, out=rows())
    assert torch.equal(w_n, w_s) and torch.equal(i_n, i_ref)
    # the contract: int32 id rows of the logits' token count, tile-layout stacks, at most 256 experts
    with pytest.raises(ValueError):
        ops.mmv_glu2_topk(x, gate, up, lg, k, N, (w_f, i_f.long()))
    with pytest.raises(ValueError):
        ops.mmv_glu2_topk(x, gate, up, lg, n + 1, N, (w_f, i_f))
    units = enc(ops, synth.weights(EA * N, K, 804), HP, 4, False, True)
    assert not ops.topk_in_gemv_supported(units, units, E, k)
    with pytest.raises(ValueError, match="tile layout"):
        ops.mmv_glu2_topk(x, units, units, lg, k, N, rows())


@pytest.mark.parametrize("E,N,K,T,k,scratch_experts", [(8, 512, 2048, 300, 4, 8), (8, 512, 2048, 300, 4, 3), (6, 96, 512, 700, 2, 1),
                                                        (16, 64, 1024, 2100, 1, 5)])
def test_two_phase_batched_product_equals_the_fused_kernel(ops, E, N, K, T, k, scratch_experts, monkeypatch):
    """bf16n_mm_ids_scratch (experts decoded once into a scratch buffer in matrix-core operand order, multiplied from
    there) writes the bits of bf16n_mm_ids (the same matrix instructions in the same order per output element): fused
    gate / up + SwiGLU, BF16 and FP32 out, the plain product and the down product, with scratch for all experts, for
    some (several groups, the last smaller) and for one; an expert without tokens is skipped."""
    gate = enc(ops, synth.weights(E * N, K, 811), HP, 32, False, True)
    up = enc(ops, synth.weights(E * N, K, 812), HP, 32, False, True)
    down = enc(ops, synth.weights(E * K, N, 813), HP, 32, False, True) if N % 512 == 0 else None
    x = tbf16(synth.activations(T, K, 814))
    rng = np.random.default_rng(11)
    ids_np = np.stack([rng.permutation(E - 1)[:k] for _ in range(T)]).astype(np.int32)  # the last expert has no tokens
    ids = torch.from_numpy(ids_np).cuda()
    routes = ops.mm_ids_route(ids, E, False)
    monkeypatch.setattr(ops, "MM_IDS_TWO_PHASE_PAIRS_PER_EXPERT", 10 ** 9)
    want16 = ops.moe_mm_ids(x, ids, gate, E, up=up, out_dtype=torch.bfloat16, routes=routes)
    want32 = ops.moe_mm_ids(x, ids, gate, E, up=up, routes=routes)
    want_g = ops.moe_mm_ids(x, ids, gate, E, routes=routes)
    monkeypatch.setattr(ops, "MM_IDS_TWO_PHASE_PAIRS_PER_EXPERT", 1)
    per = 2 * N * K * 2
    buf = torch.empty(scratch_experts * per + 4096, dtype=torch.uint8, device="cuda")
    got16 = ops.moe_mm_ids(x, ids, gate, E, up=up, out_dtype=torch.bfloat16, routes=routes, scratch=buf)
    assert torch.equal(got16.view(torch.int16), want16.view(torch.int16))
    assert torch.equal(ops.moe_mm_ids(x, ids, gate, E, up=up, routes=routes, scratch=buf), want32)
    assert torch.equal(ops.moe_mm_ids(x, ids, gate, E, routes=routes, scratch=buf), want_g)
    assert torch.equal(ops.moe_mm_ids(x, ids, gate, E, up=up, routes=routes), want32)   # the operator's own scratch
    if down is not None:
        r3 = (routes[1], routes[1], routes[2])
        monkeypatch.setattr(ops, "MM_IDS_TWO_PHASE_PAIRS_PER_EXPERT", 10 ** 9)
        want_d = ops.moe_mm_ids(want16, ids, down, E, routes=r3)
        monkeypatch.setattr(ops, "MM_IDS_TWO_PHASE_PAIRS_PER_EXPERT", 1)
        assert torch.equal(ops.moe_mm_ids(want16, ids, down, E, routes=r3, scratch=buf), want_d)
    with pytest.raises(ValueError, match="scratch"):
        ops.moe_mm_ids(x, ids, gate, E, up=up, routes=routes, scratch=buf[: per // 2])
