"""GEMV / GLU / MoE kernels on the GPU against the oracle (restates tests/core/test_kernels.py of the reference):
FP32-accumulated oracle within 1e-3 relative (1e-5 absolute floor), FP64 bound |err| <= 1e-5 * sum|w x| per output,
one-hot activations give the exact BF16 weight, BF16 outputs are the RNE of the FP32 ones."""
from __future__ import annotations

import numpy as np
import pytest
import torch

from conftest import GEMV_REL
from moe_exact import moe_layer_exact
from orin_qwen_lossless_amd import synth
from test_gpu_roundtrip import bits, enc

pytestmark = pytest.mark.gpu
NIB, HUF, HP = 1, 2, 3

LAYOUTS = [(NIB, 0, False, False), (HUF, 8, False, False), (HP, 1, False, False), (HP, 8, False, False), (HP, 16, False, False),
           (HP, 8, True, False), (HP, 4, False, True), (HP, 16, False, True)]


def tbf16(b: np.ndarray) -> torch.Tensor:
    return torch.from_numpy(np.ascontiguousarray(b).view(np.int16)).view(torch.bfloat16).cuda()


def rne_bf16(y: np.ndarray) -> np.ndarray:
    return synth.f32_to_bf16_bits(y)


def check_gemv(oracle, y: np.ndarray, w_bits: np.ndarray, x: np.ndarray, cm=False):
    """y [T, rows] against the oracle: north-star tolerance vs the FP32-accumulated result and the FP64 bound."""
    for t in range(x.shape[0]):
        ref32 = oracle.gemv_f32(w_bits, x[t], cm)
        y64, s = oracle.gemv_f64(w_bits, x[t])
        assert np.all(np.abs(y[t] - ref32) <= 1e-3 * np.abs(ref32) + 1e-5), "vs FP32-accumulated oracle"
        assert np.all(np.abs(y[t] - y64) <= GEMV_REL * s + 1e-30), "FP64 bound"


@pytest.mark.parametrize("K", [512, 1024, 2048, 4096])
@pytest.mark.parametrize("fmt,R,cm,w64", LAYOUTS)
def test_gemv_dense(ops, oracle, K, fmt, R, cm, w64):
    if cm and K == 512:
        pytest.skip("chunk-major needs K > 512")
    rows = 16 * 13
    wb = synth.weights(rows, K, K + R)
    w = enc(ops, wb, fmt, R, cm, w64)
    xb = synth.activations(3, K, 7)
    xf = synth.bf16_bits_to_f32(xb)
    y_bf = ops.mmv(tbf16(xb), w).cpu().numpy()             # BF16 activations
    y_f32 = ops.mmv(torch.from_numpy(xf).cuda(), w).cpu().numpy()   # the same values as FP32 activations
    check_gemv(oracle, y_bf, wb, xf, cm)
    check_gemv(oracle, y_f32, wb, xf, cm)
    # BF16 output = round-to-nearest-even of the FP32 output
    y16 = ops.mmv(tbf16(xb), w, out_dtype=torch.bfloat16)
    assert np.array_equal(bits(y16), rne_bf16(y_bf))
    # multi-column launches give each column the single-column result
    y1 = np.stack([ops.mmv(tbf16(xb[t: t + 1]), w).cpu().numpy()[0] for t in range(3)])
    y_sc = ops.mmv(tbf16(xb), w, multi_col=False).cpu().numpy()
    assert np.array_equal(y_sc, y1)
    assert np.array_equal(y1, y_bf)


@pytest.mark.parametrize("K", [512, 1024, 2048, 4096])
@pytest.mark.parametrize("R", [1, 4, 16])
def test_wave64_column_groups_equal_single_columns(ops, oracle, K, R):
    # one decode serves a group of up to eight token columns (fewer when K is large or the activations are FP32);
    # every batch size gives each column the bits of its single-column launch, which the oracle bounds
    if R * K % (4096 if K == 4096 else 2048):
        pytest.skip("the GEMV takes units of whole pairs (K = 4096: quadruples) of 1024-column steps")
    rows = 16 * 37
    wb = synth.weights(rows, K, 3 * K + R)
    w = enc(ops, wb, HP, R, False, True)
    xb = synth.activations(8, K, K + 11)
    xf = synth.bf16_bits_to_f32(xb)
    for x in (tbf16(xb), torch.from_numpy(xf).cuda()):
        y1 = torch.cat([ops.mmv(x[t: t + 1], w) for t in range(8)])
        check_gemv(oracle, y1.cpu().numpy(), wb, xf)
        for T in range(2, 9):
            assert torch.equal(ops.mmv(x[:T], w), y1[:T]), (T, x.dtype)
        # strided activation rows (a view of a wider buffer)
        wide = torch.zeros((8, K + 64), dtype=x.dtype, device="cuda")
        wide[:, :K] = x
        assert torch.equal(ops.mmv(wide[:, :K], w), y1)


@pytest.mark.parametrize("K", [512, 2048])
def test_nibble_column_groups_equal_single_columns(ops, oracle, K):
    # dense NIBBLE batches of 8 and more columns decode a (row, chunk) once for two or four columns; every column keeps
    # the bits of its single-column launch, plain and with the fused SwiGLU, BF16 and FP32 activations, ragged tails
    # (the plain product of BF16 activations runs on the matrix cores from nine columns on: the same bits at every
    # such batch size, within the oracle's bounds)
    rows = 2 * 88
    wb = synth.weights(rows, K, 5 * K)
    wb[3, 7] = 0x4000                                          # 2.0: an exponent outside the row table, an escape
    w = enc(ops, wb, NIB, 0, False, False)
    xb = synth.activations(19, K, K + 3)
    xf = synth.bf16_bits_to_f32(xb)
    for x in (tbf16(xb), torch.from_numpy(xf).cuda()):
        y1 = torch.cat([ops.mmv(x[t: t + 1], w) for t in range(19)])
        g1 = torch.cat([ops.mmv_glu(x[t: t + 1], w) for t in range(19)])
        check_gemv(oracle, y1[:4].cpu().numpy(), wb, xf[:4])
        y19 = ops.mmv(x, w)
        check_gemv(oracle, y19[[0, 7, 18]].cpu().numpy(), wb, xf[[0, 7, 18]])
        for T in (8, 9, 15, 16, 17, 19):
            assert torch.equal(ops.mmv(x[:T], w), y1[:T] if x.dtype == torch.float32 or T <= 8 else y19[:T]), (T, x.dtype)
            assert torch.equal(ops.mmv_glu(x[:T], w), g1[:T]), (T, x.dtype)


@pytest.mark.parametrize("rows,K,first", [(4104, 512, 2), (4104, 1024, 2), (1030, 2048, 5), (4360, 2048, 2), (2056, 4096, 3), (2048, 1536, 3)])
def test_nibble_few_columns_on_16_row_groups(ops, oracle, rows, K, first):
    """Dense NIBBLE batches of up to 16 BF16 columns over matrices whose 16-row groups fill the CUs (from two columns),
    half of them (from three) or a quarter (from five) run on the matrix cores in 16-row groups (k_nib_mm16): every step
    count per wavefront (K = 512 .. 4096), a last group of fewer than 16 rows, escaped weights there and elsewhere,
    strided activation rows, several blocks of 16 tokens; within the oracle's bounds, the BF16 output the rounding of
    the FP32 one, and a token's bits the same at every batch size and position the kernel takes.  FP32 activations keep
    the GEMV columns."""
    assert ops.cu_count() == 256, "the thresholds of this test are those of 256 CUs"
    wb = synth.weights(rows, K, rows + K)
    for r, col in ((0, 3), (17, K - 1), (rows - 1, 7), (rows - 3, K // 2)):
        wb[r, col] = 0x4500 if r % 2 else 0xC4FF                     # exponents outside the rows' tables: escapes
    w = enc(ops, wb, NIB, 0, False, False)
    xb = synth.activations(16, K, K + rows)
    xf = synth.bf16_bits_to_f32(xb)
    x = tbf16(xb)
    y16 = ops.mmv(x, w)
    assert ops.last_kernel().startswith("k_nib_mm16<")
    check_gemv(oracle, y16[[0, 9, 15]].cpu().numpy(), wb, xf[[0, 9, 15]])
    assert np.array_equal(bits(ops.mmv(x, w, out_dtype=torch.bfloat16)), rne_bf16(y16.cpu().numpy()))
    for T in range(1, 16):
        yT = ops.mmv(x[:T], w)
        took = ops.last_kernel().startswith("k_nib_mm16<")
        assert took == (T >= first), (T, ops.last_kernel())
        if took:
            assert torch.equal(yT, y16[:T]), T
        else:
            check_gemv(oracle, yT[T - 1:].cpu().numpy(), wb, xf[T - 1: T])
    wide = torch.zeros((16, K + 64), dtype=x.dtype, device="cuda")
    wide[:, :K] = x
    assert torch.equal(ops.mmv(wide[:, :K], w), y16)
    # more than 16 columns: blocks of 16 tokens, each column as in a batch of its own (two blocks per CU at most)
    x40 = torch.cat([x, x.flip(0), x[:8]])
    groups = (rows + 15) // 16
    y40 = ops.mmv(x40, w)
    assert ops.last_kernel().startswith("k_nib_mm16<") == (groups * 3 <= 512), ops.last_kernel()
    if groups * 3 <= 512:
        assert torch.equal(y40, torch.cat([y16, y16.flip(0), y16[:8]]))
    y_f32 = ops.mmv(torch.from_numpy(xf[:5]).cuda(), w)
    assert ops.last_kernel().startswith("k_nib_mmv<float")
    check_gemv(oracle, y_f32[[0, 4]].cpu().numpy(), wb, xf[[0, 4]])


@pytest.mark.parametrize("T", [6, 70])
def test_nibble_batches_over_a_row_range_through_the_c_abi(ops, T):
    """bf16n_mmv with row0 / nrows (a view of some rows of a tensor, as the engine adapter hands them over) on the
    matrix-core kernels of the 4-bit code: the product over rows [row0, row0 + nrows) is that slice of the whole
    product, bit for bit, with a first row that is no multiple of the row groups and a ragged last group."""
    import ctypes as C

    from orin_qwen_lossless_amd import _lib

    rows, K, row0, nrows = 4400, 1024, 1030, 2213
    wb = synth.weights(rows, K, 991)
    wb[row0 + 5, 9] = wb[row0 + nrows - 1, K - 3] = 0x4500        # escapes inside the range
    w = enc(ops, wb, NIB, 0, False, False)
    x = tbf16(synth.activations(T, K, 992))
    whole = ops.mmv(x, w)
    assert ops.last_kernel().startswith("k_nib_mm16<" if T <= 16 else "k_nib_mm<")
    y = torch.full((T, nrows), float("nan"), dtype=torch.float32, device="cuda")
    a = _lib.MmvArgs()
    a.x, a.y, a.ids = x.data_ptr(), y.data_ptr(), None
    a.x_tok, a.y_tok = K * 2, nrows * 4
    a.rows_per_matrix, a.row0, a.nrows, a.ncols = rows, row0, nrows, T
    a.x_bf16, a.y_bf16 = 1, 0
    _lib.check(_lib.lib().bf16n_mmv(C.byref(ops._cweight(w)), C.byref(a), C.c_void_p(torch.cuda.current_stream().cuda_stream), 1))
    torch.cuda.synchronize()
    took = ops.last_kernel()
    # (six tokens: 16-row groups for the tensor and for the range; 70 tokens, five blocks of 16, are more than two
    # blocks per CU for either: 32-row groups)
    assert took.startswith("k_nib_mm16<" if T <= 16 else "k_nib_mm<"), took
    assert torch.equal(y, whole[:, row0: row0 + nrows])


@pytest.mark.parametrize("fmt,R,cm,w64", LAYOUTS)
def test_one_hot_activations_give_exact_weights(ops, fmt, R, cm, w64):
    K, rows = 2048, 64
    wb = synth.model_like(rows, K, 3)
    wb[(wb & 0x7F80) == 0x7F80] = 0x3F80  # finite weights only: 0 * inf would poison a row
    w = enc(ops, wb, fmt, R, cm, w64)
    for k, scale in ((0, 1.0), (3, -2.0), (517, 0.5), (2047, 4.0)):
        x = np.zeros((1, K), dtype=np.float32)
        x[0, k] = scale
        want = synth.bf16_bits_to_f32(wb[:, k]) * np.float32(scale)
        for xt in (torch.from_numpy(x).cuda(), torch.from_numpy(x).cuda().to(torch.bfloat16)):
            got = ops.mmv(xt, w).cpu().numpy()[0]
            # denormal BF16 weights may be flushed by the hardware dot product: compare through abs tolerance 0 elsewhere
            nz = np.abs(want) >= np.float32(2.0 ** -126)
            assert np.array_equal(got[nz], want[nz]), (k, scale)
            assert np.all(np.abs(got[~nz] - want[~nz]) <= 2.0 ** -126)


def test_nibble_escapes_contribute_exactly(ops, oracle):
    # rows with more exponents than the table holds and exponents >= 128: escaped weights add their exact product
    wb = synth.nibble_rows_with_exponents(8, 512, 17, 5)
    wb[:, 7] = (wb[:, 7] & 0x807F) | (np.uint16(130) << 7)
    w = enc(ops, wb, NIB)
    assert w.meta.format == NIB
    ex = (wb >> 7) & 0xFF
    for k in (7, int(np.argmax(ex[0] == ex[0].min()))):
        x = np.zeros((1, 512), dtype=np.float32)
        x[0, k] = 0.5
        got = ops.mmv(torch.from_numpy(x).cuda(), w).cpu().numpy()[0]
        assert np.array_equal(got, synth.bf16_bits_to_f32(wb[:, k]) * np.float32(0.5))
    xb = synth.activations(2, 512, 9)
    y = ops.mmv(tbf16(xb), w).cpu().numpy()
    for t in range(2):
        y64, s = oracle.gemv_f64(wb, synth.bf16_bits_to_f32(xb[t]))
        assert np.all(np.abs(y[t] - y64) <= GEMV_REL * s)


@pytest.mark.parametrize("fmt,R,cm,w64", [(HP, 8, False, False), (HP, 8, True, False), (HP, 8, False, True), (HP, 16, False, True), (NIB, 0, False, False)])
@pytest.mark.parametrize("idt", [torch.int32, torch.int64])
def test_expert_ids_and_strides(ops, oracle, fmt, R, cm, w64, idt):
    E, N, K, T, k = 6, 32, 1024, 3, 2
    wb = synth.weights(E * N, K, 11)
    w = enc(ops, wb, fmt, R, cm, w64)
    ids_np = np.array([[0, 5], [3, 3], [4, 1]], dtype=np.int64)
    ids = torch.from_numpy(ids_np).to(idt).cuda()
    xb = synth.activations(T * k, K, 12).reshape(T, k, K)
    xf = synth.bf16_bits_to_f32(xb)
    # per-token activations (gate / up): x [T, K]
    y = ops.mmv(tbf16(xb[:, 0]), w, ids, N).cpu().numpy()
    assert y.shape == (T, k, N)
    for t in range(T):
        for s in range(k):
            e = ids_np[t, s]
            check_gemv(oracle, y[t, s][None], wb[e * N: (e + 1) * N], xf[t, 0][None], cm)
    # per-slot activations (down): x [T, k, K]
    y = ops.mmv(tbf16(xb), w, ids, N).cpu().numpy()
    for t in range(T):
        for s in range(k):
            e = ids_np[t, s]
            check_gemv(oracle, y[t, s][None], wb[e * N: (e + 1) * N], xf[t, s][None], cm)
    # a strided activation view (rows 16-byte aligned)
    big = torch.zeros(T, 2 * K, dtype=torch.bfloat16, device="cuda")
    big[:, :K] = tbf16(xb[:, 0])
    y2 = ops.mmv(big[:, :K], w, ids, N).cpu().numpy()
    y1 = ops.mmv(tbf16(xb[:, 0]), w, ids, N).cpu().numpy()
    assert np.array_equal(y1, y2)


def test_mmv_argument_errors(ops):
    wb = synth.weights(64, 1024, 1)
    w = enc(ops, wb, HP, 8)
    x = torch.zeros(1, 1024, dtype=torch.bfloat16, device="cuda")
    ids = torch.zeros(1, 2, dtype=torch.int32, device="cuda")
    with pytest.raises(ValueError, match="whole units"):
        ops.mmv(x, w, ids, 4)
    with pytest.raises(ValueError):
        ops.mmv(torch.zeros(1, 512, dtype=torch.bfloat16, device="cuda"), w)
    with pytest.raises(ValueError, match="whole matrix"):
        ops.mmv(x, w, None, 32)
    with pytest.raises(ValueError, match="NIBBLE"):
        ops.mmv_glu(x, w)
    wn = enc(ops, wb, NIB)
    assert ops.mmv_glu(x, wn).shape == (1, 32)


@pytest.mark.parametrize("K", [512, 2048])
def test_nibble_merged_glu_equals_unfused(ops, K):
    N = 48
    wb = synth.weights(2 * N, K, 21)
    w = enc(ops, wb, NIB)
    xb = synth.activations(2, K, 22)
    x = tbf16(xb)
    fused = ops.mmv_glu(x, w)
    g = ops.mmv(x, enc(ops, wb[:N], NIB))
    u = ops.mmv(x, enc(ops, wb[N:], NIB))
    assert torch.equal(fused, ops.swiglu(g, u))
    fused16 = ops.mmv_glu(x, w, out_dtype=torch.bfloat16)
    assert np.array_equal(bits(fused16), rne_bf16(fused.cpu().numpy()))


@pytest.mark.parametrize("fmt,R", [(NIB, 0), (HP, 8), (HP, 1), (HUF, 8)])
def test_separate_gate_up_glu_equals_unfused(ops, fmt, R):
    N, K = 64, 1024
    gb, ub = synth.weights(N, K, 23), synth.weights(N, K, 24)
    g, u = enc(ops, gb, fmt, R), enc(ops, ub, fmt, R)
    x = tbf16(synth.activations(2, K, 25))
    fused = ops.mmv_glu2(x, g, u)
    assert torch.equal(fused, ops.swiglu(ops.mmv(x, g), ops.mmv(x, u)))


@pytest.mark.parametrize("K,R", [(512, 16), (1024, 4), (2048, 8), (4096, 4)])
def test_wave64_gate_up_glu_equals_unfused(ops, K, R):
    # dense and with expert ids: the fused kernel runs the same two decode chains, so the results are identical
    E, N, T, k = 4, 64, 3, 2
    gb, ub = synth.weights(E * N, K, 26), synth.weights(E * N, K, 27)
    g, u = enc(ops, gb, HP, R, False, True), enc(ops, ub, HP, R, False, True)
    x = tbf16(synth.activations(T, K, 28))
    assert torch.equal(ops.mmv_glu2(x, g, u), ops.swiglu(ops.mmv(x, g), ops.mmv(x, u)))
    ids = torch.tensor([[0, 3], [2, 1], [3, 0]], dtype=torch.int32, device="cuda")
    fused = ops.mmv_glu2(x, g, u, ids, N)
    assert fused.shape == (T, k, N)
    assert torch.equal(fused, ops.swiglu(ops.mmv(x, g, ids, N), ops.mmv(x, u, ids, N)))
    f16 = ops.mmv_glu2(x, g, u, ids, N, out_dtype=torch.bfloat16)
    assert np.array_equal(bits(f16), rne_bf16(fused.cpu().numpy()))


def test_swiglu_and_combine(ops, oracle):
    rng = np.random.default_rng(1)
    g, u = rng.standard_normal(5000).astype(np.float32) * 3, rng.standard_normal(5000).astype(np.float32)
    got = ops.swiglu(torch.from_numpy(g).cuda(), torch.from_numpy(u).cuda()).cpu().numpy()
    assert np.allclose(got, oracle.swiglu(g, u), rtol=1e-5, atol=1e-6)
    ref = (torch.nn.functional.silu(torch.from_numpy(g).double()) * torch.from_numpy(u).double()).numpy()
    assert np.allclose(got, ref, rtol=1e-5, atol=1e-6)
    ys = rng.standard_normal((7, 8, 300)).astype(np.float32)
    wt = rng.random((7, 8)).astype(np.float32)
    got = ops.moe_combine(torch.from_numpy(ys).cuda(), torch.from_numpy(wt).cuda(), torch.float32).cpu().numpy()
    assert np.array_equal(got, oracle.moe_combine(ys, wt))  # same fmaf chain in slot order
    got16 = ops.moe_combine(torch.from_numpy(ys).cuda(), torch.from_numpy(wt).cuda(), torch.bfloat16)
    assert np.array_equal(bits(got16), rne_bf16(got))
    wt16 = torch.from_numpy(wt).cuda().to(torch.bfloat16)
    got = ops.moe_combine(torch.from_numpy(ys).cuda(), wt16, torch.float32).cpu().numpy()
    assert np.array_equal(got, oracle.moe_combine(ys, wt16.float().cpu().numpy()))


@pytest.mark.parametrize("T,k,E", [(1, 8, 256), (9, 8, 256), (130, 8, 64), (33, 3, 7), (2048, 8, 256), (1024, 4, 32), (1025, 4, 32),
                                   (8192, 8, 256), (70001, 2, 16)])  # the last one: more than one chunk of 64 rounds
@pytest.mark.parametrize("idt", [torch.int32, torch.int64])
def test_routing_lists(ops, oracle, T, k, E, idt):
    rng = np.random.default_rng(T + k)
    ids = np.stack([rng.permutation(E)[:k] for _ in range(T)]).astype(np.int32)
    if E == 64:
        ids[ids == 5] = 6 if k < E else 5  # an expert without tokens (duplicates within a token are not produced by routers)
        for t in range(T):
            if len(set(ids[t])) < k:
                ids[t] = rng.permutation(np.setdiff1d(np.arange(E), [5]))[:k]
    for per_slot in (False, True):
        src1, dst, bounds = ops.mm_ids_route(torch.from_numpy(ids).to(idt).cuda(), E, per_slot)
        o_src1, o_dst, o_bounds = oracle.route(ids, E, k if per_slot else 1, k if per_slot else 1)
        assert np.array_equal(bounds.cpu().numpy(), o_bounds)
        assert np.array_equal(dst.cpu().numpy(), o_dst)
        assert np.array_equal(src1.cpu().numpy(), o_src1)


def test_router_topk_ids_stay_valid_on_bad_logits(ops):
    # NaN / infinite logits: the ids are still k distinct experts below n_experts (they feed address arithmetic)
    lg = torch.full((4, 200), float("nan"), device="cuda")
    lg[1] = float("-inf")
    lg[2] = float("inf")
    lg[3, ::3] = 1.0
    _, ids = ops.router_topk(lg, 8)
    ids = ids.cpu().numpy()
    for t in range(4):
        assert ids[t].min() >= 0 and ids[t].max() < 200 and len(set(ids[t].tolist())) == 8
    assert ids[0].tolist() == list(range(8))          # all equal (-inf after NaN): lowest indices first
    assert ids[3].tolist() == [0, 3, 6, 9, 12, 15, 18, 21]


def test_router_topk(ops, oracle):
    rng = np.random.default_rng(4)
    lg = rng.standard_normal((5, 256)).astype(np.float32) * 2
    lg[3, 10] = lg[3, 200] = lg[3].max() + 1  # a tie at the top: the lower index comes first
    wts, ids = ops.router_topk(torch.from_numpy(lg).cuda(), 8)
    for t in range(5):
        oid, ow = oracle.router_topk(lg[t], 8)
        assert np.array_equal(ids[t].cpu().numpy(), oid)
        assert np.allclose(wts[t].cpu().numpy(), ow, rtol=1e-5, atol=1e-7)
        assert abs(float(wts[t].sum()) - 1) < 1e-5
    raw, _ = ops.router_topk(torch.from_numpy(lg).cuda(), 8, renorm=False)
    p = torch.softmax(torch.from_numpy(lg).double(), -1)
    assert np.allclose(raw.cpu().numpy(), torch.gather(p, 1, ids.cpu().long()).numpy(), rtol=1e-5)


@pytest.mark.parametrize("T", [1, 4, 8])
@pytest.mark.parametrize("w64", [False, True])
def test_moe_layer_decode(ops, oracle, T, w64):
    # the MoE decode layer at reduced expert count: router top-k on the GPU, gate/up GEMVs, SwiGLU, down, combine
    E, N, H, K, k = 16, 512, 128, 1024, 4  # down consumes N activations: N must be a multiple of 512
    gate_b, up_b, down_b = synth.weights(E * N, K, 41), synth.weights(E * N, K, 42), synth.weights(E * H, N, 43)
    gate = enc(ops, gate_b, HP, 8, not w64, w64)
    up_ = enc(ops, up_b, HP, 8, not w64, w64)
    down = enc(ops, down_b, HP, 16, False, w64)
    xb = synth.activations(T, K, 44)
    x = tbf16(xb)
    router = torch.from_numpy(synth.bf16_bits_to_f32(synth.weights(E, K, 45))).cuda()
    logits = x.float() @ router.t()
    wts, ids = ops.router_topk(logits, k)
    y = ops.moe_experts(x, gate, up_, down, wts, ids, E)
    ref = moe_layer_exact(ops, x, gate, up_, down, wts, ids.long(), E)
    err = (y.float() - ref.float()).abs()
    tol = 2.0 ** -7 * ref.float().abs() + 1e-4
    assert bool((err <= tol).all()), float(err.max())
    # FP64 check of the whole layer for token 0 from exact weights
    xf = synth.bf16_bits_to_f32(xb[0]).astype(np.float64)
    acc = np.zeros(H)
    for s in range(k):
        e = int(ids[0, s])
        gf = synth.bf16_bits_to_f32(gate_b[e * N: (e + 1) * N]).astype(np.float64) @ xf
        uf = synth.bf16_bits_to_f32(up_b[e * N: (e + 1) * N]).astype(np.float64) @ xf
        a = gf / (1 + np.exp(-gf)) * uf
        acc += float(wts[0, s]) * (synth.bf16_bits_to_f32(down_b[e * H: (e + 1) * H]).astype(np.float64) @ a)
    got = y[0].float().cpu().numpy()
    assert np.all(np.abs(got - acc) <= 2.0 ** -7 * np.abs(acc) + 1e-4)


@pytest.mark.parametrize("T", [1, 8, 9, 33])
@pytest.mark.parametrize("fmt,R,cm,w64", [(NIB, 0, False, False), (HP, 16, False, True), (HP, 8, True, False)])
def test_linear_both_token_regimes(ops, T, fmt, R, cm, w64):
    # up to 8 tokens: decode GEMV, FP32 accumulation, bias added in FP32, one rounding to BF16; more: exact dequant +
    # stock BF16 GEMM (restates the reference's linear, core/torch/torch_bindings.cpp:198-239)
    K, rows = 1024, 208
    wb = synth.weights(rows, K, 91)
    w = enc(ops, wb, fmt, R, cm, w64)
    xb = synth.activations(T, K, 92)
    bias = tbf16(synth.weights(1, rows, 93)[0])
    wf, xf = synth.bf16_bits_to_f32(wb).astype(np.float64), synth.bf16_bits_to_f32(xb).astype(np.float64)
    ref = xf @ wf.T
    for b in (None, bias):
        y = ops.linear(tbf16(xb), w, b)
        assert y.dtype == torch.bfloat16 and tuple(y.shape) == (T, rows)
        want = ref + (b.float().cpu().numpy().astype(np.float64) if b is not None else 0.0)
        got = y.float().cpu().numpy().astype(np.float64)
        # BF16 has 8 significant bits: one rounding (GEMV path) or two (GEMM path, bias added after the first)
        eps = 2.0 ** -8 if T <= 8 else 2.0 ** -7
        assert np.all(np.abs(got - want) <= eps * (np.abs(want) + 0.05))
    # leading batch dimensions are kept
    y3 = ops.linear(tbf16(xb).reshape(1, T, K), w)
    assert tuple(y3.shape) == (1, T, rows)
    with pytest.raises(ValueError):
        ops.linear(tbf16(xb).float(), w)


def test_embedding_is_the_exact_rows(ops):
    K, rows = 512, 96
    wb = synth.weights(rows, K, 94)
    for fmt, R, w64 in ((HP, 16, True), (HP, 16, False), (NIB, 0, False)):
        w = enc(ops, wb, fmt, R, False, w64)
        ids = torch.tensor([[0, 95, 17], [17, 16, 15]], dtype=torch.int64, device="cuda")
        out = ops.embedding(ids, w)
        assert tuple(out.shape) == (2, 3, K) and out.dtype == torch.bfloat16
        assert np.array_equal(bits(out).reshape(6, K), wb[ids.cpu().numpy().reshape(-1)])


@pytest.mark.parametrize("K", [512, 1024, 1536, 2048, 2560, 3072, 3584, 4096])
def test_nibble_every_chunk_count(ops, oracle, K):
    # one half-wave per (row, chunk): every K / 512 from 1 to 8, row counts that do not fill a block, plain and GLU
    rows = 2 * 13
    wb = synth.weights(rows, K, 95 + K)
    w = enc(ops, wb, NIB)
    xb = synth.activations(2, K, 96)
    xf = synth.bf16_bits_to_f32(xb)
    check_gemv(oracle, ops.mmv(tbf16(xb), w).cpu().numpy(), wb, xf)
    fused = ops.mmv_glu(tbf16(xb), w)
    g = ops.mmv(tbf16(xb), enc(ops, wb[: rows // 2], NIB))
    u = ops.mmv(tbf16(xb), enc(ops, wb[rows // 2:], NIB))
    assert torch.equal(fused, ops.swiglu(g, u))


@pytest.mark.parametrize("layout", ["nibble", "units", "tiles", "reference"])
@pytest.mark.parametrize("T", [9, 33, 512])
def test_linear_dense_through_the_c_abi(ops, layout, T):
    """The dense path for more tokens than the GEMV serves, behind the C ABI: exact dequant into the caller's scratch in
    pieces + the stock BF16 GEMM.  Against FP64 products of the exact weights (the output is BF16: one rounding of an
    FP32-accumulated sum), with a scratch buffer that forces several pieces, and captured into a HIP graph."""
    rows, K = (1000, 1024) if layout == "nibble" else (2048, 1536) if layout == "reference" else (4096, 2048)
    wb = synth.weights(rows, K, 700 + T)
    w = {"nibble": lambda: enc(ops, wb, NIB), "units": lambda: enc(ops, wb, HP, 4, False, True),
         "tiles": lambda: enc(ops, wb, HP, 32, False, True), "reference": lambda: enc(ops, wb, HP, 8, False, False)}[layout]()
    x = tbf16(synth.activations(T, K, 701))
    wd = torch.from_numpy(synth.bf16_bits_to_f32(wb)).cuda().double()
    ref, bound = x.double() @ wd.t(), x.double().abs() @ wd.abs().t()
    y = ops.linear_dense(x, w)
    assert y.dtype == torch.bfloat16 and tuple(y.shape) == (T, rows)
    assert bool(((y.double() - ref).abs() <= 2.0 ** -8 * ref.abs() + 1e-5 * bound).all())
    # a scratch buffer of 40 decoded rows: many pieces, the same result (each output element is one GEMM's dot product
    # whatever the piece it falls into; the BLAS may pick another kernel for the narrower pieces, hence the bound again)
    small = torch.empty(40 * K * 2, dtype=torch.uint8, device="cuda")
    y2 = ops.linear_dense(x, w, scratch=small)
    assert bool(((y2.double() - ref).abs() <= 2.0 ** -8 * ref.abs() + 1e-5 * bound).all())
    with pytest.raises(ValueError, match="scratch"):
        ops.linear_dense(x, w, scratch=torch.empty(K * 2, dtype=torch.uint8, device="cuda"))
    # captured: the call allocates nothing when the buffers are the caller's
    scratch = torch.empty(64 << 20, dtype=torch.uint8, device="cuda")
    wsp = torch.empty(32 << 20, dtype=torch.uint8, device="cuda")
    ops.linear_dense(x, w, scratch, wsp)
    torch.cuda.synchronize()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g):
        yg = ops.linear_dense(x, w, scratch, wsp)
    for rep in range(3):
        x.copy_(tbf16(synth.activations(T, K, 710 + rep)))
        want = ops.linear_dense(x, w, scratch, wsp).clone()
        yg.zero_()
        g.replay()
        torch.cuda.synchronize()
        assert torch.equal(yg, want), rep


@pytest.mark.parametrize("K,rows,T,row0,nrows", [(1536, 4300, 9, 7, 4200), (2560, 8200, 33, 31, 8169), (3584, 4500, 70, 0, 4500),
                                                 (4096, 4128, 12, 32, 4096)])
def test_nibble_matrix_core_batches_on_row_ranges(ops, K, rows, T, row0, nrows):
    """bf16n_mmv on a row range of a 4-bit matrix (row0, nrows of the C structure) with enough rows for the matrix-core
    path: K that is no power of two (an odd number of half chunks: the last wavefront's second turn is empty), a range
    that starts inside a group of 32 rows and ends ragged, escapes; against FP64 on the exact weights, and the GEMV
    columns (multi_col = 0) beside it."""
    import ctypes as C

    from orin_qwen_lossless_amd import _lib

    wb = synth.weights(rows, K, 3 * K + rows)
    wb[::11, ::97] = 0x4500
    w = enc(ops, wb, NIB, 0, False, False)
    x = tbf16(synth.activations(T, K, K + T))

    def product(multi_col):
        y = torch.empty((T, nrows), dtype=torch.float32, device="cuda")
        a = _lib.MmvArgs()
        a.x, a.y, a.x_bf16, a.y_bf16, a.n_used, a.x_per_slot = x.data_ptr(), y.data_ptr(), 1, 0, 1, 1
        a.ncols, a.x_tok, a.y_tok = T, x.stride(0) * 2, nrows * 4
        a.rows_per_matrix, a.row0, a.nrows = rows, row0, nrows
        cw = ops._cweight(w)
        _lib.check(_lib.lib().bf16n_mmv(C.byref(cw), C.byref(a), None, multi_col))
        return y.double()

    wd = ops.dequant(w).double()[row0: row0 + nrows]
    ref, bound = x.double() @ wd.T, x.double().abs() @ wd.abs().T
    for multi_col in (1, 0):
        assert torch.all((product(multi_col) - ref).abs() <= 1e-5 * bound), multi_col
