"""The headline configuration at its real size (output projection 248320 x 2048, HUFPAIR under the mi355x policy),
checked through properties that do not need an oracle run of that size: decode(encode(w)) == w bit for bit over the whole
matrix, a one-hot activation returns the exact weight column, and the product of a random activation stays within the
FP64 bound of the exact weights."""
from __future__ import annotations

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu
ROWS, K = 248320, 2048


@pytest.fixture(scope="module")
def head(ops):
    g = torch.Generator(device="cuda").manual_seed(1)
    w = torch.empty((ROWS, K), dtype=torch.bfloat16, device="cuda")
    for r0 in range(0, ROWS, 1 << 15):
        n = min(1 << 15, ROWS - r0)
        w[r0: r0 + n] = (torch.randn((n, K), generator=g, device="cuda") * 0.02).to(torch.bfloat16)
    # a few rows of special values: zeros, denormals, infinities, NaNs, the largest finite magnitudes
    special = torch.tensor([0x0000, 0x8000, 0x0001, 0x807F, 0x7F7F, 0xFF7F, 0x7F80, 0xFF80, 0x7FC1, 0xFFFF, 0x3F80],
                           dtype=torch.int32).to(torch.int16)
    w.view(torch.int16)[ROWS - 7, : special.numel()] = special.cuda()
    fmt, R, cm, _, w64 = ops.choose(ROWS, K, engine="mi355x")
    wbits = w.cpu().view(torch.int16).numpy().view(np.uint16)
    plane, aux, fmt_out, _ = ops.encode_bits(wbits, fmt, R, cm, wave64=w64)
    ta = torch.from_numpy(aux)
    enc = ops.upload(torch.from_numpy(plane), ta, ops.parse_header(ta), "cuda")
    assert (fmt_out, R, w64) == (3, 16, True)
    return w, enc


def test_full_size_round_trip_is_bit_exact(ops, head):
    w, enc = head
    assert ops.roundtrip_equal(enc, w)


def test_full_size_one_hot_returns_the_weight_column(ops, head):
    w, enc = head
    for col in (0, 777, K - 1):
        x = torch.zeros((1, K), dtype=torch.bfloat16, device="cuda")
        x[0, col] = 0.5
        y = ops.mmv(x, enc)[0]
        want = w[:, col].float() * 0.5
        keep = torch.ones(ROWS, dtype=torch.bool, device="cuda")
        keep[ROWS - 7] = False
        assert torch.equal(y[keep], want[keep])
        # the row that holds infinities and NaNs: 0 * inf is NaN in IEEE arithmetic, the product must not hide it
        assert bool(torch.isnan(y[ROWS - 7]))


def test_full_size_product_within_fp64_bound(ops, head):
    w, enc = head
    g = torch.Generator(device="cuda").manual_seed(2)
    x = torch.randn((4, K), generator=g, device="cuda").to(torch.bfloat16)
    y = ops.mmv(x, enc)
    keep = torch.ones(ROWS, dtype=torch.bool, device="cuda")
    keep[ROWS - 7] = False  # the row of special values has no finite bound
    for t in range(4):
        ref = torch.zeros(ROWS, dtype=torch.float64, device="cuda")
        bound = torch.zeros(ROWS, dtype=torch.float64, device="cuda")
        for r0 in range(0, ROWS, 1 << 15):
            wd = w[r0: r0 + (1 << 15)].double()
            ref[r0: r0 + wd.shape[0]] = wd @ x[t].double()
            bound[r0: r0 + wd.shape[0]] = wd.abs() @ x[t].double().abs()
        err = (y[t].double() - ref).abs()
        assert bool((err[keep] <= 1e-5 * bound[keep]).all())
    # batch columns equal single-column launches bit for bit (compared as bits: one row is NaN)
    assert torch.equal(ops.mmv(x[1:2], enc)[0].view(torch.int32), y[1].view(torch.int32))


# ---- the same matrix in the tile layout: dense products of BF16 activations run on the matrix cores, any batch size ------

@pytest.fixture(scope="module")
def head_tiles(ops, head):
    w, _ = head
    wbits = w.cpu().view(torch.int16).numpy().view(np.uint16)
    plane, aux, fmt_out, R = ops.encode_bits(wbits, 3, 32, False, wave64=True)
    assert (fmt_out, R) == (3, 32)
    ta = torch.from_numpy(aux)
    return w, ops.upload(torch.from_numpy(plane), ta, ops.parse_header(ta), "cuda")


def fp64_product(w, x):
    """x [T, K] times the exact weights, and the bound sum |w x|, in FP64, in row chunks."""
    ref = torch.empty((x.shape[0], ROWS), dtype=torch.float64, device="cuda")
    bound = torch.empty_like(ref)
    xd = x.double()
    for r0 in range(0, ROWS, 1 << 15):
        wd = w[r0: r0 + (1 << 15)].double()
        ref[:, r0: r0 + wd.shape[0]] = xd @ wd.t()
        bound[:, r0: r0 + wd.shape[0]] = xd.abs() @ wd.abs().t()
    return ref, bound


def test_full_size_tiles_round_trip_and_one_hot(ops, head_tiles):
    w, enc = head_tiles
    assert ops.roundtrip_equal(enc, w)
    assert ops.gemv_max_tokens(enc) > 8
    keep = torch.ones(ROWS, dtype=torch.bool, device="cuda")
    keep[ROWS - 7] = False
    for col in (0, 1033, K - 1):
        x = torch.zeros((1, K), dtype=torch.bfloat16, device="cuda")
        x[0, col] = 0.5
        y = ops.mmv(x, enc)[0]
        assert torch.equal(y[keep], (w[:, col].float() * 0.5)[keep])
        assert bool(torch.isnan(y[ROWS - 7]))


@pytest.mark.parametrize("T", [1, 7, 32, 33, 130])
def test_full_size_tiles_dense_product_any_batch(ops, head_tiles, T):
    w, enc = head_tiles
    g = torch.Generator(device="cuda").manual_seed(20 + T)
    x = torch.randn((T, K), generator=g, device="cuda").to(torch.bfloat16)
    y = ops.mmv(x, enc)
    keep = torch.ones(ROWS, dtype=torch.bool, device="cuda")
    keep[ROWS - 7] = False
    ref, bound = fp64_product(w, x)
    assert bool(((y.double() - ref).abs()[:, keep] <= 1e-5 * bound[:, keep]).all())
    # every column has the bits of its single-column launch, whatever the batch (passes of 32 or of 128 tokens)
    for t in {0, T // 2, T - 1}:
        assert torch.equal(ops.mmv(x[t: t + 1], enc)[0].view(torch.int32), y[t].view(torch.int32))
    # BF16 output: the round-to-nearest-even of the FP32 output; linear() takes the same path up to gemv_max_tokens
    y16 = ops.mmv(x, enc, out_dtype=torch.bfloat16)
    assert torch.equal(y16[:, keep], y[:, keep].to(torch.bfloat16))
    assert T > ops.gemv_max_tokens(enc) or torch.equal(ops.linear(x, enc).view(torch.int16), y16.view(torch.int16))
    # FP32 activations keep their precision: each column goes in as three BF16 components whose products are exact
    # (ten columns per launch); within the same bound, and every column equal to its single-column launch
    if T <= 33:
        xf = torch.randn((T, K), generator=g, device="cuda") * torch.exp(torch.randn((T, K), generator=g, device="cuda"))
        yf = ops.mmv(xf, enc)
        rf, bf = fp64_product(w, xf)
        assert bool(((yf.double() - rf).abs()[:, keep] <= 1e-5 * bf[:, keep]).all())
        for t in {0, T // 2, T - 1}:
            assert torch.equal(ops.mmv(xf[t: t + 1], enc)[0].view(torch.int32), yf[t].view(torch.int32))
        # activations that are BF16 values give the BF16 path's bits (the other two components are zero)
        assert torch.equal(ops.mmv(x.float(), enc)[:, keep], y[:, keep])


def test_full_size_tiles_row_range_and_strides(ops, head_tiles):
    """Through the C ABI: a product over a row range of the matrix, activations and outputs with padded row strides."""
    import ctypes as C

    from orin_qwen_lossless_amd import _lib
    from orin_qwen_lossless_amd.ops import _cweight, _stream

    w, enc = head_tiles
    T, row0, nrows = 5, 32 * 100, 32 * 5000
    g = torch.Generator(device="cuda").manual_seed(31)
    xw = torch.randn((T, K + 8), generator=g, device="cuda").to(torch.bfloat16)
    x = xw[:, :K]
    full = ops.mmv(x.contiguous(), enc)
    yw = torch.zeros((T, nrows + 4), dtype=torch.float32, device="cuda")
    a = _lib.MmvArgs()
    a.x, a.y, a.x_bf16, a.y_bf16 = x.data_ptr(), yw.data_ptr(), 1, 0
    a.ncols, a.n_used, a.x_per_slot = T, 1, 1
    a.x_tok, a.y_tok = x.stride(0) * 2, yw.stride(0) * 4
    a.rows_per_matrix, a.row0, a.nrows = ROWS, row0, nrows
    cw = _cweight(enc)
    _lib.check(_lib.lib().bf16n_mmv(C.byref(cw), C.byref(a), _stream(), 1))
    assert torch.equal(yw[:, :nrows], full[:, row0: row0 + nrows])
    assert not bool(yw[:, nrows:].any())


@pytest.mark.parametrize("K", [1024, 4096])
def test_dense_tiles_other_row_lengths(ops, K):
    # the smallest matrix that takes the dense matrix-core path (131072 rows), with 4 and 16 column slabs per row group
    rows = 131072
    g = torch.Generator(device="cuda").manual_seed(40 + K)
    w = torch.empty((rows, K), dtype=torch.bfloat16, device="cuda")
    for r0 in range(0, rows, 1 << 15):
        w[r0: r0 + (1 << 15)] = (torch.randn((1 << 15, K), generator=g, device="cuda") * 0.02).to(torch.bfloat16)
    assert ops.choose(rows, K, engine="mi355x", dense_frag_order=True) == (3, 32, False, False, True)
    plane, aux, _, _ = ops.encode_bits(w.cpu().view(torch.int16).numpy().view(np.uint16), 3, 32, False, wave64=True)
    ta = torch.from_numpy(aux)
    enc = ops.upload(torch.from_numpy(plane), ta, ops.parse_header(ta), "cuda")
    assert ops.roundtrip_equal(enc, w) and ops.gemv_max_tokens(enc) > 8
    for T, dt in ((3, torch.bfloat16), (40, torch.bfloat16), (2, torch.float32)):
        x = torch.randn((T, K), generator=g, device="cuda").to(dt)
        y = ops.mmv(x, enc)
        for r0 in range(0, rows, 1 << 15):
            wd = w[r0: r0 + (1 << 15)].double()
            ref, bound = x.double() @ wd.t(), x.double().abs() @ wd.abs().t()
            assert bool(((y[:, r0: r0 + (1 << 15)].double() - ref).abs() <= 1e-5 * bound).all()), (K, T, dt, r0)
        assert torch.equal(ops.mmv(x[T - 1:], enc)[0], y[T - 1])


# ---- one MoE layer of the 35B-A3B shape at its real size: 256 experts x (gate, up 512 x 2048; down 2048 x 512) -----------

E, TOPK, N = 256, 8, 512


@pytest.fixture(scope="module")
def experts(ops):
    g = torch.Generator(device="cuda").manual_seed(11)

    def make(rows_per, k):
        w = (torch.randn((E * rows_per, k), generator=g, device="cuda") * 0.02).to(torch.bfloat16)
        fmt, R, cm, _, w64 = ops.choose(rows_per, k, E, engine="mi355x", expert=True)
        assert (fmt, R, w64) == (3, 32, True)                # 32 x 256 tiles
        plane, aux, _, _ = ops.encode_bits(w.cpu().view(torch.int16).numpy().view(np.uint16), fmt, R, cm, wave64=w64)
        ta = torch.from_numpy(aux)
        return w, ops.upload(torch.from_numpy(plane), ta, ops.parse_header(ta), "cuda")

    return make(N, K), make(N, K), make(K, N)


def test_full_size_experts_round_trip(ops, experts):
    for w, enc in experts:
        assert ops.roundtrip_equal(enc, w)


def test_full_size_batched_moe_against_exact_weights_and_the_gemv_path(ops, experts):
    (wg, gate), (wu, up), (wd, down) = experts
    T = 1024                                                   # 8192 routed pairs, about 32 per expert
    g = torch.Generator(device="cuda").manual_seed(12)
    x = torch.randn((T, K), generator=g, device="cuda").to(torch.bfloat16)
    wts, ids = ops.router_topk(torch.randn((T, E), generator=g, device="cuda"), TOPK)
    src1, dst, bounds = ops.mm_ids_route(ids, E, False)
    b = bounds.cpu().numpy()
    assert b[0] == 0 and b[-1] == T * TOPK and np.all(np.diff(b) >= 0)
    # routing lists: a permutation of the pairs, sorted by expert, tokens in order inside an expert
    d = dst.cpu().numpy()
    assert np.array_equal(np.sort(d), np.arange(T * TOPK))
    flat = ids.cpu().numpy().reshape(-1)
    assert np.all(np.diff(flat[d]) >= 0)
    a = ops.moe_mm_ids(x, ids, gate, E, up=up, out_dtype=torch.float32, routes=(src1, dst, bounds))
    # sampled tokens against FP64 products with the exact weights of their experts
    for t in (0, 1, 511, T - 1):
        for s in range(TOPK):
            e = int(ids[t, s])
            xe = x[t].double()
            gg, uu = wg[e * N:(e + 1) * N].double() @ xe, wu[e * N:(e + 1) * N].double() @ xe
            want = uu * (gg / (1.0 + torch.exp(-gg)))
            assert torch.all((a[t, s].double() - want).abs() <= 1e-3 * want.abs() + 1e-5), (t, s)
    # fewer tokens take other shapes of the kernel: passes of 32 tokens at 256 tokens (the same bits for the same
    # tokens), K split over the wavefronts at 16 and 2 tokens, where few experts are active (another summation order)
    for n in (256, 16, 2):
        r = ops.mm_ids_route(ids[:n].contiguous(), E, False)
        an = ops.moe_mm_ids(x[:n], ids[:n].contiguous(), gate, E, up=up, out_dtype=torch.float32, routes=r)
        assert torch.equal(an, a[:n]) if n == 256 else torch.all((an - a[:n]).abs() <= 1e-4 * a[:n].abs() + 1e-6), n
    # the batched kernel and the routed GEMV (decode path) agree on the first tokens; so do the down products
    a8 = ops.mmv_glu2(x[:8], gate, up, ids[:8].contiguous(), N)
    assert torch.all((a8 - a[:8]).abs() <= 1e-3 * a[:8].abs() + 1e-5)
    a16 = a.to(torch.bfloat16)
    ys = ops.moe_mm_ids(a16, ids, down, E, routes=(dst, dst, bounds))
    y8 = ops.mmv(a16[:8].float(), down, ids[:8].contiguous(), K)
    assert torch.all((y8 - ys[:8]).abs() <= 1e-3 * ys[:8].abs() + 1e-5)
    for n in (256, 16, 2):
        r = ops.mm_ids_route(ids[:n].contiguous(), E, False)
        yn = ops.moe_mm_ids(a16[:n], ids[:n].contiguous(), down, E, routes=(r[1], r[1], r[2]))
        assert torch.equal(yn, ys[:n]) if n == 256 else torch.all((yn - ys[:n]).abs() <= 1e-4 * ys[:n].abs() + 1e-6), n
    # linearity in the activations: doubling them doubles every product exactly (powers of two commute with rounding)
    ys2 = ops.moe_mm_ids((a16.float() * 2).to(torch.bfloat16), ids, down, E, routes=(dst, dst, bounds))
    assert torch.equal(ys2, ys * 2)
