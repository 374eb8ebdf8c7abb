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


@pytest.mark.parametrize("T,distinct", [(1, False), (2, False), (4, False), (8, False), (16, False), (20, True), (28, False),
                                        (30, True), (40, "popular"), (70, "popular")])
def test_batched_kernels_at_every_split_of_k(ops, experts, T, distinct):
    """Few tokens through the batched kernels: the kernel that splits K over wavefronts picks its split on the device
    from the experts that are active — 8 wavefronts per item for 8 to 32 experts (an expert's K is 8 tiles), 4 up to
    64, 2 up to 128, and whole chains when the routing has more active experts than the host's estimate (20 tokens whose
    160 experts are all different: the estimate for uniform routing is 119).  More than 128 active experts give the down
    product (32 items per expert) more items than the launch holds at once: a second round, dealt out evenly over the
    blocks (28 tokens; 30 tokens whose 240 experts are all different).  An expert that every token uses has more than
    the 32 tokens of a pass: its passes are listed as work of their own and run on different blocks (40 and 70 tokens:
    two and three passes, the last one ragged).  Every (token, slot) output of the fused gate/up product and of the
    down product against FP64 products of the exact weights."""
    (wg, gate), (wu, up), (wd, down) = experts
    g = torch.Generator(device="cuda").manual_seed(300 + T)
    x = torch.randn((T, K), generator=g, device="cuda").to(torch.bfloat16)
    if distinct is True:
        ids = torch.randperm(E, generator=g, device="cuda")[: T * TOPK].to(torch.int32).view(T, TOPK).contiguous()
    else:
        logits = torch.randn((T, E), generator=g, device="cuda")
        if distinct == "popular":
            logits[:, 7] = 50.0  # every token's first choice
        _, ids = ops.router_topk(logits, TOPK)
        assert distinct != "popular" or bool((ids[:, 0] == 7).all())
    src1, dst, bounds = ops.mm_ids_route(ids, E, False)
    a = ops.moe_mm_ids(x, ids, gate, E, up=up, out_dtype=torch.float32, routes=(src1, dst, bounds))
    a16 = a.to(torch.bfloat16)
    ys = ops.moe_mm_ids(a16, ids, down, E, routes=(dst, dst, bounds))
    for t in range(T):
        xe = x[t].double()
        for s in range(TOPK):
            e = int(ids[t, s])
            gg, uu = wg[e * N:(e + 1) * N].double() @ xe, wu[e * N:(e + 1) * N].double() @ xe
            want = uu * silu64(gg)
            assert torch.all((a[t, s].double() - want).abs() <= 1e-3 * want.abs() + 1e-5), (t, s)
            h = a16[t, s].double()
            wde = wd[e * K:(e + 1) * K].double()
            err = (ys[t, s].double() - wde @ h).abs()
            assert torch.all(err <= 1e-5 * (wde.abs() @ h.abs())), (t, s)


# ---- the benchmark configurations at their stated sizes ---------------------------------------------------------------

def upload_policy(ops, w, n_matrices=1):
    """Encode a [rows, K] BF16 device tensor in the layout the mi355x policy picks and upload it."""
    rows, k = w.shape
    fmt, R, cm, _, w64 = ops.choose(rows // n_matrices, k, n_matrices, engine="mi355x", expert=n_matrices > 1)
    plane, aux, _, _ = ops.encode_bits(w.cpu().view(torch.int16).numpy().view(np.uint16), fmt, R, cm, wave64=w64)
    ta = torch.from_numpy(aux)
    return ops.upload(torch.from_numpy(plane), ta, ops.parse_header(ta), "cuda")


def silu64(g):
    return g / (1.0 + torch.exp(-g))


@pytest.mark.parametrize("T", [2048, 8192])
def test_prefill_at_the_benchmark_token_counts(ops, oracle, experts, T):
    """Batched MoE prefill of the 256-expert layer at 2048 and 8192 tokens: routing lists equal to the oracle's, and
    sampled (token, slot) outputs of the fused gate/up product and of the down product against FP64 products of the
    exact weights (1e-3 relative / 1e-5 absolute; and the reassociation bound 1e-5 * sum |w x| where the output is not
    a product of rounded intermediates); the whole layer output is bitwise equivariant under a permutation of the
    tokens."""
    (wg, gate), (wu, up), (wd, down) = experts
    g = torch.Generator(device="cuda").manual_seed(100 + T)
    x = torch.randn((T, K), generator=g, device="cuda").to(torch.bfloat16)
    wts, ids = ops.router_topk(torch.randn((T, E), generator=g, device="cuda"), TOPK)
    src1, dst, bounds = ops.mm_ids_route(ids, E, False)
    o_src1, o_dst, o_bounds = oracle.route(ids.cpu().numpy(), E, 1, 1)
    assert np.array_equal(bounds.cpu().numpy(), o_bounds)
    assert np.array_equal(dst.cpu().numpy(), o_dst) and np.array_equal(src1.cpu().numpy(), o_src1)
    load = np.diff(o_bounds)
    assert load.min() > 0 and load.max() < 2 * T * TOPK // E    # near-uniform expert load, as the configuration states
    a = ops.moe_mm_ids(x, ids, gate, E, up=up, out_dtype=torch.float32, routes=(src1, dst, bounds))
    a16 = ops.moe_mm_ids(x, ids, gate, E, up=up, out_dtype=torch.bfloat16, routes=(src1, dst, bounds))
    assert torch.equal(a16, a.to(torch.bfloat16))                # BF16 out is the rounding of the FP32 accumulators
    ys = ops.moe_mm_ids(a16, ids, down, E, routes=(dst, dst, bounds))
    rng = np.random.default_rng(T)
    tokens = [0, T - 1] + rng.integers(1, T - 1, 30).tolist()
    for t in tokens:
        xe = x[t].double()
        for s in range(TOPK):
            e = int(ids[t, s])
            gg, uu = wg[e * N:(e + 1) * N].double() @ xe, wu[e * N:(e + 1) * N].double() @ xe
            want = uu * silu64(gg)
            assert torch.all((a[t, s].double() - want).abs() <= 1e-3 * want.abs() + 1e-5), (t, s)
            h = a16[t, s].double()
            wde = wd[e * K:(e + 1) * K].double()
            want_y, bound = wde @ h, wde.abs() @ h.abs()
            err = (ys[t, s].double() - want_y).abs()
            assert torch.all(err <= 1e-5 * bound), (t, s)
            assert torch.all(err <= 1e-3 * want_y.abs() + 1e-5), (t, s)
    # the layer through moe_experts (routing lists, both products, weighted sum) for the sampled tokens
    y = ops.moe_experts(x, gate, up, down, wts, ids, E)
    comb = (ys[tokens].double() * wts[tokens].double().unsqueeze(-1)).sum(1)
    assert torch.all((y[tokens].double() - comb).abs() <= 2.0 ** -8 * comb.abs() + 1e-6)
    # over the whole output: a token's row does not depend on where the token stands in the batch (its place in the
    # routing lists and in the 32-token blocks changes, its arithmetic does not)
    perm = torch.randperm(T, generator=g, device="cuda")
    y_perm = ops.moe_experts(x[perm].contiguous(), gate, up, down, wts[perm].contiguous(), ids[perm].contiguous(), E)
    assert torch.equal(y_perm, y[perm])


@pytest.fixture(scope="module")
def moe_small_parts(ops):
    """Router 256 x 2048 and the shared expert ([gate; up] 1024 x 2048, down 2048 x 512) under the mi355x policy."""
    g = torch.Generator(device="cuda").manual_seed(21)
    ws = {name: (torch.randn(shape, generator=g, device="cuda") * 0.02).to(torch.bfloat16)
          for name, shape in (("router", (E, K)), ("sh_gate_up", (2 * N, K)), ("sh_down", (K, N)))}
    return {name: (w, upload_policy(ops, w)) for name, w in ws.items()}


def graph_of(fn):
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


@pytest.mark.parametrize("T", [1, 4])
def test_moe_decode_layer_256_experts_as_one_graph(ops, experts, moe_small_parts, T):
    """The MoE decode layer at its stated size (256 experts as 32 x 256 tiles, top-8 chosen on the device from the
    router's logits, shared expert) captured as one HIP graph: every replay on new activations equals the eager result
    bit for bit, the routing changes between replays, and the result agrees with FP64 on the exact weights."""
    (wg, gate), (wu, up), (wd, down) = experts
    (wr, router), (wsg, sh_gu), (wsd, sh_dn) = (moe_small_parts[k] for k in ("router", "sh_gate_up", "sh_down"))
    assert all(m.meta.format == 1 for m in (router, sh_gu, sh_dn))   # small matrices: the fixed 4-bit code
    g = torch.Generator(device="cuda").manual_seed(30 + T)
    xs = [torch.randn((T, K), generator=g, device="cuda").to(torch.bfloat16) for _ in range(4)]
    x = xs[0].clone()

    def layer():
        wts, ids = ops.router_topk(ops.mmv(x, router), TOPK)
        routed = ops.moe_experts(x, gate, up, down, wts, ids, E)
        shared = ops.mmv(ops.mmv_glu(x, sh_gu), sh_dn, out_dtype=torch.bfloat16)
        return routed, shared, ids, wts

    graph, outs = graph_of(layer)
    seen = set()
    for rep in range(4):
        x.copy_(xs[rep])
        want = [t.clone() for t in layer()]
        torch.cuda.synchronize()
        for t in outs:
            t.zero_()
        graph.replay()
        torch.cuda.synchronize()
        for got, ref in zip(outs, want):
            assert torch.equal(got, ref), rep
        seen.add(tuple(outs[2].cpu().numpy().reshape(-1).tolist()))
    assert len(seen) == 4
    routed, shared, ids, wts = outs
    xd = x.double()
    # the router: logits of the exact weights, the same top-8 (no ties in random data), softmax weights renormalised
    logits = xd @ wr.double().t()
    top = torch.topk(logits, TOPK, dim=-1)
    assert torch.equal(top.indices.int(), ids)
    p = torch.softmax(logits, -1).gather(1, top.indices)
    assert torch.allclose(wts.double(), p / p.sum(-1, keepdim=True), rtol=1e-4, atol=1e-7)
    for t in range(T):
        acc = torch.zeros(K, dtype=torch.float64, device="cuda")
        for s in range(TOPK):
            e = int(ids[t, s])
            h = silu64(wg[e * N:(e + 1) * N].double() @ xd[t]) * (wu[e * N:(e + 1) * N].double() @ xd[t])
            acc += float(wts[t, s]) * (wd[e * K:(e + 1) * K].double() @ h)
        assert torch.all((routed[t].double() - acc).abs() <= 2.0 ** -7 * acc.abs() + 1e-5), t
        h = silu64(wsg[:N].double() @ xd[t]) * (wsg[N:].double() @ xd[t])
        want_sh = wsd.double() @ h
        assert torch.all((shared[t].double() - want_sh).abs() <= 2.0 ** -7 * want_sh.abs() + 1e-5), t


@pytest.mark.parametrize("name,rows,k,mode,want", [
    ("qkv", 5120, 2048, "hybrid", (1, 0, False, False)), ("o", 2048, 4096, "hybrid", (1, 0, False, False)),
    ("qkv", 5120, 2048, "huffman", (3, 2, False, True)), ("o", 2048, 4096, "huffman", (3, 1, False, True)),
    ("cfg1", 2048, 2048, "huffman", (3, 2, False, True))])
def test_dense_matrices_of_the_decode_step(ops, oracle, name, rows, k, mode, want):
    """The per-layer dense projections in the layouts the mi355x policy gives them (the 4-bit code in hybrid mode, short
    wave64 units when the Huffman family is asked for), and the 2048 x 2048 matrix of the CPU reference configuration
    (its configuration names the pair code), at batch 1 and 4 against the oracle's FP32-accumulated GEMV and its FP64
    bound; the decode is bit-exact and the oracle decodes the encoder's bytes to the same weights."""
    from orin_qwen_lossless_amd import synth

    wb = synth.weights(rows, k, 500 + rows % 97)
    fmt, r, cm, _, w64 = ops.choose(rows, k, engine="mi355x", mode=mode)
    assert (fmt, r, cm, w64) == want
    plane, aux, _, _ = ops.encode_bits(wb, fmt, r, cm, wave64=w64)
    assert np.array_equal(oracle.decode(plane, aux), wb)
    ta = torch.from_numpy(aux)
    enc = ops.upload(torch.from_numpy(plane), ta, ops.parse_header(ta), "cuda")
    assert ops.roundtrip_equal(enc, torch.from_numpy(wb.view(np.int16)).view(torch.bfloat16))
    xb = synth.activations(4, k, 77)
    x = torch.from_numpy(xb.view(np.int16)).view(torch.bfloat16).cuda()
    y4 = ops.mmv(x, enc).cpu().numpy()
    on_matrix_cores = ops.last_kernel().startswith("k_nib_mm16<")   # the 4-bit code: four columns in 16-row groups
    assert on_matrix_cores == (fmt == 1)
    y4_cols = ops.mmv(x, enc, multi_col=False).cpu().numpy()         # per-column launches
    for t in range(4):
        xf = synth.bf16_bits_to_f32(xb[t])
        ref32 = oracle.gemv_f32(wb, xf)
        y64, bound = oracle.gemv_f64(wb, xf)
        y1 = ops.mmv(x[t: t + 1], enc).cpu().numpy()[0]
        assert np.array_equal(y1, y4_cols[t])                  # four batch-1 products, bit for bit
        if not on_matrix_cores:
            assert np.array_equal(y1, y4[t])                   # the column groups of the wave64 GEMV keep those bits
        for y in (y1, y4[t]):
            assert np.all(np.abs(y - ref32) <= 1e-3 * np.abs(ref32) + 1e-5)
            assert np.all(np.abs(y - y64) <= 1e-5 * bound)
    y16 = ops.linear(x, enc)
    assert np.array_equal(y16.cpu().view(torch.int16).numpy().view(np.uint16), synth.f32_to_bf16_bits(y4))


@pytest.mark.parametrize("rows,k", [(5120, 2048), (2048, 4096), (1000, 512)])
def test_nibble_projection_columns_share_a_decode_bit_for_bit(ops, oracle, rows, k):
    """Dense batches on a 4-bit matrix, escapes included.  FP32 columns, and BF16 columns on a matrix too small for the
    matrix cores, share decodes on the VALU and have the bits of their single-column products.  Up to 16 BF16 columns
    run on the matrix cores in 16-row groups where these fill the CUs (from two columns), half of them (from three) or
    a quarter (from five), also in several blocks of 16 tokens while the launch is at most two blocks per CU; larger
    batches in 32-row groups, 32 tokens per decode (with groups for a quarter of the CUs, from 25 columns with an
    eighth).  On either kernel a column has the same bits at every batch size and at every
    position (a token's sum never meets another token's), within the FP64 bound of the GEMV.  Rows that are no multiple
    of the group and batches that are no multiple of the token block leave a ragged last block."""
    from orin_qwen_lossless_amd import synth

    wb = synth.weights(rows, k, 900 + rows % 89)
    wb[::5, ::131] = np.uint16(0x4500)  # exponents outside a row's window: escape records
    plane, aux, fmt, _ = ops.encode_bits(wb, 1, 0)
    assert fmt == 1
    ta = torch.from_numpy(aux)
    enc = ops.upload(torch.from_numpy(plane), ta, ops.parse_header(ta), "cuda")
    xb = synth.activations(70, k, 78)
    x = torch.from_numpy(xb.view(np.int16)).view(torch.bfloat16).cuda()
    single = torch.cat([ops.mmv(x[t: t + 1], enc) for t in range(9)])
    cus = torch.cuda.get_device_properties(0).multi_processor_count
    g16, g32 = (rows + 15) // 16, (rows + 31) // 32
    first16 = 2 if g16 >= cus else 3 if g16 * 2 >= cus else 5 if g16 * 4 >= cus else 10 ** 9
    first32 = 5 if g32 * 2 >= cus else 9 if g32 * 4 >= cus else 25 if g32 * 8 >= cus else 10 ** 9

    def on_16_row_groups(T):  # several blocks of 16 tokens while the launch stays within two blocks per CU
        return T >= first16 and (T <= 16 or g16 * ((T + 15) // 16) <= 2 * cus)

    y70 = ops.mmv(x, enc)
    assert not on_16_row_groups(70) or first32 > 70
    by16 = torch.cat([ops.mmv(x[i: i + 16], enc) for i in range(0, 64, 16)])  # (on 16-row groups wherever a batch is)
    y16 = by16[:16]
    for T in (2, 3, 4, 5, 8, 9, 16, 17, 24, 25, 31, 32, 33, 64):
        y = ops.mmv(x[:T], enc)
        kernel = ops.last_kernel()
        if on_16_row_groups(T):
            assert kernel.startswith("k_nib_mm16<") and torch.equal(y, by16[:T]), (T, kernel)
        elif T >= first32:
            assert kernel.startswith("k_nib_mm<") and torch.equal(y, y70[:T]), (T, kernel)
        else:
            assert kernel.startswith("k_nib_mmv<") and torch.equal(y[:9], single[:T]), (T, kernel)
    if first32 <= 28 and not on_16_row_groups(28):
        assert torch.equal(ops.mmv(x[37:65], enc), y70[37:65])  # other positions in the block of 32
        assert not torch.equal(y70[:9], single)                 # (the two paths do differ: another order of summation)
    if first16 <= 9:
        assert torch.equal(ops.mmv(x[5:14], enc), y16[5:14])    # other positions in the block of 16
        assert not torch.equal(y16[:9], single)
    y70n, y16n = y70.cpu().numpy(), y16.cpu().numpy()
    for t in (0, 2, 31, 32, 69):
        y64, bound = oracle.gemv_f64(wb, synth.bf16_bits_to_f32(xb[t]))
        assert np.all(np.abs(y70n[t] - y64) <= 1e-5 * bound), t
        if t < 9:
            assert np.all(np.abs(single[t].cpu().numpy() - y64) <= 1e-5 * bound), t
            assert np.all(np.abs(y16n[t] - y64) <= 1e-5 * bound), t
    # BF16 out: the one rounding of the FP32 sums
    for n, ref in ((70, y70n), (12, y16n)):
        yb = ops.mmv(x[:n], enc, out_dtype=torch.bfloat16)
        assert np.array_equal(yb.cpu().view(torch.int16).numpy().view(np.uint16), synth.f32_to_bf16_bits(ref[:n]))
    # a caller that asks for per-column launches gets the single-column bits at any count
    assert torch.equal(ops.mmv(x[:9], enc, multi_col=False), single)
    xf = x[:4].float()
    single_f = torch.cat([ops.mmv(xf[t: t + 1], enc) for t in range(4)])
    assert torch.equal(ops.mmv(xf, enc), single_f)


# ---- the decode step (40 x [qkv, o, router, top-8, 256 experts + shared, glue]): two layers of it at real size ------------

@pytest.fixture(scope="module")
def step_sets(ops):
    from orin_qwen_lossless_amd import decode_step as D, synth

    seed = [4000]

    def gen(rows, k):
        seed[0] += 1
        return synth.weights_torch(rows, k, seed[0], "cuda")

    sets, raw, nbytes = D.make_layer_sets(ops, gen, 2, True)
    for enc_set, raw_set in zip(sets, raw):
        for name in ("qkv", "o"):
            assert ops.roundtrip_equal(enc_set[name], raw_set[name])
    # the layouts the policy gives the step's matrices: the 4-bit code for the dense ones (all below 1.5 x the dense
    # minimum), 32 x 256 tiles for the stacked experts
    m = {k: (v.meta.format, v.meta.R, v.meta.wave64) for k, v in sets[0].items()}
    assert m == {"qkv": (1, 0, False), "o": (1, 0, False), "router": (1, 0, False), "gate": (3, 32, True), "up": (3, 32, True), "down": (3, 32, True)}
    return sets, raw, nbytes


def rn(t):
    """Round an FP64 tensor to BF16 and back (the roundings the step makes between its launches)."""
    return t.float().to(torch.bfloat16).double()


def rms(t):
    return t * torch.rsqrt((t * t).mean(-1, keepdim=True) + 1e-6)


@pytest.mark.parametrize("T", [1, 4])
def test_decode_step_two_layers_as_one_graph(ops, step_sets, T):
    """Two layers of the decode step at their real size (8 launches each) captured as one HIP graph: every replay on new
    activations equals the eager step bit for bit; and one layer against an FP64 evaluation on the exact weights that
    rounds where the step rounds (BF16 between the launches), with the experts the step's router picked."""
    from orin_qwen_lossless_amd import decode_step as D, synth

    sets, raw, _ = step_sets
    step = D.Bf16nStep(ops, sets, None, 2, T)
    hs = [synth.activations_torch(T, D.K_MODEL, 4100 + i, "cuda") for i in range(3)]
    hbuf = hs[0].clone()
    graph, out = D.capture(step, hbuf)
    for rep in range(3):
        hbuf.copy_(hs[rep])
        want = step(hbuf).clone()
        torch.cuda.synchronize()
        out.zero_()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out, want), rep
    # one layer against FP64
    w, r = sets[0], raw[0]
    h = hs[1]
    x1 = ops.add_rmsnorm(h)
    x1n, hn = step.layer(w, h, x1)
    wts, ids = step.routing
    W = {k: v.double() for k, v in r.items() if k in ("qkv", "o", "router")}
    hd = h.double()
    x1r = rn(rms(hd))
    assert torch.equal(x1.double(), x1r) or bool(((x1.double() - x1r).abs() <= 2.0 ** -8 * x1r.abs()).all())
    q = rn(x1.double() @ W["qkv"].t())
    o = rn(q[:, :D.ATT] @ W["o"].t())
    s = hd + o
    h2, x2 = rn(s), rn(rms(s))
    logits = x2 @ W["router"].t()
    top = torch.topk(logits, D.TOPK, dim=-1)
    for t in range(T):  # the step's experts are the FP64 top-8 (margins in random data are far above the rounding)
        assert set(ids[t, :D.TOPK].tolist()) == set(top.indices[t].tolist()), t
    assert bool((ids[:, D.TOPK] == D.E).all()) and bool((wts[:, D.TOPK] == 1.0).all())
    comb = torch.zeros((T, D.K_MODEL), dtype=torch.float64, device="cuda")
    for t in range(T):
        for k in range(D.TOPK + 1):
            e = int(ids[t, k])
            g = r["gate"][e * D.N_MID:(e + 1) * D.N_MID].double() @ x2[t]
            u = r["up"][e * D.N_MID:(e + 1) * D.N_MID].double() @ x2[t]
            hid = (g / (1.0 + torch.exp(-g)) * u).float().double()       # the hidden activations stay FP32 in the GEMV path
            comb[t] += float(wts[t, k]) * (r["down"][e * D.K_MODEL:(e + 1) * D.K_MODEL].double() @ hid)
    s2 = h2 + comb
    href, xref = rn(s2), rn(rms(s2))
    scale = float(href.abs().max())
    assert bool(((hn.double() - href).abs() <= 2.0 ** -6 * href.abs() + 2e-3 * scale).all())
    assert bool(((x1n.double() - xref).abs() <= 2.0 ** -6 * xref.abs() + 2e-3 * float(xref.abs().max())).all())
