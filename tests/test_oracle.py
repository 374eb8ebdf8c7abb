"""Pins the CPU oracle (oracle/bf16n_oracle.c) before anything is checked against it: the reference's own encoder
output (golden fixtures made by oracle/_ref, and oracle/_ref itself where it is built), closed forms of the Huffman
construction, brute force on tiny alphabets, and numpy float64 for the GEMV references."""
from __future__ import annotations

import itertools

import numpy as np
import pytest

from conftest import golden, golden_names
from orin_qwen_lossless_amd import synth


@pytest.mark.parametrize("name", golden_names())
def test_oracle_encoder_matches_reference_bytes(oracle, name):
    z = golden(name)
    fmt, R, cm, fmt_out = (int(v) for v in z["meta"])
    plane, aux, f = oracle.encode(z["w"], fmt, R, bool(cm))
    assert f == fmt_out
    assert np.array_equal(plane, z["plane"])
    if aux.size == z["aux"].size and np.array_equal(aux, z["aux"]):
        return
    # The only licence to differ: symbols of EQUAL frequency may swap code lengths (the reference orders them with an
    # unstable sort, the oracle by symbol value).  Then the header agrees up to the stream length (lane streams are
    # padded to whole words, so swapped lengths can move a few word boundaries), the lengths differ only inside groups
    # of equal frequency, and both codes cost the same number of bits.
    assert fmt_out in (2, 3)
    h, hr = oracle.parse_header(aux), oracle.parse_header(z["aux"])
    assert {k: v for k, v in h.items() if k != "n_b"} == {k: v for k, v in hr.items() if k != "n_b"}
    assert abs(h["n_b"] - hr["n_b"]) <= 32 * h["n_a"] and aux.size - z["aux"].size == 4 * (h["n_b"] - hr["n_b"])
    ex = (z["w"].astype(np.uint32) >> 7) & 0xFF
    if fmt_out == 3:
        sym = (ex.reshape(-1)[0::2] | (ex.reshape(-1)[1::2] << 8))
    else:
        sym = ex.reshape(-1)
    freq = np.bincount(sym, minlength=65536)

    def lengths(a):
        out = np.zeros(65536, dtype=np.int64)
        if fmt_out == 3:
            lut = a[h["off_a"]: h["off_a"] + 16384].view(np.uint32)
            out[((lut >> 7) & 0xFF) | (((lut >> 23) & 0xFF) << 8)] = lut & 0x7F
        else:
            lut = a[h["off_a"]: h["off_a"] + 4096].view(np.uint32)
            out[(lut >> 7) & 0xFF] = lut & 0x7F
        return out

    lo, lr = lengths(aux), lengths(z["aux"])
    assert int((freq * lo).sum()) == int((freq * lr).sum())
    for fv in np.unique(freq[lo != lr]):
        grp = freq == fv
        assert sorted(lo[grp]) == sorted(lr[grp])
    assert np.array_equal(oracle.decode(plane, aux), z["w"])


@pytest.mark.parametrize("name", golden_names())
def test_oracle_decoder_inverts_reference_encoder(oracle, name):
    z = golden(name)
    assert np.array_equal(oracle.decode(z["plane"], z["aux"]), z["w"])


def test_header_fields_of_reference_output(oracle):
    z = golden("hp_cm_k2048_r8")
    h = oracle.parse_header(z["aux"])
    assert (h["magic"], h["format"], h["K"], h["R"], h["rows"], h["flags"]) == (0x4E363142, 3, 2048, 8, 16, 1)
    assert h["off_a"] == 256 and h["off_b"] == 256 + 16384 and h["off_c"] == h["off_b"] + 4 * 2 and h["off_d"] % 16 == 0
    assert z["aux"].size == h["off_d"] + 4 * (h["n_b"] + 32)
    z = golden("nib_k512")
    h = oracle.parse_header(z["aux"])
    assert h["off_b"] == 256 + 32 * 512 // 2 and h["off_c"] == h["off_b"] + 32 * 16 and h["off_d"] == h["off_c"] + 4 * 33


def test_fallback_boundary(oracle):
    # more than 4096 distinct exponent pairs -> single-symbol format, not at 4096 (core/tests/test_encode.cpp:262-269)
    for n, want in ((4095, 3), (4096, 3), (4097, 2)):
        w = synth.with_pairs(16, 1024, n)
        _, aux, f = oracle.encode(w, 3, 4, False)
        assert f == want and oracle.parse_header(aux)["format"] == want
        _, aux, f = oracle.encode(w, 3, 4, True)
        assert f == want and oracle.parse_header(aux)["flags"] == (1 if want == 3 else 0)


@pytest.mark.parametrize("n_exp", [14, 15, 16, 17])
def test_nibble_escape_count(oracle, n_exp):
    # 15 table entries besides exponent 0: the rarest n_exp - 15 exponents escape, with their exact counts
    # (tests/core/test_roundtrip.py:105-130)
    w = synth.nibble_rows_with_exponents(4, 512, n_exp, 20 + n_exp)
    plane, aux, _ = oracle.encode(w, 1, 0, False)
    h = oracle.parse_header(aux)
    ex = (w >> 7) & 0xFF
    want = 0
    for r in range(4):
        counts = np.sort(np.bincount(ex[r], minlength=256))[::-1]
        want += int(counts[15:].sum())
    assert h["n_a"] == want
    assert np.array_equal(oracle.decode(plane, aux), w)


def test_nibble_large_exponents_always_escape(oracle):
    z = golden("nib_exp128")
    h = oracle.parse_header(z["aux"])
    assert h["n_a"] == int((((z["w"] >> 7) & 0xFF) >= 128).sum())


def _kraft(lens):
    return sum(2.0 ** -int(l) for l in lens if l)


def _brute_force_cost(freq, L):
    """Optimal length-limited prefix code cost by exhaustive search over length multisets (tiny n)."""
    n = len(freq)
    f = sorted(freq, reverse=True)  # an optimal code gives longer codes to rarer symbols
    best = None
    for lens in itertools.combinations_with_replacement(range(1, L + 1), n):
        if sum(2.0 ** -l for l in lens) <= 1.0 + 1e-12:
            cost = sum(a * b for a, b in zip(f, lens))  # lens ascending with f descending
            best = cost if best is None or cost < best else best
    return best


@pytest.mark.parametrize("seed", range(12))
def test_package_merge_is_optimal_on_tiny_alphabets(oracle, seed):
    rng = np.random.default_rng(seed)
    n = int(rng.integers(2, 7))
    L = int(rng.integers(max(1, int(np.ceil(np.log2(n)))), 5))
    freq = rng.integers(1, 40, size=n).astype(np.uint64)
    lens = oracle.limited_lengths(freq, L)
    assert lens.max() <= L and lens.min() >= 1
    assert abs(_kraft(lens) - 1.0) < 1e-12
    assert int((freq * lens.astype(np.uint64)).sum()) == _brute_force_cost([int(v) for v in freq], L)


def test_package_merge_equals_huffman_when_unconstrained(oracle):
    # with a generous limit the cost equals the classical Huffman cost (sum of merged weights)
    import heapq

    rng = np.random.default_rng(5)
    freq = rng.integers(1, 1000, size=40).astype(np.uint64)
    h = [int(v) for v in freq]
    heapq.heapify(h)
    cost = 0
    while len(h) > 1:
        a, b = heapq.heappop(h), heapq.heappop(h)
        cost += a + b
        heapq.heappush(h, a + b)
    lens = oracle.limited_lengths(freq, 32)
    assert int((freq * lens.astype(np.uint64)).sum()) == cost


def test_package_merge_special_cases(oracle):
    assert list(oracle.limited_lengths(np.array([0, 7, 0], dtype=np.uint64), 12)) == [0, 1, 0]  # one symbol: length 1
    lens = oracle.limited_lengths(np.ones(4096, dtype=np.uint64), 12)  # full alphabet at the limit: all 12
    assert set(lens.tolist()) == {12}
    lens = oracle.limited_lengths(np.array([1, 1, 2, 4, 8, 16, 32, 64], dtype=np.uint64), 4)  # skewed, limited to 4
    assert lens.max() == 4 and abs(_kraft(lens) - 1.0) < 1e-12


def test_lut_is_a_complete_prefix_code(oracle):
    z = golden("hp_rm_k2048_r4")
    h = oracle.parse_header(z["aux"])
    lut = z["aux"][h["off_a"]: h["off_a"] + 16384].view(np.uint32)
    lens = lut & 0x7F
    assert lens.min() >= 1 and lens.max() <= 12
    # every entry with length l is shared by a run of 2^(12-l) aligned windows
    i = 0
    while i < 4096:
        span = 1 << (12 - int(lens[i]))
        assert i % span == 0 and np.all(lut[i: i + span] == lut[i])
        i += span


def test_cfg1_table_matches_reference(oracle):
    # the 2048 x 2048 N(0, 0.02) tensor of the CPU benchmark configuration: table and coded size from the reference
    z = golden("cfg1_lut")
    w = synth.weights(2048, 2048, 1)
    plane, aux, _ = oracle.encode(w, 3, 4, False)
    h = oracle.parse_header(aux)
    assert np.array_equal(aux[h["off_a"]: h["off_a"] + 16384], z["lut"])
    assert [h["n_b"], aux.size, int(plane.astype(np.uint64).sum())] == [int(v) for v in z["meta"]]


def test_against_reference_library_when_built(oracle):
    if oracle.ref() is None:
        pytest.skip("oracle/_ref is only built where the reference checkout exists")
    for K, fmt, R, cm in ((1024, 3, 8, True), (512, 3, 2, False), (1536, 2, 4, False), (3072, 1, 0, False)):
        w = synth.model_like(16, K, 1000 + K)
        p, a, f = oracle.encode(w, fmt, R, cm)
        rp, ra, rf, _ = oracle.ref_encode(w, fmt, R, cm)
        assert f == rf and np.array_equal(p, rp) and np.array_equal(a, ra)
    for bad in ((16, 500, 3, 4, False), (15, 512, 3, 4, False), (16, 512, 3, 4, True), (16, 1024, 2, 4, True), (16, 512, 1, 4, False)):
        rows, K, fmt, R, cm = bad
        w = np.zeros((rows, K), dtype=np.uint16)
        with pytest.raises(ValueError):
            oracle.ref_encode(w, fmt, R, cm)
        with pytest.raises(ValueError):
            oracle.encode(w, fmt, R, cm)


# ---------------------------------------------------------------- numeric references

def test_gemv_references_against_numpy(oracle):
    w = synth.weights(64, 1024, 7)
    x = synth.bf16_bits_to_f32(synth.activations(1, 1024, 8)[0])
    wf = synth.bf16_bits_to_f32(w).astype(np.float64)
    y64, s = oracle.gemv_f64(w, x)
    assert np.allclose(y64, wf @ x.astype(np.float64), rtol=1e-12, atol=0)
    assert np.allclose(s, np.abs(wf) @ np.abs(x.astype(np.float64)), rtol=1e-12)
    for cm in (False, True):
        y32 = oracle.gemv_f32(w, x, cm)
        assert np.all(np.abs(y32 - y64) <= 1e-5 * s)


def test_gemv_one_hot_is_exact(oracle):
    # a single activation of +-2^k picks one weight per row: the result is that BF16 value scaled, exactly
    # (llama.cpp backend tests of the reference, patch 0008:139-165)
    w = synth.model_like(32, 512, 9)
    w[(w & 0x7F80) == 0x7F80] = 0x3F80  # no Inf/NaN
    for k, scale in ((5, 0.25), (300, -4.0), (511, 1.0)):
        x = np.zeros(512, dtype=np.float32)
        x[k] = scale
        y = oracle.gemv_f32(w, x)
        assert np.array_equal(y, synth.bf16_bits_to_f32(w[:, k]) * np.float32(scale))


def test_decode_gemv_equals_gemv_on_decoded_weights(oracle):
    for name in ("hp_rm_k2048_r4", "hp_cm_k2048_r8", "nib_k2048", "huf_k1024_r8", "nib_exp17"):
        z = golden(name)
        w = z["w"].copy()
        K = w.shape[1]
        x = synth.bf16_bits_to_f32(synth.activations(1, K, 3)[0])
        h = oracle.parse_header(z["aux"])
        y = oracle.decode_gemv(z["plane"], z["aux"], x)
        finite = ((w & 0x7F80) != 0x7F80).all(axis=1)
        if h["format"] == 1:
            y64, s = oracle.gemv_f64(np.where(((w & 0x7F80) == 0x7F80), 0, w).astype(np.uint16), x)
            finite &= s < 1e30  # rows holding the largest finite BF16 overflow FP32
            assert np.all(np.abs(y[finite] - y64[finite]) <= 1e-5 * s[finite] + 1e-30)
        else:
            ref = oracle.gemv_f32(w, x, bool(h["flags"] & 1))
            assert np.array_equal(y[finite], ref[finite])


def test_swiglu_combine_route_router(oracle):
    rng = np.random.default_rng(0)
    g, u = rng.standard_normal(1000).astype(np.float32), rng.standard_normal(1000).astype(np.float32)
    want = g.astype(np.float64) / (1 + np.exp(-g.astype(np.float64))) * u
    assert np.allclose(oracle.swiglu(g, u), want, rtol=1e-6, atol=1e-7)
    ys = rng.standard_normal((5, 8, 64)).astype(np.float32)
    wt = rng.random((5, 8)).astype(np.float32)
    assert np.allclose(oracle.moe_combine(ys, wt), np.einsum("tk,tkn->tn", wt.astype(np.float64), ys), rtol=1e-5, atol=1e-6)
    # routing: brute force = stable sort of (expert, token) pairs
    T, k, E = 37, 8, 16
    ids = np.stack([rng.permutation(E)[:k] for _ in range(T)]).astype(np.int32)
    src1, dst, bounds = oracle.route(ids, E, k, k)  # activations per routed slot: row t * k + s
    pairs = sorted((int(ids[t, s]), t, s) for t in range(T) for s in range(k))
    assert [int(v) for v in dst] == [t * k + s for _, t, s in pairs]
    assert [int(v) for v in src1] == [t * k + s for _, t, s in pairs]
    assert [int(v) for v in oracle.route(ids, E, 1, 1)[0]] == [t for _, t, _ in pairs]  # one row per token
    assert [int(v) for v in bounds] == [sum(1 for e, _, _ in pairs if e < b) for b in range(E + 1)]
    # a token that names an expert twice: the last slot is listed, and later lists start behind every naming
    # (mmid_helper.cu:66-71 counts namings, not list entries), worked by hand for ids [[0, 0], [1, 2]]
    _, dst2, bounds2 = oracle.route(np.array([[0, 0], [1, 2]], dtype=np.int32), 3, 2, 2)
    assert [int(v) for v in bounds2] == [0, 2, 3, 4] and [int(dst2[j]) for j in (0, 2, 3)] == [1, 2, 3]
    # router: closed forms only (no reference counterpart)
    lg = rng.standard_normal(256).astype(np.float32)
    rid, rw = oracle.router_topk(lg, 8)
    assert list(rid) == list(np.argsort(-lg, kind="stable")[:8]) and abs(rw.sum() - 1) < 1e-6
    p = np.exp(lg.astype(np.float64) - lg.max())
    assert np.allclose(rw, p[rid] / p[rid].sum(), rtol=1e-5)
    lg[:] = 0
    assert list(oracle.router_topk(lg, 4)[0]) == [0, 1, 2, 3]  # ties: lower index first
