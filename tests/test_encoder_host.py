"""Host side of the product on the CPU: the C++ encoder and policy behind the C ABI against the golden fixtures
(reference output, byte for byte), the oracle, the reference's argument contract (core/tests/test_encode.cpp:271-306)
and policy tables (core/tests/test_policy.cpp:38-161); the library's exported symbols against include/bf16n_c.h."""
from __future__ import annotations

import csv
import os
import re

import numpy as np
import pytest

from conftest import GOLDEN, ROOT, golden, golden_names
from orin_qwen_lossless_amd import _lib, ops, synth

NIB, HUF, HP = 1, 2, 3


def test_library_exports_every_declared_symbol():
    hdr = open(os.path.join(ROOT, "include", "bf16n_c.h")).read()
    declared = set(re.findall(r"\b(bf16n_[A-Za-z0-9_]+)\s*\(", hdr))
    assert declared, "no declarations found"
    L = _lib.lib()
    for name in declared:
        assert hasattr(L, name), f"{name} is declared but not exported"
    assert declared == set(_lib.SYMBOLS), "ctypes table and header disagree"


@pytest.mark.parametrize("name", golden_names())
def test_encoder_matches_reference_bytes(name):
    z = golden(name)
    fmt, R, cm, fmt_out = (int(v) for v in z["meta"])
    plane, aux, f, r_out = ops.encode_bits(z["w"], fmt, R, bool(cm))
    assert f == fmt_out and r_out == (0 if fmt == NIB else R)
    assert np.array_equal(plane, z["plane"])
    assert aux.size == z["aux"].size and np.array_equal(aux, z["aux"])


def test_encoder_is_thread_count_independent():
    w = synth.model_like(64, 2048, 77)
    ops.set_encode_threads(1)
    a1 = ops.encode_bits(w, HP, 8, True)
    ops.set_encode_threads(7)
    a7 = ops.encode_bits(w, HP, 8, True)
    ops.set_encode_threads(0)
    assert np.array_equal(a1[0], a7[0]) and np.array_equal(a1[1], a7[1])


@pytest.mark.parametrize("K", [512, 2048, 4096])
def test_round_trip_every_layout_through_the_oracle_decoder(oracle, K):
    # every format and layout the kernels support (core/tests/test_encode.cpp:243-259), decoded by the oracle
    w = synth.model_like(32, K, K)
    cases = [(NIB, 0, False, False)]
    for R in (1, 2, 4, 8, 16):
        cases += [(HUF, R, False, False), (HP, R, False, False)]
        if K > 512 and R >= 4:
            cases.append((HP, R, True, False))
        if (R * K // 512) % 2 == 0:
            cases.append((HP, R, False, True))
    for fmt, R, cm, w64 in cases:
        plane, aux, f, _ = ops.encode_bits(w, fmt, R, cm, wave64=w64)
        h = oracle.parse_header(aux)
        assert f == fmt and h["flags"] == (1 if cm else 0) | (4 if w64 else 0)
        assert np.array_equal(oracle.decode(plane, aux), w), (fmt, R, cm, w64)


def test_wave64_layout_keeps_plane_and_code(oracle):
    w = synth.model_like(32, 2048, 5)
    p_ref, a_ref, _, _ = ops.encode_bits(w, HP, 8, False)
    p, a, _, _ = ops.encode_bits(w, HP, 8, False, wave64=True)
    assert np.array_equal(p, p_ref)
    h, hr = oracle.parse_header(a), oracle.parse_header(a_ref)
    lut = a[h["off_a"]: h["off_a"] + 16384].view(np.uint32)
    lut_ref = a_ref[hr["off_a"]: hr["off_a"] + 16384].view(np.uint32)
    rev = np.array([int(f"{i:012b}"[::-1], 2) for i in range(4096)])
    assert np.array_equal(lut[rev], lut_ref)  # same table, index bits reversed
    assert h["off_c"] == h["off_d"] and h["off_d"] % 16 == 0
    ub = a[h["off_b"]: h["off_b"] + 4 * (h["n_a"] + 1)].view(np.uint32)
    assert ub[0] == 0 and ub[-1] == h["n_b"] and np.all(np.diff(ub.astype(np.int64)) >= 192)
    assert a.size == h["off_d"] + 4 * (h["n_b"] + 1024)


def test_fallback_and_single_symbol():
    for n, want in ((4095, HP), (4096, HP), (4097, HUF)):
        w = synth.with_pairs(16, 1024, n)
        for cm, w64 in ((False, False), (True, False), (False, True)):
            _, aux, f, _ = ops.encode_bits(w, HP, 4, cm, wave64=w64)
            assert f == want
            flags = ops.HEADER.unpack(aux[:80].tobytes())[11]
            assert flags == ((1 if cm else 0) | (4 if w64 else 0) if want == HP else 0)  # HUFFMAN has no layouts


def test_argument_contract():
    z = np.zeros((64, 4096 + 512), dtype=np.uint16)

    def enc(rows, K, fmt, R, cm, fo=False, w64=False):
        return lambda: ops.encode_bits(z[:rows, :K] if K <= z.shape[1] and rows > 0 else np.zeros((max(rows, 0), max(K, 1)), np.uint16),
                                       fmt, R, cm, fo, w64)

    def throws(f):
        try:
            f()
        except ValueError as e:
            assert str(e).startswith("bf16n encode: ")
            return True
        return False

    for K in (511, 513, 4095, 4097, 4608):
        assert throws(enc(16, K, HP, 4, False)), K
    for K in (512, 4096):
        assert not throws(enc(16, K, HP, 4, False)), K
    assert throws(enc(0, 512, NIB, 0, False)) and not throws(enc(1, 512, NIB, 0, False))
    assert throws(enc(16, 512, NIB, 4, False)) and throws(enc(16, 1024, NIB, 0, True))
    for R in (0, 3, 32):
        assert throws(enc(96, 512, HUF, R, False)), R
    assert throws(enc(15, 512, HP, 4, False)) and not throws(enc(16, 512, HP, 4, False)) and throws(enc(17, 512, HP, 4, False))
    assert throws(enc(16, 1024, HUF, 4, True))
    assert throws(enc(16, 512, HP, 4, True)) and not throws(enc(16, 1024, HP, 4, True)) and throws(enc(16, 1024, HP, 2, True))
    assert throws(enc(16, 512, 0, 4, False)) and throws(enc(16, 512, 4, 4, False))
    # fragment order is the NVIDIA mma register layout: always rejected here, with the reference's wording first
    for args in ((16, 512, HP, 16, False), (16, 512, HP, 8, False), (32, 1024, HP, 16, True), (16, 512, HUF, 16, False), (16, 512, NIB, 0, False)):
        with pytest.raises(ValueError, match="fragment order|fragment-order"):
            enc(*args, fo=True)()
    with pytest.raises(ValueError, match="multiple of R"):
        enc(15, 512, HP, 4, False)()
    with pytest.raises(ValueError, match="chunk-major"):
        enc(16, 512, HP, 4, True)()
    # wave64: HUFPAIR, row-major, even number of chunks per unit
    assert throws(enc(16, 512, HP, 1, False, w64=True)) and not throws(enc(16, 512, HP, 2, False, w64=True))
    assert throws(enc(16, 1024, HP, 4, True, w64=True)) and throws(enc(16, 512, HUF, 4, False, w64=True))
    assert throws(enc(16, 512, NIB, 0, False, w64=True)) and not throws(enc(16, 1024, HP, 1, False, w64=True))


def test_policy_matches_reference_table():
    n = 0
    with open(os.path.join(GOLDEN, "policy.csv")) as f:
        for row in csv.DictReader(f):
            got = ops.choose(int(row["rows"]), int(row["K"]), int(row["n"]), row["engine"], row["mode"], 8 << 20, bool(int(row["expert"])))
            want = (int(row["format"]), int(row["R"]), bool(int(row["chunk_major"])), bool(int(row["frag_order"])))
            assert (got[:4] if got else (0, 0, False, False)) == want, row
            assert got is None or got[4] is False
            n += 1
    assert n > 6000


def test_policy_contract_cases():
    # spot checks restated from core/tests/test_policy.cpp (the CSV above holds the full grid from the reference)
    c = lambda *a, **k: ops.choose(*a, **k)  # noqa: E731
    assert c(248320, 2048, 1, "llama")[:3] == (HP, 16, False) and c(2048, 4096, 1, "llama")[:3] == (HP, 4, False)
    assert c(12288, 2048, 1, "llama")[1] == 16 and c(12288, 2048, 1, "vllm")[1] == 8 and c(9216, 2048, 1, "vllm")[1] == 2
    assert c(16388, 512, 1, "vllm")[1] == 2 and c(18436, 512, 1, "vllm")[1] == 2 and c(20484, 512, 1, "vllm")[1] == 4
    for engine in ("llama", "vllm", "mi355x"):
        for rows in (16383, 16384, 16385):
            # (mi355x keeps the 4-bit code beyond the dense minimum where its units would be 4096 weights)
            assert c(rows, 512, 1, engine)[0] == (NIB if rows < 16384 or engine == "mi355x" else HP)
            assert c(rows, 512, 1, engine, "huffman")[0] == HP
        assert c(512, 2048, 2, engine, "nibble", 0, True)[0] == NIB
        for K in (-1, 0, 1, 256, 511, 513, 1000, 4095, 4097, 4608):
            assert c(2048, K, 1, engine) is None and c(2048, K, 2, engine) is None
        assert c(0, 512, 1, engine) is None and c(1, 512, 0, engine) is None
    big = 2 ** 63 - 1
    assert c(big - 3, 4096, big, "llama", "hybrid", big)[:3] == (HP, 4, True)
    assert c(big, 4096, 1, "vllm")[:2] == (HP, 1)
    for m, want in ((1023, HP), (1024, HP), (1025, NIB)):
        assert c(1, 512, 2, "llama", "hybrid", m)[0] == want


def test_policy_mi355x():
    # the benchmark shapes: wave64 row-major units; 16 rows for a matrix that streams (more than 4096 units), the
    # shortest units that fit one round of 4096 wavefronts for a smaller one
    assert ops.choose(248320, 2048) == (HP, 16, False, False, True)
    assert ops.choose(16384, 2048) == (HP, 4, False, False, True)
    assert ops.choose(65536, 2048) == (HP, 16, False, False, True)
    assert ops.choose(8192, 2048) == (HP, 2, False, False, True) and ops.choose(32768, 512) == (HP, 8, False, False, True)
    huf = lambda rows, K: ops.choose(rows, K, mode="huffman")  # noqa: E731
    assert huf(5120, 2048) == (HP, 2, False, False, True)
    assert huf(2048, 4096) == (HP, 1, False, False, True)
    assert huf(16384, 512) == (HP, 8, False, False, True)              # units of at least 4096 weights
    assert huf(4096, 2048) == (HP, 2, False, False, True)
    assert huf(8192, 1024) == (HP, 4, False, False, True)
    # ... and in hybrid mode a matrix of less than 1.5 x the dense minimum whose units would be that small (4096 weights
    # compress no better than the 4-bit code, whose GEMV has no decode chain) takes the 4-bit code
    for shape in ((5120, 2048), (2048, 4096), (16384, 512), (4096, 2048), (8192, 1024), (6143, 2048)):
        assert ops.choose(*shape)[0] == NIB and ops.choose(*shape, dense_frag_order=True)[0] == NIB
    assert ops.choose(6144, 2048)[:2] == (HP, 2) and ops.choose(3072, 4096)[:2] == (HP, 1)
    assert ops.choose(5120, 2048, dense_min=4 << 20)[:2] == (HP, 2) and ops.choose(5120, 2048, dense_min=0)[:2] == (HP, 2)
    # experts: 32 x 256 tiles in matrix-core operand order where the rows per expert allow it, else units of 4 rows
    assert ops.choose(512, 2048, 256, expert=True) == (HP, 32, False, False, True)
    assert ops.choose(2048, 512, 256, expert=True) == (HP, 32, False, False, True)
    assert ops.choose(96, 1536, 8, expert=True) == (HP, 32, False, False, True)
    assert ops.choose(144, 2048, 8, expert=True) == (HP, 4, False, False, True)
    # a stack of several matrices is an expert stack with or without the caller's flag (a C++ caller that leaves
    # policy_options::expert at its default gets the same layout as one that sets it)
    for shape in ((512, 2048, 256), (2048, 512, 256), (144, 2048, 8), (64, 512, 4)):
        assert ops.choose(*shape, expert=False) == ops.choose(*shape, expert=True) and ops.choose(*shape)[0] == HP
    assert ops.choose(512, 2048)[0] == NIB and ops.choose(2048, 512)[0] == NIB and ops.choose(256, 2048)[0] == NIB
    # dense matrices of at least 131072 rows take the tiles when the caller asks for the matrix-core order
    assert ops.choose(248320, 2048, dense_frag_order=True) == (HP, 32, False, False, True)
    assert ops.choose(131072, 1024, dense_frag_order=True) == (HP, 32, False, False, True)
    assert ops.choose(131040, 2048, dense_frag_order=True) == (HP, 16, False, False, True)   # too few rows
    assert ops.choose(248336, 2048, dense_frag_order=True) == (HP, 16, False, False, True)   # not a multiple of 32
    assert ops.choose(248320, 512, dense_frag_order=True) == (HP, 16, False, False, True)    # K too short
    assert ops.choose(5120, 2048, mode="huffman", dense_frag_order=True) == (HP, 2, False, False, True)
    # shapes without a wave64 GEMV instance keep the reference layouts
    assert ops.choose(16384, 1536) == (HP, 4, False, False, False)
    assert ops.choose(520, 1536, 8, expert=True) == (HP, 8, True, False, False)


def test_parse_header_rejects_garbage():
    import torch

    z = golden("hp_rm_k512_r1")
    aux = torch.from_numpy(z["aux"].copy())
    m = ops.parse_header(aux)
    assert (m.format, m.K, m.rows, m.R, m.chunk_major, m.wave64) == (3, 512, 32, 1, False, False)
    aux[0] ^= 1
    with pytest.raises(ValueError):
        ops.parse_header(aux)
    with pytest.raises(ValueError):
        ops.parse_header(torch.zeros(10, dtype=torch.uint8))


def tile32_virtual(w: np.ndarray) -> np.ndarray:
    """The 512-column matrix V whose wave64 units (16 rows) are the 32 x 256 tiles of w, from the layout's definition:
    V[16u + 2s + h][128j + 4l + q] = w[32g + l][256t + 32s + 16(j//2) + 8h + 4(j%2) + q], u = g * (K/256) + t."""
    rows, K = w.shape
    u, s, h, j, l, q = np.meshgrid(np.arange(rows * K // 8192), np.arange(8), np.arange(2), np.arange(4), np.arange(32),
                                   np.arange(4), indexing="ij")
    g, t = u // (K // 256), u % (K // 256)
    v = np.empty((rows * K // 512, 512), dtype=w.dtype)
    v[16 * u + 2 * s + h, 128 * j + 4 * l + q] = w[32 * g + l, 256 * t + 32 * s + 16 * (j // 2) + 8 * h + 4 * (j % 2) + q]
    return v


@pytest.mark.parametrize("rows,K", [(32, 512), (64, 2048), (96, 1024)])
def test_tile32_layout_is_the_wave64_layout_of_the_permuted_matrix(oracle, rows, K):
    w = synth.model_like(rows, K, rows + K)
    plane, aux, f, R = ops.encode_bits(w, HP, 32, False, wave64=True)
    h = oracle.parse_header(aux)
    assert (f, R, h["R"], h["K"], h["rows"], h["flags"]) == (HP, 32, 32, K, rows, 4)
    assert np.array_equal(oracle.decode(plane, aux), w)
    v = tile32_virtual(w)
    pv, av, _, _ = ops.encode_bits(v, HP, 16, False, wave64=True)
    assert np.array_equal(plane.reshape(-1), pv.reshape(-1))
    assert np.array_equal(aux[256:], av[256:])          # table, unit bases and stream; the headers differ in K, R, rows
    # a lane's 16 weights of a step are two runs of 8 consecutive columns of one row: the A operand of two 32x32x16
    # matrix instructions (lane l: row l % 32, columns 8 (l // 32) .. + 8 of each 16-column block)
    vi = tile32_virtual(np.arange(rows * K, dtype=np.int64).reshape(rows, K))
    for step, lane in ((0, 0), (3, 17), (7, 63), (5, 32)):
        slots = [vi[2 * step + lane // 32, 128 * (i // 4) + 4 * (lane % 32) + i % 4] for i in range(16)]
        r0, k0 = lane % 32, 32 * step + 8 * (lane // 32)
        assert slots == [r0 * K + k0 + i for i in range(8)] + [r0 * K + k0 + 16 + i for i in range(8)]


def test_tile32_contract():
    w = synth.model_like(64, 1024, 5)
    for bad in (lambda: ops.encode_bits(w, HP, 32, False),                      # only with the wave64 layout
                lambda: ops.encode_bits(w, HUF, 32, False, wave64=True),
                lambda: ops.encode_bits(w, HP, 32, True, wave64=True),
                lambda: ops.encode_bits(w[:48], HP, 32, False, wave64=True)):   # rows must be a multiple of 32
        with pytest.raises(ValueError):
            bad()
