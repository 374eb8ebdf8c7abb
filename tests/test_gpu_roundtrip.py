"""GPU decode is bit-exact: encode on the host, dequant on the device through the C ABI, compare with the source and
with the oracle's decode (restates tests/core/test_roundtrip.py of the reference for HIP)."""
from __future__ import annotations

import numpy as np
import pytest
import torch

from conftest import golden, golden_names
from orin_qwen_lossless_amd import synth

pytestmark = pytest.mark.gpu
NIB, HUF, HP = 1, 2, 3


def up(ops, plane, aux):
    tp, ta = torch.from_numpy(np.ascontiguousarray(plane)), torch.from_numpy(np.ascontiguousarray(aux))
    return ops.upload(tp, ta, ops.parse_header(ta), "cuda")


def enc(ops, w, fmt, R=0, cm=False, w64=False):
    plane, aux, _, _ = ops.encode_bits(w, fmt, R, cm, wave64=w64)
    return up(ops, plane, aux)


def bits(t: torch.Tensor) -> np.ndarray:
    return t.contiguous().view(torch.int16).cpu().numpy().view(np.uint16)


@pytest.mark.parametrize("name", golden_names())
def test_dequant_of_reference_buffers(ops, oracle, name):
    # buffers made by the reference encoder decode unchanged
    z = golden(name)
    w = up(ops, z["plane"], z["aux"])
    got = bits(ops.dequant(w))
    assert np.array_equal(got, z["w"])
    assert np.array_equal(got, oracle.decode(z["plane"], z["aux"]))


@pytest.mark.parametrize("K", [512, 1024, 2048, 4096])
@pytest.mark.parametrize("units", [1, 2, 5, 64])
def test_roundtrip_layouts(ops, K, units):
    for fmt, R, cm, w64 in [(NIB, 0, False, False), (HUF, 8, False, False), (HP, 1, False, False), (HP, 4, False, False),
                            (HP, 16, False, False), (HP, 8, True, False), (HP, 4, False, True), (HP, 16, False, True),
                            (HP, 2, False, True)]:
        if cm and K == 512:
            continue
        rows = units * max(R, 1)
        src = synth.model_like(rows, K, 100 * K + units + R)
        w = enc(ops, src, fmt, R, cm, w64)
        assert np.array_equal(bits(ops.dequant(w)), src), (fmt, R, cm, w64)
        assert ops.roundtrip_equal(w, torch.from_numpy(src.view(np.int16)).view(torch.bfloat16))


def test_specials_every_format(ops):
    # zeros, denormals, largest finite, infinities, NaNs with payload, in every slot class
    specials = np.array(synth.SPECIALS + (0x7FFF, 0x0080, 0x8080, 0x7F00), dtype=np.uint16)
    src = np.resize(specials, (16, 1024)).copy()
    src[3] = np.roll(src[3], 5)
    for fmt, R, cm, w64 in [(NIB, 0, False, False), (HUF, 4, False, False), (HP, 4, False, False), (HP, 4, True, False), (HP, 4, False, True)]:
        w = enc(ops, src, fmt, R, cm, w64)
        assert np.array_equal(bits(ops.dequant(w)), src), (fmt, R, cm, w64)


def test_row_range_dequant_equals_slice(ops):
    src = synth.model_like(96, 2048, 31)
    for fmt, R, cm, w64 in [(NIB, 0, False, False), (HP, 8, False, False), (HP, 8, True, False), (HP, 8, False, True), (HUF, 8, False, False)]:
        w = enc(ops, src, fmt, R, cm, w64)
        full = bits(ops.dequant(w))
        for r0, nr in ((0, 8), (16, 40), (88, 8), (32, 0)):
            assert np.array_equal(bits(ops.dequant(w, r0, nr)), full[r0: r0 + nr])
    w = enc(ops, src, HP, 8)
    with pytest.raises(ValueError, match="whole units"):
        ops.dequant(w, 4, 8)
    with pytest.raises(ValueError, match="whole units"):
        ops.dequant(w, 0, 12)
    w = enc(ops, src, NIB)
    assert np.array_equal(bits(ops.dequant(w, 5, 7)), src[5:12])  # NIBBLE rows are independent


def test_flipped_bit_is_detected(ops):
    src = synth.model_like(64, 1024, 32)
    t = torch.from_numpy(src.view(np.int16)).view(torch.bfloat16)
    for w64 in (False, True):
        w = enc(ops, src, HP, 8, False, w64)
        assert ops.roundtrip_equal(w, t)
        w.plane.view(-1)[1000] ^= 1
        assert not ops.roundtrip_equal(w, t)
        w.plane.view(-1)[1000] ^= 1
        off = w.meta.off_d + 4 * 200
        w.aux[off] ^= 0x10
        assert not ops.roundtrip_equal(w, t)


def test_wave64_many_units_per_wave(ops):
    # enough units that every wave walks several of them through its stream ring, with ragged tails
    for rows, K, R in ((16 * 300 + 16, 512, 16), (4 * 9001, 2048, 4), (2 * 4099, 4096, 2)):
        src = synth.weights(rows, K, rows)
        w = enc(ops, src, HP, R, False, True)
        assert np.array_equal(bits(ops.dequant(w)), src)


def test_high_entropy_exponents_wave64(ops):
    # near-uniform exponent pairs: every code is 12 bits long, every lane refills at (almost) every check, so the stream
    # ring is drained at its maximum rate
    rng = np.random.default_rng(3)
    pairs = rng.integers(0, 4096, size=(64, 1024)).astype(np.uint32)
    src = np.zeros((64, 2048), dtype=np.uint16)
    src[:, 0::2] = ((pairs & 63) + 60) << 7
    src[:, 1::2] = ((pairs >> 6) + 60) << 7
    src |= rng.integers(0, 128, size=src.shape).astype(np.uint16)
    for R in (2, 16):
        w = enc(ops, src, HP, R, False, True)
        assert w.meta.format == HP
        assert np.array_equal(bits(ops.dequant(w)), src)


def test_get_rows(ops):
    src = synth.model_like(64, 2048, 33)
    ids = torch.tensor([0, 63, 17, 17, 8, 31], device="cuda")
    for fmt, R, w64 in [(NIB, 0, False), (HP, 8, False), (HP, 8, True), (HP, 1, False)]:
        w = enc(ops, src, fmt, R, False, w64)
        for idt in (torch.int32, torch.int64):
            got = ops.get_rows(ids.to(idt), w, torch.bfloat16)
            assert np.array_equal(bits(got), src[ids.cpu().numpy()])
        finite = src.copy()
        got32 = ops.get_rows(ids.to(torch.int32), w, torch.float32).cpu().numpy()
        assert np.array_equal(got32.view(np.uint32), synth.bf16_bits_to_f32(finite[ids.cpu().numpy()]).view(np.uint32))
        assert np.array_equal(bits(ops.get_rows(torch.tensor([3, 5], device="cuda", dtype=torch.int32), w, torch.bfloat16, row0=12)), src[[15, 17]])
    w = enc(ops, src, HP, 8, True)
    with pytest.raises(ValueError, match="chunk-major"):
        ops.get_rows(ids, w)
    w = enc(ops, src, HUF, 8)
    with pytest.raises(ValueError, match="Huffman"):
        ops.get_rows(ids, w)
