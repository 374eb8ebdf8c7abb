"""Seeded sweep of the host encoder on the CPU: for random shapes, unit sizes and layouts the product encoder's output
decodes back to the input through the oracle's decoder (an independent restatement of the format), and — where the
reference's own encoder was built from its sources — equals its plane and aux byte for byte in the reference layouts."""
from __future__ import annotations

import numpy as np
import pytest

from orin_qwen_lossless_amd import ops, synth

NIB, HUF, HP = 1, 2, 3


def cases(n: int):
    rng = np.random.default_rng(777)
    out = []
    while len(out) < n:
        K = int(rng.choice([512, 1024, 1536, 2048, 3072, 4096]))
        fmt = int(rng.choice([NIB, HUF, HP, HP, HP]))
        R = 0 if fmt == NIB else int(rng.choice([1, 2, 4, 8, 16]))
        cm = bool(fmt == HP and K > 512 and R >= 4 and rng.random() < 0.3)
        w64 = bool(fmt == HP and not cm and (R * (K // 512)) % 2 == 0 and rng.random() < 0.5)
        rows = int(rng.integers(1, 12)) * max(R, 1)
        kind = int(rng.integers(0, 3))
        out.append((K, fmt, R, cm, w64, rows, kind, int(rng.integers(1 << 30))))
    for _ in range(n // 4):  # the tile form of the wave64 layout: R = 32, any K
        K = int(rng.choice([512, 1024, 1536, 2048, 3072, 4096]))
        out.append((K, HP, 32, False, True, 32 * int(rng.integers(1, 5)), int(rng.integers(0, 3)), int(rng.integers(1 << 30))))
    return out


@pytest.mark.parametrize("K,fmt,R,cm,w64,rows,kind,seed", cases(60))
def test_random_encode(oracle, K, fmt, R, cm, w64, rows, kind, seed):
    if kind == 0:
        w = synth.weights(rows, K, seed)
    elif kind == 1:
        w = synth.model_like(rows, K, seed)
    else:  # a wide exponent alphabet: long codes, NIBBLE escapes
        rng = np.random.default_rng(seed)
        w = (rng.integers(0, 2, (rows, K)) << 15 | rng.integers(90, 140, (rows, K)) << 7 | rng.integers(0, 128, (rows, K))).astype(np.uint16)
    plane, aux, fmt_out, R_out = ops.encode_bits(w, fmt, R, cm, wave64=w64)
    # more than 4096 distinct exponent pairs: the single-symbol format, which has no tiles (units of 16 rows instead)
    assert fmt_out in (fmt, HUF) and R_out == (16 if R == 32 and fmt_out == HUF else R)
    assert np.array_equal(oracle.decode(plane, aux), w)
    if oracle.ref() is not None and not w64:
        rp, ra, rf, _ = oracle.ref_encode(w, fmt, R, cm)
        assert rf == fmt_out
        assert np.array_equal(plane, rp) and np.array_equal(aux, ra)
