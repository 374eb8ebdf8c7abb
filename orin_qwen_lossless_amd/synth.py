"""Seeded synthetic tensors for tests and benchmarks (numpy only, identical on every machine).

The generator is counter-based: element i of stream `seed` is splitmix64(seed * 2^32 + i); normals come from
Box-Muller on two such uniforms. Weights are N(0, scale) rounded to BF16 (round to nearest even), as the reference's
benchmarks and tests do with their own generators (core/tests/test_encode.cpp:167-189, tests/conftest.py:32-39)."""
from __future__ import annotations

import numpy as np

_M64 = np.uint64(0xFFFFFFFFFFFFFFFF)


def splitmix64(x: np.ndarray) -> np.ndarray:
    with np.errstate(over="ignore"):
        z = (x + np.uint64(0x9E3779B97F4A7C15)) & _M64
        z = ((z ^ (z >> np.uint64(30))) * np.uint64(0xBF58476D1CE4E5B9)) & _M64
        z = ((z ^ (z >> np.uint64(27))) * np.uint64(0x94D049BB133111EB)) & _M64
        return z ^ (z >> np.uint64(31))


def uniform(n: int, seed: int, stream: int = 0) -> np.ndarray:
    """n float64 uniforms in (0, 1)."""
    with np.errstate(over="ignore"):
        ctr = np.arange(n, dtype=np.uint64) + (np.uint64(seed) << np.uint64(32)) + (np.uint64(stream) << np.uint64(56))
    return ((splitmix64(ctr) >> np.uint64(11)).astype(np.float64) + 0.5) * (1.0 / (1 << 53))


def normal(n: int, seed: int) -> np.ndarray:
    """n float32 standard normals."""
    m = (n + 1) // 2
    u1, u2 = uniform(m, seed, 1), uniform(m, seed, 2)
    r = np.sqrt(-2.0 * np.log(u1))
    out = np.empty(2 * m, dtype=np.float64)
    out[0::2] = r * np.cos(2 * np.pi * u2)
    out[1::2] = r * np.sin(2 * np.pi * u2)
    return out[:n].astype(np.float32)


def f32_to_bf16_bits(x: np.ndarray) -> np.ndarray:
    b = np.ascontiguousarray(x, dtype=np.float32).view(np.uint32).astype(np.uint64)
    return ((b + 0x7FFF + ((b >> 16) & 1)) >> 16).astype(np.uint16)


def bf16_bits_to_f32(bits: np.ndarray) -> np.ndarray:
    return (np.ascontiguousarray(bits).astype(np.uint32) << 16).view(np.float32)


def weights(rows: int, K: int, seed: int, scale: float = 0.02) -> np.ndarray:
    """rows x K BF16 bit patterns of N(0, scale)."""
    return f32_to_bf16_bits(normal(rows * K, seed) * np.float32(scale)).reshape(rows, K)


def activations(T: int, K: int, seed: int) -> np.ndarray:
    """T x K BF16 bit patterns of N(0, 1)."""
    return f32_to_bf16_bits(normal(T * K, seed)).reshape(T, K)


SPECIALS = (0x0000, 0x8000, 0x0001, 0x807F, 0x7F7F, 0xFF7F, 0x7F80, 0xFF80, 0x7FC1, 0xFFFF, 0x3F80)


def model_like(rows: int, K: int, seed: int) -> np.ndarray:
    """N(0, 0.02) with 1e-3 outliers (x3000: exponents >= 128) and every special BF16 class at seeded positions,
    the data shape of core/tests/test_encode.cpp:167-189."""
    n = rows * K
    f = normal(n, seed) * np.float32(0.02)
    f = np.where(uniform(n, seed, 3) < 1e-3, f * np.float32(3000.0), f).astype(np.float32)
    w = (f.view(np.uint32) >> 16).astype(np.uint16)  # truncation, as the reference test does
    pos = (uniform(4 * len(SPECIALS), seed, 4) * n).astype(np.int64)
    for i, p in enumerate(pos):
        w[p] = SPECIALS[i % len(SPECIALS)]
    return w.reshape(rows, K)


def with_pairs(rows: int, K: int, n: int) -> np.ndarray:
    """Weights whose (even, odd) exponent pairs take exactly n distinct values (core/tests/test_encode.cpp:221-229)."""
    p = (np.arange(rows * K // 2) % n).astype(np.uint32)
    w = np.zeros(rows * K, dtype=np.uint16)
    w[0::2] = ((p & 0xFF) << 7).astype(np.uint16)
    w[1::2] = ((p >> 8) << 7).astype(np.uint16)
    return w.reshape(rows, K)


def nibble_rows_with_exponents(rows: int, K: int, n_exp: int, seed: int) -> np.ndarray:
    """Rows that use exactly n_exp distinct nonzero exponents < 128 with strictly decreasing counts, so the NIBBLE row
    table (15 entries besides exponent 0) leaves the n_exp - 15 rarest as escapes (tests/core/test_roundtrip.py:105-130)."""
    counts = np.arange(n_exp, 0, -1, dtype=np.int64)
    counts = counts * (K // counts.sum())
    counts[0] += K - counts.sum()
    exps = np.repeat(np.arange(100, 100 + n_exp, dtype=np.uint16), counts)
    out = np.empty((rows, K), dtype=np.uint16)
    for r in range(rows):
        perm = np.argsort(uniform(K, seed + r, 5), kind="stable")
        mant = (uniform(K, seed + r, 6) * 128).astype(np.uint16) & 0x7F
        sign = (uniform(K, seed + r, 7) < 0.5).astype(np.uint16)
        out[r] = (sign << 15) | (exps[perm] << 7) | mant
    return out


# ---------------------------------------------------------------- the same generator on a torch device

def _i64(c: int) -> int:
    """A 64-bit constant as the two's-complement int64 torch holds."""
    return c - (1 << 64) if c >= (1 << 63) else c


def _splitmix64_torch(x):
    """splitmix64 on int64 tensors: additions and multiplications wrap modulo 2^64 as the unsigned ones do; the right
    shifts are made logical by masking the sign extension away."""
    def shr(v, s):
        return (v >> s) & ((1 << (64 - s)) - 1)

    z = x + _i64(0x9E3779B97F4A7C15)
    z = (z ^ shr(z, 30)) * _i64(0xBF58476D1CE4E5B9)
    z = (z ^ shr(z, 27)) * _i64(0x94D049BB133111EB)
    return z ^ shr(z, 31)


def normal_torch(n: int, seed: int, device, first: int = 0):
    """Elements [first, first + n) of normal(., seed) as a float32 tensor on `device` (first even): the same counters,
    the same Box-Muller in float64.  The integer part is exact; log / sqrt / cos / sin come from the device's math
    library, whose last-bit differences from numpy's survive the rounding to float32 in about one element in 10^8."""
    import math

    import torch

    assert first % 2 == 0
    m = (n + 1) // 2
    i = torch.arange(first // 2, first // 2 + m, dtype=torch.int64, device=device)
    u = []
    for stream in (1, 2):
        z = _splitmix64_torch(i + _i64(((seed << 32) + (stream << 56)) & ((1 << 64) - 1)))
        u.append((((z >> 11) & ((1 << 53) - 1)).to(torch.float64) + 0.5) * (1.0 / (1 << 53)))
    r = torch.sqrt(-2.0 * torch.log(u[0]))
    ang = (2 * math.pi) * u[1]
    out = torch.stack((r * torch.cos(ang), r * torch.sin(ang)), dim=1).reshape(-1)
    return out[:n].to(torch.float32)


def weights_torch(rows: int, K: int, seed: int, device, scale: float = 0.02, block_rows: int = 1 << 15):
    """weights(rows, K, seed) as a BF16 tensor on `device`, generated there in blocks of rows."""
    import torch

    w = torch.empty((rows, K), dtype=torch.bfloat16, device=device)
    assert K % 2 == 0
    for r0 in range(0, rows, block_rows):
        nr = min(block_rows, rows - r0)
        f = normal_torch(nr * K, seed, device, first=r0 * K) * torch.tensor(scale, dtype=torch.float32, device=device)
        w[r0: r0 + nr] = f.to(torch.bfloat16).view(nr, K)
    return w


def activations_torch(T: int, K: int, seed: int, device):
    """activations(T, K, seed) as a BF16 tensor on `device`."""
    import torch

    return normal_torch(T * K, seed, device).to(torch.bfloat16).view(T, K)
