"""TEST INFRASTRUCTURE ONLY: ctypes access to the CPU oracle (liboracle.so) and, where it was built, to the reference's
own host encoder/policy (oracle/_ref/libbf16n_ref.so).  Imported only by tests/, __graft_entry__.smoke() and the
cpu_baseline leg of bench.py; the shipped package never imports this module."""
from __future__ import annotations

import ctypes as C
import os
import struct
import subprocess

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
HEADER = struct.Struct("<IIIIQQQQQQQII")
FMT_NIBBLE, FMT_HUFFMAN, FMT_HUFPAIR = 1, 2, 3

_u8p, _u16p, _f32p, _f64p, _i32p = (C.POINTER(t) for t in (C.c_uint8, C.c_uint16, C.c_float, C.c_double, C.c_int32))


def build(ref: bool = True) -> None:
    """Compile the oracle (and oracle/_ref when the reference checkout exists). Building the checker is not using it."""
    subprocess.run(["make", "-C", HERE, "-s"], check=True)


def _load(path):
    if not os.path.exists(path):
        return None
    return C.CDLL(path)


_lib = None
_ref = None


def lib():
    global _lib
    if _lib is None:
        p = os.path.join(HERE, "liboracle.so")
        if not os.path.exists(p):
            build()
        _lib = C.CDLL(p)
        _lib.orc_last_error.restype = C.c_char_p
    return _lib


def ref():
    """The reference's own encoder/policy, or None when oracle/_ref was not built (no reference checkout)."""
    global _ref
    if _ref is None:
        _ref = _load(os.path.join(HERE, "_ref", "libbf16n_ref.so")) or False
        if _ref:
            _ref.ref_last_error.restype = C.c_char_p
    return _ref or None


def _p(a, t):
    return a.ctypes.data_as(t)


def parse_header(aux: np.ndarray) -> dict:
    f = HEADER.unpack(aux[: HEADER.size].tobytes())
    k = ("magic", "format", "K", "R", "rows", "off_a", "off_b", "off_c", "off_d", "n_a", "n_b", "flags", "pad")
    return dict(zip(k, f))


def _encode_with(fn, free, w, fmt, R, cm, extra=()):
    w = np.ascontiguousarray(w, dtype=np.uint16)
    rows, K = w.shape
    plane = np.zeros((max(rows, 0), max(K, 0)), dtype=np.uint8)
    aux = _u8p()
    nbytes = C.c_uint64()
    fmt_out = C.c_int()
    return w, rows, K, plane, aux, nbytes, fmt_out


def encode(w: np.ndarray, fmt: int, R: int = 0, cm: bool = False):
    """Oracle encoder. Returns (plane[rows,K] u8, aux u8, format). Raises ValueError on a contract violation."""
    L = lib()
    w = np.ascontiguousarray(w, dtype=np.uint16)
    rows, K = w.shape
    plane = np.zeros((rows, K), dtype=np.uint8)
    aux = _u8p()
    nbytes = C.c_uint64()
    fmt_out = C.c_int()
    rc = L.orc_encode(_p(w, _u16p), C.c_int64(rows), C.c_int64(K), fmt, R, int(cm), _p(plane, _u8p), C.byref(aux),
                      C.byref(nbytes), C.byref(fmt_out))
    if rc != 0:
        raise ValueError(L.orc_last_error().decode())
    out = np.ctypeslib.as_array(aux, shape=(nbytes.value,)).copy()
    L.orc_free(aux)
    return plane, out, fmt_out.value


def ref_encode(w: np.ndarray, fmt: int, R: int = 0, cm: bool = False, fo: bool = False):
    """The reference's encode(). Returns (plane, aux, format, R). Raises ValueError for std::invalid_argument."""
    L = ref()
    assert L is not None, "oracle/_ref is not built"
    w = np.ascontiguousarray(w, dtype=np.uint16)
    rows, K = w.shape
    plane = np.zeros((max(rows, 1), max(K, 1)), dtype=np.uint8)
    aux = _u8p()
    nbytes = C.c_uint64()
    fmt_out, r_out = C.c_int(), C.c_int()
    rc = L.ref_encode(_p(w, _u16p), C.c_int64(rows), C.c_int64(K), fmt, R, int(cm), int(fo), _p(plane, _u8p),
                      C.byref(aux), C.byref(nbytes), C.byref(fmt_out), C.byref(r_out))
    if rc == 1:
        raise ValueError(L.ref_last_error().decode())
    if rc != 0:
        raise RuntimeError(L.ref_last_error().decode())
    out = np.ctypeslib.as_array(aux, shape=(nbytes.value,)).copy()
    L.ref_free(aux)
    return plane[:rows, :K], out, fmt_out.value, r_out.value


def ref_choose(rows, K, n=1, engine="vllm", mode="hybrid", dense_min=8 << 20, expert=False, dense_frag_order=False):
    L = ref()
    assert L is not None, "oracle/_ref is not built"
    out = (C.c_int * 4)()
    ok = L.ref_choose(C.c_int64(rows), C.c_int64(K), C.c_int64(n), {"llama": 0, "vllm": 1}[engine],
                      {"hybrid": 0, "huffman": 1, "nibble": 2}[mode], C.c_int64(dense_min), int(expert),
                      int(dense_frag_order), out)
    return None if not ok else (out[0], out[1], bool(out[2]), bool(out[3]))


def decode(plane: np.ndarray, aux: np.ndarray) -> np.ndarray:
    L = lib()
    h = parse_header(aux)
    plane = np.ascontiguousarray(plane, dtype=np.uint8)
    aux = np.ascontiguousarray(aux, dtype=np.uint8)
    out = np.zeros((h["rows"], h["K"]), dtype=np.uint16)
    rc = L.orc_decode(_p(plane, _u8p), _p(aux, _u8p), C.c_uint64(aux.size), _p(out, _u16p))
    if rc != 0:
        raise ValueError("oracle decode: malformed buffers")
    return out


def limited_lengths(freq: np.ndarray, L_: int) -> np.ndarray:
    freq = np.ascontiguousarray(freq, dtype=np.uint64)
    out = np.zeros(freq.size, dtype=np.int32)
    lib().orc_limited_lengths(freq.ctypes.data_as(C.POINTER(C.c_uint64)), int(freq.size), int(L_), _p(out, _i32p))
    return out


def bf16_to_f32(bits: np.ndarray) -> np.ndarray:
    return (bits.astype(np.uint32) << 16).view(np.float32)


def f32_to_bf16(x: np.ndarray) -> np.ndarray:
    """Round to nearest even (finite inputs)."""
    b = np.ascontiguousarray(x, dtype=np.float32).view(np.uint32)
    return ((b + 0x7FFF + ((b >> 16) & 1)) >> 16).astype(np.uint16)


def gemv_f32(w_bits: np.ndarray, x: np.ndarray, cm: bool = False) -> np.ndarray:
    w_bits = np.ascontiguousarray(w_bits, dtype=np.uint16)
    x = np.ascontiguousarray(x, dtype=np.float32)
    rows, K = w_bits.shape
    y = np.zeros(rows, dtype=np.float32)
    lib().orc_gemv_f32(_p(w_bits, _u16p), C.c_int64(rows), C.c_int64(K), _p(x, _f32p), int(cm), _p(y, _f32p))
    return y


def gemv_f64(w_bits: np.ndarray, x: np.ndarray):
    w_bits = np.ascontiguousarray(w_bits, dtype=np.uint16)
    x = np.ascontiguousarray(x, dtype=np.float32)
    rows, K = w_bits.shape
    y = np.zeros(rows, dtype=np.float64)
    s = np.zeros(rows, dtype=np.float64)
    lib().orc_gemv_f64(_p(w_bits, _u16p), C.c_int64(rows), C.c_int64(K), _p(x, _f32p), _p(y, _f64p), _p(s, _f64p))
    return y, s


def decode_gemv(plane, aux, x, row0=0, nrows=None, threads=1) -> np.ndarray:
    h = parse_header(aux)
    nrows = h["rows"] - row0 if nrows is None else nrows
    plane = np.ascontiguousarray(plane, dtype=np.uint8)
    aux = np.ascontiguousarray(aux, dtype=np.uint8)
    x = np.ascontiguousarray(x, dtype=np.float32)
    y = np.zeros(nrows, dtype=np.float32)
    rc = lib().orc_decode_gemv(_p(plane, _u8p), _p(aux, _u8p), C.c_uint64(aux.size), C.c_int64(row0), C.c_int64(nrows),
                               _p(x, _f32p), _p(y, _f32p), int(threads))
    if rc != 0:
        raise ValueError("oracle decode_gemv: bad arguments")
    return y


def swiglu(g, u):
    g = np.ascontiguousarray(g, dtype=np.float32)
    u = np.ascontiguousarray(u, dtype=np.float32)
    y = np.zeros_like(g)
    lib().orc_swiglu(_p(g, _f32p), _p(u, _f32p), _p(y, _f32p), C.c_int64(g.size))
    return y


def moe_combine(ys, w):
    ys = np.ascontiguousarray(ys, dtype=np.float32)
    w = np.ascontiguousarray(w, dtype=np.float32)
    T, k, n = ys.shape
    y = np.zeros((T, n), dtype=np.float32)
    lib().orc_moe_combine(_p(ys, _f32p), _p(w, _f32p), _p(y, _f32p), T, k, C.c_int64(n))
    return y


def route(ids, n_experts, nchannels_y=None, sis1=1):
    ids = np.ascontiguousarray(ids, dtype=np.int32)
    T, k = ids.shape
    nchannels_y = k if nchannels_y is None else nchannels_y
    src1 = np.zeros(T * k, dtype=np.int32)
    dst = np.zeros(T * k, dtype=np.int32)
    bounds = np.zeros(n_experts + 1, dtype=np.int32)
    lib().orc_route(_p(ids, _i32p), C.c_int64(k), n_experts, T, k, nchannels_y, sis1, _p(src1, _i32p), _p(dst, _i32p),
                    _p(bounds, _i32p))
    return src1, dst, bounds


def router_topk(logits, k):
    logits = np.ascontiguousarray(logits, dtype=np.float32)
    ids = np.zeros(k, dtype=np.int32)
    w = np.zeros(k, dtype=np.float32)
    lib().orc_router_topk(_p(logits, _f32p), int(logits.size), int(k), _p(ids, _i32p), _p(w, _f32p))
    return ids, w
