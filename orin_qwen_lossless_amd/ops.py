"""Host-side operator layer over the C ABI, with the names, argument meaning and error behaviour of the reference's
Python operator module (engines/vllm/vllm_bf16n/ops.py) so that code and tests written against it carry over:
encode / upload / dequant / roundtrip_equal / mmv / mmv_glu / linear / get_rows / embedding / moe_mm_ids /
moe_combine / swiglu / moe_experts, plus router_topk and choose.

torch is used for device memory and streams only; every product runs in libbf16n_hip.so.  Weights are passed
explicitly as plane + aux uint8 tensors with metadata parsed once from the aux header on the host."""
from __future__ import annotations

import ctypes as C
import struct
from dataclasses import dataclass

import numpy as np
import torch

from . import _lib

FMT_NIBBLE, FMT_HUFFMAN, FMT_HUFPAIR = 1, 2, 3
FORMAT_NAMES = {FMT_NIBBLE: "nibble", FMT_HUFFMAN: "huffman", FMT_HUFPAIR: "hufpair"}
MAGIC = 0x4E363142
HEADER = struct.Struct("<IIIIQQQQQQQII")  # include/bf16n/format.h aux_header
FLAG_CHUNK_MAJOR, FLAG_FRAG_ORDER, FLAG_WAVE64 = 1, 2, 4

# up to 8 tokens through the GEMV kernels, more through the batched MoE kernel / dequant + GEMM
# (engines/vllm/vllm_bf16n/ops.py:25-27, core/torch/torch_bindings.cpp:195)
GEMV_MAX_TOKENS = 8
# moe_experts: expert GEMVs up to this many routed (token, slot) pairs per expert (tile layout, other layouts), and in
# the tile layout up to this many pairs whatever the number of experts
MOE_GEMV_PAIRS_PER_EXPERT = (0.14, 0.7, 0.5)  # tiles, other wave64 / reference layouts, the 4-bit code
MOE_GEMV_MIN_PAIRS = 24
DEQUANT_CHUNK_BYTES = 64 << 20

ENGINES = {"llama": 0, "vllm": 1, "mi355x": 2}
MODES = {"hybrid": 0, "huffman": 1, "nibble": 2}


_HEADER_FIELDS = ("magic", "format", "K", "R", "rows", "off_a", "off_b", "off_c", "off_d", "n_a", "n_b", "flags", "reserved")
_KNOWN_FLAGS = FLAG_CHUNK_MAJOR | FLAG_FRAG_ORDER | FLAG_WAVE64


@dataclass(frozen=True)
class Meta:
    """What the launchers need to know about one encoded matrix (the fields of bf16n_weight that are not pointers).

    Field names and order are those of the reference's Meta (engines/vllm/vllm_bf16n/ops.py:33-50) so that code
    written against it keeps working; wave64 is this build's layout bit and comes last."""

    format: int
    K: int
    rows: int
    R: int
    chunk_major: bool
    frag_order: bool
    off_a: int
    off_b: int
    off_c: int
    off_d: int
    wave64: bool = False

    @property
    def flags(self) -> int:
        bits = 0
        for on, bit in ((self.chunk_major, FLAG_CHUNK_MAJOR), (self.frag_order, FLAG_FRAG_ORDER), (self.wave64, FLAG_WAVE64)):
            bits |= bit if on else 0
        return bits

    def as_list(self) -> list[int]:
        """The nine integers of the torch.ops.bf16n `meta` argument: format, K, rows, R, flags, off_a .. off_d."""
        return [self.format, self.K, self.rows, self.R, self.flags, self.off_a, self.off_b, self.off_c, self.off_d]


def parse_header(aux: torch.Tensor) -> Meta:
    """Meta of an encoded matrix from the aux_header at the start of its host aux buffer (include/bf16n/format.h).

    ValueError when the buffer is not host uint8 memory holding a whole 256-byte header block, when the magic or the
    format number is wrong, or when a layout flag is set that this build does not know."""
    on_host = aux.device.type == "cpu"
    if not on_host or aux.dtype != torch.uint8 or aux.numel() < 256:
        raise ValueError("bf16n: aux must be a CPU uint8 tensor of at least 256 bytes")
    raw = aux.reshape(-1)[: HEADER.size].contiguous().numpy().tobytes()
    h = dict(zip(_HEADER_FIELDS, HEADER.unpack(raw)))
    if h["magic"] != MAGIC or h["format"] not in FORMAT_NAMES:
        raise ValueError(f"bf16n: bad aux header (magic {h['magic']:#x}, format {h['format']})")
    flags = h["flags"]
    if flags & ~_KNOWN_FLAGS:
        raise ValueError(f"bf16n: unknown layout flags {flags:#x}")
    return Meta(format=h["format"], K=h["K"], rows=h["rows"], R=h["R"], chunk_major=bool(flags & FLAG_CHUNK_MAJOR),
                frag_order=bool(flags & FLAG_FRAG_ORDER), off_a=h["off_a"], off_b=h["off_b"], off_c=h["off_c"],
                off_d=h["off_d"], wave64=bool(flags & FLAG_WAVE64))


@dataclass
class Weight:
    """An encoded matrix resident on a device: the two uint8 buffers the encoder produced (plane: one sign|mantissa byte
    per weight; aux: header, tables and exponent streams) and the Meta parsed from the aux header on the host."""

    plane: torch.Tensor
    aux: torch.Tensor
    meta: Meta

    @property
    def m(self) -> list[int]:
        return self.meta.as_list()

    @property
    def nbytes(self) -> int:
        """Bytes the matrix occupies in device memory."""
        return int(self.plane.numel()) + int(self.aux.numel())


def _stream() -> C.c_void_p:
    return C.c_void_p(torch.cuda.current_stream().cuda_stream)


def _cweight(w: Weight) -> _lib.Weight:
    m = w.meta
    if not (w.plane.is_cuda and w.aux.is_cuda):
        raise ValueError("bf16n: plane and aux must be device tensors")
    if w.plane.dtype != torch.uint8 or w.aux.dtype != torch.uint8:
        raise ValueError("bf16n: plane and aux must be uint8")
    if not (w.plane.is_contiguous() and w.aux.is_contiguous()):
        raise ValueError("bf16n: plane and aux must be contiguous")
    if w.plane.numel() != m.rows * m.K:
        raise ValueError(f"bf16n: plane has {w.plane.numel()} bytes, meta says {m.rows} x {m.K}")
    if max(m.off_a, m.off_b, m.off_c, m.off_d) >= w.aux.numel():
        raise ValueError(f"bf16n: aux ({w.aux.numel()} bytes) shorter than its offsets")
    if w.plane.data_ptr() % 16 or w.aux.data_ptr() % 16:
        raise ValueError("bf16n: plane/aux must be 16-byte aligned")
    return _lib.Weight(w.plane.data_ptr(), w.aux.data_ptr(), m.format, m.R, m.K, m.rows, m.flags, 0, m.off_a, m.off_b,
                       m.off_c, m.off_d)


def _check_x(x: torch.Tensor, K: int, what: str) -> None:
    if not x.is_cuda:
        raise ValueError(f"bf16n: {what} must be a device tensor")
    if x.dtype not in (torch.bfloat16, torch.float32):
        raise ValueError(f"bf16n: {what} must be bf16 or f32")
    if x.shape[-1] != K or x.stride(-1) != 1:
        raise ValueError(f"bf16n: {what} last dim must be K = {K} and contiguous")
    if x.data_ptr() % 16:
        raise ValueError(f"bf16n: {what} must be 16-byte aligned")
    for d in range(x.dim() - 1):
        if (x.stride(d) * x.element_size()) % 16:
            raise ValueError(f"bf16n: {what} row strides must be multiples of 16 bytes")


def _check_ids(ids: torch.Tensor) -> None:
    if not ids.is_cuda or ids.dim() != 2:
        raise ValueError("bf16n: ids must be a 2-D device tensor [tokens, n_used]")
    if ids.dtype not in (torch.int32, torch.int64):
        raise ValueError("bf16n: ids must be int32 or int64")
    if ids.stride(1) != 1:
        raise ValueError("bf16n: ids must be contiguous along the slot dimension")


def init() -> None:
    """Device attributes and kernel shared-memory limits; once per process, before any launch / graph capture."""
    _lib.check(_lib.lib().bf16n_init())


def cu_count() -> int:
    n = C.c_int()
    _lib.check(_lib.lib().bf16n_cu_count(C.byref(n)))
    return n.value


def set_encode_threads(n: int) -> None:
    _lib.lib().bf16n_set_encode_threads(int(n))


def choose(rows: int, K: int, n_matrices: int = 1, engine: str = "mi355x", mode: str = "hybrid",
           dense_min: int = 8 << 20, expert: bool = False, dense_frag_order: bool = False):
    """Shape policy (core/src/policy.cpp). Returns None (stay BF16) or (format, R, chunk_major, frag_order, wave64)."""
    out = (C.c_int * 5)()
    ok = _lib.lib().bf16n_choose(rows, K, n_matrices, ENGINES[engine], MODES[mode], dense_min, int(expert),
                                 int(dense_frag_order), out)
    return None if not ok else (out[0], out[1], bool(out[2]), bool(out[3]), bool(out[4]))


def encode_bits(w_bits: np.ndarray, fmt: int, R: int, chunk_major: bool = False, frag_order: bool = False,
                wave64: bool = False) -> tuple[np.ndarray, np.ndarray, int, int]:
    """Encode rows x K BF16 bit patterns (numpy uint16). Returns (plane, aux, format produced, R)."""
    w_bits = np.ascontiguousarray(w_bits, dtype=np.uint16)
    if w_bits.ndim < 2:
        raise ValueError("bf16n.encode: weight must be at least 2-D (rows x K)")
    K = w_bits.shape[-1]
    rows = w_bits.size // max(K, 1)
    flags = (FLAG_CHUNK_MAJOR if chunk_major else 0) | (FLAG_FRAG_ORDER if frag_order else 0) | (FLAG_WAVE64 if wave64 else 0)
    L = _lib.lib()
    h = C.c_void_p()
    _lib.check(L.bf16n_encode(w_bits.ctypes.data, rows, K, fmt, R, flags, C.byref(h)))
    # the arrays are views of the encoder's buffers (no copy of hundreds of megabytes); the buffers are freed when the
    # last view is gone
    owner = _EncodedOwner(L, h)
    n = C.c_uint64()
    p = L.bf16n_encoded_plane(h, C.byref(n))
    plane = _view(p, n.value, owner).reshape(rows, K)
    p = L.bf16n_encoded_aux(h, C.byref(n))
    aux = _view(p, n.value, owner)
    return plane, aux, L.bf16n_encoded_format(h), L.bf16n_encoded_R(h)


class _EncodedOwner:
    """Keeps a bf16n_encoded handle alive for the numpy views of its buffers."""

    def __init__(self, L, h):
        self._free, self._h = L.bf16n_encoded_free, h

    def __del__(self):
        self._free(self._h)


def _view(ptr: int, n: int, owner: _EncodedOwner) -> np.ndarray:
    buf = (C.c_uint8 * n).from_address(ptr)
    buf._bf16n_owner = owner  # numpy keeps `buf` as the base of the array, and `buf` keeps the handle
    return np.frombuffer(buf, dtype=np.uint8)


def encode(w: torch.Tensor, fmt: int, R: int, chunk_major: bool, frag_order: bool = False, wave64: bool = False
           ) -> tuple[torch.Tensor, torch.Tensor, Meta]:
    """Encode a BF16 CPU tensor (..., K) on the host cores. FMT_HUFPAIR falls back to FMT_HUFFMAN when the tensor has
    more than 4096 distinct exponent pairs; the returned Meta holds the format and layout actually produced."""
    if w.device.type != "cpu":
        raise ValueError("bf16n.encode: weight must be on the CPU")
    if w.dtype != torch.bfloat16:
        raise ValueError("bf16n.encode: weight must be bfloat16")
    if w.dim() < 2:
        raise ValueError("bf16n.encode: weight must be at least 2-D (rows x K)")
    bits = w.contiguous().view(torch.int16).numpy().view(np.uint16)
    plane, aux, _, _ = encode_bits(bits, fmt, R, chunk_major, frag_order, wave64)
    tp, ta = torch.from_numpy(plane), torch.from_numpy(aux)
    return tp, ta, parse_header(ta)


def upload(plane: torch.Tensor, aux: torch.Tensor, meta: Meta, device: torch.device | str) -> Weight:
    return Weight(plane.to(device), aux.to(device), meta)


def dequant(w: Weight, row0: int = 0, nrows: int | None = None) -> torch.Tensor:
    nrows = w.meta.rows - row0 if nrows is None else nrows
    cw = _cweight(w)
    if row0 < 0 or nrows < 0 or row0 + nrows > w.meta.rows:
        raise ValueError("bf16n.dequant: rows out of range")
    out = torch.empty((nrows, w.meta.K), dtype=torch.bfloat16, device=w.plane.device)
    with torch.cuda.device(w.plane.device):
        _lib.check(_lib.lib().bf16n_dequant(C.byref(cw), row0, nrows, out.data_ptr(), _stream()))
    return out


def roundtrip_equal(w: Weight, src: torch.Tensor, chunk_bytes: int = 64 << 20) -> bool:
    """True when the device decode of w reproduces every BF16 bit pattern of src (rows x K values on any device).

    The matrix is decoded in pieces of at most chunk_bytes of BF16 output, each a whole number of units, and each piece
    is compared on the device; the first differing piece ends the check (engines/vllm/vllm_bf16n/ops.py:104-116)."""
    meta = w.meta
    want = src.reshape(meta.rows, meta.K)
    if want.element_size() != 2:
        raise ValueError("bf16n.roundtrip_equal: the source must hold 16-bit values (bfloat16)")
    rows_per_unit = meta.R if meta.R > 0 else 1
    piece = chunk_bytes // (2 * meta.K) // rows_per_unit * rows_per_unit
    piece = piece if piece >= rows_per_unit else rows_per_unit
    first = 0
    while first < meta.rows:
        n = piece if first + piece <= meta.rows else meta.rows - first
        decoded = dequant(w, first, n)
        expect = want.narrow(0, first, n).to(decoded.device, non_blocking=False)
        # compare bit patterns, not values: NaN payloads and signed zeros count
        if not bool((decoded.view(torch.int16) == expect.view(torch.int16)).all()):
            return False
        first += n
    return True


def _mmv_common(x: torch.Tensor, w: Weight, ids: torch.Tensor | None, rows_per_matrix: int, out_bf16: bool, glu: bool,
                multi_col: bool = True, up: Weight | None = None, topk=None) -> torch.Tensor:
    """glu: w holds [gate; up] per matrix.  up given: w is the gate matrix and up a separate matrix of the same shape
    (the product is silu(gate x) * (up x) with as many rows as either)."""
    cw = _cweight(w)
    cu = _cweight(up) if up is not None else None
    K, rows = w.meta.K, w.meta.rows
    _check_x(x, K, "x")
    a = _lib.MmvArgs()
    a.x = x.data_ptr()
    a.x_bf16 = int(x.dtype == torch.bfloat16)
    a.y_bf16 = int(out_bf16)
    odt = torch.bfloat16 if out_bf16 else torch.float32
    osz = 2 if out_bf16 else 4
    a.n_used, a.x_per_slot = 1, 1
    if ids is None:
        if x.dim() != 2:
            raise ValueError("bf16n.mmv: dense x must be [tokens, K]")
        rpm = rows_per_matrix if rows_per_matrix > 0 else rows
        if rpm != rows:
            raise ValueError("bf16n.mmv: a dense product uses the whole matrix")
        if glu and rpm % 2:
            raise ValueError("bf16n.mmv_glu: odd row count")
        n_out = rpm // 2 if glu else rpm
        T = x.shape[0]
        y = torch.empty((T, n_out), dtype=odt, device=x.device)
        if T == 0:
            return y
        a.y = y.data_ptr()
        a.ncols = T
        a.x_tok = x.stride(0) * x.element_size()
        a.y_tok = n_out * osz
        a.rows_per_matrix = rpm
        a.nrows = n_out
    else:
        _check_ids(ids)
        if ids.device != w.plane.device:
            raise ValueError("bf16n.mmv: ids on another device")
        T, n_used = ids.shape
        if rows_per_matrix <= 0 or rows % rows_per_matrix:
            raise ValueError("bf16n.mmv: rows_per_matrix must divide the rows")
        if glu and rows_per_matrix % 2:
            raise ValueError("bf16n.mmv_glu: odd rows per matrix")
        n_out = rows_per_matrix // 2 if glu else rows_per_matrix
        if not ((x.dim() == 2 and x.shape[0] == T) or (x.dim() == 3 and x.shape[0] == T and x.shape[1] == n_used)):
            raise ValueError("bf16n.mmv: x must be [tokens, K] or [tokens, n_used, K]")
        y = torch.empty((T, n_used, n_out), dtype=odt, device=x.device)
        if T == 0 or n_used == 0:
            return y
        a.y = y.data_ptr()
        a.ncols = T * n_used
        a.ids = ids.data_ptr()
        a.ids_s0 = ids.element_size()
        a.ids_s1 = ids.stride(0) * ids.element_size()
        a.n_used = n_used
        a.x_tok = x.stride(0) * x.element_size()
        a.x_per_slot = n_used if x.dim() == 3 else 1
        a.x_slot = x.stride(1) * x.element_size() if x.dim() == 3 else 0
        a.y_tok = n_used * n_out * osz
        a.y_slot = n_out * osz
        a.rows_per_matrix = rows_per_matrix
        a.nrows = n_out
    L = _lib.lib()
    with torch.cuda.device(x.device):
        if topk is not None:
            logits, k, renorm, wts = topk
            _lib.check(L.bf16n_mmv_glu2_topk(C.byref(cw), C.byref(cu), C.byref(a), logits.data_ptr(), logits.stride(0), logits.shape[1],
                                             k, int(renorm), wts.data_ptr(), wts.stride(0), _stream()))
        elif cu is not None:
            _lib.check(L.bf16n_mmv_glu2(C.byref(cw), C.byref(cu), C.byref(a), _stream()))
        elif glu:
            _lib.check(L.bf16n_mmv_glu(C.byref(cw), C.byref(a), _stream()))
        else:
            _lib.check(L.bf16n_mmv(C.byref(cw), C.byref(a), _stream(), int(multi_col)))
    return y


def mmv(x: torch.Tensor, w: Weight, ids: torch.Tensor | None = None, rows_per_matrix: int = 0,
        out_dtype: torch.dtype = torch.float32, multi_col: bool = True) -> torch.Tensor:
    return _mmv_common(x, w, ids, rows_per_matrix, out_dtype == torch.bfloat16, False, multi_col)


def mmv_glu(x: torch.Tensor, w: Weight, ids: torch.Tensor | None = None, rows_per_matrix: int = 0,
            out_dtype: torch.dtype = torch.float32) -> torch.Tensor:
    """silu(gate x) * (up x) for a NIBBLE matrix whose rows per matrix are [gate; up]."""
    return _mmv_common(x, w, ids, rows_per_matrix or w.meta.rows, out_dtype == torch.bfloat16, True)


def mmv_glu2(x: torch.Tensor, gate: Weight, up: Weight, ids: torch.Tensor | None = None, rows_per_matrix: int = 0,
             out_dtype: torch.dtype = torch.float32) -> torch.Tensor:
    """silu(gate x) * (up x) for separate gate / up matrices of one shape, dense or with expert ids
    (bf16n::mmv_glu(gate, up), core launch.h:56-61)."""
    if (gate.meta.K, gate.meta.rows) != (up.meta.K, up.meta.rows):
        raise ValueError("bf16n.mmv_glu: gate/up shapes must match")
    return _mmv_common(x, gate, ids, rows_per_matrix, out_dtype == torch.bfloat16, False, True, up)


# the routed gate / up GEMV can select the experts itself (bf16n_mmv_glu2_topk): one launch fewer in a decode step
TOPK_IN_EXPERT_GEMV = True


def topk_in_gemv_supported(gate: Weight, up: Weight, n_experts: int, k: int) -> bool:
    """Whether mmv_glu2_topk takes these expert stacks: the tile layout, at most 256 experts to select from."""
    tiles = all(m.meta.wave64 and m.meta.R == 32 and m.meta.format == FMT_HUFPAIR for m in (gate, up))
    return TOPK_IN_EXPERT_GEMV and tiles and n_experts <= 256 and 0 < k <= 64 and (gate.meta.K, gate.meta.rows) == (up.meta.K, up.meta.rows)


def mmv_glu2_topk(x: torch.Tensor, gate: Weight, up: Weight, logits: torch.Tensor, k: int, rows_per_matrix: int,
                  out: tuple[torch.Tensor, torch.Tensor], renorm: bool = True, out_dtype: torch.dtype = torch.float32) -> torch.Tensor:
    """router_topk(logits, k, renorm, out) and mmv_glu2(x, gate, up, ids, rows_per_matrix) in one launch
    (bf16n_mmv_glu2_topk): every block of the GEMV selects its token's experts from the logits in its prologue.
    out = (weights f32, ids int32) [tokens, m >= k]: columns 0..k-1 are written, the columns from k on are read as
    further slots of every token (experts that all tokens use).  x: BF16 [tokens, K].  Returns [tokens, m, rows]."""
    wts, ids = out
    if not (logits.is_cuda and logits.dim() == 2 and logits.dtype == torch.float32 and logits.stride(1) == 1):
        raise ValueError("bf16n.mmv_glu2_topk: logits must be f32 [tokens, n_experts], contiguous along experts")
    if not (wts.dtype == torch.float32 and ids.dtype == torch.int32 and wts.shape == ids.shape and wts.dim() == 2
            and wts.shape[0] == logits.shape[0] and wts.shape[1] >= k and wts.is_contiguous() and ids.is_contiguous()
            and wts.device == logits.device and ids.device == logits.device):
        raise ValueError("bf16n.mmv_glu2_topk: out must be contiguous (f32, int32) [tokens, m >= k] tensors on the logits' device")
    if x.dtype != torch.bfloat16 or x.dim() != 2:
        raise ValueError("bf16n.mmv_glu2_topk: x must be bf16 [tokens, K]")
    return _mmv_common(x, gate, ids, rows_per_matrix, out_dtype == torch.bfloat16, False, True, up, (logits, k, renorm, wts))


def gemv_max_tokens(w: Weight) -> int:
    """BF16 token columns up to which mmv is the faster dense path for this matrix: GEMV_MAX_TOKENS (the reference's
    rule, ops.py:25-27), or more for matrices whose dense products run on the matrix cores."""
    n = C.c_int(0)
    cw = _cweight(w)
    _lib.check(_lib.lib().bf16n_gemv_max_tokens(C.byref(cw), C.byref(n)))
    return n.value


def linear(x: torch.Tensor, w: Weight, bias: torch.Tensor | None = None) -> torch.Tensor:
    """y = x W^T (+ bias) in BF16: up to gemv_max_tokens(w) tokens through the decode GEMV (FP32 accumulation, the bias
    added in FP32 before the one rounding to BF16), more through exact dequant in row chunks + a stock BF16 GEMM
    (core/torch/torch_bindings.cpp:198-239)."""
    if x.dtype != torch.bfloat16:
        raise ValueError("bf16n.linear: x must be bf16")
    K, rows = w.meta.K, w.meta.rows
    if x.shape[-1] != K:
        raise ValueError(f"bf16n.linear: x last dim must be K = {K}")
    oshape = list(x.shape[:-1]) + [rows]
    x2 = x.reshape(-1, K)
    T = x2.shape[0]
    if T <= GEMV_MAX_TOKENS or T <= gemv_max_tokens(w):
        ok = x2.stride(1) == 1 and (x2.stride(0) * 2) % 16 == 0 and x2.data_ptr() % 16 == 0
        xc = x2 if ok else x2.contiguous()
        if bias is not None:
            y = _mmv_common(xc, w, None, 0, False, False).add_(bias).to(torch.bfloat16)
        else:
            y = _mmv_common(xc, w, None, 0, True, False)
    else:
        unit = 1 if w.meta.format == FMT_NIBBLE else w.meta.R
        chunk = min(max(DEQUANT_CHUNK_BYTES // (K * 2) // unit * unit, unit), rows)
        if chunk == rows:
            # one piece: the stock linear adds the bias before its single rounding to BF16, as the reference's does
            y = torch.nn.functional.linear(x2, dequant(w, 0, rows), bias)
        else:
            y = torch.empty((T, rows), dtype=x.dtype, device=x.device)
            for r0 in range(0, rows, chunk):
                nr = min(chunk, rows - r0)
                wc = dequant(w, r0, nr)
                ys = y.narrow(1, r0, nr)
                if bias is None:
                    torch.mm(x2, wc.t(), out=ys)
                else:
                    torch.addmm(bias.narrow(0, r0, nr), x2, wc.t(), out=ys)
    return y.view(oshape)


def linear_dense(x: torch.Tensor, w: Weight, scratch: torch.Tensor | None = None, gemm_workspace: torch.Tensor | None = None
                 ) -> torch.Tensor:
    """y = x W^T in BF16 through the library's dense path (bf16n_linear_dense: exact dequant in pieces into `scratch`
    + hipBLASLt BF16 GEMM, FP32 accumulation), the path of linear() above gemv_max_tokens without torch's GEMM.  scratch /
    gemm_workspace: uint8 device buffers (allocated here when not given; a caller under graph capture passes its own)."""
    if x.dtype != torch.bfloat16 or x.dim() != 2 or x.shape[1] != w.meta.K or not x.is_cuda:
        raise ValueError("bf16n.linear_dense: x must be a bf16 device tensor [tokens, K]")
    _check_x(x, w.meta.K, "x")
    cw = _cweight(w)
    need_s, need_g = C.c_uint64(), C.c_uint64()
    L = _lib.lib()
    _lib.check(L.bf16n_linear_dense_sizes(C.byref(cw), C.byref(need_s), C.byref(need_g)))
    if scratch is None:
        scratch = torch.empty(need_s.value, dtype=torch.uint8, device=x.device)
    if gemm_workspace is None:
        gemm_workspace = torch.empty(need_g.value, dtype=torch.uint8, device=x.device)
    T = x.shape[0]
    y = torch.empty((T, w.meta.rows), dtype=torch.bfloat16, device=x.device)
    if T == 0:
        return y
    with torch.cuda.device(x.device):
        _lib.check(L.bf16n_linear_dense(C.byref(cw), x.data_ptr(), x.stride(0), T, y.data_ptr(), y.stride(0), scratch.data_ptr(),
                                        scratch.numel(), gemm_workspace.data_ptr(), gemm_workspace.numel(), _stream()))
    return y


def get_rows(ids: torch.Tensor, w: Weight, out_dtype: torch.dtype = torch.bfloat16, row0: int = 0) -> torch.Tensor:
    cw = _cweight(w)
    if not ids.is_cuda or ids.dim() != 1:
        raise ValueError("bf16n.get_rows: ids must be a 1-D device tensor")
    if ids.dtype not in (torch.int32, torch.int64):
        raise ValueError("bf16n.get_rows: ids must be int32 or int64")
    n = ids.shape[0]
    out = torch.empty((n, w.meta.K), dtype=out_dtype, device=w.plane.device)
    with torch.cuda.device(w.plane.device):
        _lib.check(_lib.lib().bf16n_get_rows(C.byref(cw), ids.data_ptr(), ids.stride(0) * ids.element_size(), n,
                                             out.data_ptr(), int(out_dtype == torch.bfloat16),
                                             w.meta.K * out.element_size(), _stream(), row0))
    return out


def embedding(ids: torch.Tensor, w: Weight) -> torch.Tensor:
    flat = ids.reshape(-1)
    return get_rows(flat, w).view(*ids.shape, w.meta.K)


def mm_ids_supported(w: Weight, up: Weight | None = None) -> bool:
    """Shapes with a batched (prefill) MoE kernel (bf16n::mm_ids_supported, core/src/launch.cu:446-456)."""
    cw = _cweight(w)
    cu = _cweight(up) if up is not None else None
    return bool(_lib.lib().bf16n_mm_ids_supported(C.byref(cw), C.byref(cu) if cu is not None else None))


def mm_ids_route(topk_ids: torch.Tensor, n_experts: int, per_slot: bool):
    """Expert-sorted routing lists on the device (bf16n::mm_ids_route): (ids_src1, ids_dst, bounds) int32."""
    _check_ids(topk_ids)
    T, n_used = topk_ids.shape
    dev = topk_ids.device
    src1 = torch.empty(T * n_used, dtype=torch.int32, device=dev)
    dst = torch.empty(T * n_used, dtype=torch.int32, device=dev)
    bounds = torch.empty(n_experts + 1, dtype=torch.int32, device=dev)
    nch = n_used if per_slot else 1
    with torch.cuda.device(dev):
        _lib.check(_lib.lib().bf16n_mm_ids_route(topk_ids.data_ptr(), int(topk_ids.dtype == torch.int64), topk_ids.stride(0),
                                                 src1.data_ptr(), dst.data_ptr(), bounds.data_ptr(), n_experts, T, n_used,
                                                 nch, nch, _stream()))
    return src1, dst, bounds


# moe_mm_ids: routed pairs per expert from which the tile layout's two-phase form (decode a group of experts into
# scratch once, multiply from there) replaces the fused kernel, which decodes an expert once per 128 of its tokens.
# Off by default: measured on a 256-expert layer it is behind the fused kernel at every token count (1.86 against 1.09
# ms at 8192 tokens, 1.03 against 0.40 ms at 2048): writing and re-reading the experts as BF16 (1.6 GB a layer) costs
# more than the second decode it saves.  Callers that pass `scratch` and lower this value get it.
MM_IDS_TWO_PHASE_PAIRS_PER_EXPERT = 1 << 30
_mm_scratch: dict = {}


def mm_ids_scratch(w: Weight, up: Weight | None, n_experts: int) -> torch.Tensor:
    """The scratch buffer of the two-phase batched product for these expert stacks (the size the library advises: groups
    of experts that stay in the last-level cache), one per device and size, kept for later calls."""
    per, adv = C.c_uint64(0), C.c_uint64(0)
    cw, cu = _cweight(w), _cweight(up) if up is not None else None
    _lib.check(_lib.lib().bf16n_mm_ids_scratch_bytes(C.byref(cw), C.byref(cu) if cu is not None else None, n_experts, C.byref(per), C.byref(adv)))
    key = (w.plane.device, adv.value)
    if key not in _mm_scratch:
        _mm_scratch[key] = torch.empty(adv.value, dtype=torch.uint8, device=w.plane.device)
    return _mm_scratch[key]


def moe_mm_ids(x: torch.Tensor, topk_ids: torch.Tensor, w: Weight, n_experts: int, up: Weight | None = None,
               out_dtype: torch.dtype = torch.float32, routes=None, scratch: torch.Tensor | None = None) -> torch.Tensor:
    """Batched MUL_MAT_ID over routed tokens (core/torch/torch_bindings.cpp:307-345): x [T, K] (gate / up) or
    [T, n_used, K] (down), BF16; out [T, n_used, N]; up given: fused gate/up + SwiGLU.  routes: the lists of
    mm_ids_route(topk_ids, n_experts, x.dim() == 3) if the caller already has them (they are computed otherwise).
    scratch: a uint8 device buffer for the two-phase form (tile layout, from MM_IDS_TWO_PHASE_PAIRS_PER_EXPERT routed
    pairs per expert on); None: the operator keeps one of the advised size per device (mm_ids_scratch)."""
    cw = _cweight(w)
    cu = _cweight(up) if up is not None else None
    _check_ids(topk_ids)
    _check_x(x, w.meta.K, "x")
    if x.dtype != torch.bfloat16 or not x.is_contiguous():
        raise ValueError("bf16n.moe_mm_ids: x must be contiguous bf16 (BF16 activations)")
    if n_experts <= 0 or w.meta.rows % n_experts:
        raise ValueError("bf16n.moe_mm_ids: rows must split into n_experts")
    T, n_used = topk_ids.shape
    N = w.meta.rows // n_experts
    per_slot = x.dim() == 3
    if not ((x.dim() == 2 and x.shape[0] == T) or (per_slot and x.shape[0] == T and x.shape[1] == n_used)):
        raise ValueError("bf16n.moe_mm_ids: x must be [tokens, K] or [tokens, n_used, K]")
    y = torch.empty((T, n_used, N), dtype=out_dtype, device=x.device)
    if T == 0:
        return y
    L = _lib.lib()
    if not L.bf16n_mm_ids_supported(C.byref(cw), C.byref(cu) if cu is not None else None):
        raise ValueError("bf16n.moe_mm_ids: no batched kernel for this matrix (format/K/R/layout)")
    src1, dst, bounds = routes if routes is not None else mm_ids_route(topk_ids, n_experts, per_slot)
    tiles = w.meta.wave64 and w.meta.R == 32 and w.meta.format == FMT_HUFPAIR and (up is None or (up.meta.wave64 and up.meta.R == 32))
    if tiles and T * n_used >= MM_IDS_TWO_PHASE_PAIRS_PER_EXPERT * n_experts:
        buf = scratch if scratch is not None else mm_ids_scratch(w, up, n_experts)
        with torch.cuda.device(x.device):
            _lib.check(L.bf16n_mm_ids_scratch(C.byref(cw), C.byref(cu) if cu is not None else None, x.data_ptr(), w.meta.K,
                                              src1.data_ptr(), dst.data_ptr(), bounds.data_ptr(), y.data_ptr(),
                                              int(out_dtype == torch.bfloat16), N, n_experts, buf.data_ptr(), buf.numel(), _stream()))
        return y
    with torch.cuda.device(x.device):
        _lib.check(L.bf16n_mm_ids(C.byref(cw), C.byref(cu) if cu is not None else None, x.data_ptr(), w.meta.K,
                                  src1.data_ptr(), dst.data_ptr(), bounds.data_ptr(), y.data_ptr(),
                                  int(out_dtype == torch.bfloat16), N, n_experts, T, n_used, _stream()))
    return y


def moe_combine(ys: torch.Tensor, topk_weights: torch.Tensor, out_dtype: torch.dtype = torch.bfloat16) -> torch.Tensor:
    if not (ys.is_cuda and ys.dim() == 3 and ys.dtype == torch.float32 and ys.is_contiguous()):
        raise ValueError("bf16n.moe_combine: ys must be contiguous f32 [tokens, n_used, N]")
    if not (topk_weights.is_cuda and topk_weights.dim() == 2 and topk_weights.is_contiguous()
            and topk_weights.dtype in (torch.float32, torch.bfloat16)):
        raise ValueError("bf16n.moe_combine: topk_weights must be contiguous f32/bf16 [tokens, n_used]")
    T, n_used, N = ys.shape
    if tuple(topk_weights.shape) != (T, n_used):
        raise ValueError("bf16n.moe_combine: shape mismatch")
    y = torch.empty((T, N), dtype=out_dtype, device=ys.device)
    with torch.cuda.device(ys.device):
        _lib.check(_lib.lib().bf16n_moe_combine(ys.data_ptr(), topk_weights.data_ptr(), int(topk_weights.dtype == torch.bfloat16),
                                                y.data_ptr(), int(out_dtype == torch.bfloat16), T, n_used, N, _stream()))
    return y


def add_rmsnorm(a: torch.Tensor, b: torch.Tensor | None = None, c: torch.Tensor | None = None, ys: torch.Tensor | None = None,
                topk_weights: torch.Tensor | None = None, gamma: torch.Tensor | None = None, eps: float = 1e-6,
                want_sum: bool = False):
    """Engine glue of a decode step in one launch: s = a + b + c + moe_combine(ys, topk_weights) in FP32 (every addend
    but a optional), returns bf16(s * rsqrt(mean(s^2) + eps) * gamma), and bf16(s) too when want_sum.
    a, b, c: [T, n] BF16 contiguous; ys: [T, n_used, n] FP32 with topk_weights [T, n_used]; gamma: [n] BF16."""
    for t in (a, b, c):
        if t is not None and not (t.is_cuda and t.dtype == torch.bfloat16 and t.is_contiguous() and t.shape == a.shape and t.dim() == 2):
            raise ValueError("bf16n.add_rmsnorm: inputs must be contiguous bf16 [tokens, n] of one shape")
    if gamma is not None and not (gamma.is_cuda and gamma.dtype == torch.bfloat16 and gamma.is_contiguous() and gamma.numel() == a.shape[1]):
        raise ValueError("bf16n.add_rmsnorm: gamma must be contiguous bf16 [n]")
    T, n = a.shape
    n_used = 0
    if ys is not None:
        if not (ys.is_cuda and ys.dtype == torch.float32 and ys.is_contiguous() and ys.dim() == 3 and ys.shape[0] == T and ys.shape[2] == n):
            raise ValueError("bf16n.add_rmsnorm: ys must be contiguous f32 [tokens, n_used, n]")
        n_used = ys.shape[1]
        w = topk_weights
        if w is None or not (w.is_cuda and w.is_contiguous() and tuple(w.shape) == (T, n_used) and w.dtype in (torch.float32, torch.bfloat16)):
            raise ValueError("bf16n.add_rmsnorm: topk_weights must be contiguous f32/bf16 [tokens, n_used]")
    y = torch.empty_like(a)
    ysum = torch.empty_like(a) if want_sum else None
    ptr = lambda t: t.data_ptr() if t is not None else None  # noqa: E731
    with torch.cuda.device(a.device):
        _lib.check(_lib.lib().bf16n_add_rmsnorm(
            a.data_ptr(), ptr(b), ptr(c), ptr(ys), ptr(topk_weights) if ys is not None else None,
            int(ys is not None and topk_weights.dtype == torch.bfloat16), n_used, ptr(gamma), ptr(ysum), y.data_ptr(), T, n,
            C.c_float(eps), _stream()))
    return (y, ysum) if want_sum else y


def swiglu(g: torch.Tensor, u: torch.Tensor) -> torch.Tensor:
    if not (g.is_cuda and g.dtype == torch.float32 and g.is_contiguous() and u.shape == g.shape
            and u.dtype == torch.float32 and u.is_contiguous()):
        raise ValueError("bf16n.swiglu: g and u must be contiguous f32 of one shape")
    y = torch.empty_like(g)
    with torch.cuda.device(g.device):
        _lib.check(_lib.lib().bf16n_swiglu(g.data_ptr(), u.data_ptr(), y.data_ptr(), g.numel(), _stream()))
    return y


def router_topk(logits: torch.Tensor, k: int, renorm: bool = True, out: tuple[torch.Tensor, torch.Tensor] | None = None
                ) -> tuple[torch.Tensor, torch.Tensor]:
    """Softmax over experts + k largest on the device: (topk_weights f32 [T, k], topk_ids int32 [T, k]).
    out = (weights, ids): contiguous [T, m >= k] tensors whose first k columns are written (a caller that runs fixed
    experts beside the routed ones keeps their weights and ids in the columns from k on); they are returned."""
    if not (logits.is_cuda and logits.dim() == 2 and logits.dtype == torch.float32 and logits.stride(1) == 1):
        raise ValueError("bf16n.router_topk: logits must be f32 [tokens, n_experts], contiguous along experts")
    T, E = logits.shape
    if out is None:
        ids = torch.empty((T, k), dtype=torch.int32, device=logits.device)
        wts = torch.empty((T, k), dtype=torch.float32, device=logits.device)
    else:
        wts, ids = out
        if not (wts.dtype == torch.float32 and ids.dtype == torch.int32 and wts.shape == ids.shape and wts.dim() == 2
                and wts.shape[0] == T and wts.shape[1] >= k and wts.is_contiguous() and ids.is_contiguous()
                and wts.device == logits.device and ids.device == logits.device):
            raise ValueError("bf16n.router_topk: out must be contiguous (f32, int32) [tokens, m >= k] tensors on the logits' device")
    with torch.cuda.device(logits.device):
        _lib.check(_lib.lib().bf16n_router_topk_strided(logits.data_ptr(), logits.stride(0), T, E, k, int(renorm), ids.data_ptr(),
                                                        wts.data_ptr(), ids.shape[1], _stream()))
    return wts, ids


# router_topk_routes: tokens up to which one block that selects and sorts beats the two launches (its one CU runs a
# wavefront per token: 7.7 / 8.6 / 12.4 us at 4 / 8 / 16 tokens against 4.6 + 5.4 us and the gap between two launches)
TOPK_ROUTE_ONE_LAUNCH_TOKENS = 8


def router_topk_routes(logits: torch.Tensor, k: int, n_listed: int, renorm: bool = True,
                       out: tuple[torch.Tensor, torch.Tensor] | None = None):
    """router_topk followed by mm_ids_route(ids, n_listed, False) over every column of the id rows: (weights, ids,
    (ids_src1, ids_dst, bounds)).  One launch (bf16n_router_topk_route) up to TOPK_ROUTE_ONE_LAUNCH_TOKENS tokens, two
    beyond."""
    if out is not None and not (out[1].dim() == 2 and out[1].shape[1] >= k):
        raise ValueError("bf16n.router_topk_routes: out must be (f32, int32) [tokens, m >= k] tensors")
    T = logits.shape[0] if logits.dim() == 2 else 0
    n_slots = out[1].shape[1] if out is not None else k
    L = _lib.lib()
    if T == 0 or T > TOPK_ROUTE_ONE_LAUNCH_TOKENS or not L.bf16n_router_topk_route_fits(T, n_slots, n_listed):
        wts, ids = router_topk(logits, k, renorm, out)
        return wts, ids, mm_ids_route(ids, n_listed, False)
    if not (logits.is_cuda and logits.dtype == torch.float32 and logits.stride(1) == 1):
        raise ValueError("bf16n.router_topk: logits must be f32 [tokens, n_experts], contiguous along experts")
    dev = logits.device
    if out is None:
        ids = torch.empty((T, k), dtype=torch.int32, device=dev)
        wts = torch.empty((T, k), dtype=torch.float32, device=dev)
    else:
        wts, ids = out
        if not (wts.dtype == torch.float32 and ids.dtype == torch.int32 and wts.shape == ids.shape and wts.shape[0] == T
                and wts.is_contiguous() and ids.is_contiguous() and wts.device == dev and ids.device == dev):
            raise ValueError("bf16n.router_topk: out must be contiguous (f32, int32) [tokens, m >= k] tensors on the logits' device")
    src1 = torch.empty(T * n_slots, dtype=torch.int32, device=dev)
    dst = torch.empty(T * n_slots, dtype=torch.int32, device=dev)
    bounds = torch.empty(n_listed + 1, dtype=torch.int32, device=dev)
    with torch.cuda.device(dev):
        _lib.check(L.bf16n_router_topk_route(logits.data_ptr(), logits.stride(0), T, logits.shape[1], k, int(renorm), ids.data_ptr(),
                                             wts.data_ptr(), n_slots, n_slots, n_listed, src1.data_ptr(), dst.data_ptr(),
                                             bounds.data_ptr(), 1, 1, _stream()))
    return wts, ids, (src1, dst, bounds)


def last_kernel() -> str:
    """The kernel instance the calling thread's last dense product launch chose, as a profiler prints it
    (bf16n_last_kernel; "" where the path leaves no note)."""
    return _lib.lib().bf16n_last_kernel().decode()


def glu2_supported(gate: Weight, up: Weight) -> bool:
    """Layouts with a fused gate / up + SwiGLU GEMV (the rule of bf16n::mmv_glu(gate, up), core launch.h:56-61, plus
    this build's wave64 units): same format, K, R and layout, not chunk-major."""
    g, u = gate.meta, up.meta
    return ((g.format, g.K, g.R, g.flags) == (u.format, u.K, u.R, u.flags) and not g.chunk_major
            and (not g.wave64 or g.K in (512, 1024, 2048, 4096)))


def _experts_batched(x, gate, up, down, topk_ids, n_experts, routes=None):
    """Per-pair FP32 outputs of the routed experts through the batched kernels: one routing pass serves both products
    (with one activation row per (token, slot), as down takes them, the source row of a pair is its destination row)."""
    src1, dst, bounds = routes if routes is not None else mm_ids_route(topk_ids, n_experts, False)
    hidden = moe_mm_ids(x, topk_ids, gate, n_experts, up=up, out_dtype=torch.bfloat16, routes=(src1, dst, bounds))
    return moe_mm_ids(hidden, topk_ids, down, n_experts, out_dtype=torch.float32, routes=(dst, dst, bounds))


def _experts_gemv_hidden(x, gate, up, topk_ids, n_mid):
    """silu(gate x) * (up x) per (token, slot) in FP32 through one GEMV column each, fused where a kernel is."""
    if glu2_supported(gate, up):
        return mmv_glu2(x, gate, up, topk_ids, n_mid)
    return swiglu(mmv(x, gate, topk_ids, n_mid), mmv(x, up, topk_ids, n_mid))


def moe_experts_batched(n_tokens: int, n_used: int, gate: Weight, up: Weight, down: Weight, n_experts: int) -> bool:
    """Whether moe_experts_rows runs these experts through the batched kernels (then it takes routing lists) rather than
    through one GEMV column per (token, slot); the thresholds are explained there."""
    tiles = all(m.meta.wave64 and m.meta.R == 32 for m in (gate, up, down))
    if tiles:
        gemv = n_tokens * n_used <= max(MOE_GEMV_MIN_PAIRS, MOE_GEMV_PAIRS_PER_EXPERT[0] * n_experts)
    elif all(m.meta.format == FMT_NIBBLE for m in (gate, up, down)):
        # the 4-bit code: its GEMV columns have no decode chain and stay ahead for longer (40 layers of 257 experts,
        # top-8 + 1: 182 / 202 / 221 us per layer at 12 / 14 / 16 tokens against 195 / 199 / 203 batched)
        gemv = n_tokens <= max(GEMV_MAX_TOKENS, int(MOE_GEMV_PAIRS_PER_EXPERT[2] * n_experts) // n_used)
    else:
        gemv = n_tokens <= max(GEMV_MAX_TOKENS, int(MOE_GEMV_PAIRS_PER_EXPERT[1] * n_experts) // n_used)
    return not gemv and mm_ids_supported(gate, up) and mm_ids_supported(down)


def moe_experts_rows(x: torch.Tensor, gate: Weight, up: Weight, down: Weight, topk_ids: torch.Tensor, n_experts: int,
                     routes=None) -> torch.Tensor:
    """The per-(token, slot) outputs down_e(silu(gate_e x) * (up_e x)) of the routed experts, FP32 [T, n_used, H]:
    moe_experts before the weighted sum (callers that fold the sum into their own next launch, add_rmsnorm, stop here).
    routes: mm_ids_route(topk_ids, n_experts, False) if the caller has it (router_topk_routes), used by the batched kernels.

    The reference switches from expert GEMVs to the batched kernels above 8 tokens.  Here the GEMVs stay ahead only
    while the routed pairs are few against the experts (each pair decodes one expert matrix in its own GEMV column; the
    batched kernel decodes every active expert once).  Tile layout: up to 0.14 pairs per expert and never below 24 pairs
    (top-8 of 256: 4 tokens; with a ninth slot that every token shares, 3; measured, GEMVs against batched kernels, at
    4 / 5 / 6 tokens: 50 / 64 / 68 against 55 / 67 / 64 us with 8 slots, 61 / 67 / 80 against 57 / 69 / 67 us with 9),
    its batched kernel splits K over wavefronts while few experts are active; other layouts: 0.7 pairs per expert and
    never below the reference's 8 tokens."""
    n_tokens, n_used = x.shape[0], max(int(topk_ids.shape[1]), 1)
    n_mid, n_out = gate.meta.rows // n_experts, down.meta.rows // n_experts
    x = x.contiguous()
    if moe_experts_batched(n_tokens, n_used, gate, up, down, n_experts):
        return _experts_batched(x, gate, up, down, topk_ids, n_experts, routes)
    # one GEMV column per (token, slot), FP32 between the products
    return mmv(_experts_gemv_hidden(x, gate, up, topk_ids, n_mid), down, topk_ids, n_out)


def moe_experts(x: torch.Tensor, gate: Weight, up: Weight, down: Weight, topk_weights: torch.Tensor,
                topk_ids: torch.Tensor, n_experts: int) -> torch.Tensor:
    """Routed experts of one MoE layer, BF16 out: for every token the weighted sum over its top-k experts of
    down_e(silu(gate_e x) * (up_e x)) (engines/vllm/vllm_bf16n/ops.py:251-271); see moe_experts_rows for the paths."""
    return moe_combine(moe_experts_rows(x, gate, up, down, topk_ids, n_experts), topk_weights, torch.bfloat16)
