"""`torch.ops.bf16n.*`: the operator schema of the reference's torch extension (core/torch/torch_bindings.cpp:373-389)
registered from Python over the C ABI, with the reference's fake (meta) implementations
(engines/vllm/vllm_bf16n/ops.py:292-369) so that the ops trace under torch.compile and FakeTensor.

    import orin_qwen_lossless_amd.torch_ops        # registers the library once
    plane, aux = torch.ops.bf16n.encode(w_cpu_bf16, 3, 16, False)          # reference layouts
    plane, aux = torch.ops.bf16n.encode_auto(w_cpu_bf16, 1, "mi355x")      # this build's policy (wave64 units)
    meta = meta_of(aux)                                                    # [format, K, rows, R, flags, off_a..off_d]
    y = torch.ops.bf16n.mmv(x, plane.cuda(), aux.cuda(), meta, None, 0, False)

`meta` is the reference's list; bit 2 of meta[4] (flags) marks the wave64 layout.  The int4 / int2 baseline ops of the
reference extension are not part of the BF16N path and are not registered.  encode_auto is this build's addition."""
from __future__ import annotations

import torch

from . import ops

_lib = torch.library.Library("bf16n", "DEF")
_lib.define("init() -> ()")
_lib.define("encode(Tensor w, int format, int R, bool chunk_major, bool frag_order=False) -> (Tensor, Tensor)")
_lib.define("encode_auto(Tensor w, int n_matrices, str engine) -> (Tensor, Tensor)")
_lib.define("dequant(Tensor plane, Tensor aux, int[] meta, int row0, int nrows) -> Tensor")
_lib.define("mmv(Tensor x, Tensor plane, Tensor aux, int[] meta, Tensor? ids, int rows_per_matrix, bool out_bf16) -> Tensor")
_lib.define("mmv_glu(Tensor x, Tensor plane, Tensor aux, int[] meta, Tensor? ids, int rows_per_matrix, bool out_bf16) -> Tensor")
_lib.define("linear(Tensor x, Tensor plane, Tensor aux, int[] meta, Tensor? bias) -> Tensor")
_lib.define("get_rows(Tensor ids, Tensor plane, Tensor aux, int[] meta, bool out_bf16) -> Tensor")
_lib.define("moe_mm_ids(Tensor x, Tensor topk_ids, Tensor plane, Tensor aux, int[] meta, Tensor? up_plane, Tensor? up_aux, "
            "int[] up_meta, int n_experts, bool out_bf16) -> Tensor")
_lib.define("moe_combine(Tensor ys, Tensor topk_weights, bool out_bf16) -> Tensor")
_lib.define("swiglu(Tensor g, Tensor u) -> Tensor")
_lib.define("router_topk(Tensor logits, int k, bool renorm) -> (Tensor, Tensor)")


def meta_of(aux: torch.Tensor) -> list[int]:
    """The meta list of an encoded matrix from its (CPU) aux tensor."""
    return ops.parse_header(aux.cpu() if aux.is_cuda else aux).as_list()


def _weight(plane: torch.Tensor, aux: torch.Tensor, meta) -> ops.Weight:
    if len(meta) != 9:
        raise ValueError("bf16n: meta must be [format, K, rows, R, flags, off_a, off_b, off_c, off_d]")
    fmt, K, rows, R, flags, a, b, c, d = (int(v) for v in meta)
    return ops.Weight(plane, aux, ops.Meta(fmt, K, rows, R, bool(flags & ops.FLAG_CHUNK_MAJOR), bool(flags & ops.FLAG_FRAG_ORDER),
                                           a, b, c, d, bool(flags & ops.FLAG_WAVE64)))


def _dt(out_bf16: bool) -> torch.dtype:
    return torch.bfloat16 if out_bf16 else torch.float32


# ---------------------------------------------------------------- implementations

def _init():
    ops.init()


def _encode_cpu(w, fmt, R, chunk_major, frag_order=False):
    plane, aux, _ = ops.encode(w, fmt, R, chunk_major, frag_order)
    return plane.view(-1, w.shape[-1]), aux


def _encode_auto_cpu(w, n_matrices, engine):
    K = w.shape[-1]
    rows = w.numel() // K
    if n_matrices <= 0 or rows % n_matrices:
        raise ValueError("bf16n.encode_auto: rows must split into n_matrices")
    ch = ops.choose(rows // n_matrices, K, n_matrices, engine=engine, expert=n_matrices > 1)
    if ch is None:
        raise ValueError("bf16n.encode_auto: the policy keeps this shape in BF16")
    fmt, R, cm, fo, w64 = ch
    plane, aux, _ = ops.encode(w, fmt, R, cm, fo, w64)
    return plane.view(-1, K), aux


def _dequant(plane, aux, meta, row0, nrows):
    return ops.dequant(_weight(plane, aux, meta), row0, nrows)


def _mmv(x, plane, aux, meta, ids, rows_per_matrix, out_bf16):
    return ops.mmv(x, _weight(plane, aux, meta), ids, rows_per_matrix, _dt(out_bf16))


def _mmv_glu(x, plane, aux, meta, ids, rows_per_matrix, out_bf16):
    return ops.mmv_glu(x, _weight(plane, aux, meta), ids, rows_per_matrix, _dt(out_bf16))


def _linear(x, plane, aux, meta, bias):
    return ops.linear(x, _weight(plane, aux, meta), bias)


def _get_rows(ids, plane, aux, meta, out_bf16):
    return ops.get_rows(ids, _weight(plane, aux, meta), _dt(out_bf16))


def _moe_mm_ids(x, topk_ids, plane, aux, meta, up_plane, up_aux, up_meta, n_experts, out_bf16):
    up = _weight(up_plane, up_aux, up_meta) if up_plane is not None else None
    return ops.moe_mm_ids(x, topk_ids, _weight(plane, aux, meta), n_experts, up, _dt(out_bf16))


def _moe_combine(ys, topk_weights, out_bf16):
    return ops.moe_combine(ys, topk_weights, _dt(out_bf16))


def _swiglu(g, u):
    return ops.swiglu(g, u)


def _router_topk(logits, k, renorm):
    return ops.router_topk(logits, k, renorm)


_lib.impl("init", _init, "CompositeExplicitAutograd")
_lib.impl("encode", _encode_cpu, "CPU")
_lib.impl("encode_auto", _encode_auto_cpu, "CPU")
for _name, _fn in (("dequant", _dequant), ("mmv", _mmv), ("mmv_glu", _mmv_glu), ("linear", _linear), ("get_rows", _get_rows),
                   ("moe_mm_ids", _moe_mm_ids), ("moe_combine", _moe_combine), ("swiglu", _swiglu), ("router_topk", _router_topk)):
    _lib.impl(_name, _fn, "CUDA")


# ---------------------------------------------------------------- fake (meta) implementations

@torch.library.register_fake("bf16n::encode")
def _encode_fake(w, fmt, R, chunk_major, frag_order=False):
    ctx = torch.library.get_ctx()
    K = w.shape[-1]
    return w.new_empty((w.numel() // K, K), dtype=torch.uint8), w.new_empty((ctx.new_dynamic_size(),), dtype=torch.uint8)


@torch.library.register_fake("bf16n::encode_auto")
def _encode_auto_fake(w, n_matrices, engine):
    ctx = torch.library.get_ctx()
    K = w.shape[-1]
    return w.new_empty((w.numel() // K, K), dtype=torch.uint8), w.new_empty((ctx.new_dynamic_size(),), dtype=torch.uint8)


@torch.library.register_fake("bf16n::dequant")
def _dequant_fake(plane, aux, meta, row0, nrows):
    return plane.new_empty((nrows, meta[1]), dtype=torch.bfloat16)


def _mmv_shape(x, meta, ids, rows_per_matrix, glu):
    if ids is None:
        return (x.shape[0], meta[2] // 2 if glu else meta[2])
    return (ids.shape[0], ids.shape[1], rows_per_matrix // 2 if glu else rows_per_matrix)


@torch.library.register_fake("bf16n::mmv")
def _mmv_fake(x, plane, aux, meta, ids, rows_per_matrix, out_bf16):
    return x.new_empty(_mmv_shape(x, meta, ids, rows_per_matrix, False), dtype=_dt(out_bf16))


@torch.library.register_fake("bf16n::mmv_glu")
def _mmv_glu_fake(x, plane, aux, meta, ids, rows_per_matrix, out_bf16):
    return x.new_empty(_mmv_shape(x, meta, ids, rows_per_matrix, True), dtype=_dt(out_bf16))


@torch.library.register_fake("bf16n::linear")
def _linear_fake(x, plane, aux, meta, bias):
    return x.new_empty((*x.shape[:-1], meta[2]))


@torch.library.register_fake("bf16n::get_rows")
def _get_rows_fake(ids, plane, aux, meta, out_bf16):
    return plane.new_empty((ids.shape[0], meta[1]), dtype=_dt(out_bf16))


@torch.library.register_fake("bf16n::moe_mm_ids")
def _moe_mm_ids_fake(x, topk_ids, plane, aux, meta, up_plane, up_aux, up_meta, n_experts, out_bf16):
    return x.new_empty((topk_ids.shape[0], topk_ids.shape[1], meta[2] // n_experts), dtype=_dt(out_bf16))


@torch.library.register_fake("bf16n::moe_combine")
def _moe_combine_fake(ys, topk_weights, out_bf16):
    return ys.new_empty((ys.shape[0], ys.shape[2]), dtype=_dt(out_bf16))


@torch.library.register_fake("bf16n::swiglu")
def _swiglu_fake(g, u):
    return torch.empty_like(g)


@torch.library.register_fake("bf16n::router_topk")
def _router_topk_fake(logits, k, renorm):
    return logits.new_empty((logits.shape[0], k), dtype=torch.float32), logits.new_empty((logits.shape[0], k), dtype=torch.int32)
