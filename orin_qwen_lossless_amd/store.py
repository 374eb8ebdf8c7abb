"""Encoded tensors on disk: plane + aux of every matrix in one safetensors file, so that a model is encoded and verified
once and later loads skip the encoder (the reference leaves this to its roadmap, docs/ROADMAP.md "Stage 8"; its engines
re-encode from the BF16 checkpoint at every load).  Nothing is interpreted here: the aux buffer carries its own header,
and load() parses it with ops.parse_header exactly as a fresh encode would be parsed.

    store.save("model.bf16n.safetensors", {"lm_head": (plane, aux), ...})
    weights = store.load("model.bf16n.safetensors", device="cuda:0")      # name -> ops.Weight
"""
from __future__ import annotations

import numpy as np
import torch
from safetensors import safe_open
from safetensors.torch import save_file

from . import ops

FORMAT_TAG = "bf16n-encoded-1"


def _u8(a) -> torch.Tensor:
    t = torch.from_numpy(np.ascontiguousarray(a)) if isinstance(a, np.ndarray) else a
    if t.dtype != torch.uint8:
        raise ValueError("bf16n.store: plane and aux must be uint8")
    return t.detach().cpu().contiguous().reshape(-1)


def save(path: str, tensors: dict) -> None:
    """tensors: name -> (plane, aux) (numpy or torch uint8, as ops.encode_bits / ops.encode return them) or ops.Weight."""
    out = {}
    for name, v in tensors.items():
        plane, aux = (v.plane, v.aux) if isinstance(v, ops.Weight) else v
        plane, aux = _u8(plane), _u8(aux)
        m = ops.parse_header(aux)                      # refuses anything that is not an aux buffer
        if plane.numel() != m.rows * m.K:
            raise ValueError(f"bf16n.store: {name}: plane has {plane.numel()} bytes, header says {m.rows} x {m.K}")
        out[name + ".plane"], out[name + ".aux"] = plane, aux
    save_file(out, path, metadata={"format": FORMAT_TAG})


def load(path: str, device: str | torch.device = "cpu", names=None) -> dict:
    """name -> ops.Weight on `device` (plane reshaped to rows x K); names: only these matrices."""
    res = {}
    with safe_open(path, framework="pt", device="cpu") as f:
        if (f.metadata() or {}).get("format") != FORMAT_TAG:
            raise ValueError(f"bf16n.store: {path} is not a {FORMAT_TAG} file")
        stems = sorted({k[: -len(".aux")] for k in f.keys() if k.endswith(".aux")})
        for name in stems:
            if names is not None and name not in names:
                continue
            aux = f.get_tensor(name + ".aux")
            m = ops.parse_header(aux)
            plane = f.get_tensor(name + ".plane")
            if plane.numel() != m.rows * m.K:
                raise ValueError(f"bf16n.store: {name}: plane size does not match its header")
            res[name] = ops.upload(plane.reshape(m.rows, m.K), aux, m, device)
    return res
