"""torch.ops.bf16n.*: the reference extension's operator schema (core/torch/torch_bindings.cpp:373-389) registered over
the C ABI.  CPU part: schemas, the CPU encode ops against the fixtures, fake (meta) shapes as in the reference's
tests/core/test_opcheck.py.  GPU part: the ops give what the Python layer gives."""
from __future__ import annotations

import numpy as np
import pytest
import torch

from conftest import golden
from orin_qwen_lossless_amd import ops, synth, torch_ops

B = torch.ops.bf16n


def bf16(bits: np.ndarray) -> torch.Tensor:
    return torch.from_numpy(np.ascontiguousarray(bits).view(np.int16)).view(torch.bfloat16)


def test_schemas_match_the_reference_extension():
    want = {
        "encode": "bf16n::encode(Tensor w, int format, int R, bool chunk_major, bool frag_order=False) -> (Tensor, Tensor)",
        "dequant": "bf16n::dequant(Tensor plane, Tensor aux, int[] meta, int row0, int nrows) -> Tensor",
        "mmv": "bf16n::mmv(Tensor x, Tensor plane, Tensor aux, int[] meta, Tensor? ids, int rows_per_matrix, bool out_bf16) -> Tensor",
        "mmv_glu": "bf16n::mmv_glu(Tensor x, Tensor plane, Tensor aux, int[] meta, Tensor? ids, int rows_per_matrix, bool out_bf16) -> Tensor",
        "linear": "bf16n::linear(Tensor x, Tensor plane, Tensor aux, int[] meta, Tensor? bias) -> Tensor",
        "get_rows": "bf16n::get_rows(Tensor ids, Tensor plane, Tensor aux, int[] meta, bool out_bf16) -> Tensor",
        "moe_mm_ids": "bf16n::moe_mm_ids(Tensor x, Tensor topk_ids, Tensor plane, Tensor aux, int[] meta, Tensor? up_plane, "
                      "Tensor? up_aux, int[] up_meta, int n_experts, bool out_bf16) -> Tensor",
        "moe_combine": "bf16n::moe_combine(Tensor ys, Tensor topk_weights, bool out_bf16) -> Tensor",
        "swiglu": "bf16n::swiglu(Tensor g, Tensor u) -> Tensor",
        "init": "bf16n::init() -> ()",
    }
    for name, schema in want.items():
        assert str(getattr(B, name).default._schema) == schema, name


def test_encode_op_reproduces_the_reference_bytes():
    z = golden("hp_rm_k2048_r4")
    plane, aux = B.encode(bf16(z["w"]), 3, 4, False)
    assert plane.shape == z["w"].shape and plane.dtype == torch.uint8
    assert np.array_equal(plane.numpy().reshape(-1), z["plane"].reshape(-1))
    assert np.array_equal(aux.numpy(), z["aux"])
    meta = torch_ops.meta_of(aux)
    assert meta[:5] == [3, 2048, z["w"].shape[0], 4, 0]
    with pytest.raises((ValueError, RuntimeError), match="multiple of R"):
        B.encode(bf16(z["w"][:6]), 3, 4, False)


def test_encode_auto_uses_the_policy():
    w = bf16(synth.weights(8192, 2048, 5))
    plane, aux = B.encode_auto(w, 1, "mi355x")
    meta = torch_ops.meta_of(aux)
    assert meta[0] == 3 and meta[4] & ops.FLAG_WAVE64
    plane2, aux2 = B.encode_auto(w, 1, "llama")
    assert torch_ops.meta_of(aux2)[4] == 0 and torch.equal(plane, plane2)  # the plane is the same in both layouts


def test_fake_implementations_give_the_output_shapes():
    from torch._subclasses.fake_tensor import FakeTensorMode

    meta = [3, 2048, 4096, 16, 4, 256, 16640, 17672, 17672]
    with FakeTensorMode():
        x = torch.empty((3, 2048), dtype=torch.bfloat16, device="cuda")
        plane = torch.empty((4096, 2048), dtype=torch.uint8, device="cuda")
        aux = torch.empty((1 << 20,), dtype=torch.uint8, device="cuda")
        ids = torch.empty((3, 8), dtype=torch.int32, device="cuda")
        assert B.mmv(x, plane, aux, meta, None, 0, False).shape == (3, 4096)
        assert B.mmv(x, plane, aux, meta, ids, 512, True).shape == (3, 8, 512)
        assert B.mmv(x, plane, aux, meta, ids, 512, True).dtype == torch.bfloat16
        assert B.mmv_glu(x, plane, aux, meta, None, 0, False).shape == (3, 2048)
        assert B.linear(x, plane, aux, meta, None).shape == (3, 4096)
        assert B.dequant(plane, aux, meta, 16, 32).shape == (32, 2048)
        assert B.get_rows(ids[:, 0], plane, aux, meta, True).shape == (3, 2048)
        assert B.moe_mm_ids(x, ids, plane, aux, meta, None, None, [], 8, False).shape == (3, 8, 512)
        ys = torch.empty((3, 8, 512), dtype=torch.float32, device="cuda")
        assert B.moe_combine(ys, torch.empty((3, 8), device="cuda"), True).shape == (3, 512)
        assert B.swiglu(ys, ys).shape == ys.shape
        w, i = B.router_topk(torch.empty((3, 256), device="cuda"), 8, True)
        assert w.shape == (3, 8) and i.dtype == torch.int32


@pytest.mark.gpu
def test_ops_equal_the_python_layer():
    B.init()
    K, rows = 2048, 256
    wb = synth.weights(rows, K, 71)
    plane, aux = B.encode_auto(bf16(wb), 1, "llama")  # below the dense threshold: NIBBLE
    plane2, aux2 = B.encode(bf16(wb), 3, 16, False)
    for p, a in ((plane, aux), (plane2, aux2)):
        meta = torch_ops.meta_of(a)
        pd, ad = p.cuda(), a.cuda()
        w = ops.Weight(pd.view(-1), ad, ops.parse_header(a))
        x = bf16(synth.activations(2, K, 72)).cuda()
        assert torch.equal(B.dequant(pd.view(-1), ad, meta, 0, rows), ops.dequant(w))
        assert torch.equal(B.mmv(x, pd.view(-1), ad, meta, None, 0, False), ops.mmv(x, w))
        assert torch.equal(B.linear(x, pd.view(-1), ad, meta, None), ops.linear(x, w))
        if meta[0] == 1:
            continue
        ids = torch.tensor([3, 200, 17], dtype=torch.int32, device="cuda")
        assert torch.equal(B.get_rows(ids, pd.view(-1), ad, meta, True), ops.get_rows(ids, w))
    g = torch.randn((5, 300), device="cuda")
    assert torch.equal(B.swiglu(g, g * 2), ops.swiglu(g, g * 2))
    wts, ids = B.router_topk(torch.randn((4, 64), device="cuda"), 4, True)
    assert ids.shape == (4, 4) and torch.allclose(wts.sum(-1), torch.ones(4, device="cuda"), atol=1e-6)


@pytest.mark.gpu
def test_opcheck_and_compile():
    # schema and fake-tensor consistency of the registered ops, and a traced function without graph breaks
    # (restates tests/core/test_opcheck.py of the reference)
    B.init()
    K, rows = 1024, 128
    plane, aux = B.encode(bf16(synth.weights(rows, K, 81)), 3, 8, False)
    meta = torch_ops.meta_of(aux)
    pd, ad = plane.cuda().view(-1), aux.cuda()
    x = bf16(synth.activations(2, K, 82)).cuda()
    ids = torch.tensor([[0, 1], [1, 0]], dtype=torch.int32, device="cuda")
    checks = ("test_schema", "test_faketensor")
    torch.library.opcheck(B.mmv.default, (x, pd, ad, meta, None, 0, False), test_utils=checks)
    torch.library.opcheck(B.mmv.default, (x, pd, ad, meta, ids, 64, True), test_utils=checks)
    torch.library.opcheck(B.dequant.default, (pd, ad, meta, 8, 16), test_utils=checks)
    torch.library.opcheck(B.linear.default, (x, pd, ad, meta, None), test_utils=checks)
    torch.library.opcheck(B.swiglu.default, (torch.randn(4, 8, device="cuda"), torch.randn(4, 8, device="cuda")), test_utils=checks)

    def f(x):
        return B.swiglu(B.mmv(x, pd, ad, meta, None, 0, False), B.mmv(x, pd, ad, meta, None, 0, False))

    got = torch.compile(f, fullgraph=True, backend="eager")(x)
    assert torch.equal(got, f(x))
