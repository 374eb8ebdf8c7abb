"""bf16n_moe_mm_ids_static, the entry point that allocates nothing: routing lists in the library's own device array.
Called through the C ABI and compared bit for bit with bf16n_mm_ids_route + bf16n_mm_ids on the same inputs, on two calls
in a row, the second with fewer tokens (the array keeps the first call's lists), and with the device allocator watched."""
from __future__ import annotations

import ctypes as C

import numpy as np
import pytest
import torch

from orin_qwen_lossless_amd import _lib, synth
from test_gpu_kernels import tbf16
from test_gpu_roundtrip import enc

pytestmark = pytest.mark.gpu
HP = 3


def static_call(ops, x, ids, w, n_experts, up=None, out_dtype=torch.float32):
    from orin_qwen_lossless_amd.ops import _cweight, _stream

    T, n_used = ids.shape
    N = w.meta.rows // n_experts
    y = torch.empty((T, n_used, N), dtype=out_dtype, device=x.device)
    cw = _cweight(w)
    cu = _cweight(up) if up is not None else None
    before = torch.cuda.memory_stats()["allocation.all.allocated"]
    free_before, _ = torch.cuda.mem_get_info()
    _lib.check(_lib.lib().bf16n_moe_mm_ids_static(
        C.byref(cw), C.byref(cu) if cu is not None else None, x.data_ptr(), w.meta.K, ids.data_ptr(),
        int(ids.dtype == torch.int64), ids.stride(0), int(x.dim() == 3), y.data_ptr(), int(out_dtype == torch.bfloat16), N,
        n_experts, T, n_used, _stream()))
    torch.cuda.synchronize()
    assert torch.cuda.memory_stats()["allocation.all.allocated"] == before   # nothing from torch's allocator
    assert torch.cuda.mem_get_info()[0] == free_before                        # and nothing from the device
    return y


@pytest.mark.parametrize("layout", ["tiles", "units", "nibble"])
def test_static_routing_lists_match_the_allocating_path(ops, layout):
    E, k, K, N = 24, 4, 2048, 512
    if layout == "nibble":  # expert stacks in the 4-bit code: the third dispatch branch of the entry point
        gate, up, down = (enc(ops, synth.weights(r, c, 201 + i), 1, 0, False) for i, (r, c) in enumerate(((E * N, K), (E * N, K), (E * K, N))))
    else:
        r_gu, r_dn = (32, 32) if layout == "tiles" else (4, 16)
        gate = enc(ops, synth.weights(E * N, K, 201), HP, r_gu, False, True)
        up = enc(ops, synth.weights(E * N, K, 202), HP, r_gu, False, True)
        down = enc(ops, synth.weights(E * K, N, 203), HP, r_dn, False, True)
    rng = np.random.default_rng(7)
    for T in (300, 41):  # the second call is smaller: entries of the first call's lists stay behind it in the array
        x = tbf16(synth.activations(T, K, 210 + T))
        ids = torch.from_numpy(np.stack([rng.permutation(E)[:k] for _ in range(T)]).astype(np.int32)).cuda()
        for idt in (torch.int32, torch.int64):
            idx = ids.to(idt)
            want = ops.moe_mm_ids(x, idx, gate, E, up=up, out_dtype=torch.bfloat16)
            got = static_call(ops, x, idx, gate, E, up=up, out_dtype=torch.bfloat16)
            assert torch.equal(got.view(torch.int16), want.view(torch.int16)), (T, idt)
        want_dn = ops.moe_mm_ids(want, ids, down, E)
        got_dn = static_call(ops, want, ids, down, E)
        assert torch.equal(got_dn, want_dn), T
        want_g = ops.moe_mm_ids(x, ids, gate, E)   # without the fused up matrix
        assert torch.equal(static_call(ops, x, ids, gate, E), want_g), T


def test_static_entry_rejects_sizes_beyond_its_array(ops):
    E, k, K, N = 8, 8, 2048, 64
    gate = enc(ops, synth.weights(E * N, K, 220), HP, 32, False, True)
    T = 65536 // k + 1
    x = torch.zeros((T, K), dtype=torch.bfloat16, device="cuda")
    ids = torch.zeros((T, k), dtype=torch.int32, device="cuda")
    with pytest.raises(ValueError, match="at most 65536 routed pairs"):
        static_call(ops, x, ids, gate, E)
