"""Encoded tensors on disk (orin_qwen_lossless_amd/store.py): what is saved is what the encoder produced, byte for byte,
for every format and layout; a file that is not one is refused; on the GPU a loaded tensor decodes bit-exactly."""
import numpy as np
import pytest
import torch

from orin_qwen_lossless_amd import ops, store, synth

NIB, HUF, HP = 1, 2, 3


def make():
    w1, w2, w3 = synth.model_like(64, 1024, 1), synth.weights(32, 512, 2), synth.weights(96, 2048, 3)
    enc = {"dense.w64": ops.encode_bits(w1, HP, 8, False, wave64=True)[:2], "small.nibble": ops.encode_bits(w2, NIB, 0)[:2],
           "experts.tiles": ops.encode_bits(w3, HP, 32, False, wave64=True)[:2], "ref.cm": ops.encode_bits(w3, HP, 8, True)[:2],
           "ref.huffman": ops.encode_bits(w2, HUF, 4)[:2]}
    return {"dense.w64": w1, "small.nibble": w2, "experts.tiles": w3, "ref.cm": w3, "ref.huffman": w2}, enc


def test_save_load_round_trip(tmp_path, oracle):
    src, enc = make()
    path = str(tmp_path / "m.safetensors")
    store.save(path, enc)
    got = store.load(path)
    assert sorted(got) == sorted(enc)
    for name, (plane, aux) in enc.items():
        w = got[name]
        assert np.array_equal(w.plane.numpy().reshape(-1), plane.reshape(-1)) and np.array_equal(w.aux.numpy(), aux)
        assert w.meta == ops.parse_header(torch.from_numpy(aux))
        assert np.array_equal(oracle.decode(w.plane.numpy(), w.aux.numpy()), src[name])
    assert sorted(store.load(path, names={"ref.cm"})) == ["ref.cm"]


def test_refuses_foreign_files_and_buffers(tmp_path):
    from safetensors.torch import save_file

    path = str(tmp_path / "x.safetensors")
    save_file({"a.aux": torch.zeros(300, dtype=torch.uint8), "a.plane": torch.zeros(4, dtype=torch.uint8)}, path)
    with pytest.raises(ValueError, match="not a bf16n-encoded-1 file"):
        store.load(path)
    _, enc = make()
    plane, aux = enc["small.nibble"]
    with pytest.raises(ValueError):
        store.save(path, {"bad": (plane[:-1], aux)})            # plane size against the header
    with pytest.raises(ValueError):
        store.save(path, {"bad": (plane, aux[:100])})           # not an aux buffer


@pytest.mark.gpu
def test_loaded_tensors_decode_bit_exactly_on_the_device(tmp_path):
    o = ops
    o.init()
    src, enc = make()
    path = str(tmp_path / "m.safetensors")
    store.save(path, enc)
    for name, w in store.load(path, device="cuda").items():
        ref = torch.from_numpy(src[name].view(np.int16)).view(torch.bfloat16)
        assert o.roundtrip_equal(w, ref), name
