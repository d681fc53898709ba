"""The safetensors container, the strict loader's errors and the random-weights mode (CPU).

Loader vectors from the reference's tests/unit/model/test_config_and_loader.py:96-131.
"""

from __future__ import annotations

import json
import shutil

import numpy as np
import pytest
import torch
from safetensors.torch import load_file, save_file

from dli_amd.weights import CheckpointError, SafetensorsFile, load_model, write_random_model, write_safetensors
from dli_amd.weights.safetensors_io import SafetensorsFormatError, bfloat16_bits_to_float32, float32_to_bfloat16_bits
from tiny_configs import TINY_A, TINY_B


def make_folder(tmp_path, raw=TINY_B, **kw):
    return write_random_model(tmp_path / "m", raw, seed=4, **kw)


def test_own_writer_is_read_by_the_safetensors_library_and_back(tmp_path):
    d = make_folder(tmp_path)
    theirs = load_file(str(d / "model.safetensors"))
    with SafetensorsFile(d / "model.safetensors") as f:
        assert sorted(f.names()) == sorted(theirs)
        for name in f.names():
            e = f.get(name)
            assert e.tag == "BF16" and e.shape == tuple(theirs[name].shape)
            mine = torch.from_numpy(bfloat16_bits_to_float32(np.array(e.bits)))
            assert torch.equal(mine, theirs[name].float())
    # and a file written by the library is read by the own reader, all supported types
    tensors = {"a": torch.randn(3, 5), "b": torch.randn(7).bfloat16(), "c": torch.arange(6, dtype=torch.int64),
               "d": torch.arange(4, dtype=torch.int32).view(2, 2), "e": torch.randn(2, 2).half()}
    save_file(tensors, str(tmp_path / "lib.safetensors"))
    with SafetensorsFile(tmp_path / "lib.safetensors") as f:
        assert np.array_equal(f.get("a").bits, tensors["a"].numpy())
        assert np.array_equal(f.get("c").bits, tensors["c"].numpy())
        assert np.array_equal(f.get("d").bits, tensors["d"].numpy())
        assert f.get("b").tag == "BF16" and f.get("e").tag == "F16"
        assert np.array_equal(bfloat16_bits_to_float32(np.array(f.get("b").bits)), tensors["b"].float().numpy())


def test_bfloat16_rounding_is_nearest_even():
    x = torch.randn(10000) * 3
    x[:4] = torch.tensor([1.00390625, 1.01171875, float("inf"), -0.0])  # two exact ties
    bits = float32_to_bfloat16_bits(x.numpy())
    assert torch.equal(torch.from_numpy(bfloat16_bits_to_float32(bits)), x.bfloat16().float())


@pytest.mark.parametrize("damage,match", [
    (lambda b: b[:5], "shorter"),
    (lambda b: (2 ** 40).to_bytes(8, "little") + b[8:], "exceeds"),
    (lambda b: b[:8] + b"x" + b[9:], "not JSON"),
    (lambda b: b[:-3], "outside|bytes"),
])
def test_malformed_files_are_refused(tmp_path, damage, match):
    write_safetensors(tmp_path / "ok.safetensors", {"w": ("F32", np.ones((2, 3), np.float32))})
    raw = (tmp_path / "ok.safetensors").read_bytes()
    (tmp_path / "bad.safetensors").write_bytes(damage(raw))
    with pytest.raises(SafetensorsFormatError, match=match):
        SafetensorsFile(tmp_path / "bad.safetensors")


def _rewrite(folder, change):
    path = folder / "model.safetensors"
    state = load_file(str(path))
    change(state)
    save_file(state, str(path))


def test_pickle_only_folder_is_refused(tmp_path):
    d = make_folder(tmp_path)
    (d / "model.safetensors").rename(d / "pytorch_model.bin")
    with pytest.raises(CheckpointError, match="pickle"):
        load_model(d, dtype="float32", device="cpu")
    (d / "pytorch_model.bin").unlink()
    with pytest.raises(CheckpointError, match="no \\*.safetensors"):
        load_model(d, dtype="float32", device="cpu")


def test_one_error_lists_missing_unexpected_and_misshapen(tmp_path):
    d = make_folder(tmp_path)

    def change(state):
        del state["model.layers.1.mlp.up_proj.weight"]
        del state["model.layers.2.self_attn.k_proj.weight"]
        state["model.norm.weight"] = torch.ones(191).bfloat16()
        state["model.layers.0.self_attn.rotary_emb.inv_freq"] = torch.ones(16)
    _rewrite(d, change)
    with pytest.raises(CheckpointError) as exc:
        load_model(d, dtype="float32", device="cpu")
    msg = str(exc.value)
    assert "missing" in msg and "model.layers.1.mlp.up_proj.weight" in msg
    assert "model.layers.2.self_attn.k_proj.weight" in msg
    assert "unexpected" in msg and "rotary_emb.inv_freq" in msg
    assert "shape" in msg and "model.norm.weight" in msg and "[191]" in msg and "[192]" in msg


def test_tied_head_in_the_file_must_equal_the_embedding(tmp_path):
    d = make_folder(tmp_path, raw=TINY_A)
    _rewrite(d, lambda s: s.__setitem__("lm_head.weight", s["model.embed_tokens.weight"].clone()))
    load_model(d, dtype="float32", device="cpu")  # an exact copy is accepted and dropped
    _rewrite(d, lambda s: s.__setitem__("lm_head.weight", torch.randn_like(s["model.embed_tokens.weight"])))
    with pytest.raises(CheckpointError, match="tie_word_embeddings"):
        load_model(d, dtype="float32", device="cpu")


def test_untied_model_needs_its_head(tmp_path):
    d = make_folder(tmp_path)
    _rewrite(d, lambda s: s.pop("lm_head.weight"))
    with pytest.raises(CheckpointError, match="missing.*lm_head.weight"):
        load_model(d, dtype="float32", device="cpu")


def test_stored_types_after_loading(tmp_path):
    d = make_folder(tmp_path)
    for dtype, want in (("float32", torch.float32), ("bfloat16", torch.bfloat16)):
        m = load_model(d, dtype=dtype, device="cpu")
        attn = m.layers[0].parts["mixer"]
        assert attn.w_qkv.dtype == want and attn.w_qkv.shape == ((6 + 2 * 2) * 32, 192)
        assert m.layers[0].parts["mixer_norm"].weight.dtype == torch.float32  # norms stay 32-bit
        assert m.head.weight.dtype == want and m.embedding.weight.dtype == want
    # sharded folders are merged
    state = load_file(str(d / "model.safetensors"))
    names = sorted(state)
    save_file({n: state[n] for n in names[::2]}, str(d / "model-00001-of-00002.safetensors"))
    save_file({n: state[n] for n in names[1::2]}, str(d / "model-00002-of-00002.safetensors"))
    (d / "model.safetensors").unlink()
    m2 = load_model(d, dtype="float32", device="cpu")
    assert torch.equal(m2.head.weight, load_model(make_folder(tmp_path / "x"), dtype="float32", device="cpu").head.weight)


def test_random_weights_depend_on_seed_and_name_only(tmp_path):
    a = load_file(str(write_random_model(tmp_path / "a", TINY_A, seed=1) / "model.safetensors"))
    b = load_file(str(write_random_model(tmp_path / "b", TINY_A, seed=1) / "model.safetensors"))
    c = load_file(str(write_random_model(tmp_path / "c", TINY_A, seed=2) / "model.safetensors"))
    assert all(torch.equal(a[k], b[k]) for k in a)
    assert not torch.equal(a["model.embed_tokens.weight"], c["model.embed_tokens.weight"])
    # a tensor's values do not depend on what else the model holds: 3 layers instead of 2
    bigger = load_file(str(write_random_model(tmp_path / "d", {**TINY_A, "num_hidden_layers": 3}, seed=1)
                           / "model.safetensors"))
    assert all(torch.equal(a[k], bigger[k]) for k in a)
    w = a["model.layers.0.mlp.down_proj.weight"].float()
    assert abs(w.std().item() - 0.02) < 0.002 and abs(w.mean().item()) < 0.002
    assert torch.all(a["model.norm.weight"] == 1)
    assert "lm_head.weight" not in a and json.loads((tmp_path / "a" / "config.json").read_text()) == TINY_A
    f32 = load_file(str(write_random_model(tmp_path / "e", TINY_A, seed=1, storage="float32") / "model.safetensors"))
    assert f32["model.norm.weight"].dtype == torch.float32
    assert torch.equal(f32["model.embed_tokens.weight"].bfloat16(), a["model.embed_tokens.weight"])
