"""Safetensors reading and writing, the one error for a checkpoint that does not fit, random weights (no GPU)."""
import json
import os
import struct

import pytest
import torch

from conftest import TINY_A, TINY_B
from rust_inference_amd.config import config_from_dict
from rust_inference_amd.errors import UnsupportedError, WeightsError
from rust_inference_amd.parts import expected_tensors
from rust_inference_amd.weights import ModelFolder, SafeTensorFile, load_checked, save_file, write_random_model


def spec_of(raw):
    arch, c = config_from_dict(raw)
    return arch.build_spec(c)


def test_round_trip_and_dtypes_are_kept(tmp_path):
    t = {"a": torch.randn(3, 5).to(torch.bfloat16), "b": torch.randn(7), "idx": torch.arange(4, dtype=torch.int32)}
    path = str(tmp_path / "x.safetensors")
    save_file(t, path)
    f = SafeTensorFile(path)
    assert sorted(f.names()) == ["a", "b", "idx"]
    for name, want in t.items():
        got = f.load(name)
        assert got.dtype == want.dtype and torch.equal(got, want)      # bfloat16 stays, float32 stays
    # the safetensors package reads the same file
    from safetensors import safe_open
    with safe_open(path, framework="pt") as g:
        assert torch.equal(g.get_tensor("a"), t["a"])


def test_files_written_by_the_safetensors_package_are_read(tmp_path):
    from safetensors.torch import save_file as st_save
    t = {"w": torch.randn(4, 6).to(torch.bfloat16)}
    st_save(t, str(tmp_path / "model.safetensors"))
    assert torch.equal(ModelFolder(str(tmp_path)).load("w"), t["w"])


def test_bad_files_are_refused(tmp_path):
    p = tmp_path / "model.safetensors"
    p.write_bytes(b"abc")
    with pytest.raises(WeightsError, match="too small"):
        SafeTensorFile(str(p))
    p.write_bytes(struct.pack("<Q", 1000) + b"{}")
    with pytest.raises(WeightsError, match="past the end"):
        SafeTensorFile(str(p))
    header = json.dumps({"w": {"dtype": "F32", "shape": [4], "data_offsets": [0, 8]}}).encode()
    p.write_bytes(struct.pack("<Q", len(header)) + header + b"\0" * 8)
    with pytest.raises(WeightsError, match="bad data offsets for w"):         # src/safetensors.rs:76-79
        SafeTensorFile(str(p))
    header = json.dumps({"w": {"dtype": "F8_E4M3", "shape": [4], "data_offsets": [0, 4]}}).encode()
    p.write_bytes(struct.pack("<Q", len(header)) + header + b"\0" * 4)
    f8 = SafeTensorFile(str(p))                          # a format this library does not read is refused when
    assert f8.tensors["w"].dtype is None                 # the tensor is asked for, not when the file is opened
    with pytest.raises(UnsupportedError, match="F8_E4M3"):
        f8.load("w")
    with pytest.raises(WeightsError, match="neither"):
        ModelFolder(str(tmp_path / "nowhere"))


def test_sharded_folder(tmp_path):
    a, b = {"x": torch.ones(2)}, {"y": torch.zeros(3)}
    save_file(a, str(tmp_path / "s1.safetensors"))
    save_file(b, str(tmp_path / "s2.safetensors"))
    (tmp_path / "model.safetensors.index.json").write_text(
        json.dumps({"weight_map": {"x": "s1.safetensors", "y": "s2.safetensors"}}))
    f = ModelFolder(str(tmp_path))
    assert f.names() == ["x", "y"] and torch.equal(f.load("y"), b["y"]) and "x" in f and "z" not in f


def test_random_model_folder_loads_and_is_seeded(tmp_path):
    d1 = write_random_model(str(tmp_path / "m1"), TINY_B, seed=5)
    d2 = write_random_model(str(tmp_path / "m2"), TINY_B, seed=5)
    d3 = write_random_model(str(tmp_path / "m3"), TINY_B, seed=6)
    exp = expected_tensors(spec_of(TINY_B))
    w1, w2, w3 = load_checked(d1, exp), load_checked(d2, exp), load_checked(d3, exp)
    assert set(w1) == set(exp)                                    # untied: lm_head.weight is written
    assert all(torch.equal(w1[n], w2[n]) for n in w1) and not torch.equal(w1["lm_head.weight"], w3["lm_head.weight"])
    assert w1["model.norm.weight"].dtype == torch.bfloat16
    q = w1["model.layers.1.self_attn.q_proj.weight"].float()
    assert abs(q.std().item() - 0.02) < 0.004 and abs(w1["model.norm.weight"].float().mean().item() - 1.0) < 0.1
    assert json.load(open(os.path.join(d1, "config.json")))["num_hidden_layers"] == 3
    tied = write_random_model(str(tmp_path / "m4"), TINY_A, seed=0, dtype=torch.float32)
    wt = load_checked(tied, expected_tensors(spec_of(TINY_A)))
    assert "lm_head.weight" not in wt and wt["model.embed_tokens.weight"].dtype == torch.float32


def test_tensors_the_model_does_not_read_are_ignored_with_a_warning(tmp_path):
    """The reference looks tensors up by name and never lists the rest (src/safetensors.rs:157-174): a folder
    with a buffer of another kind beside the model's tensors loads; an expected tensor in such a format does not."""
    d = write_random_model(str(tmp_path / "m"), TINY_A, seed=0)
    f = ModelFolder(d)
    t = {n: f.load(n).clone() for n in f.names()}
    t["model.layers.1.self_attn.rotary_emb.inv_freq"] = torch.zeros(8, dtype=torch.float16)
    t["model.masked_bias"] = torch.zeros(3, dtype=torch.uint8)
    os.remove(os.path.join(d, "model.safetensors"))
    from safetensors.torch import save_file as st_save
    st_save(t, os.path.join(d, "model.safetensors"))
    exp = expected_tensors(spec_of(TINY_A))
    with pytest.warns(UserWarning, match="2 tensors that the model does not read are ignored.*masked_bias"):
        w = load_checked(d, exp)
    assert set(w) == set(exp) - {"lm_head.weight"}
    t["model.norm.weight"] = t["model.norm.weight"].to(torch.float16)
    st_save(t, os.path.join(d, "model.safetensors"))
    with pytest.raises(WeightsError, match=r"wrong dtype \(1\): model.norm.weight: stored as F16"):
        load_checked(d, exp)


def test_one_error_lists_missing_unexpected_and_misshapen(tmp_path):
    d = write_random_model(str(tmp_path / "m"), TINY_A, seed=0)
    f = ModelFolder(d)
    t = {n: f.load(n).clone() for n in f.names()}
    del t["model.layers.0.mlp.up_proj.weight"], t["model.norm.weight"]
    t["model.layers.1.self_attn.rotary_emb.inv_freq"] = torch.zeros(8)
    t["model.layers.1.self_attn.k_proj.weight"] = torch.zeros(16, 64, dtype=torch.bfloat16)
    t["model.layers.1.input_layernorm.weight"] = torch.zeros(64, dtype=torch.int32)
    os.remove(os.path.join(d, "model.safetensors"))
    save_file(t, os.path.join(d, "model.safetensors"))
    with pytest.raises(WeightsError) as e:
        load_checked(d, expected_tensors(spec_of(TINY_A)))
    msg = str(e.value)
    assert "missing (2)" in msg and "model.layers.0.mlp.up_proj.weight" in msg and "model.norm.weight" in msg
    assert "unexpected (1)" in msg and "rotary_emb.inv_freq" in msg
    assert "wrong shape (1)" in msg and "k_proj.weight: file has [16, 64], model wants [32, 64]" in msg
    assert "wrong dtype (1)" in msg and "input_layernorm" in msg
