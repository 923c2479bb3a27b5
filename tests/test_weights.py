"""Weights: the file format, loading by name, the one error that lists everything (no GPU)."""
import json
import struct

import numpy as np
import pytest
import torch

from flambeau_amd.models.decoder import DecoderModel
from flambeau_amd.registry import config_from_dict
from flambeau_amd.weights import (SafetensorsDir, SafetensorsFile, WeightError, WeightFileError,
                                  check_against_manifest, write_random_model, write_safetensors)
from tiny_configs import TINY, write_tiny


def _manifest(name):
    arch, cfg = config_from_dict(TINY[name]["config"])
    return DecoderModel(arch.build_spec(cfg), rt=None).manifest()


def test_written_file_is_read_by_the_safetensors_package(tmp_path):
    """The format is pinned by a second reader: the installed safetensors package."""
    from safetensors.torch import load_file
    for store in ("float32", "bfloat16"):
        d = write_tiny("A", tmp_path / store, store)
        theirs = load_file(str(d / "model.safetensors"))
        ours = SafetensorsFile(d / "model.safetensors")
        assert set(theirs) == set(ours.names())
        for n, t in theirs.items():
            mine = ours.read(n)
            assert mine.dtype == t.dtype and torch.equal(mine, t)
        ours.close()


def test_file_written_by_the_safetensors_package_is_read(tmp_path):
    from safetensors.torch import save_file
    t = {"a": torch.randn(3, 5), "b": torch.randn(7).to(torch.bfloat16), "c": torch.arange(6, dtype=torch.int32).reshape(2, 3)}
    save_file(t, str(tmp_path / "x.safetensors"))
    f = SafetensorsFile(tmp_path / "x.safetensors")
    for n in t:
        assert torch.equal(f.read(n), t[n])
    with pytest.raises(KeyError, match="no tensor named 'zzz'"):
        f.read("zzz")


def test_random_weights_are_seeded_and_have_the_stated_moments(tmp_path):
    a = write_tiny("B", tmp_path / "a", "float32")
    b = write_tiny("B", tmp_path / "b", "float32")
    fa, fb = SafetensorsFile(a / "model.safetensors"), SafetensorsFile(b / "model.safetensors")
    for n in fa.names():
        assert torch.equal(fa.read(n), fb.read(n))
    other = write_random_model(TINY["B"]["config"], tmp_path / "c", seed=99, std=0.05, gain_std=0.01,
                               store_dtype=torch.float32)
    fc = SafetensorsFile(other / "model.safetensors")
    assert not torch.equal(fa.read("lm_head.weight"), fc.read("lm_head.weight"))
    w = fa.read("model.embed_tokens.weight")
    assert abs(float(w.std()) - 0.05) < 0.003 and abs(float(w.mean())) < 0.002
    g = fa.read("model.layers.1.input_layernorm.weight")
    assert abs(float(g.mean()) - 1.0) < 0.01 and 0.003 < float(g.std()) < 0.02
    assert set(fa.names()) == set(_manifest("B"))
    assert json.loads((a / "config.json").read_text())["torch_dtype"] == "float32"


def test_tied_head_has_no_matrix_of_its_own():
    assert "lm_head.weight" not in _manifest("C") and "lm_head.weight" in _manifest("A")


def test_one_error_lists_missing_unexpected_and_wrong_shapes(tmp_path):
    d = write_tiny("A", tmp_path / "m", "float32")
    f = SafetensorsFile(d / "model.safetensors")
    t = {n: f.read(n) for n in f.names()}
    f.close()
    del t["model.layers.1.mlp.up_proj.weight"]
    del t["model.norm.weight"]
    t["model.layers.0.self_attn.rotary_emb.inv_freq"] = torch.zeros(8)
    t["model.layers.0.self_attn.q_proj.bias"] = torch.zeros(64)
    t["model.layers.0.self_attn.k_proj.weight"] = torch.zeros(16, 64)       # should be [32, 64]
    t["lm_head.weight"] = torch.zeros(64, 256)                              # transposed
    write_safetensors(d / "model.safetensors", t)
    src = SafetensorsDir(d)
    with pytest.raises(WeightError) as ei:
        check_against_manifest(_manifest("A"), src)
    e = ei.value
    assert e.missing == ["model.layers.1.mlp.up_proj.weight", "model.norm.weight"]
    assert e.unexpected == ["model.layers.0.self_attn.q_proj.bias", "model.layers.0.self_attn.rotary_emb.inv_freq"]
    # tensors the architecture says a file may hold without the model reading them are no error
    with pytest.warns(UserWarning, match="rotary_emb.inv_freq"), pytest.raises(WeightError) as ei:
        check_against_manifest(_manifest("A"), src, ignored=("*.rotary_emb.inv_freq",))
    assert ei.value.unexpected == ["model.layers.0.self_attn.q_proj.bias"]
    assert sorted(n for n, _, _ in e.wrong_shape) == ["lm_head.weight", "model.layers.0.self_attn.k_proj.weight"]
    msg = str(e)
    for piece in ("missing (2)", "unexpected (2)", "model.norm.weight", "rotary_emb.inv_freq",
                  "lm_head.weight is [64, 256], expected [256, 64]"):
        assert piece in msg


def test_vocab_size_must_match_the_table(tmp_path):
    d = write_tiny("A", tmp_path / "m", "float32")
    raw = dict(TINY["A"]["config"], vocab_size=250)
    arch, cfg = config_from_dict(raw)
    with pytest.raises(WeightError, match="model.embed_tokens.weight is \\[256, 64\\], expected \\[250, 64\\]"):
        check_against_manifest(DecoderModel(arch.build_spec(cfg), rt=None).manifest(), SafetensorsDir(d))


def test_integer_tensor_where_a_float_is_expected(tmp_path):
    d = write_tiny("A", tmp_path / "m", "float32")
    f = SafetensorsFile(d / "model.safetensors")
    t = {n: f.read(n) for n in f.names()}
    f.close()
    t["model.norm.weight"] = torch.ones(64, dtype=torch.int32)
    write_safetensors(d / "model.safetensors", t)
    with pytest.raises(WeightError, match="wrong dtype: model.norm.weight is I32"):
        check_against_manifest(_manifest("A"), SafetensorsDir(d))


def test_damaged_files_are_refused(tmp_path):
    d = write_tiny("A", tmp_path / "m", "float32")
    blob = (d / "model.safetensors").read_bytes()
    p = tmp_path / "cut.safetensors"
    p.write_bytes(blob[:len(blob) // 2])
    with pytest.raises(WeightFileError, match="truncated"):
        SafetensorsFile(p)
    p.write_bytes(blob[:4])
    with pytest.raises(WeightFileError, match="truncated"):
        SafetensorsFile(p)
    (hlen,) = struct.unpack("<Q", blob[:8])
    header = json.loads(blob[8:8 + hlen])
    names = [n for n in header if n != "__metadata__"]
    header[names[1]]["data_offsets"] = header[names[0]]["data_offsets"]
    header[names[1]]["shape"] = header[names[0]]["shape"]
    hb = json.dumps(header).encode()
    p.write_bytes(struct.pack("<Q", len(hb)) + hb + blob[8 + hlen:])
    with pytest.raises(WeightFileError, match="overlap"):
        SafetensorsFile(p)
    p.write_bytes(struct.pack("<Q", 5) + b"{oops" + b"\0" * 16)
    with pytest.raises(WeightFileError, match="JSON"):
        SafetensorsFile(p)
    with pytest.raises(WeightFileError, match="neither"):
        SafetensorsDir(tmp_path)


def test_sharded_folder(tmp_path):
    d = write_tiny("A", tmp_path / "m", "bfloat16")
    f = SafetensorsFile(d / "model.safetensors")
    names = f.names()
    half = len(names) // 2
    write_safetensors(d / "model-00001-of-00002.safetensors", {n: f.read(n) for n in names[:half]})
    write_safetensors(d / "model-00002-of-00002.safetensors", {n: f.read(n) for n in names[half:]})
    wm = {n: ("model-00001-of-00002.safetensors" if i < half else "model-00002-of-00002.safetensors")
          for i, n in enumerate(names)}
    (d / "model.safetensors.index.json").write_text(json.dumps({"weight_map": wm}))
    whole = {n: f.read(n) for n in names}
    f.close()
    (d / "model.safetensors").unlink()
    src = SafetensorsDir(d)
    check_against_manifest(_manifest("A"), src)
    for n in names:
        assert torch.equal(src.read(n), whole[n])


def test_random_weights_follow_what_a_tensor_says_of_itself():
    """By role a vector is a gain (1 + noise) and a matrix noise; a part whose vector is a bias, a
    decay rate or an integer table says so in its TensorSpec, and the defaults' values stay what they were."""
    import torch
    from flambeau_amd.parts import TensorSpec
    from flambeau_amd.weights.random_init import RandomSource

    def decay(generator, shape, device):
        return -torch.rand(shape, generator=generator, device=device) - 0.5

    def table(generator, shape, device):
        return torch.randint(0, 7, shape, generator=generator, device=device)
    manifest = {"gain": (0, "g", TensorSpec((64,), "vector32")), "matrix": (0, "m", TensorSpec((8, 16))),
                "bias": (0, "b", TensorSpec((64,), "vector32", init="normal")), "zero": (0, "z", TensorSpec((5,), "vector32", init="zeros")),
                "one": (0, "o", TensorSpec((5, 2), init="ones")), "decay": (0, "d", TensorSpec((32,), "vector32", init=decay)),
                "ids": (0, "i", TensorSpec((9,), "int32", init=table)), "bad": (0, "x", TensorSpec((3,), "int32"))}
    src = RandomSource(manifest, seed=4, std=0.05, gain_std=0.01, store_dtype=torch.float32)
    gain, bias = src.read("gain"), src.read("bias")
    assert abs(float(gain.mean()) - 1) < 0.01 and float(gain.std()) < 0.03
    assert abs(float(bias.mean())) < 0.03 and 0.02 < float(bias.std()) < 0.08
    assert float(src.read("zero").abs().max()) == 0 and torch.equal(src.read("one"), torch.ones(5, 2))
    d = src.read("decay")
    assert float(d.max()) <= -0.5 and float(d.min()) >= -1.5
    ids = src.read("ids")
    assert ids.dtype == torch.int32 and src.info("ids") == ((9,), "I32") and 0 <= int(ids.min()) and int(ids.max()) < 7
    with pytest.raises(ValueError, match="no rule for the integer table"):
        src.read("bad")
    # a tensor's values depend on the seed and its name alone
    again = RandomSource({"matrix": manifest["matrix"]}, seed=4, std=0.05, gain_std=0.5, store_dtype=torch.float32)
    assert torch.equal(again.read("matrix"), src.read("matrix"))
