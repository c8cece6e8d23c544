"""Weights: reading by name, the one error that lists everything wrong, random folders."""

import json

import pytest
import torch
from safetensors import safe_open
from safetensors.torch import save_file

from tiny_models import CONFIG_A, CONFIG_B
from tokasaurus_amd.models import architecture_of, build_model
from tokasaurus_amd.weights import WeightError, read_tensors, write_random_model


def _model(cfgd):
    arch = architecture_of(cfgd)
    return build_model(arch, arch.config_from_dict(cfgd))


def _all(folder):
    with safe_open(str(folder / "model.safetensors"), framework="pt") as f:
        return {k: f.get_tensor(k) for k in f.keys()}


def test_random_folder_round_trip_and_determinism(tmp_path):
    a = write_random_model(tmp_path / "a", CONFIG_B, seed=5)
    b = write_random_model(tmp_path / "b", CONFIG_B, seed=5)
    c = write_random_model(tmp_path / "c", CONFIG_B, seed=6)
    assert json.loads((a / "config.json").read_text()) == CONFIG_B
    ta, tb, tc = _all(a), _all(b), _all(c)
    assert ta.keys() == tb.keys() and all(torch.equal(ta[k], tb[k]) for k in ta)
    assert any(not torch.equal(ta[k], tc[k]) for k in ta)
    specs = _model(CONFIG_B).tensor_specs()
    got = read_tensors(a, specs)
    assert set(got) == {s.name for s in specs}
    assert all(t.dtype == torch.bfloat16 for t in got.values())  # stored and kept in bfloat16
    w = got["model.layers.1.mlp.up_proj.weight"].float()
    assert abs(float(w.std()) - 0.02) < 0.002 and abs(float(w.mean())) < 0.002
    n = got["model.layers.0.input_layernorm.weight"].float()
    assert abs(float(n.mean()) - 1.0) < 0.01 and 0.003 < float(n.std()) < 0.02


def test_tied_head_is_not_drawn_and_may_be_present(tmp_path):
    a = write_random_model(tmp_path / "a", CONFIG_A, seed=1)
    t = _all(a)
    assert "lm_head.weight" not in t
    t["lm_head.weight"] = t["model.embed_tokens.weight"].clone()
    save_file(t, str(a / "model.safetensors"))
    specs = _model(CONFIG_A).tensor_specs()
    with pytest.raises(WeightError, match="unexpected"):
        read_tensors(a, specs)
    assert "lm_head.weight" not in read_tensors(a, specs, allow_unexpected=("lm_head.weight",))


def test_one_error_lists_missing_unexpected_and_wrong_shapes(tmp_path):
    a = write_random_model(tmp_path / "a", CONFIG_B, seed=1)
    t = _all(a)
    del t["model.layers.2.mlp.down_proj.weight"], t["model.norm.weight"]
    t["model.layers.0.self_attn.q_proj.weight"] = torch.zeros(96, 95, dtype=torch.bfloat16)
    t["model.layers.7.extra.weight"] = torch.zeros(3, dtype=torch.bfloat16)
    save_file(t, str(a / "model.safetensors"))
    with pytest.raises(WeightError) as e:
        read_tensors(a, _model(CONFIG_B).tensor_specs())
    err = e.value
    assert err.missing == ["model.layers.2.mlp.down_proj.weight", "model.norm.weight"]
    assert err.unexpected == ["model.layers.7.extra.weight"]
    assert [(n, list(h), list(w)) for n, h, w in err.wrong_shape] == [
        ("model.layers.0.self_attn.q_proj.weight", [96, 95], [96, 96])]
    text = str(err)
    for piece in ("missing tensors (2)", "unexpected tensors (1)", "wrong shapes (1)", "has [96, 95], wanted [96, 96]"):
        assert piece in text


def test_sharded_checkpoint_and_no_checkpoint(tmp_path):
    a = write_random_model(tmp_path / "a", CONFIG_A, seed=2)
    t = _all(a)
    names = sorted(t)
    half = len(names) // 2
    (a / "model.safetensors").unlink()
    save_file({k: t[k] for k in names[:half]}, str(a / "model-00001-of-00002.safetensors"))
    save_file({k: t[k] for k in names[half:]}, str(a / "model-00002-of-00002.safetensors"))
    weight_map = {k: ("model-00001-of-00002.safetensors" if i < half else "model-00002-of-00002.safetensors")
                  for i, k in enumerate(names)}
    (a / "model.safetensors.index.json").write_text(json.dumps({"weight_map": weight_map}))
    got = read_tensors(a, _model(CONFIG_A).tensor_specs())
    assert all(torch.equal(got[k], t[k]) for k in t)
    (tmp_path / "empty").mkdir()
    with pytest.raises(FileNotFoundError):
        read_tensors(tmp_path / "empty", [])


def test_a_tensor_stored_in_32_bit_stays_so(tmp_path):
    a = write_random_model(tmp_path / "a", CONFIG_A, seed=2)
    t = _all(a)
    t["model.norm.weight"] = t["model.norm.weight"].float()
    save_file(t, str(a / "model.safetensors"))
    got = read_tensors(a, _model(CONFIG_A).tensor_specs())
    assert got["model.norm.weight"].dtype == torch.float32
    assert got["model.embed_tokens.weight"].dtype == torch.bfloat16
