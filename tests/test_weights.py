"""The weight loader's errors and the random-weights mode (no GPU)."""
from __future__ import annotations

import json

import pytest
import torch
from safetensors import safe_open
from safetensors.torch import save_file

from holon_amd.engine.loading import load_model
from holon_amd.weights import WeightError, write_random_model
from tests.helpers import CONFIG_A, CONFIG_B
from tests.plain.ops import TorchKernels


def _tensors(folder):
    with safe_open(str(folder / "model.safetensors"), "pt") as f:
        return {k: f.get_tensor(k) for k in f.keys()}


def _load(folder, dtype="float32"):
    return load_model(folder, device="cpu", dtype=dtype, kernels=TorchKernels(), page_size=8, max_seqs=2,
                      max_model_len=64, cache_tokens=64)


def test_random_folder_is_seeded_and_typed(tmp_path):
    a = write_random_model(CONFIG_B, 1, tmp_path / "a")
    b = write_random_model(CONFIG_B, 1, tmp_path / "b")
    c = write_random_model(CONFIG_B, 2, tmp_path / "c")
    ta, tb, tc = _tensors(a), _tensors(b), _tensors(c)
    assert ta.keys() == tb.keys() and all(torch.equal(ta[k], tb[k]) for k in ta)
    assert not torch.equal(ta["lm_head.weight"], tc["lm_head.weight"])
    assert all(t.dtype == torch.bfloat16 for t in ta.values())
    assert json.loads((a / "config.json").read_text())["architectures"] == ["Qwen3ForCausalLM"]
    lin, norm = ta["model.layers.0.mlp.up_proj.weight"].float(), ta["model.layers.1.input_layernorm.weight"].float()
    assert abs(lin.std().item() - 0.02) < 0.002 and abs(lin.mean().item()) < 0.002
    assert abs(norm.mean().item() - 1) < 0.05 and 0.05 < norm.std().item() < 0.15
    assert "lm_head.weight" not in _tensors(write_random_model(CONFIG_A, 0, tmp_path / "tied"))
    f32 = _tensors(write_random_model(CONFIG_B, 1, tmp_path / "f32", torch.float32))
    assert all(t.dtype == torch.float32 for t in f32.values())
    assert torch.equal(f32["lm_head.weight"], ta["lm_head.weight"].float())      # the same bfloat16-exact values


def test_weights_are_kept_in_the_engine_dtype_and_merged(tmp_path):
    folder = write_random_model(CONFIG_B, 1, tmp_path / "m")
    t = _tensors(folder)
    for dtype in ("float32", "bfloat16"):
        model = _load(folder, dtype).model
        assert all(getattr(o, n).dtype == getattr(torch, dtype) for _, o, n, _ in model.named_params())
        mixer = model.blocks[0].mixer
        want = torch.cat([t[f"model.layers.0.self_attn.{p}_proj.weight"] for p in "qkv"]).to(getattr(torch, dtype))
        assert torch.equal(mixer.qkv.weight, want) and mixer.q_proj is None
        ffn = model.blocks[2].ffn
        assert ffn.gate_up.weight.shape == (320, 96) and ffn.gate_proj is None
        assert torch.equal(ffn.gate_up.weight[160:], t["model.layers.2.mlp.up_proj.weight"].to(getattr(torch, dtype)))
    tied = _load(write_random_model(CONFIG_A, 0, tmp_path / "tied")).model
    assert tied.lm_head.tied and "lm_head.weight" not in dict((p, 1) for p, *_ in tied.named_params())


def test_one_error_lists_missing_unexpected_and_wrong_shapes(tmp_path):
    folder = write_random_model(CONFIG_B, 1, tmp_path / "m")
    t = _tensors(folder)
    del t["model.layers.1.mlp.down_proj.weight"], t["model.norm.weight"]
    t["model.layers.0.self_attn.k_proj.weight"] = torch.zeros(96, 97, dtype=torch.bfloat16)
    t["model.layers.7.mlp.up_proj.weight"] = torch.zeros(2, 2)
    t["model.layers.0.self_attn.rotary.inv_freq"] = torch.zeros(4)
    t["something.else"] = torch.zeros(1)
    save_file(t, str(folder / "model.safetensors"))
    with pytest.raises(WeightError) as e:
        _load(folder)
    err = e.value
    assert err.missing == ["model.layers.1.mlp.down_proj.weight", "model.norm.weight"]
    assert err.unexpected == ["model.layers.0.self_attn.rotary.inv_freq", "model.layers.7.mlp.up_proj.weight", "something.else"]
    assert err.wrong_shape == [("model.layers.0.self_attn.k_proj.weight", (96, 97), (96, 96))]
    text = str(err)
    for piece in ("missing tensors (2)", "unexpected tensors (3)", "wrong shapes (1)", "[96, 97]", "[96, 96]", "something.else"):
        assert piece in text


def test_shards_and_other_errors(tmp_path):
    folder = write_random_model(CONFIG_B, 1, tmp_path / "m")
    t = _tensors(folder)
    names = sorted(t)
    (folder / "model.safetensors").unlink()
    save_file({k: t[k] for k in names[:10]}, str(folder / "model-00001-of-00002.safetensors"))
    save_file({k: t[k] for k in names[10:]}, str(folder / "model-00002-of-00002.safetensors"))
    assert _load(folder).model.norm.weight is not None                       # every shard is read
    save_file({k: t[k] for k in names[9:]}, str(folder / "model-00002-of-00002.safetensors"))
    with pytest.raises(WeightError, match="is in both"):
        _load(folder)
    tied = write_random_model(CONFIG_A, 0, tmp_path / "tied")
    tt = _tensors(tied)
    tt["lm_head.weight"] = torch.zeros(256, 64)                               # a tied model reads past a stored head
    save_file(tt, str(tied / "model.safetensors"))
    _load(tied)
    with pytest.raises(FileNotFoundError):
        _load(tmp_path / "nothing-here")
    (tmp_path / "empty").mkdir()
    (tmp_path / "empty" / "config.json").write_text(json.dumps(CONFIG_A))
    with pytest.raises(FileNotFoundError, match="safetensors"):
        _load(tmp_path / "empty")


def test_no_cpu_path_in_the_product(tmp_path):
    folder = write_random_model(CONFIG_A, 0, tmp_path / "m")
    with pytest.raises(RuntimeError, match="no CPU path"):
        load_model(folder, device="cpu", dtype="float32")
