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


def test_one_tensor_per_expert_fills_a_stacked_parameter(tmp_path):
    """A rule with `stack` sends tensor `...experts.{e}...` to slice e of a parameter [experts, ...]; a missing
    expert, one beyond the parameter and a wrong slice shape are all listed in the one error."""
    from holon_amd.engine.loading import build_from_spec
    from holon_amd.registry import register_part, unregister_part
    from holon_amd.spec import LayerSpec, ModelSpec, PartRef, in_order
    from holon_amd.weights.loader import checkpoint_names, load_weights, locate
    from tests.toy_parts import STACKED_RULES, StackedTopOne
    register_part("ffn", "test-stacked-top-one")(StackedTopOne)
    try:
        norm = PartRef("norm", "rmsnorm", eps=1e-6)
        mixer = PartRef("mixer", "gqa", heads=2, kv_heads=1, head_dim=8)
        layer = LayerSpec(PartRef("block", "prenorm"), mixer, PartRef("ffn", "test-stacked-top-one", inter=12, experts=3), norm)
        spec = ModelSpec(hidden=16, vocab=20, layers=(layer,), order=in_order(1), embed=PartRef("embed", "table"),
                         norm=norm, head=PartRef("head", "linear", tied=True), rules=STACKED_RULES)
        assert locate(STACKED_RULES, "model.layers.0.mlp.experts.2.down.weight") == ("layers.0.ffn.down", 2)
        assert checkpoint_names(STACKED_RULES, "layers.0.ffn.down", (3, 16, 12)) == [
            (f"model.layers.0.mlp.experts.{e}.down.weight", e) for e in range(3)]
        shape = dict(device=torch.device("cpu"), dtype=torch.float32, kernels=TorchKernels(), page_size=4, max_seqs=2,
                     max_model_len=16, max_step_tokens=16)
        model, _ = build_from_spec(spec, **shape)
        g = torch.Generator().manual_seed(0)
        tensors = {}
        for path, _, _, decl in model.named_params():
            for name, index in checkpoint_names(STACKED_RULES, path, decl.shape):
                tensors[name] = torch.randn(decl.shape if index is None else decl.shape[1:], generator=g)
        assert "model.layers.0.mlp.experts.1.gate_up.weight" in tensors and len(tensors) == 9 + 6
        folder = tmp_path / "stacked"
        folder.mkdir()
        save_file(tensors, str(folder / "model.safetensors"))
        load_weights(model, spec, folder, shape["device"], shape["dtype"])
        ffn = model.blocks[0].ffn
        for e in range(3):
            assert torch.equal(ffn.gate_up[e], tensors[f"model.layers.0.mlp.experts.{e}.gate_up.weight"])
            assert torch.equal(ffn.down[e], tensors[f"model.layers.0.mlp.experts.{e}.down.weight"])
        broken = dict(tensors)
        del broken["model.layers.0.mlp.experts.1.down.weight"]
        broken["model.layers.0.mlp.experts.3.down.weight"] = torch.zeros(16, 12)
        broken["model.layers.0.mlp.experts.0.gate_up.weight"] = torch.zeros(24, 15)
        save_file(broken, str(folder / "model.safetensors"))
        model, _ = build_from_spec(spec, **shape)
        with pytest.raises(WeightError) as err:
            load_weights(model, spec, folder, shape["device"], shape["dtype"])
        assert err.value.missing == ["model.layers.0.mlp.experts.1.down.weight"]
        assert err.value.unexpected == ["model.layers.0.mlp.experts.3.down.weight"]
        assert err.value.wrong_shape == [("model.layers.0.mlp.experts.0.gate_up.weight", (24, 15), (24, 16))]
    finally:
        unregister_part("ffn", "test-stacked-top-one")
