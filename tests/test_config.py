"""Configuration, registry and command-line flags (no GPU)."""
from __future__ import annotations

import subprocess
import sys

import pytest

from holon_amd.config import ConfigError, EngineConfig, SamplingParams
from holon_amd.models.qwen3 import Qwen3Config
from holon_amd.registry import RegistryError, architectures, part_class, register_part, resolve, unregister_part
from holon_amd.spec import ModelSpec, PartRef, Run, WeightRule
from tests.helpers import CONFIG_A, CONFIG_B, CONFIG_C


def test_importing_the_configuration_imports_no_torch():
    code = "import sys, holon_amd.config, holon_amd.spec, holon_amd.registry; assert 'torch' not in sys.modules"
    subprocess.run([sys.executable, "-c", code], check=True)


def test_every_size_comes_from_config_json():
    a, b = Qwen3Config.from_dict(CONFIG_A), Qwen3Config.from_dict(CONFIG_B)
    assert (a.hidden_size, a.head_dim, a.num_key_value_heads, a.tie_word_embeddings, a.rope_theta) == (64, 16, 1, True, 1e4)
    assert (b.hidden_size, b.head_dim, b.num_key_value_heads, b.tie_word_embeddings, b.rms_norm_eps) == (96, 32, 3, False, 1e-5)
    assert Qwen3Config.from_dict(CONFIG_C).rope_theta == 50000.0            # the rope_parameters style of config
    for key in Qwen3Config.REQUIRED + ("rope_theta",):
        broken = {k: v for k, v in CONFIG_A.items() if k != key}
        with pytest.raises(ConfigError, match=key):
            Qwen3Config.from_dict(broken)
    assert Qwen3Config.from_dict(a.to_dict()) == a


def test_what_the_reference_refuses_is_refused():
    for extra in ({"attention_bias": True}, {"use_sliding_window": True}, {"rope_scaling": {"rope_type": "yarn", "factor": 4}},
                  {"rope_parameters": {"rope_theta": 1e6, "rope_type": "linear"}}):
        with pytest.raises(NotImplementedError):
            Qwen3Config.from_dict(CONFIG_A | extra)
    with pytest.raises(ConfigError):
        Qwen3Config.from_dict(CONFIG_A | {"num_key_value_heads": 3})
    with pytest.raises(ConfigError):
        Qwen3Config.from_dict(CONFIG_A | {"hidden_size": 0})
    ok = Qwen3Config.from_dict(CONFIG_A | {"use_sliding_window": False, "sliding_window": 4096, "hidden_act": "silu",
                                            "eos_token_id": 7}, {"eos_token_id": [7, 9]})
    assert ok.eos_token_ids == (7, 9)


def test_registry_maps_the_architecture_name_to_its_model():
    assert "Qwen3ForCausalLM" in architectures()
    cfg, spec = resolve(CONFIG_B)
    assert isinstance(cfg, Qwen3Config) and isinstance(spec, ModelSpec)
    assert len(spec.layers) == 3 and [r.layer for r in spec.order] == [0, 1, 2]
    mixer = spec.layers[0].mixer.get()
    assert (mixer["heads"], mixer["kv_heads"], mixer["head_dim"]) == (6, 3, 32)
    assert mixer["position"].get()["theta"] == 1e6 and mixer["qk_norm"].get()["eps"] == 1e-5
    assert spec.skip == () and resolve(CONFIG_A)[1].skip == ("lm_head.",)
    assert resolve(CONFIG_B)[1].identity() == spec.identity() != resolve(CONFIG_A)[1].identity()
    with pytest.raises(RegistryError, match="LlamaForCausalLM"):
        resolve(CONFIG_A | {"architectures": ["LlamaForCausalLM"]})
    with pytest.raises(RegistryError):
        part_class(PartRef("mixer", "no-such-mixer"))
    with pytest.raises(RegistryError):
        register_part("mixer", "gqa")(object)                 # a name is registered once
    register_part("ffn", "test-only")(object)
    assert part_class(PartRef("ffn", "test-only")) is object
    unregister_part("ffn", "test-only")


def test_the_run_order_is_checked():
    _, spec = resolve(CONFIG_A)
    import dataclasses
    dataclasses.replace(spec, order=(Run(0), Run(1), Run(0, reads=0), Run(1)))          # a layer twice, a shared cache
    for bad in ((Run(2),), (Run(0, reads=0),), (Run(0), Run(1, reads=0), Run(1, reads=1))):
        with pytest.raises(ValueError):
            dataclasses.replace(spec, order=bad)


def test_weight_rules():
    rule = WeightRule("model.layers.{i}.self_attn.{rest}", "layers.{i}.mixer.{rest}")
    m = rule.compile().match("model.layers.12.self_attn.q_proj.weight")
    assert m and rule.target.format(**m.groupdict()) == "layers.12.mixer.q_proj.weight"
    assert rule.compile().match("model.layers.x.self_attn.q_proj.weight") is None
    assert rule.compile().match("prefix.model.layers.1.self_attn.w") is None


def test_engine_config_and_sampling_params():
    with pytest.raises(ValueError):
        EngineConfig(model="m", page_size=0)
    with pytest.raises(ValueError):
        EngineConfig(model="m", dtype="float16")
    with pytest.raises(ValueError):
        EngineConfig(model="m", max_seqs=64, max_step_tokens=64, chunk_with_decode=16)
    SamplingParams().check()
    for bad in (SamplingParams(temperature=-1), SamplingParams(top_p=0), SamplingParams(top_k=-1), SamplingParams(max_tokens=0)):
        with pytest.raises(ValueError):
            bad.check()
    with pytest.raises(NotImplementedError):
        SamplingParams(presence_penalty=0.5).check()


def test_command_line_has_a_flag_per_engine_setting():
    import argparse
    import dataclasses

    from holon_amd.cli import engine_config, engine_flags
    ap = argparse.ArgumentParser()
    engine_flags(ap)
    a = ap.parse_args(["--dtype", "float32", "--page-size", "8", "--max-seqs", "3", "--no-graphs", "--chunk-with-decode", "0"])
    cfg = engine_config("folder", a)
    assert (cfg.model, cfg.dtype, cfg.page_size, cfg.max_seqs, cfg.graphs) == ("folder", "float32", 8, 3, False)
    assert not engine_config("folder", ap.parse_args(["--no-cuda-graphs"])).graphs     # the reference's name for the flag
    flags = {x.dest for x in ap._actions}
    assert {f.name for f in dataclasses.fields(EngineConfig)} - {"model"} <= flags
    out = subprocess.run([sys.executable, "-m", "holon_amd", "models"], capture_output=True, text=True, check=True)
    assert "Qwen3ForCausalLM" in out.stdout


def test_command_line_makes_engine_settings_and_takes_auto_for_the_context(tmp_path):
    """One flag a field of EngineConfig; `--max-model-len auto` is the model's trained context, at most 32,768."""
    import argparse
    import json
    from holon_amd import cli
    ap = argparse.ArgumentParser()
    cli.engine_flags(ap)
    (tmp_path / "config.json").write_text(json.dumps({"architectures": ["Qwen3ForCausalLM"],
                                                       "max_position_embeddings": 40960}))
    got = cli.engine_config(str(tmp_path), ap.parse_args(["--max-model-len", "auto", "--no-prefix-cache", "--page-size", "32"]))
    assert (got.max_model_len, got.prefix_cache, got.page_size, got.overlap) == (32768, False, 32, True)
    (tmp_path / "config.json").write_text(json.dumps({"architectures": ["Qwen3ForCausalLM"], "max_position_embeddings": 512}))
    assert cli.engine_config(str(tmp_path), ap.parse_args(["--max-model-len", "auto"])).max_model_len == 512
    assert cli.engine_config(str(tmp_path), ap.parse_args(["--max-model-len", "100"])).max_model_len == 100


def test_product_choices_resolve_pinned_then_by_mode_then_timed_at_start_only():
    """Which form a matrix product takes where several serve it: a pin wins, else the engine's mode; mode `timed`
    times once while the engine starts and falls back to this package's form, recorded as untimed, afterwards. The
    reference's order is pinned, preferred, priority (core/holon/core/build.py:89-106)."""
    import argparse

    from holon_amd import cli
    from holon_amd.config.products import ProductError, ProductPlan, key_of, row_bucket
    assert [row_bucket(r) for r in (17, 32, 33, 64, 65, 128, 129, 512, 513, 768, 769, 1000)] == \
        [32, 32, 64, 64, 128, 128, 256, 512, 768, 768, 1024, 1024]
    assert key_of("parts", (4096, 12288), 64) == "parts:4096x12288:64"
    calls = []

    def timer():
        calls.append(1)
        return "vendor"
    own = ProductPlan("own", {"parts:8x16:64": "vendor"})
    assert own.choose("parts", (8, 16), 64, timer) == "vendor" and own.how["parts:8x16:64"] == "pinned"
    assert own.choose("parts", (8, 16), 32, timer) == "parts" and own.choose("vendor", (8, 16), 32, timer) == "bf16"
    assert own.choose("glu", (8, 16), 32) == "rows" and not calls
    vendor = ProductPlan("vendor")
    assert [vendor.choose(k, (8, 16), 32, timer) for k in ("rows", "glu", "parts", "vendor")] == ["vendor"] * 3 + ["bf16"]
    timed = ProductPlan("timed", {"rows:8x16:32": "rows"})
    assert timed.choose("parts", (8, 16), 32, timer) == "parts" and timed.how["parts:8x16:32"] == "untimed" and not calls
    timed.resolving = True
    assert timed.choose("parts", (8, 16), 32, timer) == "parts" and not calls          # kept: one answer a key, for good
    assert timed.choose("parts", (8, 16), 64, timer) == "vendor" and calls == [1] and timed.how["parts:8x16:64"] == "timed"
    assert timed.choose("parts", (8, 16), 64, timer) == "vendor" and calls == [1]
    assert timed.choose("rows", (8, 16), 32, timer) == "rows" and calls == [1]          # pinned: not timed
    assert timed.report() == {"parts:8x16:32": "parts", "parts:8x16:64": "vendor", "rows:8x16:32": "rows"}
    assert ProductPlan("own", timed.report()).choose("parts", (8, 16), 64) == "vendor"   # a report is a set of pins
    timed.resolving = True
    with pytest.raises(ProductError, match="not one of"):
        timed.choose("vendor", (8, 16), 32, lambda: "rows")
    for bad in ({"parts:8x16": "parts"}, {"shares:8x16:32": "parts"}, {"parts:8x16:32": "f32"}, {"parts:ax16:32": "parts"}):
        with pytest.raises(ProductError):
            ProductPlan("own", bad)
    with pytest.raises(ProductError):
        ProductPlan("fastest")
    with pytest.raises(ValueError, match="products"):
        EngineConfig(model="m", products="fastest")
    with pytest.raises(ValueError):
        EngineConfig(model="m", product_pins={"parts:8x16:32": "rows"})
    ap = argparse.ArgumentParser()
    cli.engine_flags(ap)
    got = cli.engine_config("m", ap.parse_args(["--products", "timed", "--product-pins",
                                                "parts:8x16:32=vendor, vendor:8x16:512=f32x2"]))
    assert got.products == "timed" and got.product_pins == {"parts:8x16:32": "vendor", "vendor:8x16:512": "f32x2"}
