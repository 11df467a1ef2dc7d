"""The engine against the plain model at the shapes its measurements are quoted for. GPU only.

* the whole Qwen3-8B shape: 36 layers, vocabulary 151,936 (what 36 layers of rounding add up to, and the head over
  the full vocabulary);
* the layer sizes of Qwen3-32B (hidden 5120, 64 heads over 8 kv heads, feed-forward 25600: head groups of 8, widths that
  differ from heads x head_dim, the gated product in eight waves a block), two layers, with 32 and 64 rows decoded
  together from graphs;
* the layer sizes of Qwen3-4B (hidden 2560, feed-forward 9728, the head tied to an embedding of 151,936 rows), two layers;
* a narrow model at 16,400 and at 69,700 tokens: prompt portions of 4,096 tokens behind tens of thousands of cached ones,
  a decode tail from graphs across a length bucket's edge, and a block table past the 4,096 pages the LDS-staged
  attention kernels copy (the kernel that reads operands straight from the cache).

Each in float32 and bfloat16: every request whole, most of one with its last 32 tokens one by one, in portions of
changing size, and mixed with the others in a pool so small that pages are used again. Models of these sizes are not
written to folders: the engine draws its weights on the device (`random_config`), and the plain model is handed the
same tensors, drawn again from (seed, tensor name), under their checkpoint names. The assertion messages report the
distance from the plain float32 model as rms and as the largest element (relative to the logits' rms), the same for
the plain model run in bfloat16 (the rounding floor), and how often the most likely token agrees.
"""
from __future__ import annotations

import functools

import pytest
import torch

from tests import helpers as H
from tests.plain.qwen3 import PlainQwen3

pytestmark = pytest.mark.gpu

BASE = {"architectures": ["Qwen3ForCausalLM"], "head_dim": 128, "num_key_value_heads": 8, "rope_theta": 1e6,
        "rms_norm_eps": 1e-6, "max_position_embeddings": 40960}
SHAPES = {
    "8b": dict(BASE, num_hidden_layers=36, hidden_size=4096, num_attention_heads=32, intermediate_size=12288,
               vocab_size=151936, tie_word_embeddings=False),
    "32b-layers": dict(BASE, num_hidden_layers=2, hidden_size=5120, num_attention_heads=64, intermediate_size=25600,
                       vocab_size=4096, tie_word_embeddings=False),
    "4b-layers": dict(BASE, num_hidden_layers=2, hidden_size=2560, num_attention_heads=32, intermediate_size=9728,
                      vocab_size=151936, tie_word_embeddings=True),
    "narrow": dict(BASE, num_hidden_layers=2, hidden_size=256, num_attention_heads=2, num_key_value_heads=1,
                   intermediate_size=512, vocab_size=512, tie_word_embeddings=False, max_position_embeddings=131072),
}
SEED = {"8b": 21, "32b-layers": 22, "4b-layers": 23, "narrow": 24}
GAIN = {"8b": 1.0, "32b-layers": 2.0, "4b-layers": 2.0, "narrow": 2.5}      # q/k norm weights times this: peaked scores
LENGTHS = (300, 130, 70, 45)


def _sharpen(t: torch.Tensor, gain: float) -> torch.Tensor:
    return (t.float() * gain).bfloat16().to(t.dtype)


@functools.lru_cache(maxsize=2)
def _tensors(shape: str) -> dict[str, torch.Tensor]:
    """Every tensor of the shape's model under its checkpoint name, float32 on the GPU: drawn from (seed, name) as the
    engine's random weights are."""
    from holon_amd.weights.loader import checkpoint_names
    from holon_amd.weights.random_init import meta_model, random_tensor
    _, spec, model = meta_model(SHAPES[shape])
    out = {}
    for path, _, _, decl in model.named_params():
        for name, index in checkpoint_names(spec.rules, path, decl.shape):
            assert index is None
            t = random_tensor(name, decl, SEED[shape], "cuda")
            out[name] = _sharpen(t, GAIN[shape]) if name.endswith(("q_norm.weight", "k_norm.weight")) else t
    return out


@functools.lru_cache(maxsize=2)
def _plain(shape: str, dtype: str) -> PlainQwen3:
    return PlainQwen3.from_tensors(SHAPES[shape], _tensors(shape), getattr(torch, dtype))


@functools.lru_cache(maxsize=None)
def _plain_logits(shape: str, dtype: str, ids: tuple[int, ...], rows: tuple[int, ...] | None = None) -> torch.Tensor:
    logits = _plain(shape, dtype).logits(list(ids))
    return (logits if rows is None else logits[list(rows)]).cpu()


def _load(shape: str, dtype: str, **engine):
    """The engine over the shape's random weights, the q/k norm weights sharpened as the plain model's are."""
    from holon_amd.engine.loading import load_model
    loaded = load_model(f"random:{shape}", device="cuda", dtype=dtype, page_size=16, random_config=SHAPES[shape],
                        seed=SEED[shape], **engine)
    for block in loaded.model.blocks:
        for norm in (block.mixer.q_norm, block.mixer.k_norm):
            norm.weight.copy_(_sharpen(norm.weight, GAIN[shape]))
    return loaded


def closeness(got: torch.Tensor, want32: torch.Tensor, floor16: torch.Tensor | None) -> str:
    def top1(a, b):
        return (a.argmax(-1) == b.argmax(-1)).float().mean().item()
    text = (f"rms {H.rel_rms(got, want32):.3g}, max {H.max_over_rms(got, want32):.3g}, "
            f"top-1 agrees on {top1(got, want32):.4f} of {got.shape[0]} rows")
    if floor16 is not None:
        text += (f"; plain bfloat16: rms {H.rel_rms(floor16, want32):.3g}, max {H.max_over_rms(floor16, want32):.3g}, "
                 f"top-1 {top1(floor16, want32):.4f}")
    return text


def _check(shape, dtype, requests, got, what):
    want = {r: _plain_logits(shape, "float32", tuple(ids)) for r, ids in requests.items()}
    g, w = H.gather(want, got)
    floor = None
    if dtype == "bfloat16":
        _, floor = H.gather({r: _plain_logits(shape, "bfloat16", tuple(ids)) for r, ids in requests.items()}, got)
    report = f"{shape} {dtype} {what}: {closeness(g, w, floor)}"
    print(report)
    try:
        if dtype == "float32":
            H.assert_fp32_close(g, w, report)
        else:
            H.assert_bf16_close(g, w, floor, report)
            agree = (g.argmax(-1) == w.argmax(-1)).float().mean().item()
            floor_agree = (floor.argmax(-1) == w.argmax(-1)).float().mean().item()
            assert agree >= floor_agree - 0.03, report
    except AssertionError as e:
        raise AssertionError(f"{report}\n{e}") from None


def _requests(shape: str) -> dict[str, list[int]]:
    vocab = SHAPES[shape]["vocab_size"]
    return {f"r{i}": H.random_ids(n, vocab, 400 + i) for i, n in enumerate(LENGTHS)}


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("shape", ["8b", "32b-layers", "4b-layers"])
def test_every_way_of_cutting_at_the_measured_shapes(shape, dtype):
    from holon_amd.engine.replay import Replayer
    requests = _requests(shape)
    mixed = H.trace_mixed(requests, 7, decode_tail=6, max_chunk=70)
    tokens = max(H.peak_live_tokens(mixed), 320)
    loaded = _load(shape, dtype, max_seqs=4, max_model_len=512, max_step_tokens=512, cache_tokens=tokens, graphs=True)
    rep = Replayer(loaded)
    got = H.run_trace(rep, H.trace_whole(requests))
    _check(shape, dtype, requests, got, "whole")
    if dtype == "bfloat16":        # the prompts of 300 and 130 tokens took this package's product for the down projection
        taken, cfg = loaded.kernels.plan.report(), SHAPES[shape]
        for bucket in (256, 512):
            key = f"parts:{cfg['hidden_size']}x{cfg['intermediate_size']}:{bucket}"
            assert taken.get(key) == "parts", (key, taken)
    got = H.run_trace(rep, H.trace_decode_tail("r0", requests["r0"], 32))          # the tail replays from graphs
    _check(shape, dtype, requests, got, "decode tail")
    assert loaded.runner.graph_replays >= 30
    got = H.run_trace(rep, H.trace_chunks("r0", requests["r0"], [70, 2, 33, 17, 100, 2]))
    _check(shape, dtype, requests, got, "portions")
    got = H.run_trace(rep, mixed)
    assert len(got) == sum(LENGTHS)
    _check(shape, dtype, requests, got, "mixed")
    rep.cache.check()
    assert all(g.pool.free == g.pool.usable for g in rep.cache.groups)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_32_and_64_rows_decode_together_at_the_32b_layer_sizes(dtype):
    """64 requests decode together from graphs, the batch shrinking through the buckets of 64, 48, 32, 24, 16 and 8
    rows: the products of this package's own for 17 to 64 rows at these widths (the gated one in eight waves a block,
    the output and down projections in shares of K), the decode attention with head groups of 8."""
    from holon_amd.engine.replay import Replayer
    from tests.test_replay_wide import _wide_batch_requests, _wide_batch_trace
    requests = {rid: v for rid, v in _wide_batch_requests().items() if rid not in ("long", "mid")}
    trace = _wide_batch_trace(requests, 2304)
    loaded = _load("32b-layers", dtype, max_seqs=64, max_model_len=512, max_step_tokens=2304,
                   cache_tokens=H.peak_live_tokens(trace), graphs=True, products="own")
    rep = Replayer(loaded)
    got = H.run_trace(rep, trace)
    assert {(64, 1024), (48, 1024), (32, 1024), (24, 1024), (16, 1024), (8, 1024)} <= set(loaded.runner.graphs)
    assert loaded.runner.graph_replays >= 40
    if dtype == "bfloat16":
        taken = loaded.kernels.plan.report()
        assert taken["glu:51200x5120:64"] == "rows" and taken["parts:5120x25600:32"] == "parts", taken
    _check("32b-layers", dtype, {rid: ids for rid, (ids, _) in requests.items()}, got, "62 rows decoding together")
    rep.cache.check()


def _long_trace(ids: list[int], other: list[int], portion: int, tail: int, every: int = 509) -> H.Trace:
    """Request `long`: portions of `portion` tokens, then `tail` tokens one by one. Wanted: every `every`-th place and
    the last 40 of every portion, and every decoded token. Request `short` joins when the decoding starts, with a
    prompt of 8 tokens and then a token a step, so that the decode steps hold rows of unlike lengths."""
    t = H.Trace()
    head = len(ids) - tail
    for at in range(0, head, portion):
        n = min(portion, head - at)
        want = sorted(set(range(0, n, every)) | set(range(max(0, n - 40), n)))
        t.add([("long", at, ids[at: at + n], want)])
    for i, p in enumerate(range(head, len(ids))):
        entries = [("long", p, [ids[p]], [0])]
        if i == 0:
            entries.append(("short", 0, other[:8], [7]))
        elif 7 + i < len(other):
            entries.append(("short", 7 + i, [other[7 + i]], [0]))
        t.add(entries, end=["long", "short"] if p == len(ids) - 1 else [])
    return t


@pytest.mark.parametrize("dtype,length", [("float32", 16400), ("bfloat16", 16400), ("bfloat16", 69700)])
def test_long_contexts_in_portions_and_a_decode_tail_across_a_length_bucket(dtype, length):
    """A narrow model (2 query heads over 1 kv head of 128) far beyond the other tests' lengths. 16,400 tokens: four
    portions of 4,096 (the last three behind thousands of cached tokens), then 30 decoded tokens from graphs whose
    length bucket changes at 16,384. 69,700 tokens: the block table grows past the 4,096 pages that the LDS-staged
    attention kernels keep a copy of, and the last portions and decode rows (length bucket 131,072) run the kernels that
    do without. The q/k norm weights are sharpened so that single far keys carry weight; a second, short request
    shares the decode steps."""
    from holon_amd.engine.replay import Replayer
    ids = H.random_ids(length, SHAPES["narrow"]["vocab_size"], 500 + length)
    other = H.random_ids(40, SHAPES["narrow"]["vocab_size"], 501)
    tail = 30 if length < 65536 else 12
    trace = _long_trace(ids, other, 4096, tail)
    loaded = _load("narrow", dtype, max_seqs=4, max_model_len=length + 64, max_step_tokens=4096,
                   cache_tokens=length + 256, graphs=True)
    rep = Replayer(loaded)
    got = H.run_trace(rep, trace)
    keys = sorted(k for k in got if k[0] == "long")
    rows = tuple(p for _, p in keys)
    assert rows[-1] == length - 1 and len(rows) > 40 * (length // 4096)
    buckets = {k[1] for k in loaded.runner.graphs}
    assert buckets == ({16384, 32768} if length < 65536 else {131072}), buckets
    assert loaded.runner.graph_replays >= tail - 4
    short_keys = sorted(k for k in got if k[0] == "short")
    assert len(short_keys) == tail
    g = torch.stack([got[k] for k in keys + short_keys])
    both = lambda dt: torch.cat((_plain_logits("narrow", dt, tuple(ids), rows),
                                 _plain_logits("narrow", dt, tuple(other), tuple(p for _, p in short_keys))))
    w = both("float32")
    floor = both("bfloat16") if dtype == "bfloat16" else None
    report = f"narrow {dtype} {length} tokens: {closeness(g, w, floor)}"
    print(report)
    if dtype == "float32":
        H.assert_fp32_close(g, w, report)
    else:
        H.assert_bf16_close(g, w, floor, report)
    rep.cache.check()
    assert all(gr.pool.free == gr.pool.usable for gr in rep.cache.groups)
