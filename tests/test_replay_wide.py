"""The engine at the layer sizes of the measured model (hidden 4096, 32 query heads over 8 kv heads of 128, feed-forward
12288; two layers and a small vocabulary keep the plain model affordable): the kernels and launch shapes that the
measurements use (matrix-core attention in its three forms, the few-row weight-streaming product with its tiled
weights, the vendor product for prompts, graph replay) against the plain model, in float32 and bfloat16, for every
way of cutting. GPU only."""
from __future__ import annotations

import functools

import pytest
import torch

from tests import helpers as H
from tests.plain.qwen3 import PlainQwen3

pytestmark = pytest.mark.gpu
WIDE = {"architectures": ["Qwen3ForCausalLM"], "num_hidden_layers": 2, "hidden_size": 4096, "num_attention_heads": 32,
        "num_key_value_heads": 8, "head_dim": 128, "intermediate_size": 12288, "vocab_size": 4096, "rope_theta": 1e6,
        "rms_norm_eps": 1e-6, "tie_word_embeddings": False, "max_position_embeddings": 4096}
LENGTHS = (300, 130, 70, 45)


@pytest.fixture(scope="module")
def folder(tmp_path_factory):
    return H.make_folder(tmp_path_factory.mktemp("wide") / "m", WIDE, 11, qk_gain=2.0)


@functools.lru_cache(maxsize=None)
def _plain(folder: str, dtype: str) -> PlainQwen3:
    """The plain model's own functions, run on the GPU: at these widths the CPU needs minutes for them."""
    return PlainQwen3(folder, getattr(torch, dtype), device="cuda")


@functools.lru_cache(maxsize=None)
def _plain_logits(folder: str, dtype: str, ids: tuple[int, ...]) -> torch.Tensor:
    return _plain(folder, dtype).logits(list(ids)).cpu()


def _requests():
    return {f"r{i}": H.random_ids(n, WIDE["vocab_size"], 200 + i) for i, n in enumerate(LENGTHS)}


def _check(folder, dtype, requests, got, what):
    want = {r: _plain_logits(str(folder), "float32", tuple(ids)) for r, ids in requests.items()}
    g, w = H.gather(want, got)
    if dtype == "float32":
        H.assert_fp32_close(g, w, what)
    else:
        floor = {r: _plain_logits(str(folder), "bfloat16", tuple(ids)) for r, ids in requests.items()}
        _, f = H.gather(floor, got)
        H.assert_bf16_close(g, w, f, what)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_wide_layers_every_way_of_cutting(folder, dtype):
    from holon_amd.engine.loading import load_model
    from holon_amd.engine.replay import Replayer
    requests = _requests()
    mixed = H.trace_mixed(requests, 5, decode_tail=6, max_chunk=70)
    tokens = max(H.peak_live_tokens(mixed), 320)
    loaded = load_model(folder, device="cuda", dtype=dtype, page_size=16, max_seqs=4, max_model_len=512,
                        max_step_tokens=512, cache_tokens=tokens, graphs=True)
    rep = Replayer(loaded)
    block = loaded.model.blocks[0]                 # in bfloat16 the norms are folded into the products that read them
    assert block._mixer_defers == block._ffn_defers == (dtype == "bfloat16")
    got = H.run_trace(rep, H.trace_whole(requests))
    _check(folder, dtype, requests, got, f"wide {dtype} whole")
    got = H.run_trace(rep, H.trace_decode_tail("r0", requests["r0"], 32))          # the tail replays from graphs
    _check(folder, dtype, requests, got, f"wide {dtype} decode tail")
    assert loaded.runner.graph_replays >= 30
    got = H.run_trace(rep, H.trace_chunks("r0", requests["r0"], [70, 2, 33, 17, 100, 2]))
    _check(folder, dtype, requests, got, f"wide {dtype} portions")
    got = H.run_trace(rep, mixed)
    assert len(got) == sum(LENGTHS)
    _check(folder, dtype, requests, got, f"wide {dtype} mixed")
    rep.cache.check()
    assert all(g.pool.free == g.pool.usable for g in rep.cache.groups)


def test_portions_of_17_to_64_rows_with_some_rows_wanted_over_partial_sums(folder):
    """Prompt portions of 40, 17 and 64 rows of which a few rows' logits are wanted, with the output and down
    projections' products forced to come as partial sums over shares of K: the rows are then selected from the
    residual stream and from its pending term, the last down projection's shares, alike."""
    from holon_amd.engine.loading import load_model
    from holon_amd.engine.replay import Replayer
    ids = _requests()["r1"]                                           # 130 tokens
    loaded = load_model(folder, device="cuda", dtype="bfloat16", page_size=16, max_seqs=4, max_model_len=512,
                        max_step_tokens=512, cache_tokens=256, products="own")
    trace = H.Trace()
    trace.add([("r1", 0, ids[:40], [0, 39])])
    trace.add([("r1", 40, ids[40:57], [16])])
    trace.add([("r1", 57, ids[57:121], [3, 40, 63])])
    trace.add([("r1", 121, ids[121:], [len(ids) - 122])], end=["r1"])  # nine rows: the few-row kernels
    got = H.run_trace(Replayer(loaded), trace)
    assert len(got) == 7
    taken = loaded.kernels.plan.report()
    assert taken["parts:4096x4096:64"] == taken["parts:4096x12288:64"] == taken["parts:4096x12288:32"] == "parts", taken
    _check(folder, "bfloat16", {"r1": ids}, got, "wide bfloat16, some rows of portions over partial sums")


def _wide_batch_requests() -> dict[str, tuple[list[int], int]]:
    """64 requests as (token ids, prompt length): the rest of each is decoded one token a step, all together. The
    decode counts make the batch shrink 64 -> 45 -> 30 -> 20 -> 12 -> 7 (padded to 48, 32, 24, 16, 8); request `long` goes from 2,042 to 2,062 tokens
    (the longest row crosses 2,048 while 64 rows decode) and leaves after 20 steps; request `mid` goes from 990 to
    1,050, so that the longest row crosses 1,024 while 8 rows decode. Prompt lengths sit on and around page edges."""
    decodes = [60] * 6 + [8] * 19 + [14] * 15 + [20] * 9 + [26] * 8 + [32] * 5
    prompts = [1, 2, 15, 16, 17, 31, 32, 33, 47, 48, 49, 63, 64, 65, 100, 127, 128, 129, 255, 256, 257, 300]
    out = {}
    for i, d in enumerate(decodes):         # the first slots go to short requests that stay to the end: what a padding
        p = prompts[(7 * i) % len(prompts)]  # row wrongly wrote there would be one of their few keys
        out[f"s{i}"] = (H.random_ids(p + d, WIDE["vocab_size"], 1000 + i), p)
    out["long"] = (H.random_ids(2042 + 20, WIDE["vocab_size"], 900), 2042)
    out["mid"] = (H.random_ids(990 + 60, WIDE["vocab_size"], 901), 990)
    assert len(out) == 64
    return out


def _wide_batch_trace(requests: dict[str, tuple[list[int], int]], budget: int) -> H.Trace:
    """Prompts first, several to a step under `budget` tokens, their last logits wanted; then every live request's
    next token in one step, every row's logits wanted, until all are done."""
    t = H.Trace()
    entries, used = [], 0
    for rid, (ids, p) in requests.items():
        if used + p > budget:
            t.add(entries)
            entries, used = [], 0
        entries.append((rid, 0, ids[:p], [p - 1]))
        used += p
    t.add(entries)
    at = {rid: p for rid, (_, p) in requests.items()}
    while at:
        entries = [(rid, pos, [requests[rid][0][pos]], [0]) for rid, pos in at.items()]
        end = [rid for rid, pos in at.items() if pos + 1 == len(requests[rid][0])]
        t.add(entries, end)
        at = {rid: pos + 1 for rid, pos in at.items() if rid not in end}
    return t


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("products", ["own", "vendor"])
def test_sixty_four_rows_decode_together_from_graphs(folder, dtype, products):
    """Decode steps of 64 rows shrinking to 7, replayed from graphs of every batch bucket on the way (all but the
    first with padding rows) and of three length buckets (1,024, 2,048, 4,096): the products for more than 16 rows,
    the decode attention with 64 rows, the few-row kernels below. Once with the kernels of our own for 17 to 64 rows
    (the gated product shares the rows through LDS and reads the folded weights over rows normed without the norm's
    weight; the output and down projections split K over blocks and hand partial sums to the norm that adds them),
    once with the vendor library's products (the engine's `products` setting). Every row's logits in every step
    against the plain model."""
    from holon_amd.engine.loading import load_model
    from holon_amd.engine.replay import Replayer
    requests = _wide_batch_requests()
    trace = _wide_batch_trace(requests, 2304)
    loaded = load_model(folder, device="cuda", dtype=dtype, page_size=16, max_seqs=64, max_model_len=2304,
                        max_step_tokens=2304, cache_tokens=H.peak_live_tokens(trace), graphs=True, products=products)
    rep = Replayer(loaded)
    got = H.run_trace(rep, trace)
    assert len(got) == 64 + sum(len(ids) - p for ids, p in requests.values())
    keys = set(loaded.runner.graphs)
    assert {(64, 2048), (64, 4096), (48, 4096), (32, 4096), (24, 1024), (16, 1024), (8, 1024), (8, 2048)} <= keys, keys
    assert loaded.runner.graph_replays >= 40
    _check(folder, dtype, {rid: ids for rid, (ids, _) in requests.items()}, got, f"wide {dtype} 64 rows")
    rep.cache.check()
    assert all(g.pool.free == g.pool.usable for g in rep.cache.groups)
    if dtype == "bfloat16":
        taken = set(loaded.kernels.plan.report().values())
        assert taken <= ({"rows", "parts", "bf16"} if products == "own" else {"vendor", "bf16"}), loaded.kernels.plan.report()


def test_timed_choices_are_made_at_start_reported_and_repeatable_when_pinned(folder):
    """Mode `timed` times every product with a choice while the model is put together, in every row bucket the engine
    can reach, and never later; what each took is reported in the syntax pins are given in. Two further launches with
    those pins (whatever their mode) then compute a 64-row decode trace bit for bit alike."""
    from holon_amd.engine.loading import load_model
    from holon_amd.engine.replay import Replayer
    requests = {rid: v for rid, v in _wide_batch_requests().items() if rid not in ("long", "mid")}
    trace = _wide_batch_trace(requests, 2304)
    shape = dict(device="cuda", dtype="bfloat16", page_size=16, max_seqs=64, max_model_len=512, max_step_tokens=2304,
                 cache_tokens=H.peak_live_tokens(trace), graphs=True)
    timed = load_model(folder, products="timed", **shape)
    plan = timed.kernels.plan
    taken = plan.report()
    assert plan.seconds > 0 and not plan.resolving and set(plan.how.values()) == {"timed"}, plan.how
    for key in ("glu:24576x4096:32", "glu:24576x4096:64", "parts:4096x12288:32", "parts:4096x12288:64",
                "parts:4096x4096:64", "parts:4096x12288:128", "vendor:6144x4096:64"):
        assert key in taken or key.startswith("vendor:"), (key, taken)
    first = H.run_trace(Replayer(timed), trace)
    assert plan.report() == taken and set(plan.how.values()) == {"timed"}        # nothing was chosen inside a step
    del timed
    again = []
    for mode in ("own", "vendor"):
        loaded = load_model(folder, products=mode, product_pins=taken, **shape)
        again.append(H.run_trace(Replayer(loaded), trace))
        reached = loaded.kernels.plan.report()                                     # what the trace's steps came to
        assert reached and reached.items() <= taken.items(), (mode, reached)
        assert set(loaded.kernels.plan.how.values()) == {"pinned"}
        del loaded
    for key, row in first.items():
        assert torch.equal(row, again[0][key]) and torch.equal(row, again[1][key]), key
    _check(folder, "bfloat16", {rid: ids for rid, (ids, _) in requests.items()}, first, "wide bfloat16 timed products")


def test_a_hundred_rows_decode_together(folder):
    """Decode steps of 100 rows shrinking to 70 (graph buckets 128 and 96), the output and down projections' products
    as partial sums over shares of K, which serve up to 128 rows: every row's logits against the plain model."""
    from holon_amd.engine.loading import load_model
    from holon_amd.engine.replay import Replayer
    requests = {f"q{i}": (H.random_ids(1 + (5 * i) % 37 + (3 if i < 70 else 2), WIDE["vocab_size"], 1500 + i),
                          1 + (5 * i) % 37) for i in range(100)}          # 70 decode three tokens, 30 two
    trace = _wide_batch_trace(requests, 2304)
    loaded = load_model(folder, device="cuda", dtype="bfloat16", page_size=16, max_seqs=128, max_model_len=256,
                        max_step_tokens=2304, cache_tokens=H.peak_live_tokens(trace), graphs=True, products="own")
    rep = Replayer(loaded)
    got = H.run_trace(rep, trace)
    assert len(got) == 100 + 70 * 3 + 30 * 2
    assert {(128, 1024), (96, 1024)} <= set(loaded.runner.graphs), set(loaded.runner.graphs)
    assert loaded.kernels.plan.report()["parts:4096x12288:128"] == "parts"
    _check(folder, "bfloat16", {rid: ids for rid, (ids, _) in requests.items()}, got, "wide bfloat16 100 rows")
    rep.cache.check()


@pytest.mark.parametrize("products", ["timed", "own"])
def test_engine_at_the_wide_sizes_with_everything_on(folder, products):
    """The whole engine in bfloat16 at the measured layer sizes (matrix-core attention, the few-row products over
    tiled weights, the residual add and the gated form inside them). One step in flight changes no launch, so it must
    change no token, greedy or seeded. Graph replay shapes the decode attention for its length bucket (other splits
    of the keys, other roundings) and shared prefixes cut the prompts elsewhere, and 20 requests make steps of more
    than 16 rows (their products once as timing chooses, once in the kernels of our own): there the greedy tokens are
    held to the plain model's own greedy decoding in bfloat16."""
    from holon_amd.config import EngineConfig, SamplingParams
    from holon_amd.engine.engine import Engine
    start = H.random_ids(40, WIDE["vocab_size"], 300)
    prompts = [start[: 8 + 4 * (i % 9)] + H.random_ids(3 + 5 * i, WIDE["vocab_size"], 301 + i) for i in range(20)]
    shape = dict(model=str(folder), device="cuda", dtype="bfloat16", page_size=16, max_seqs=24, max_model_len=256,
                 max_step_tokens=256, cache_tokens=24 * 256, products=products)
    bare = Engine(EngineConfig(overlap=False, graphs=False, prefix_cache=False, **shape))
    if products == "timed":                  # the next engines take what this one's timings chose: pinned, repeatable
        assert bare.kernels.plan.seconds > 0 and set(bare.kernels.plan.how.values()) == {"timed"}
        shape["product_pins"] = bare.products()
    ahead = Engine(EngineConfig(overlap=True, graphs=False, prefix_cache=False, **shape))
    for params in (SamplingParams(temperature=0.0, max_tokens=24, ignore_eos=True),
                   SamplingParams(temperature=0.8, top_k=40, top_p=0.95, seed=5, max_tokens=24, ignore_eos=True)):
        assert ahead.generate(prompts, params) == bare.generate(prompts, params)
    full = Engine(EngineConfig(overlap=True, graphs=True, prefix_cache=True, **shape))
    plain = _plain(str(folder), "bfloat16")
    params = SamplingParams(temperature=0.0, max_tokens=12, ignore_eos=True)
    for _ in range(2):                                           # the second time the prompts come from the cache
        for prompt, got in zip(prompts, full.generate(prompts, params)):
            H.assert_greedy_follows(plain, prompt, got)
    assert full.cache.tokens_saved > 0 and full.stats()["graphs"] >= 1 and full.runner.graph_replays > 10
    how = {"timed": "pinned", "own": "own"}[products]
    assert full.stats()["products"].items() <= bare.products().items()           # (a rival's own form is not met again)
    assert set(full.kernels.plan.how.values()) == {how}, full.kernels.plan.how


def test_long_context_attention_kernels():
    """Matrix-core attention far beyond the other tests' lengths: a 512-token portion behind 16,384 cached tokens (the
    LDS-staged kernel), a 40-token portion behind 70,000 (past the LDS table: the direct kernel), decode rows at 32,767
    and 70,039 keys; and one key that carries all the weight at the far end of each."""
    from holon_amd.kernels import load_hip
    from tests.plain.ops import TorchKernels
    from tests.test_kernels_gpu import _paged_case
    hip, plain = load_hip(), TorchKernels()
    heads, kv_heads, head_dim, page = 8, 2, 128, 16
    for rows in ([(16384, 512)], [(70000, 40)], [(32766, 1), (70039, 1), (5, 1)]):
        q, pages, table, attn = _paged_case(rows, heads, kv_heads, head_dim, page, torch.bfloat16, seed=len(rows), max_seqs=4)
        for target in (0, rows[0][0] - 1):
            slot = int(attn.slots[0])
            unit, off = int(table[slot, target // page]), target % page
            kp = pages[:, 0].view(-1, kv_heads, page, head_dim)
            for h in range(heads):
                q[0, h] = kp[unit, h // (heads // kv_heads), off].float().mul(3.0).to(torch.bfloat16)
            want = plain.paged_attention(q.float(), pages.float(), table, attn, page, head_dim ** -0.5, 0)
            got = hip.paged_attention(q, pages, table, attn, page, head_dim ** -0.5, 0)
            assert H.op_budget_usage(got, want.double(), torch.bfloat16, head_dim + rows[0][0]) <= 1, (rows, target)
