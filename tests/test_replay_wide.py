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
def _plain_logits(folder: str, dtype: str, ids: tuple[int, ...]) -> torch.Tensor:
    return PlainQwen3(folder, getattr(torch, dtype)).logits(list(ids))


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
