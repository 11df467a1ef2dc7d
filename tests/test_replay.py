"""The engine against the plain model, through the step function: the same requests whole, with the last tokens one by
one, in portions of changing size, and mixed with other requests in a pool so small that pages are used again; in
float32 and in bfloat16. On the CPU the plain kernel twins stand in for the HIP kernels (this checks the cache, the
batch layout and the step function); the `gpu` cases run the HIP kernels."""
from __future__ import annotations

import functools

import pytest
import torch

from tests import helpers as H
from tests.plain.ops import TorchKernels
from tests.plain.qwen3 import PlainQwen3

DEVICES = [pytest.param("cpu", id="cpu-twin"), pytest.param("cuda", marks=pytest.mark.gpu, id="hip")]
DTYPES = ["float32", "bfloat16"]
MODELS = {"A": (H.CONFIG_A, 0, 1.0, 16), "B": (H.CONFIG_B, 1, 1.0, 8), "C": (H.CONFIG_C, 2, 1.0, 16),
          "A-sharp": (H.CONFIG_A, 3, 3.0, 16), "B-sharp": (H.CONFIG_B, 4, 2.5, 8), "C-sharp": (H.CONFIG_C, 5, 3.0, 32)}
LENGTHS = (40, 70, 33, 90, 50, 64, 21)


@pytest.fixture(scope="module")
def folders(tmp_path_factory):
    root = tmp_path_factory.mktemp("models")
    return {name: H.make_folder(root / name, cfg, seed, gain) for name, (cfg, seed, gain, _) in MODELS.items()}


@functools.lru_cache(maxsize=None)
def _plain(folder: str, dtype: str) -> PlainQwen3:
    return PlainQwen3(folder, getattr(torch, dtype))


@functools.lru_cache(maxsize=None)
def _plain_logits(folder: str, dtype: str, ids: tuple[int, ...]) -> torch.Tensor:
    return _plain(folder, dtype).logits(list(ids))


def _requests(name: str, lengths=LENGTHS) -> dict[str, list[int]]:
    vocab = MODELS[name][0]["vocab_size"]
    return {f"r{i}": H.random_ids(n, vocab, 100 + i) for i, n in enumerate(lengths)}


def _replayer(folder, name, device, dtype, cache_tokens, max_seqs=4, max_model_len=512):
    from holon_amd.engine.loading import load_model
    from holon_amd.engine.replay import Replayer
    loaded = load_model(folder, device=device, dtype=dtype, kernels=TorchKernels() if device == "cpu" else None,
                        page_size=MODELS[name][3], max_seqs=max_seqs, max_model_len=max_model_len,
                        max_step_tokens=max_model_len, cache_tokens=cache_tokens)
    return Replayer(loaded)


def _check(folder, dtype, requests, got, what):
    want = {r: _plain_logits(str(folder), "float32", tuple(ids)) for r, ids in requests.items()}
    g, w = H.gather(want, got)
    if dtype == "float32":
        H.assert_fp32_close(g, w, what)
    else:
        floor = {r: _plain_logits(str(folder), "bfloat16", tuple(ids)) for r, ids in requests.items()}
        _, f = H.gather(floor, got)
        H.assert_bf16_close(g, w, f, what)


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", list(MODELS))
def test_every_way_of_cutting(folders, name, dtype, device):
    folder, requests = folders[name], _requests(name)
    page = MODELS[name][3]
    # whole, one request at a time, in a pool that holds only the longest: pages are used again by each request
    rep = _replayer(folder, name, device, dtype, cache_tokens=-(-max(LENGTHS) // page) * page)
    got = H.run_trace(rep, H.trace_whole(requests))
    assert len(got) == sum(LENGTHS)
    _check(folder, dtype, requests, got, f"{name} {dtype} whole")
    rep.cache.check()
    # most of it in one step, the last 32 tokens one by one
    for rid in ("r1", "r3"):
        got = H.run_trace(rep, H.trace_decode_tail(rid, requests[rid], 32))
        _check(folder, dtype, requests, got, f"{name} {dtype} decode tail {rid}")
    # portions of changing size, down to two tokens, off the page edges
    for rid, sizes in (("r3", [7, 2, 13, 3, 2, 30, 5]), ("r1", [2, 2, 17, 16, 1 + page, 2])):
        got = H.run_trace(rep, H.trace_chunks(rid, requests[rid], sizes))
        assert len(got) == len(requests[rid])
        _check(folder, dtype, requests, got, f"{name} {dtype} portions {rid}")
    rep.cache.check()
    assert all(g.pool.free == g.pool.usable for g in rep.cache.groups)


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", ["A", "B", "C-sharp", "B-sharp"])
def test_mixed_batches_in_a_tight_pool(folders, name, dtype, device):
    folder, requests = folders[name], _requests(name)
    for seed in (0, 1):
        trace = H.trace_mixed(requests, seed)
        tokens = H.peak_live_tokens(trace, 64)
        rep = _replayer(folder, name, device, dtype, cache_tokens=tokens)
        got = H.run_trace(rep, trace)
        assert len(got) == sum(LENGTHS)
        _check(folder, dtype, requests, got, f"{name} {dtype} mixed seed {seed}")
        rep.cache.check()
        assert all(g.pool.free == g.pool.usable for g in rep.cache.groups)
        assert rep.cache.free_slots == rep.cache.max_seqs


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", ["A", "B-sharp"])
def test_long_decoding_and_first_tokens(folders, name, dtype, device):
    folder = folders[name]
    vocab = MODELS[name][0]["vocab_size"]
    requests = {"long": H.random_ids(300, vocab, 7), "one": H.random_ids(1, vocab, 8), "two": H.random_ids(2, vocab, 9),
                "three": H.random_ids(3, vocab, 10)}
    rep = _replayer(folder, name, device, dtype, cache_tokens=320)
    trace = H.Trace()
    trace.add([("long", 0, requests["long"][:4], [0, 1, 2, 3])])
    for p in range(4, 300):                        # 296 single-token steps across many page edges
        trace.add([("long", p, [requests["long"][p]], [0])], end=["long"] if p == 299 else [])
    got = H.run_trace(rep, trace)
    _check(folder, dtype, {"long": requests["long"]}, got, f"{name} {dtype} long decoding")
    trace = H.Trace()                              # the first tokens of sequences: whole, and one by one from nothing
    trace.add([("one", 0, requests["one"], [0]), ("two", 0, requests["two"], [0, 1]),
               ("three", 0, requests["three"][:1], [0])], end=["one", "two"])
    trace.add([("three", 1, requests["three"][1:2], [0])])
    trace.add([("three", 2, requests["three"][2:3], [0])], end=["three"])
    got = H.run_trace(rep, trace)
    _check(folder, dtype, {k: requests[k] for k in ("one", "two", "three")}, got, f"{name} {dtype} first tokens")
    rep.cache.check()


@pytest.mark.parametrize("shares", [0, 2])
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", ["A", "B-sharp"])
def test_norms_folded_into_the_products_that_read_them(folders, name, dtype, shares):
    """Steps of few rows fold each block's norms into the q/k/v and the gate/up products (weights times the norm's
    weight, rows scaled by the norm's factor from statistics the kernel before left). On the CPU the kernel twin
    stands in for that path: the parts' logic of deferring a norm, passing the rows' statistics along the residual
    stream and falling back for portions of more than 16 rows is what runs here. Same logits, every way of cutting.
    With `shares`, steps of 17 to 64 rows also get the products that are added to the residual stream (output and
    down projection) as partial sums over shares of K, which the next norm's add, or the final one, takes as they
    are."""
    from holon_amd.engine.loading import load_model
    from holon_amd.engine.replay import Replayer
    folder, requests = folders[name], _requests(name)
    kernels = TorchKernels()
    kernels.fold_norms = True
    kernels.split_products = shares
    taken = []
    if shares:
        plain_add = kernels.add_rmsnorm
        kernels.add_rmsnorm = lambda x, residual, w, eps: (taken.append(x.dim() - residual.dim()), plain_add(x, residual, w, eps))[1]
    loaded = load_model(folder, device="cpu", dtype=dtype, kernels=kernels, page_size=MODELS[name][3], max_seqs=4,
                        max_model_len=512, max_step_tokens=512, cache_tokens=256)
    block = loaded.model.blocks[0]
    assert block._mixer_defers and block._ffn_defers and block.mixer.qkv.folded is block.input_norm
    rep = Replayer(loaded)
    got = H.run_trace(rep, H.trace_decode_tail("r1", requests["r1"], 40))         # 30 rows whole, then one by one
    _check(folder, dtype, requests, got, f"{name} {dtype} folded norms, decode tail")
    got = H.run_trace(rep, H.trace_chunks("r3", requests["r3"], [7, 2, 13, 16, 17, 30, 5]))
    _check(folder, dtype, requests, got, f"{name} {dtype} folded norms, portions")
    got = H.run_trace(rep, H.trace_mixed(requests, 2))
    _check(folder, dtype, requests, got, f"{name} {dtype} folded norms, mixed")
    some = H.Trace()                               # a portion of which only some rows are wanted: rows are selected from
    ids = requests["r1"]                           # the stream and from its pending term alike
    some.add([("r1", 0, ids[:33], [3, 32])], end=["r1"])
    _check(folder, dtype, requests, H.run_trace(rep, some), f"{name} {dtype} folded norms, some rows of a portion")
    assert not shares or 1 in taken, taken                        # terms went through the norms' adds as partial sums


@pytest.mark.parametrize("device", DEVICES)
def test_logits_do_not_depend_on_the_cut_in_float32(folders, device):
    """Beyond the comparison with the plain model: the same position computed whole, in portions and one by one
    agrees within the same float32 budget as the comparison with the plain model."""
    folder, name = folders["B-sharp"], "B-sharp"
    ids = _requests(name)["r3"]
    rep = _replayer(folder, name, device, "float32", cache_tokens=128)
    whole = H.run_trace(rep, H.trace_whole({"r3": ids}))
    parts = H.run_trace(rep, H.trace_chunks("r3", ids, [5, 2, 9, 24, 3]))
    tail = H.run_trace(rep, H.trace_decode_tail("r3", ids, 40))
    a = torch.stack([whole[k] for k in sorted(whole)])
    for other in (parts, tail):
        b = torch.stack([other[k] for k in sorted(whole)])
        H.assert_fp32_close(b, a, "cut independence")


@pytest.mark.gpu
@pytest.mark.parametrize("name", ["A", "B", "C-sharp"])
def test_float32_logits_are_bit_for_bit_the_same_however_they_are_cut(folders, name):
    """In 32-bit every sum of the engine is taken in an order that the position alone decides (the product's order
    depends on K alone, attention walks a query's keys from the first, norms work by row). So the logits at a
    position are the same bits whole, with the last tokens one by one (from graphs too), in portions of changing
    size, and mixed with other requests in a pool so small that pages are used again."""
    from holon_amd.engine.loading import load_model
    from holon_amd.engine.replay import Replayer
    folder, requests = folders[name], _requests(name)
    whole = H.run_trace(_replayer(folder, name, "cuda", "float32", cache_tokens=96), H.trace_whole(requests))

    def same(got, what):
        assert got.keys() <= whole.keys() and got
        bad = [k for k in got if not torch.equal(got[k], whole[k])]
        assert not bad, f"{name} {what}: {len(bad)} of {len(got)} positions differ in their bits, first {min(bad)}"
    for rid in ("r1", "r3"):
        rep = _replayer(folder, name, "cuda", "float32", cache_tokens=96)
        same(H.run_trace(rep, H.trace_decode_tail(rid, requests[rid], 32)), f"decode tail {rid}")
        same(H.run_trace(rep, H.trace_chunks(rid, requests[rid], [7, 2, 13, 3, 2, 30, 5])), f"portions {rid}")
    loaded = load_model(folder, device="cuda", dtype="float32", page_size=MODELS[name][3], max_seqs=4,
                        max_model_len=512, max_step_tokens=512, cache_tokens=96, graphs=True)
    same(H.run_trace(Replayer(loaded), H.trace_decode_tail("r3", requests["r3"], 40)), "decode tail from graphs")
    assert loaded.runner.graph_replays >= 30
    for seed in (0, 1):
        trace = H.trace_mixed(requests, seed)
        rep = _replayer(folder, name, "cuda", "float32", cache_tokens=H.peak_live_tokens(trace, 64))
        got = H.run_trace(rep, trace)
        assert len(got) == sum(LENGTHS)
        same(got, f"mixed seed {seed}")


@pytest.mark.gpu
@pytest.mark.parametrize("head_dim", [64, 80])
def test_float32_stays_within_its_budget_at_1700_tokens(tmp_path, head_dim):
    """A sharp model (q/k norm weights times 3) over a 1,700-token prompt, whole and in portions that end off the page
    edges: the 32-bit engine stays within the same budget of the plain 32-bit model as at 300 tokens. (Both are then
    about 7e-5 from the same formulas in float64: the rotation angle position * frequency is a float32 product in the
    reference's formula, 1e-4 rad off at these positions, and the engine and the plain model share it.)"""
    cfg = dict(H.CONFIG_C, head_dim=head_dim, max_position_embeddings=2048)
    folder = H.make_folder(tmp_path / "m", cfg, 21, qk_gain=3.0)
    ids = H.random_ids(1700, cfg["vocab_size"], 5)
    want = PlainQwen3(folder).logits(ids)
    from holon_amd.engine.loading import load_model
    from holon_amd.engine.replay import Replayer
    loaded = load_model(folder, device="cuda", dtype="float32", page_size=16, max_seqs=2, max_model_len=2048,
                        max_step_tokens=2048, cache_tokens=1712)
    rep = Replayer(loaded)
    whole = H.run_trace(rep, H.trace_whole({"r": ids}))
    H.assert_fp32_close(torch.stack([whole[("r", i)] for i in range(1700)]), want, f"1,700 tokens whole, head_dim {head_dim}")
    parts = H.run_trace(rep, H.trace_chunks("r", ids, [501, 2, 333, 700, 17]))
    assert all(torch.equal(parts[k], whole[k]) for k in whole)


@pytest.mark.gpu
@pytest.mark.parametrize("shape", [dict(hidden_size=1024, num_attention_heads=5, num_key_value_heads=1, head_dim=80,
                                        intermediate_size=520, vocab_size=1000, tie_word_embeddings=True),
                                   dict(hidden_size=200, num_attention_heads=4, num_key_value_heads=1, head_dim=32,
                                        intermediate_size=160, vocab_size=3001, tie_word_embeddings=False)])
def test_float32_is_as_near_the_formulas_as_the_plain_float32_model(tmp_path, shape):
    """Three sharp layers (q/k norm weights times 3) over 1,500 tokens amplify every rounding: there the plain model in
    float32 is itself 6e-5 to 1.5e-4 (rms) from the same formulas in float64, and two float32 evaluations that round
    in different orders differ by 1e-5 to 3e-5, past the budget that shallower models are held to. What can be asked
    of the engine is that it is no further from the float64 formulas than the plain float32 model is."""
    cfg = dict(H.CONFIG_C, num_hidden_layers=3, max_position_embeddings=2048, **shape)
    folder = H.make_folder(tmp_path / "m", cfg, 5055, qk_gain=3.0)
    ids = H.random_ids(1500, cfg["vocab_size"], 6)
    truth = PlainQwen3(folder, torch.float64).logits(ids)
    plain = PlainQwen3(folder).logits(ids).double()
    from holon_amd.engine.loading import load_model
    from holon_amd.engine.replay import Replayer
    loaded = load_model(folder, device="cuda", dtype="float32", page_size=16, max_seqs=2, max_model_len=2048,
                        max_step_tokens=2048, cache_tokens=1504)
    got = H.run_trace(Replayer(loaded), H.trace_whole({"r": ids}))
    engine = torch.stack([got[("r", i)] for i in range(1500)]).double().cpu()
    floor_rms, floor_max = H.rel_rms(plain, truth), H.max_over_rms(plain, truth)
    assert floor_rms > 5e-6                                           # the model does amplify: the floor is well above one rounding
    assert H.rel_rms(engine, truth) <= 1.25 * floor_rms + 1e-6, (H.rel_rms(engine, truth), floor_rms)
    assert H.max_over_rms(engine, truth) <= 1.25 * floor_max + 1e-5, (H.max_over_rms(engine, truth), floor_max)
    assert H.rel_rms(engine, plain) <= floor_rms                      # and nearer the plain model than either is to them


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", DTYPES)
def test_the_trace_run_program(folders, tmp_path, dtype):
    """bin/trace_run as a user runs it: steps on standard input, `done <step>` lines, logits files [wanted, vocab] as
    little-endian float32; a step that wants nothing writes no file."""
    import pathlib
    import subprocess
    import sys

    import numpy as np
    folder, name = folders["B-sharp"], "B-sharp"
    requests = _requests(name, (40, 70, 33, 90))
    trace = H.trace_mixed(requests, 3)
    trace.steps[2]["entries"][0]["want"] = []                  # one step computes without reporting
    dropped = trace.expect[2][: len(trace.steps[2]["entries"][0]["tokens"])]
    trace.expect[2] = trace.expect[2][len(dropped):]
    out = tmp_path / "out"
    program = pathlib.Path(__file__).resolve().parent.parent / "bin" / "trace_run"
    run = subprocess.run([sys.executable, str(program), "--model", str(folder), "--dtype", dtype, "--out", str(out),
                          "--max-tokens", str(H.peak_live_tokens(trace)), "--page-size", "8"],
                         input=trace.jsonl(), capture_output=True, text=True, timeout=110)
    assert run.returncode == 0, run.stderr[-2000:]
    assert run.stdout.split("\n")[:-1] == [f"done {i}" for i in range(len(trace.steps))]
    vocab = MODELS[name][0]["vocab_size"]
    got = {}
    for i, expect in enumerate(trace.expect):
        path = out / f"{i}.f32"
        assert path.exists() == bool(expect)
        if expect:
            rows = torch.from_numpy(np.fromfile(path, dtype="<f4").reshape(len(expect), vocab))
            got.update(zip(expect, rows))
    assert len(got) == sum(map(len, requests.values())) - len(dropped)
    _check(folder, dtype, requests, got, f"trace_run {dtype}")


def test_a_refused_step_leaves_nothing_behind(folders):
    """Steps that the step function refuses (no tokens, a wanted place beyond the tokens, a token outside the
    vocabulary, a request longer than the model length, a request twice in a step) raise, and a request that such a
    step brought holds neither a slot nor a page afterwards."""
    rep = _replayer(folders["A"], "A", "cpu", "float32", cache_tokens=128, max_model_len=128)
    assert rep.step([{"id": "a", "tokens": [1, 2, 3], "want": []}]) is None          # nothing wanted: no logits
    free = [g.pool.free for g in rep.cache.groups]
    for bad in ([{"id": "c", "tokens": [], "want": []}], [{"id": "c", "tokens": [1, 2], "want": [2]}],
                [{"id": "c", "tokens": [999], "want": [0]}], [{"id": "c", "tokens": [1] * 200, "want": [0]}],
                [{"id": "c", "tokens": [1, 2], "want": [0]}, {"id": "c", "tokens": [3], "want": [0]}]):
        with pytest.raises((ValueError, RuntimeError)):
            rep.step(bad)
        assert set(rep.slots) == {"a"} and [g.pool.free for g in rep.cache.groups] == free
        rep.cache.check()
    assert rep.step([{"id": "a", "tokens": [4], "want": [0]}], end=["a"]).shape == (1, 256)
    assert all(g.pool.free == g.pool.usable for g in rep.cache.groups) and rep.cache.free_slots == rep.cache.max_seqs
