"""Generation through the entry point (`Engine`), against the plain model: greedy and seeded temperature sampling,
chunked prompts, mixed steps, preemption, rejections. CPU cases run the plain kernel twins; `gpu` cases the HIP kernels.
Workloads: the two tiny configurations' own (3 prompts of 5/17/33 tokens with 16 greedy tokens; 4 prompts of
1/8/31/64 tokens with portions of 16 beside decode tokens and seeded sampling) and the reference's engine tests
(plugins/tests/test_engine.py:25-106)."""
from __future__ import annotations

import pytest
import torch

from holon_amd.cache import OutOfPages
from holon_amd.config import EngineConfig, SamplingParams
from tests import helpers as H
from tests.plain import sampling as S
from tests.plain.ops import TorchKernels
from tests.plain.qwen3 import PlainQwen3

DEVICES = [pytest.param("cpu", id="cpu-twin"), pytest.param("cuda", marks=pytest.mark.gpu, id="hip")]


@pytest.fixture(scope="module")
def folders(tmp_path_factory):
    root = tmp_path_factory.mktemp("engine-models")
    return {"A": H.make_folder(root / "A", H.CONFIG_A, 0), "B": H.make_folder(root / "B", H.CONFIG_B, 1, qk_gain=2.0),
            "Bu": H.make_folder(root / "Bu", H.CONFIG_B, 6, scale=3.0)}


def _engine(folder, device, **kw):
    from holon_amd.engine.engine import Engine
    kw.setdefault("dtype", "float32")
    return Engine(EngineConfig(model=str(folder), device=device, **kw),
                  kernels=TorchKernels() if device == "cpu" else None)


def _released(engine):
    """No request holds anything: every page is free or held by the prefix index alone."""
    engine.cache.check()
    cached = len(engine.cache.prefix.entries) if engine.cache.prefix is not None else 0
    return all(g.pool.free + cached == g.pool.usable for g in engine.cache.groups) and \
        engine.cache.free_slots == engine.cache.max_seqs


@pytest.mark.parametrize("device", DEVICES)
def test_greedy_generation_is_the_plain_model(folders, device):
    """Tiny A's workload: 3 requests of 5/17/33 tokens, 16 greedy tokens each, pages of 16."""
    plain = PlainQwen3(folders["Bu"])
    prompts = [H.random_ids(n, 384, 40 + n) for n in (5, 17, 33)]
    engine = _engine(folders["Bu"], device, page_size=16, max_seqs=3, max_model_len=64, max_step_tokens=64)
    out = engine.generate(prompts, SamplingParams(temperature=0.0, max_tokens=16, ignore_eos=True))
    assert out == [plain.greedy(p, 16) for p in prompts]
    assert len({tuple(o) for o in out}) == 3 and all(len(set(o)) > 2 for o in out)   # not a degenerate model
    assert _released(engine)
    # the reference's shape: short pages, few slots, a step budget that cuts prompts, requests that wait
    prompts = [H.random_ids(n, 384, 50 + n) for n in (3, 17, 8, 25)]
    engine = _engine(folders["Bu"], device, page_size=4, max_seqs=3, max_step_tokens=10, max_model_len=40)
    out = engine.generate(prompts, SamplingParams(temperature=0.0, max_tokens=12, ignore_eos=True))
    assert out == [plain.greedy(p, 12) for p in prompts]
    assert _released(engine)


@pytest.mark.parametrize("device", DEVICES)
def test_tied_tiny_model_greedy(folders, device):
    plain = PlainQwen3(folders["A"])
    prompts = [H.random_ids(n, 256, n) for n in (5, 17, 33)]
    engine = _engine(folders["A"], device, page_size=16, max_seqs=4, max_model_len=128)
    out = engine.generate(prompts, SamplingParams(temperature=0.0, max_tokens=16, ignore_eos=True))
    assert out == [plain.greedy(p, 16) for p in prompts]


def _plain_sampled(plain, prompt, n, seed, temperature, **filters):
    ids, out = list(prompt), []
    for _ in range(n):
        logits = plain.logits(ids)[-1]
        q = S.probs(logits, temperature, **filters)
        token = S.draw(q, S.uniform(seed, len(ids)), S.drawing_order(logits, temperature, **filters))
        out.append(token)
        ids.append(token)
    return out


@pytest.mark.parametrize("device", DEVICES)
def test_seeded_sampling_mixed_with_chunked_prompts(folders, device):
    """Tiny B's workload: prompts of 1/8/31/64 tokens, portions of 16 beside decode tokens, 24 tokens at temperature
    0.8 with a fixed seed, pages of 8. Every draw is the plain model's law at the plain uniform of (seed, position)."""
    plain = PlainQwen3(folders["B"])
    prompts = [H.random_ids(n, 384, 60 + n) for n in (1, 8, 31, 64)]
    engine = _engine(folders["B"], device, page_size=8, max_seqs=4, max_model_len=96, max_step_tokens=32,
                     chunk_with_decode=16)
    params = SamplingParams(temperature=0.8, max_tokens=24, ignore_eos=True, seed=1234)
    out = engine.generate(prompts, params)
    assert out == [_plain_sampled(plain, p, 24, 1234, 0.8) for p in prompts]
    assert engine.stats()["mixed_steps"] > 0
    assert _released(engine)
    filtered = SamplingParams(temperature=0.9, top_k=12, top_p=0.9, min_p=0.02, max_tokens=10, ignore_eos=True, seed=7)
    out = engine.generate(prompts[:2], filtered)
    assert out == [_plain_sampled(plain, p, 10, 7, 0.9, top_k=12, top_p=0.9, min_p=0.02) for p in prompts[:2]]


@pytest.mark.parametrize("device", DEVICES)
def test_preemption_changes_nothing(folders, device):
    prompts = [H.random_ids(n, 384, 70 + n) for n in (3, 17, 8, 25)]
    params = SamplingParams(temperature=1.0, top_k=50, seed=7, max_tokens=12, ignore_eos=True)
    shape = dict(page_size=4, max_seqs=3, max_step_tokens=10, max_model_len=40)
    roomy = _engine(folders["Bu"], device, **shape)
    want = roomy.generate(prompts, params)
    tight = _engine(folders["Bu"], device, cache_tokens=48, **shape)          # 12 pages
    assert tight.generate(prompts, params) == want
    assert tight.stats()["preemptions"] > 0 and roomy.stats()["preemptions"] == 0
    assert _released(tight)
    greedy = SamplingParams(temperature=0.0, max_tokens=12, ignore_eos=True)
    assert tight.generate(prompts, greedy) == roomy.generate(prompts, greedy)


@pytest.mark.parametrize("device", DEVICES)
def test_prompts_that_start_alike_share_their_cache_and_generate_the_same(folders, device):
    """Four prompts over one 37-token start, then the same four again, with sampling: every draw is still the plain
    model's at the plain uniform. The second round (and, within a round, every prompt admitted after the first has
    published) computes only what the cache does not hold; a tight pool evicts cached pages and preempts between."""
    plain = PlainQwen3(folders["Bu"])
    start = H.random_ids(37, 384, 90)
    prompts = [start + H.random_ids(n, 384, 91 + n) for n in (1, 6, 12, 3)] + [start[:33]]
    params = SamplingParams(temperature=0.7, seed=11, max_tokens=10, ignore_eos=True)
    want = [_plain_sampled(plain, p, 10, 11, 0.7) for p in prompts]
    shape = dict(page_size=4, max_seqs=3, max_step_tokens=24, max_model_len=64)
    engine = _engine(folders["Bu"], device, **shape)
    assert engine.generate(prompts, params) == want
    first = engine.stats()["prefix_tokens_saved"]
    assert first >= 36                                     # the third and later prompts were admitted after a publish
    assert engine.generate(prompts, params) == want
    assert engine.stats()["prefix_tokens_saved"] - first >= 4 * 36 + 32      # all but a tail of every prompt
    assert _released(engine)
    two = engine.generate([prompts[1], prompts[1]], params)                 # the same prompt twice, side by side
    assert two == [want[1], want[1]]
    off = _engine(folders["Bu"], device, prefix_cache=False, **shape)
    assert off.generate(prompts, params) == want and off.stats()["prefix_tokens_saved"] == 0
    tight = _engine(folders["Bu"], device, cache_tokens=72, **shape)        # 18 pages: one request of 64, little more
    assert tight.generate(prompts, params) == want
    assert tight.generate(prompts[::-1], params) == want[::-1]
    assert tight.cache.prefix.evictions > 0 and tight.stats()["preemptions"] > 0
    assert _released(tight)
    tight.flush_prefix()
    assert all(g.pool.free == g.pool.usable for g in tight.cache.groups)
    assert tight.generate(prompts[:2], params) == want[:2]


@pytest.mark.parametrize("device,seed", [pytest.param("cpu", s, id=f"cpu-twin-{s}") for s in range(6)] +
                         [pytest.param("cuda", s, marks=pytest.mark.gpu, id=f"hip-{s}") for s in range(4)])
def test_random_traffic_generates_what_the_plain_model_generates(folders, device, seed):
    """Requests arrive while others run: prompts that share starts, pools so tight that cached pages are evicted and
    requests preempted, portions beside decode rows or not, several sequences of a prompt. Every sequence is the
    plain model's, drawn at the plain uniforms, whatever happened to it on the way. On the GPU the steps really
    overlap: a step is launched while the one before it still runs, and pages freed by a request that just finished
    are written by the next."""
    import random
    rng = random.Random(seed)
    plain = PlainQwen3(folders["Bu"])
    page = rng.choice([4, 8])
    max_len = 64
    mixed = rng.choice([0, 6])
    engine = _engine(folders["Bu"], device, page_size=page, max_seqs=rng.choice([2, 3, 5]), max_model_len=max_len,
                     max_step_tokens=rng.choice([16, 24]), chunk_with_decode=mixed,
                     cache_tokens=rng.choice([64, 96, 160]), prefix_cache=rng.random() < 0.8,
                     overlap=rng.random() < 0.7)
    starts = [H.random_ids(40, 384, 1000 * seed + i) for i in range(2)]
    todo = []
    for i in range(10):
        cut = rng.randrange(0, 30)
        prompt = rng.choice(starts)[:cut] + H.random_ids(rng.randrange(1, 12), 384, 2000 * seed + i)
        greedy = rng.random() < 0.4
        params = SamplingParams(temperature=0.0 if greedy else 0.9, seed=50 + i, ignore_eos=True,
                                max_tokens=rng.randrange(1, 14), n=1 if greedy else rng.choice([1, 1, 2]),
                                top_k=rng.choice([0, 0, 20]))
        todo.append((f"r{i}", prompt, params))
    want = {}
    for rid, prompt, p in todo:
        for i in range(p.n):
            want[rid, i] = plain.greedy(prompt, p.max_tokens) if p.greedy else \
                _plain_sampled(plain, prompt, p.max_tokens, S.sequence_seed(p.seed, i), p.temperature, top_k=p.top_k)
    got = {key: [] for key in want}
    done = set()
    pending = list(todo)
    for _ in range(3000):
        while pending and rng.random() < 0.3:
            rid, prompt, p = pending.pop(0)
            engine.add(prompt, p, rid=rid)
        if not engine.has_work():
            if not pending:
                break
            continue
        for d in engine.step():
            got[d.rid, d.index] += d.token_ids
            if d.finish_reason:
                assert d.finish_reason == "length" and (d.rid, d.index) not in done
                done.add((d.rid, d.index))
        engine.cache.check()
    assert done == set(want) and got == want
    assert _released(engine)


@pytest.mark.parametrize("device,seed", [pytest.param("cpu", s, id=f"cpu-twin-{s}") for s in range(3)] +
                         [pytest.param("cuda", s, marks=pytest.mark.gpu, id=f"hip-{s}") for s in range(2)])
def test_random_traffic_with_aborts(folders, device, seed):
    """The same traffic with requests aborted at random moments (waiting, in a prompt, decoding, with a step in
    flight): what an aborted request gave until then is the plain model's, the others never notice, and every page
    and slot comes back."""
    import random
    rng = random.Random(10_000 + seed)
    plain = PlainQwen3(folders["Bu"])
    engine = _engine(folders["Bu"], device, page_size=rng.choice([4, 8]), max_seqs=rng.choice([2, 3, 5]), max_model_len=64,
                     max_step_tokens=rng.choice([16, 24]), chunk_with_decode=rng.choice([0, 6]),
                     cache_tokens=rng.choice([64, 96, 160]), prefix_cache=rng.random() < 0.8, overlap=rng.random() < 0.7)
    starts = [H.random_ids(40, 384, 1000 * seed + i) for i in range(2)]
    todo = {}
    for i in range(12):
        prompt = rng.choice(starts)[:rng.randrange(0, 30)] + H.random_ids(rng.randrange(1, 12), 384, 2000 * seed + i)
        greedy = rng.random() < 0.4
        todo[f"r{i}"] = (prompt, SamplingParams(temperature=0.0 if greedy else 0.9, seed=50 + i, ignore_eos=True,
                                                max_tokens=rng.randrange(1, 14), n=1 if greedy else rng.choice([1, 1, 2]),
                                                top_k=rng.choice([0, 0, 20])))
    want = {}
    for rid, (prompt, p) in todo.items():
        for i in range(p.n):
            want[rid, i] = plain.greedy(prompt, p.max_tokens) if p.greedy else \
                _plain_sampled(plain, prompt, p.max_tokens, S.sequence_seed(p.seed, i), p.temperature, top_k=p.top_k)
    got = {key: [] for key in want}
    done, aborted, added = set(), set(), []
    pending = list(todo)
    for _ in range(3000):
        while pending and rng.random() < 0.3:
            rid = pending.pop(0)
            engine.add(todo[rid][0], todo[rid][1], rid=rid)
            added.append(rid)
        if added and rng.random() < 0.08:
            rid = rng.choice(added)
            if rid not in aborted and not all((rid, i) in done for i in range(todo[rid][1].n)):
                engine.abort(rid)
                aborted.add(rid)
        if not engine.has_work():
            if not pending:
                break
            continue
        for d in engine.step():
            assert d.rid not in aborted, "a delta of an aborted request"
            got[d.rid, d.index] += d.token_ids
            if d.finish_reason:
                assert d.finish_reason == "length" and (d.rid, d.index) not in done
                done.add((d.rid, d.index))
        engine.cache.check()
    assert aborted, "the seed aborts nothing"
    for (rid, i), tokens in got.items():
        if rid in aborted:
            assert tokens == want[rid, i][: len(tokens)]
        else:
            assert tokens == want[rid, i] and (rid, i) in done
    assert _released(engine)


@pytest.mark.parametrize("device", DEVICES)
def test_a_step_in_flight_changes_no_token(folders, device):
    """With `overlap` a step is scheduled and launched before the one before it has been committed: a decode row
    takes its token from the device, a request that ends on an end-of-sequence token has one more row in flight (it
    is dropped), a preempted request waits for its token. The tokens are those of the engine that commits every step
    at once, and the plain model's."""
    plain = PlainQwen3(folders["Bu"])
    prompts = [H.random_ids(n, 384, 300 + n) for n in (3, 17, 8, 25, 12)]
    free = [plain.greedy(p, 12) for p in prompts]
    stops = tuple({f[5] for f in free})                       # every request stops on some token another one draws too
    params = SamplingParams(temperature=0.0, max_tokens=12, stop_token_ids=stops)
    want = []
    for f in free:
        cut = min(i for i, t in enumerate(f) if t in stops)
        want.append(f[: cut + 1])
    assert any(len(w) < 6 for w in want) or all(len(w) == 6 for w in want)
    shape = dict(page_size=4, max_seqs=3, max_step_tokens=10, max_model_len=40, cache_tokens=48)
    outs = {}
    for overlap in (True, False):
        engine = _engine(folders["Bu"], device, overlap=overlap, **shape)
        outs[overlap] = engine.generate(prompts, params)
        assert outs[overlap] == want, overlap
        assert _released(engine) and not engine.has_work()
        stats = engine.stats()
    lagging = _engine(folders["Bu"], device, overlap=True, **shape)
    rid = lagging.add(prompts[1], SamplingParams(temperature=0.0, max_tokens=4, ignore_eos=True))
    seen = []
    while lagging.has_work():
        seen.append([d.token_ids for d in lagging.step()])
    assert seen[0] == [] and sum(len(s) for s in seen) == 4     # the first step's token comes with the second step
    assert [t for s in seen for ts in s for t in ts] == plain.greedy(prompts[1], 4)


@pytest.mark.parametrize("device", DEVICES)
def test_rejections_and_limits(folders, device):
    engine = _engine(folders["Bu"], device, page_size=4, max_seqs=3, max_step_tokens=10, max_model_len=40)
    with pytest.raises(ValueError):
        engine.add([])
    with pytest.raises(ValueError):
        engine.add(list(range(40)))
    with pytest.raises(ValueError):
        engine.add([1, 2, 384])
    with pytest.raises(NotImplementedError):
        engine.add([1, 2], SamplingParams(repetition_penalty=1.1))
    with pytest.raises(OutOfPages):
        _engine(folders["Bu"], device, page_size=4, max_seqs=3, max_model_len=40, cache_tokens=36)
    out = engine.generate([H.random_ids(30, 384, 1)], SamplingParams(temperature=0.0, ignore_eos=True))
    assert len(out[0]) == 10                                                  # stops at max_model_len
    # stop tokens and abort
    first = engine.generate([[5, 6, 7]], SamplingParams(temperature=0.0, max_tokens=5, ignore_eos=True))[0]
    out = engine.generate([[5, 6, 7]], SamplingParams(temperature=0.0, max_tokens=5, stop_token_ids=(first[1],)))
    assert out[0] == first[: first.index(first[1]) + 1]
    rid = engine.add([1, 2, 3], SamplingParams(temperature=0.0, max_tokens=50))
    engine.step()
    assert [d.finish_reason for d in engine.abort(rid)] == ["abort"]
    assert not engine.has_work() and _released(engine)


@pytest.mark.gpu
def test_bfloat16_generation_stays_with_the_plain_model(folders):
    """In bfloat16 rounding may decide between two tokens whose logits nearly tie, and only there: every token the
    engine picks is the most likely one of the plain model run in bfloat16 on the same tokens, wherever that model's
    two best logits are further apart than a twentieth of the logits' spread. Most places are that clear."""
    plain16 = PlainQwen3(folders["Bu"], torch.bfloat16)
    prompts = [H.random_ids(n, 384, 40 + n) for n in (5, 17, 33)]
    engine = _engine(folders["Bu"], "cuda", dtype="bfloat16", page_size=16, max_seqs=3, max_model_len=64)
    out = engine.generate(prompts, SamplingParams(temperature=0.0, max_tokens=16, ignore_eos=True))
    held = sum(H.assert_greedy_follows(plain16, prompt, tokens) for prompt, tokens in zip(prompts, out))
    assert held >= 36, f"only {held} of 48 places were clear enough to hold the engine to"


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_graph_replays_equal_eager_steps(folders, dtype):
    """Decode steps replayed from HIP graphs give the tokens of eager steps, over many replays with the program's own
    eager work (prompt steps, sampling, host synchronisation) between them, while the batch shrinks through the
    buckets and pages are taken and given back."""
    prompts = [H.random_ids(n, 384, 80 + n) for n in (3, 17, 8, 25, 40, 1)]
    shape = dict(dtype=dtype, page_size=8, max_seqs=6, max_model_len=128, max_step_tokens=64)
    outs = {}
    for graphs in (False, True):
        engine = _engine(folders["Bu"], "cuda", graphs=graphs, **shape)
        rids = [engine.add(p, SamplingParams(temperature=0.0 if i % 2 else 0.7, seed=5, max_tokens=20 + 7 * i,
                                             ignore_eos=True)) for i, p in enumerate(prompts)]
        got = {r: [] for r in rids}
        while engine.has_work():
            for d in engine.step():
                got[d.rid].extend(d.token_ids)
        outs[graphs] = [got[r] for r in rids]
        assert _released(engine)
        if graphs:
            assert engine.runner.graph_replays > 20 and len(engine.runner.graphs) >= 3
    assert outs[True] == outs[False]


@pytest.mark.gpu
def test_command_line_generates_and_sizes_its_cache(folders):
    """`python -m holon_amd generate` on the GPU, the cache sized from free memory (no --cache-tokens)."""
    import subprocess
    import sys
    plain = PlainQwen3(folders["Bu"])
    prompts = [H.random_ids(n, 384, 90 + n) for n in (4, 11)]
    cmd = [sys.executable, "-m", "holon_amd", "generate", str(folders["Bu"]), "--dtype", "float32", "--max-tokens", "6",
           "--temperature", "0", "--ignore-eos", "--max-seqs", "2", "--max-model-len", "64", "--max-step-tokens", "32",
           "--stats"]
    for p in prompts:
        cmd += ["--prompt-ids", " ".join(map(str, p))]
    run = subprocess.run(cmd, capture_output=True, text=True, timeout=110)
    assert run.returncode == 0, run.stderr[-2000:]
    got = [[int(t) for t in line.split()] for line in run.stdout.strip().splitlines()]
    assert got == [plain.greedy(p, 6) for p in prompts]
    assert "for the cache" in run.stderr and '"preemptions": 0' in run.stderr


@pytest.mark.gpu
def test_command_line_takes_text_with_the_folders_tokenizer(folders, tmp_path):
    """`--prompt TEXT` is encoded with the folder's tokenizer.json and answered as text; `--n` sequences a prompt, one
    a line. The tokenizer is a word list made here ("w0" ... "w383"), so ids and words map one to one."""
    import shutil
    import subprocess
    import sys
    from tokenizers import Tokenizer, models, pre_tokenizers
    plain = PlainQwen3(folders["Bu"])
    folder = tmp_path / "with-tokenizer"
    shutil.copytree(folders["Bu"], folder)
    tok = Tokenizer(models.WordLevel({f"w{i}": i for i in range(384)}, unk_token="w0"))
    tok.pre_tokenizer = pre_tokenizers.WhitespaceSplit()
    tok.save(str(folder / "tokenizer.json"))
    prompt = H.random_ids(9, 384, 77)
    cmd = [sys.executable, "-m", "holon_amd", "generate", str(folder), "--dtype", "float32", "--max-tokens", "5",
           "--temperature", "0.8", "--seed", "3", "--n", "2", "--ignore-eos", "--max-seqs", "4", "--max-model-len", "64",
           "--cache-tokens", "256", "--prompt", " ".join(f"w{t}" for t in prompt), "--prompt-ids",
           " ".join(map(str, prompt))]
    run = subprocess.run(cmd, capture_output=True, text=True, timeout=110)
    assert run.returncode == 0, run.stderr[-2000:]
    want = [_plain_sampled(plain, prompt, 5, S.sequence_seed(3, i), 0.8) for i in range(2)]
    lines = run.stdout.strip().splitlines()
    assert lines[:2] == [" ".join(map(str, w)) for w in want]                 # the prompt given as ids, answered as ids
    assert lines[2:] == [" ".join(f"w{t}" for t in w) for w in want]          # the prompt given as text, as text
    missing = subprocess.run(cmd[:4] + [str(folders["Bu"]), "--prompt", "w1"], capture_output=True, text=True, timeout=110)
    assert missing.returncode != 0 and "tokenizer.json" in missing.stderr


def test_bench_refuses_more_than_one_gpu():
    import pathlib
    import subprocess
    import sys
    bench = pathlib.Path(__file__).resolve().parent.parent / "bench.py"
    run = subprocess.run([sys.executable, str(bench), "--gpus", "2"], capture_output=True, text=True, timeout=60)
    assert run.returncode == 2 and len(run.stdout.strip().splitlines()) == 1 and "one GPU" in run.stdout


@pytest.mark.parametrize("device", DEVICES)
def test_logprobs_of_generated_tokens(folders, device):
    plain = PlainQwen3(folders["Bu"])
    engine = _engine(folders["Bu"], device, page_size=8, max_seqs=2, max_model_len=64)
    prompt = H.random_ids(9, 384, 3)
    engine.add(prompt, SamplingParams(temperature=0.0, max_tokens=4, ignore_eos=True, logprobs=3), rid="a")
    engine.add(prompt[:5], SamplingParams(temperature=0.0, max_tokens=4, ignore_eos=True), rid="b")
    ids, got = list(prompt), []
    while engine.has_work():
        for d in engine.step():
            if d.rid == "b":
                assert d.logprobs is None
                continue
            want = plain.logits(ids)[-1].log_softmax(-1)
            top = want.topk(3)
            assert d.logprobs.top_ids == [top.indices.tolist()] and d.token_ids == [int(top.indices[0])]
            torch.testing.assert_close(torch.tensor(d.logprobs.top[0]), top.values, rtol=1e-4, atol=1e-4)
            torch.testing.assert_close(torch.tensor(d.logprobs.token), top.values[:1], rtol=1e-4, atol=1e-4)
            ids += d.token_ids
            got += d.token_ids
    assert len(got) == 4
    with pytest.raises(ValueError):
        engine.add(prompt, SamplingParams(logprobs=33))


@pytest.mark.parametrize("device", DEVICES)
def test_several_sequences_of_one_prompt_and_prompt_logprobs(folders, device):
    """`n` sequences of one prompt: sequence i draws with `sequence_seed(seed, i)`; with the prefix cache the siblings
    start from the first one's cached prompt. `prompt_logprobs`: every prompt token's log-probability given the tokens
    before it, with the first delta; such a request computes every position, in portions, also when it is preempted
    in its prompt and runs part of it again."""
    plain = PlainQwen3(folders["Bu"])
    prompt = H.random_ids(29, 384, 123)
    engine = _engine(folders["Bu"], device, page_size=4, max_seqs=4, max_step_tokens=10, max_model_len=48)
    params = SamplingParams(temperature=0.8, seed=5, n=3, max_tokens=6, ignore_eos=True, prompt_logprobs=2)
    rid = engine.add(prompt, params)
    out, first = {0: [], 1: [], 2: []}, {}
    while engine.has_work():
        for d in engine.step():
            assert d.rid == rid
            first.setdefault(d.index, d)
            assert (d.cached_tokens is None) == (d is not first[d.index])
            out[d.index] += d.token_ids
    assert out == {i: _plain_sampled(plain, prompt, 6, S.sequence_seed(5, i), 0.8) for i in range(3)}
    assert len({tuple(o) for o in out.values()}) == 3
    assert [first[i].cached_tokens for i in range(3)] == [0, 28, 28]        # 7 whole pages of the 29 tokens
    want = plain.logits(prompt)[:-1].log_softmax(-1)
    top = want.topk(2)
    lp = first[0].prompt_logprobs
    assert first[1].prompt_logprobs is None and len(lp.token) == 28
    assert lp.top_ids == top.indices.tolist()
    torch.testing.assert_close(torch.tensor(lp.top), top.values, rtol=1e-4, atol=1e-4)
    torch.testing.assert_close(torch.tensor(lp.token), want.gather(-1, torch.tensor(prompt[1:])[:, None])[:, 0],
                               rtol=1e-4, atol=1e-4)
    assert _released(engine)
    with pytest.raises(ValueError):
        engine.generate([prompt], params)
    with pytest.raises(ValueError):
        engine.add(prompt, SamplingParams(n=0))
    engine.add(prompt, params, rid="gone")
    engine.step()
    assert sorted(d.index for d in engine.abort("gone")) == [0, 1, 2] and not engine.has_work()
    assert engine.idle_for() is None and engine.drain() == [] and _released(engine)
    # preempted in its prompt: the older requests grow, the youngest gives way and later runs its prompt again
    tight = _engine(folders["Bu"], device, page_size=4, max_seqs=3, max_step_tokens=10, max_model_len=48,
                    cache_tokens=60, chunk_with_decode=6, prefix_cache=False)
    greedy = SamplingParams(temperature=0.0, max_tokens=14, ignore_eos=True)
    for n in (12, 9):
        tight.add(H.random_ids(n, 384, 130 + n), greedy)
    for _ in range(2):
        tight.step()
    tight.add(prompt, SamplingParams(temperature=0.0, max_tokens=3, ignore_eos=True, prompt_logprobs=0), rid="lp")
    got = None
    while tight.has_work():
        for d in tight.step():
            if d.rid == "lp" and d.prompt_logprobs is not None:
                got = d.prompt_logprobs
    assert tight.stats()["preemptions"] > 0
    assert got.top_ids == [[]] * 28
    torch.testing.assert_close(torch.tensor(got.token), want.gather(-1, torch.tensor(prompt[1:])[:, None])[:, 0],
                               rtol=1e-4, atol=1e-4)


@pytest.mark.parametrize("device", DEVICES)
def test_end_of_sequence_tokens_stop_a_request(folders, tmp_path, device):
    """eos_token_id of config.json and generation_config.json (an int or a list) ends a request with "stop" and the
    token is delivered; ignore_eos generates on."""
    import json
    import shutil
    plain = PlainQwen3(folders["Bu"])
    prompt = H.random_ids(7, 384, 21)
    free = plain.greedy(prompt, 8)
    folder = tmp_path / "with-eos"
    shutil.copytree(folders["Bu"], folder)
    cfg = json.loads((folder / "config.json").read_text())
    cfg["eos_token_id"] = free[2]
    (folder / "config.json").write_text(json.dumps(cfg))
    (folder / "generation_config.json").write_text(json.dumps({"eos_token_id": [free[2], free[5]]}))
    engine = _engine(folder, device, page_size=8, max_seqs=2, max_model_len=64)
    assert engine.eos == {free[2], free[5]}
    rid = engine.add(prompt, SamplingParams(temperature=0.0, max_tokens=8))
    deltas = []
    while engine.has_work():
        deltas += engine.step()
    assert [t for d in deltas for t in d.token_ids] == free[: free.index(free[2]) + 1]
    assert deltas[-1].finish_reason == "stop" and deltas[-1].rid == rid
    out = engine.generate([prompt], SamplingParams(temperature=0.0, max_tokens=8, ignore_eos=True))
    assert out == [free]
