"""Decode and prefill throughput of the engine at the Qwen3-8B shape with random weights, on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--batch 8] [--layers L] [--no-points]
    python -m holon_amd bench ...          (the same)

    python bench.py --workload mixed|long [--layers L]

One JSON line: decoded tokens a second at the given batch (default 8) with every request near a context of 4,096 tokens
(the far end of a 2,048-token prompt and 2,048 generated tokens: the requests are given prompts that leave just the
timed steps, `config.decode_prompt_len`), plus the prefill of one 2,048-token prompt (`prefill.ms` is the best of three
prompts, `prefill.ms_median` their median), the decode step's memory roofline, and `points`: decode at batch 1, 16, 32
and 64 at the same context and at batch 8 at a context of 32,768 (tokens a second, ms a step, the gigabytes a step
must read, the fraction of the memory roofline), and prompts of 512 and 8,192 tokens (tokens a second, best and median
ms, TFLOP, the fraction of the matrix peak; the longer one takes two steps under the step budget of 4,096 tokens).
`latency` holds the time to the first token of the 2,048-token prompt and the median time between two tokens of a
request, as the reference's driver reports them (bench/driver.py:102-134); `products` what every matrix product with
a choice of kernels took. A step is one decode step of the engine: scheduling, the model, sampling and the commit.
The engine is one process on one GPU; for --gpus > 1 a line says so and the exit code is 2.

--workload runs a whole job through the engine instead and prints its own line: `mixed` is 32 requests of 128 to 4,096
prompt tokens at the Qwen3-32B shape, portions of 512 tokens beside decode rows, 256 greedy tokens each; `long` is 8
prompts of 32,768 tokens at the Qwen3-4B shape, 512 tokens each at temperature 0.7.
"""
from __future__ import annotations

import argparse
import json
import sys
import time

HBM_GBS = 8000.0                 # MI355X published peaks
PEAK_FLOPS = {"bfloat16": 2.5e15, "float32": 157.3e12}
QWEN3_8B = {"architectures": ["Qwen3ForCausalLM"], "num_hidden_layers": 36, "hidden_size": 4096,
            "num_attention_heads": 32, "num_key_value_heads": 8, "head_dim": 128, "intermediate_size": 12288,
            "vocab_size": 151936, "rope_theta": 1e6, "rms_norm_eps": 1e-6, "tie_word_embeddings": False,
            "max_position_embeddings": 40960}
CONTEXT, PROMPT = 4096, 2048
LONG_CONTEXT = 32768            # the context of the long decode point (batch 8)
POINT_BATCHES = (1, 16, 32, 64)
POINT_PROMPTS = (512, 8192)
QWEN3_32B = dict(QWEN3_8B, num_hidden_layers=64, hidden_size=5120, num_attention_heads=64, intermediate_size=25600)
QWEN3_4B = dict(QWEN3_8B, hidden_size=2560, intermediate_size=9728, tie_word_embeddings=True)


def workload(name: str, layers: int | None, dtype: str, products: str = "timed") -> int:
    """A whole job: every request added at once, stepped until all are finished."""
    import random

    import torch

    from .config import EngineConfig, SamplingParams
    from .engine.engine import Engine
    rng = random.Random(0)
    if name == "mixed":
        shape, model = QWEN3_32B, "Qwen3-32B shape"
        prompts = [[rng.randrange(shape["vocab_size"]) for _ in range(rng.randint(128, 4096))] for _ in range(32)]
        params = SamplingParams(temperature=0.0, max_tokens=256, ignore_eos=True)
        ecfg = dict(max_seqs=32, max_model_len=4096 + 256 + 16, max_step_tokens=1024, chunk_with_decode=512)
    else:
        shape, model = QWEN3_4B, "Qwen3-4B shape"
        prompts = [[rng.randrange(shape["vocab_size"]) for _ in range(32768)] for _ in range(8)]
        params = SamplingParams(temperature=0.7, seed=1, max_tokens=512, ignore_eos=True)
        ecfg = dict(max_seqs=8, max_model_len=40960, max_step_tokens=4096)
    cfg_json = dict(shape, num_hidden_layers=layers or shape["num_hidden_layers"])
    engine = Engine.from_random(cfg_json, seed=0, cfg=EngineConfig(
        model=f"random:{name}", device="cuda:0", dtype=dtype, page_size=16, products=products,
        cache_tokens=len(prompts) * (max(map(len, prompts)) + params.max_tokens + 64), **ecfg))
    for p in prompts:
        engine.add(p, params)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    out = steps = out_at = 0
    t_prompts = None
    while engine.has_work():
        out += sum(len(d.token_ids) for d in engine.step())
        steps += 1
        if t_prompts is None and not engine.sched.waiting and all(
                s.num_computed >= s.prompt_len for s in engine.sched.running):
            torch.cuda.synchronize()
            t_prompts, out_at = time.perf_counter() - t0, out
    torch.cuda.synchronize()
    total = time.perf_counter() - t0
    stats = engine.stats()
    prompt_tokens = sum(map(len, prompts))
    print(json.dumps({
        "metric": f"{name} workload, {model}: tokens/s over the whole job", "value": round((prompt_tokens + out) / total, 1),
        "unit": "tokens/s", "n_gpus": 1, "seconds": round(total, 3), "dtype": "bf16" if dtype == "bfloat16" else "fp32",
        "data": "synthetic (random weights, uniform random token ids)",
        "config": {"model": model, "layers": cfg_json["num_hidden_layers"], "layers_of_config": shape["num_hidden_layers"],
                   "requests": len(prompts), "prompt_tokens": prompt_tokens, "output_tokens": out, **ecfg},
        "until_prompts_done": {"seconds": round(t_prompts, 3), "prompt_tokens_per_s": round(prompt_tokens / t_prompts, 1)},
        "decode_tail": {"tokens_per_s": round((out - out_at) / max(total - t_prompts, 1e-9), 1)},
        "steps": steps, "mixed_steps": stats["mixed_steps"], "preemptions": stats["preemptions"],
        "products": {"mode": products, "took": stats["products"]}}), flush=True)
    return 0


def main(argv: list[str] | None = None) -> int:
    ap = argparse.ArgumentParser(prog="bench", description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=64)
    ap.add_argument("--warmup", type=int, default=24,
                    help="untimed decode steps first (the first 15 or so after the prompts run 3%% slower)")
    ap.add_argument("--batch", type=int, default=8)
    ap.add_argument("--layers", type=int, default=QWEN3_8B["num_hidden_layers"],
                    help="fewer layers than the configuration has (recorded in config)")
    ap.add_argument("--dtype", choices=("bfloat16", "float32"), default="bfloat16")
    ap.add_argument("--no-points", action="store_true", help="skip the further decode and prefill points")
    ap.add_argument("--context", type=int, default=CONTEXT, help="the context the timed decode steps end at")
    ap.add_argument("--prompt", type=int, default=PROMPT, help="tokens of the timed prompt")
    ap.add_argument("--no-graphs", action="store_true")
    ap.add_argument("--workload", choices=("decode", "mixed", "long"), default="decode")
    ap.add_argument("--products", choices=("own", "vendor", "timed"), default="timed",
                    help="EngineConfig.products: which kernel products of 17 to 1,024 rows take (reported in the line)")
    a = ap.parse_args(argv)
    if a.gpus != 1:
        print(f"bench.py: this engine serves on one GPU; --gpus {a.gpus} is not a configuration it has", flush=True)
        return 2
    if a.workload != "decode":
        from .kernels import build as kernel_build
        if kernel_build.find_library() is None:
            kernel_build.build()
        return workload(a.workload, None if "--layers" not in (argv or sys.argv) else a.layers, a.dtype, a.products)

    import torch

    from .config import EngineConfig, SamplingParams
    from .engine.engine import Engine
    from .kernels import build as kernel_build

    if kernel_build.find_library() is None:
        kernel_build.build()
    cfg_json = dict(QWEN3_8B, num_hidden_layers=a.layers)
    max_batch = max(a.batch, 1 if a.no_points else max(POINT_BATCHES))
    longest = max(a.context, a.prompt, 0 if a.no_points else max(LONG_CONTEXT, max(POINT_PROMPTS)))
    engine = Engine.from_random(cfg_json, seed=0, cfg=EngineConfig(
        model="random:qwen3-8b", device="cuda:0", dtype=a.dtype, page_size=16, max_seqs=max_batch,
        max_model_len=longest + 16, max_step_tokens=4096,
        cache_tokens=max(max_batch * (CONTEXT + 16), a.batch * (a.context + 16), a.prompt + 16,
                         0 if a.no_points else 8 * (LONG_CONTEXT + 16)),
        graphs=not a.no_graphs, products=a.products))
    spec, c = engine.spec, cfg_json
    item = 2 if a.dtype == "bfloat16" else 4
    g = torch.Generator().manual_seed(0)
    greedy = lambda n: SamplingParams(temperature=0.0, max_tokens=n, ignore_eos=True)

    def decode(batch: int, steps: int, warmup: int, context: int = CONTEXT) -> tuple[float, float, float, int]:
        """(ms per decode step, mean context, median ms between two steps' ends, prompt length) for `batch` requests
        whose contexts end at `context`. The requests go on for two steps after the timed ones, so that the host's work
        for finished requests (not part of a decode step) falls outside the timed region."""
        after = 2
        start = context - steps - warmup - 1 - after
        for _ in range(batch):
            engine.add(torch.randint(0, c["vocab_size"], (start,), generator=g).tolist(),
                       greedy(steps + warmup + 1 + after))
        while engine.sched.waiting:                              # prompts, cut by the step budget
            engine.step()
        for _ in range(warmup):
            engine.step()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        ends = []
        for _ in range(steps):
            engine.step()                      # returns when the step before has been committed: one step's time apart
            ends.append(time.perf_counter())
        torch.cuda.synchronize()
        ms = (time.perf_counter() - t0) * 1e3 / steps
        gaps = sorted(b - a for a, b in zip(ends, ends[1:])) or [ms * 1e-3]
        while engine.has_work():
            engine.step()
        return ms, start + 1 + warmup + steps / 2, gaps[len(gaps) // 2] * 1e3, start

    def prefill(tokens: int) -> tuple[float, float]:
        """(best, median) ms from adding a prompt of `tokens` to its first generated token on the host: one step, or as
        many as the step budget cuts the prompt into."""
        times = []
        for _ in range(3):                     # another prompt each time: nothing of it is in the prefix cache
            ids = torch.randint(0, c["vocab_size"], (tokens,), generator=g).tolist()
            engine.add(ids, greedy(1))
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            while engine.has_work():
                engine.step()
            engine.drain()                     # the last step's one token on the host: the request is finished
            torch.cuda.synchronize()
            times.append((time.perf_counter() - t0) * 1e3)
            assert not engine.has_work()
        return min(times), sorted(times)[1]

    h, hq, hkv, d, inter, v, layers = (c["hidden_size"], c["num_attention_heads"], c["num_key_value_heads"],
                                       c["head_dim"], c["intermediate_size"], c["vocab_size"], a.layers)
    layer_params = h * (hq + 2 * hkv) * d + hq * d * h + 3 * h * inter
    weight_bytes = (layers * (layer_params + 2 * h + 2 * d) + h + h * v) * item      # every weight a decode step reads
    kv_token_bytes = layers * 2 * hkv * d * item
    def prompt_flops(tokens: int) -> float:
        """Products of every layer over `tokens` rows, causal attention (half of the square), the head on one row."""
        return layers * (2 * tokens * layer_params + 2 * hq * d * tokens * tokens) + 2 * h * v

    pre_ms, ttft_ms = prefill(a.prompt)
    pre_flops = prompt_flops(a.prompt)
    ms, ctx, tpot_ms, decode_prompt = decode(a.batch, a.steps, a.warmup, a.context)
    step_bytes = weight_bytes + a.batch * ctx * kv_token_bytes
    achieved = step_bytes / (ms * 1e-3) / 1e9
    points = {}
    if not a.no_points:
        def decode_point(name: str, b: int, context: int) -> None:
            pms, pctx, _, _ = decode(b, a.steps, a.warmup, context)
            gb = (weight_bytes + b * pctx * kv_token_bytes) / 1e9
            points[name] = round(b / (pms * 1e-3), 1)
            points[f"{name}_ms"] = round(pms, 4)
            points[f"{name}_gb"] = round(gb, 2)
            points[f"{name}_frac"] = round(gb / (pms * 1e-3) / HBM_GBS, 4)
        for b in POINT_BATCHES:
            decode_point(f"decode_b{b}", b, CONTEXT)
        decode_point(f"decode_b8_ctx{LONG_CONTEXT}", 8, LONG_CONTEXT)
        for tokens in POINT_PROMPTS:
            best, median = prefill(tokens)
            points[f"prefill_{tokens}"] = round(tokens / (best * 1e-3), 1)
            points[f"prefill_{tokens}_ms"] = round(best, 3)
            points[f"prefill_{tokens}_ms_median"] = round(median, 3)
            points[f"prefill_{tokens}_tflop"] = round(prompt_flops(tokens) / 1e12, 2)
            points[f"prefill_{tokens}_frac"] = round(prompt_flops(tokens) / (best * 1e-3) / PEAK_FLOPS[a.dtype], 4)
    line = {
        "metric": f"decode tok/s at batch {a.batch} (context {a.context:,}), Qwen3-8B shape", "value": round(a.batch / (ms * 1e-3), 1),
        "unit": "tokens/s", "n_gpus": 1, "steps": a.steps, "warmup": a.warmup, "ms_per_step": round(ms, 4),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "bf16" if a.dtype == "bfloat16" else "fp32",
        "data": "synthetic (random weights, uniform random token ids)",
        "config": {"model": "Qwen3-8B shape", "layers": layers, "layers_of_config": QWEN3_8B["num_hidden_layers"],
                   "hidden": h, "heads": hq, "kv_heads": hkv, "head_dim": d, "intermediate": inter, "vocab": v,
                   "tied": False, "global_batch": a.batch, "seq_len": a.context, "prefill_tokens": a.prompt,
                   "decode_prompt_len": decode_prompt, "page_size": 16,
                   "parallelism": "single GPU", "graphs": not a.no_graphs, "mean_context": round(ctx, 1),
                   "products": a.products},
        "prefill": {"value": round(a.prompt / (pre_ms * 1e-3), 1), "tokens": a.prompt, "ms": round(pre_ms, 3),
                    "ms_is": "best of 3 prompts", "ms_median": round(ttft_ms, 3),
                    "frac": round(pre_flops / (pre_ms * 1e-3) / PEAK_FLOPS[a.dtype], 4)},
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_GBS, "unit": "GB/s",
                     "frac": round(achieved / HBM_GBS, 4)},
        "points": points,
        "products": engine.products(),
        "latency": {"ttft_ms_p50": round(ttft_ms, 3), "ttft_tokens": a.prompt, "tpot_ms_p50": round(tpot_ms, 4),
                    "tpot_batch": a.batch},
    }
    if engine.stats()["prefix_tokens_saved"]:
        raise RuntimeError("the prefix cache served part of a timed prompt: the figures above would count work not done")
    print(json.dumps(line), flush=True)
    return 0


if __name__ == "__main__":
    sys.exit(main())
