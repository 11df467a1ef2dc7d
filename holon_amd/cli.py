"""The command line: `python -m holon_amd <command>`.

    generate MODEL   generate token ids for prompts given as token ids (in process, no server)
    random           write a model folder with random weights from a configuration and a seed
    replay           trace replay (what bin/trace_run runs)
    models           the architectures this build serves
    bench            decode and prefill throughput at the Qwen3-8B shape (what bench.py at the repository's root runs)

Engine flags are made from `EngineConfig`'s fields, one flag a field with the field's help line, booleans as
--x / --no-x, as the reference's `holon serve` makes them (core/holon/core/cli.py:52-80).
"""
from __future__ import annotations

import argparse
import dataclasses
import json
import pathlib
import sys
import typing

from .config import EngineConfig, SamplingParams


AUTO_CONTEXT = 32768      # `--max-model-len auto`: the model's trained context, at most this


def engine_flags(parser: argparse.ArgumentParser | argparse._ArgumentGroup) -> None:
    hints = typing.get_type_hints(EngineConfig)
    for f in dataclasses.fields(EngineConfig):
        if f.name == "model":
            continue
        flag, kind = "--" + f.name.replace("_", "-"), hints[f.name]
        help_ = f.metadata["help"] + (f" (default: {f.default})" if f.default is not None else "")
        if kind is bool:
            # (`--cuda-graphs` is the reference's name for `--graphs`, core/holon/core/engine.py:83; both are taken)
            also = ["--cuda-graphs", "--no-cuda-graphs"] if f.name == "graphs" else []
            parser.add_argument(flag, *also[:1], action=argparse.BooleanOptionalAction, default=f.default, help=help_)
        elif f.name == "max_model_len":            # also `auto` (core/holon/core/cli.py:44-47, 76)
            parser.add_argument(flag, type=lambda s: s if s == "auto" else int(s), default=f.default,
                                help=help_ + f"; auto: the model's trained context, at most {AUTO_CONTEXT}")
        elif f.name == "product_pins":
            parser.add_argument(flag, type=_pins, default=None, help=help_)
        elif kind in (int, float, str):
            parser.add_argument(flag, type=kind, default=f.default, help=help_)
        else:                                         # int | None
            parser.add_argument(flag, type=int, default=f.default, help=help_)


def _pins(text: str) -> dict[str, str]:
    """`kind:NxK:rows=form,kind:NxK:rows=form` -> {key: form}."""
    pairs = [item.split("=", 1) for item in text.split(",") if item.strip()]
    if any(len(pair) != 2 for pair in pairs):
        raise argparse.ArgumentTypeError("expected kind:NxK:rows=form, separated by commas")
    return {key.strip(): form.strip() for key, form in pairs}


def engine_config(model: str, args: argparse.Namespace) -> EngineConfig:
    names = {f.name for f in dataclasses.fields(EngineConfig)} - {"model"}
    settings = {k: v for k, v in vars(args).items() if k in names}
    if settings.get("max_model_len") == "auto":
        from .config.model import read_config_json
        trained = read_config_json(model)[0].get("max_position_embeddings")
        settings["max_model_len"] = min(int(trained), AUTO_CONTEXT) if trained else AUTO_CONTEXT
    return EngineConfig(model=model, **settings)


def _ids(text: str) -> list[int]:
    return [int(t) for t in text.replace(",", " ").split()]


def _tokenizer(folder: str):
    """The checkpoint's own tokenizer (tokenizer.json), for prompts given as text. core/holon/api/frontend.py:55-70
    keeps tokenisation outside the engine; so does this: the engine sees ids only."""
    path = pathlib.Path(folder) / "tokenizer.json"
    if not path.is_file():
        raise SystemExit(f"--prompt needs {path}; give token ids with --prompt-ids instead")
    from tokenizers import Tokenizer
    return Tokenizer.from_file(str(path))


def generate_main(argv: list[str]) -> int:
    ap = argparse.ArgumentParser(prog="holon_amd generate", description="Generate tokens for prompts of token ids "
                                 "(printed as ids) or of text (printed as text, with the folder's tokenizer.json).")
    ap.add_argument("model", help="model folder (config.json, *.safetensors)")
    ap.add_argument("--prompt-ids", action="append", default=[], metavar="IDS",
                    help="a prompt as token ids separated by spaces or commas; may be given several times")
    ap.add_argument("--prompt-file", help="a file with one prompt of token ids per line")
    ap.add_argument("--prompt", action="append", default=[], metavar="TEXT",
                    help="a prompt as text, encoded with the model folder's tokenizer.json; may be given several times")
    ap.add_argument("--max-tokens", type=int, default=16)
    ap.add_argument("--temperature", type=float, default=0.0)
    ap.add_argument("--top-k", type=int, default=0)
    ap.add_argument("--top-p", type=float, default=1.0)
    ap.add_argument("--min-p", type=float, default=0.0)
    ap.add_argument("--seed", type=int, default=None)
    ap.add_argument("--n", type=int, default=1, help="sequences per prompt, printed one a line in order")
    ap.add_argument("--ignore-eos", action=argparse.BooleanOptionalAction, default=False)
    ap.add_argument("--stats", action="store_true", help="print the engine's counters to stderr at the end")
    engine_flags(ap.add_argument_group("engine"))
    a = ap.parse_args(argv)
    prompts = [_ids(p) for p in a.prompt_ids]
    if a.prompt_file:
        prompts += [_ids(line) for line in pathlib.Path(a.prompt_file).read_text().splitlines() if line.strip()]
    as_text = len(prompts)                          # prompts from here on were given as text and are answered as text
    tokenizer = _tokenizer(a.model) if a.prompt else None
    prompts += [tokenizer.encode(text).ids for text in a.prompt]
    if not prompts:
        ap.error("give at least one prompt (--prompt-ids, --prompt-file or --prompt)")
    from .engine.engine import Engine
    engine = Engine(engine_config(a.model, a))
    params = SamplingParams(temperature=a.temperature, top_k=a.top_k, top_p=a.top_p, min_p=a.min_p, seed=a.seed,
                            max_tokens=a.max_tokens, ignore_eos=a.ignore_eos, n=a.n)
    rids = [engine.add(p, params) for p in prompts]
    out: dict[tuple[str, int], list[int]] = {(rid, i): [] for rid in rids for i in range(a.n)}
    while engine.has_work():
        for d in engine.step():
            out[d.rid, d.index] += d.token_ids
    for at, rid in enumerate(rids):
        for i in range(a.n):
            ids = out[rid, i]
            print(tokenizer.decode(ids) if at >= as_text else " ".join(str(t) for t in ids), flush=True)
    if a.stats:
        print(json.dumps(engine.stats()), file=sys.stderr)
    engine.close()
    return 0


def random_main(argv: list[str]) -> int:
    ap = argparse.ArgumentParser(prog="holon_amd random",
                                 description="Write a model folder with random weights (config.json, model.safetensors).")
    ap.add_argument("--config", required=True, help="a config.json to take the architecture and sizes from")
    ap.add_argument("--seed", type=int, default=0)
    ap.add_argument("--out", required=True, help="the folder to write")
    ap.add_argument("--store-dtype", choices=("bfloat16", "float32"), default="bfloat16")
    a = ap.parse_args(argv)
    import torch

    from .weights import write_random_model
    cfg = json.loads(pathlib.Path(a.config).read_text())
    write_random_model(cfg, a.seed, a.out, getattr(torch, a.store_dtype))
    print(a.out)
    return 0


def replay_main(argv: list[str]) -> int:
    ap = argparse.ArgumentParser(prog="trace_run", description="Trace replay: token ids in, logits out, step by step.")
    ap.add_argument("--model", required=True)
    ap.add_argument("--dtype", choices=("bfloat16", "float32"), required=True)
    ap.add_argument("--out", required=True)
    ap.add_argument("--max-tokens", type=int, required=True,
                    help="the most tokens live requests hold at any time (each rounded up to a multiple of 64)")
    ap.add_argument("--page-size", type=int, default=16)
    ap.add_argument("--max-seqs", type=int, default=8)
    a = ap.parse_args(argv)
    if a.max_tokens < 1 or a.page_size < 1 or 64 % a.page_size:
        ap.error("--max-tokens must be positive and --page-size must divide 64")
    from .engine.loading import load_model
    from .engine.replay import Replayer
    out = pathlib.Path(a.out)
    out.mkdir(parents=True, exist_ok=True)
    tokens = -(-a.max_tokens // a.page_size) * a.page_size
    loaded = load_model(a.model, device="cuda", dtype=a.dtype, page_size=a.page_size, max_seqs=a.max_seqs,
                        max_model_len=tokens, max_step_tokens=tokens, cache_tokens=tokens)
    replayer = Replayer(loaded)
    for line in sys.stdin:
        line = line.strip()
        if not line:
            continue
        step = json.loads(line)
        logits = replayer.step(step.get("entries", []), step.get("end", []))
        if logits is not None:
            logits.cpu().numpy().astype("<f4", copy=False).tofile(out / f"{step['step']}.f32")
        print(f"done {step['step']}", flush=True)
    return 0


def models_main(argv: list[str]) -> int:
    from .registry import architectures
    for name in architectures():
        print(name)
    return 0


def bench_main(argv: list[str]) -> int:
    from .benchmark import main as bench
    return bench(argv)


COMMANDS = {"generate": generate_main, "random": random_main, "replay": replay_main, "models": models_main,
            "bench": bench_main}


def main(argv: list[str] | None = None) -> int:
    argv = sys.argv[1:] if argv is None else argv
    if not argv or argv[0] in ("-h", "--help") or argv[0] not in COMMANDS:
        print(__doc__.strip(), file=sys.stderr)
        return 0 if argv and argv[0] in ("-h", "--help") else 2
    return COMMANDS[argv[0]](argv[1:])
