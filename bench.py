#!/usr/bin/env python3
"""Decode and prefill throughput of the engine at the Qwen3-8B shape with random weights, on one MI355X: one JSON line.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--batch 8] [--layers L] [--no-points]

The measurement itself is `holon_amd/benchmark.py` (also `python -m holon_amd bench`)."""
import pathlib
import sys

sys.path.insert(0, str(pathlib.Path(__file__).resolve().parent))

from holon_amd.benchmark import main  # noqa: E402

if __name__ == "__main__":
    sys.exit(main())
