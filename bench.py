#!/usr/bin/env python3
"""python bench.py [--gpus 1] [--steps K] [--warmup W] [--layers L] [--batch B] [--no-points]

Decode and prefill throughput of the engine at the Llama-3-8B shape on one MI355X, as one
JSON line; see rbitnet_amd/benchmark.py for what is measured and how."""
import os
import sys

sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))

from rbitnet_amd.benchmark import LLAMA3_8B, main  # noqa: E402,F401

if __name__ == "__main__":
    sys.exit(main())
