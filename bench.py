"""Benchmark entry point: decode tokens per second of Gemma-2 at 2B layer sizes on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] ...

One JSON line on standard output; the options, the contract and what is measured are described in
trapetum_amd/measure.py, which `python -m trapetum_amd bench` runs as well.  More than one GPU is not
measured: this library runs on a single MI355X, and `--gpus N` with N > 1 prints one line saying so and exits
with 2.
"""
import os
import sys

sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))

if __name__ == "__main__":
    from trapetum_amd.measure import main
    sys.exit(main())
