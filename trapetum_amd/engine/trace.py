"""Trace replay: feed given token ids through a model step by step and write logits; nothing is sampled.

It drives the same model, step function, cache and kernels as generation.  The reference's nearest tool is
its `generate` binary, which feeds a prompt one token per forward and compares each position's logits with a
file (runtime/src/bin/generate.rs:45-96).

Input, one JSON object per line:
    {"step": 0, "entries": [{"id": "a", "tokens": [5, 17, 3], "want": [0, 2]}], "end": []}
A step may bring any number of tokens for each of its requests, whether they start or go on, and a request may
join after others have started.  For a step with wanted places the
logits go to <out>/<step>.f32 as little-endian float32 [wanted, vocab], in the order of entries and of want.
After every step "done <step>" is printed and flushed.
"""
import json
import os
import sys

import numpy as np

from ..registry import config_from_folder
from ..weights import load_folder
from .model import Model
from .runtime import Runtime

PAGE = 64


class TraceError(ValueError):
    pass


class TraceRunner:
    def __init__(self, folder, dtype, max_tokens, device="cuda:0", ops=None):
        arch, self.config = config_from_folder(folder)
        self.model = Model(arch.build_spec(self.config), Runtime(dtype=dtype, device=device, ops=ops))
        load_folder(self.model, folder)
        self.cache = self.model.new_cache(max_tokens, max_context=max_tokens, page_size=PAGE)
        self.slot_of = {}

    def run_step(self, record):
        """Returns the logits of the wanted places as a float32 array [wanted, vocab], or None."""
        entries = record.get("entries", [])
        if not isinstance(entries, list):
            raise TraceError("'entries' must be a list")
        slots, counts, flat, want, offset = [], [], [], [], 0
        fresh = []
        for e in entries:
            rid, toks = e["id"], e["tokens"]
            if not toks:
                raise TraceError(f"request {rid!r} brings no tokens in step {record.get('step')}")
            if rid not in self.slot_of:
                self.slot_of[rid] = self.cache.acquire()
                fresh.append(rid)
            slots.append(self.slot_of[rid])
            counts.append(len(toks))
            flat.extend(int(t) for t in toks)
            for w in e.get("want", []):
                if not 0 <= w < len(toks):
                    raise TraceError(f"request {rid!r}: wanted place {w} is outside its {len(toks)} tokens")
                want.append(offset + int(w))
            offset += len(toks)
        out = None
        if entries:
            try:
                logits = self.model.step(self.cache, slots, flat, counts=counts, want=want)
            except Exception:
                for rid in fresh:                       # a refused step leaves nothing behind
                    self.cache.release(self.slot_of.pop(rid))
                raise
            if logits is not None:
                out = logits.float().cpu().numpy().astype("<f4", copy=False)
        for rid in record.get("end", []):
            if rid not in self.slot_of:
                raise TraceError(f"request {rid!r} ends in step {record.get('step')} but is not live")
            self.cache.release(self.slot_of.pop(rid))
        return out


def main(argv=None, stdin=None, stdout=None):
    import argparse
    ap = argparse.ArgumentParser(prog="trace_run", description=__doc__.split("\n\n")[0])
    ap.add_argument("--model", required=True, help="folder with config.json and model.safetensors")
    ap.add_argument("--dtype", required=True, choices=["bfloat16", "float32"])
    ap.add_argument("--out", required=True, help="folder the logits files go to")
    ap.add_argument("--max-tokens", type=int, required=True,
                    help="most tokens live requests hold at any time, each rounded up to a multiple of 64")
    ap.add_argument("--device", default="cuda:0")
    args = ap.parse_args(argv)
    stdin = stdin or sys.stdin
    stdout = stdout or sys.stdout
    os.makedirs(args.out, exist_ok=True)
    runner = TraceRunner(args.model, args.dtype, args.max_tokens, device=args.device)
    for line in stdin:
        line = line.strip()
        if not line:
            continue
        record = json.loads(line)
        step = record["step"]
        logits = runner.run_step(record)
        if logits is not None:
            logits.tofile(os.path.join(args.out, f"{step}.f32"))
        stdout.write(f"done {step}\n")
        stdout.flush()
    return 0
