"""bin/trace_run as a user runs it: the same requests whole, with the last 32 tokens one by one, and in
batches of unequal lengths, in float32 and bfloat16, against the plain implementation."""
import json
import os
import subprocess
import sys

import numpy as np
import pytest
import torch

from .plain import gemma2_plain as plain
from .tiny import CONFIGS, make_folder, random_tokens, rel_l2
from . import trace_schedules as ts

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
TOL = {"float32": 1e-5, "bfloat16": 2e-2}


def replay(folder, dtype, steps, out_dir, max_tokens):
    p = subprocess.run([sys.executable, os.path.join(ROOT, "bin", "trace_run"), "--model", folder, "--dtype", dtype,
                        "--out", out_dir, "--max-tokens", str(max_tokens)],
                       input="".join(json.dumps(s) + "\n" for s in steps), capture_output=True, text=True, timeout=300)
    assert p.returncode == 0, p.stderr[-2000:]
    assert [l for l in p.stdout.splitlines() if l.startswith("done")] == [f"done {s['step']}" for s in steps]
    out = {}
    for s in steps:
        f = os.path.join(out_dir, f"{s['step']}.f32")
        wanted = sum(len(e.get("want", [])) for e in s["entries"])
        assert os.path.exists(f) == (wanted > 0)
        if wanted:
            out[s["step"]] = np.fromfile(f, dtype="<f4")
    return out


@pytest.mark.parametrize("which", ["A", "B", "D"])
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_replay_schedules_agree_with_plain(which, dtype, tmp_path):
    folder = make_folder(tmp_path, which)
    pcfg, pw = plain.read_folder(folder)
    vocab = pcfg["vocab_size"]
    lens = [70, 41, 97, 5, 33, 1, 64]
    requests = {f"r{i}": random_tokens(n, vocab, 10 + i) for i, n in enumerate(lens)}
    ref = {rid: plain.forward(pcfg, pw, toks) for rid, toks in requests.items()}
    schedules = {"whole": ts.whole(requests), "tail": ts.last_one_by_one(requests, 32), "batches": ts.batches(requests, 3),
                 "portions of 16": ts.chunked(requests, [16]), "portions of 1, 7, 32": ts.chunked(requests, [1, 7, 32]),
                 "joining a running batch": ts.joining(requests)}
    for name, steps in schedules.items():
        out_dir = str(tmp_path / ("out_" + name.replace(" ", "_").replace(",", "")))
        got = ts.collect(steps, replay(folder, dtype, steps, out_dir, ts.held_tokens(steps)), vocab)
        for rid in requests:
            assert got[rid].shape == tuple(ref[rid].shape), (name, rid)
            assert rel_l2(torch.from_numpy(got[rid]), ref[rid]) < TOL[dtype], (name, rid)
