"""The command line as a user runs it: `python -m trapetum_amd random`, then `run` and `generate` on the folder it
wrote, and `run --random`; the ids must be the plain implementation's (the reference's entry point is such a
binary: runtime/src/bin/gemma_run.rs:1-19)."""
import json
import os
import subprocess
import sys

import numpy as np
import pytest

from .plain import gemma2_plain as plain
from .tiny import TINY_A, TINY_A_INIT, random_tokens

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def cli(*args):
    p = subprocess.run([sys.executable, "-m", "trapetum_amd"] + [str(a) for a in args], cwd=ROOT, capture_output=True,
                       text=True, timeout=300)
    assert p.returncode == 0, p.stderr[-2000:]
    return p.stdout


def test_random_run_generate(tmp_path):
    config = tmp_path / "config.json"
    config.write_text(json.dumps(dict(TINY_A, architectures=["Gemma2ForCausalLM"])))
    folder = tmp_path / "model"
    init = ["--seed", TINY_A_INIT["seed"], "--sigma", TINY_A_INIT["sigma"], "--sigma-norm", TINY_A_INIT["sigma_norm"]]
    assert "wrote" in cli("random", "--config", config, "--out", folder, *init)
    pcfg, pw = plain.read_folder(str(folder))
    prompts = [random_tokens(n, pcfg["vocab_size"], 90 + n) for n in (5, 11, 17)]
    want = [plain.greedy_generate(pcfg, pw, p, 8) for p in prompts]
    ids_file = tmp_path / "prompt.bin"
    np.asarray(prompts[1], dtype="<i4").tofile(ids_file)
    out = cli("run", folder, ids_file, "--max-tokens", 8, "--dtype", "float32", "--no-stop")
    assert out.strip() == f"continuation ids: {want[1]}"
    out = cli("run", folder, "--prompt-ids", ",".join(map(str, prompts[0])), "--max-tokens", 8, "--dtype", "float32", "--no-stop")
    assert out.strip() == f"continuation ids: {want[0]}"
    lines = tmp_path / "prompts.txt"
    lines.write_text("".join(" ".join(map(str, p)) + "\n" for p in prompts))
    out = cli("generate", folder, "--prompts-file", lines, "--max-tokens", 8, "--dtype", "float32", "--no-stop")
    assert [[int(t) for t in l.split()] for l in out.strip().splitlines()] == want
    # the same model without a folder: random weights of the configuration, by the same seed
    out = cli("run", "--random", config, "--weights-seed", TINY_A_INIT["seed"], "--sigma", TINY_A_INIT["sigma"],
              "--sigma-norm", TINY_A_INIT["sigma_norm"], "--prompt-ids", ",".join(map(str, prompts[2])), "--max-tokens", 8,
              "--dtype", "float32", "--no-stop")
    assert out.strip() == f"continuation ids: {want[2]}"
    # a stop token ends the continuation before it
    out = cli("run", folder, "--prompt-ids", ",".join(map(str, prompts[1])), "--max-tokens", 8, "--dtype", "float32",
              "--stop-id", want[1][3])
    assert out.strip() == f"continuation ids: {want[1][:want[1].index(want[1][3])]}"


def test_a_text_prompt_goes_through_the_folders_tokenizer(tmp_path):
    """`run DIR --prompt "text"`: the ids are the tokenizer.json's (no special tokens added, as the reference's server
    encodes: runtime/src/bin/serve.rs:312), the continuation is the one the same ids give, and it comes back as ids and
    as text; a folder without a tokenizer.json refuses a text prompt with an error that names the file."""
    from tokenizers import Tokenizer
    from tokenizers.models import WordLevel
    from tokenizers.pre_tokenizers import Whitespace
    config = tmp_path / "config.json"
    config.write_text(json.dumps(dict(TINY_A, architectures=["Gemma2ForCausalLM"])))
    folder = tmp_path / "model"
    cli("random", "--config", config, "--out", folder, "--seed", 3)
    p = subprocess.run([sys.executable, "-m", "trapetum_amd", "run", str(folder), "--prompt", "w5 w17 w3"], cwd=ROOT,
                       capture_output=True, text=True, timeout=300)
    assert p.returncode != 0 and "tokenizer.json" in p.stderr
    vocab = {f"w{i}": i for i in range(TINY_A["vocab_size"])}
    tok = Tokenizer(WordLevel(vocab, unk_token="w0"))
    tok.pre_tokenizer = Whitespace()
    tok.save(str(folder / "tokenizer.json"))
    by_ids = cli("run", folder, "--prompt-ids", "5,17,3,9", "--max-tokens", 6, "--dtype", "float32", "--no-stop").strip()
    by_text = cli("run", folder, "--prompt", "w5 w17 w3 w9", "--max-tokens", 6, "--dtype", "float32", "--no-stop").strip().splitlines()
    assert by_text[0] == by_ids
    ids = json.loads(by_ids.split(":", 1)[1])
    assert by_text[1] == "continuation text: " + " ".join(f"w{i}" for i in ids)


def test_float32_weights_are_kept_as_drawn(tmp_path):
    """`random --store-dtype float32` stores the drawn values unrounded, and the float32 engine keeps them so: its
    logits follow a plain run on the unrounded values, not one on their bfloat16 roundings."""
    import torch

    from .tiny import rel_l2
    config = tmp_path / "config.json"
    config.write_text(json.dumps(dict(TINY_A, architectures=["Gemma2ForCausalLM"])))
    folder = tmp_path / "model32"
    cli("random", "--config", config, "--out", folder, "--seed", 4, "--sigma", 0.05, "--sigma-norm", 0.2, "--store-dtype", "float32")
    pcfg, pw = plain.read_folder(str(folder))
    assert any((t.float().to(torch.bfloat16).double() != t).any() for t in pw.values())     # not bfloat16 values
    from .gpu_engine import load_gpu_model
    model, cfg = load_gpu_model(str(folder), "float32")
    toks = random_tokens(30, cfg.vocab_size, 8)
    cache = model.new_cache(max_tokens=64)
    s = cache.acquire()
    got = model.step(cache, [s], toks, counts=[30], want=list(range(30)))
    assert rel_l2(got, plain.forward(pcfg, pw, toks)) < 1e-5
    rounded = {k: v.float().to(torch.bfloat16).double() for k, v in pw.items()}
    assert rel_l2(got, plain.forward(pcfg, rounded, toks)) > 1e-4


def test_switches(tmp_path):
    """TRAPETUM_AMD_PROFILE=1 prints the time per entry point of the kernel library when the process ends;
    TRAPETUM_AMD_FORCE_PLAIN=1 runs bfloat16 on the plain kernels, with the same tokens where the model is sure."""
    config = tmp_path / "config.json"
    config.write_text(json.dumps(dict(TINY_A, architectures=["Gemma2ForCausalLM"])))
    args = [sys.executable, "-m", "trapetum_amd", "run", "--random", str(config), "--prompt-ids", "5,6,7,8", "--max-tokens", "6",
            "--no-stop"]
    p = subprocess.run(args, cwd=ROOT, capture_output=True, text=True, timeout=300, env=dict(os.environ, TRAPETUM_AMD_PROFILE="1"))
    assert p.returncode == 0, p.stderr[-2000:]
    prof = [l for l in p.stderr.splitlines() if l.startswith("[profile] op=")]
    ops = {l.split()[1][3:]: int(l.split()[2][6:]) for l in prof}
    assert ops["tp_linear"] > 0 and ops["tp_add_rms_norm"] > 0 and "tp_attn_decode_fused" in ops, p.stderr[-2000:]
    ids = p.stdout.strip()
    p = subprocess.run(args, cwd=ROOT, capture_output=True, text=True, timeout=300, env=dict(os.environ, TRAPETUM_AMD_FORCE_PLAIN="1", TRAPETUM_AMD_PROFILE="1"))
    assert p.returncode == 0, p.stderr[-2000:]
    assert "tp_attn_decode_fused" not in p.stderr and "tp_attn_simple_decode" in p.stderr
    assert p.stdout.strip() == ids


def test_bench_line(tmp_path):
    """The measurement's one JSON line with two layers of the 2B sizes: the keys its readers rely on, a flat `config` of at
    most 20 keys, fewer layers named beside the full number; more than one GPU is refused in one line with exit code 2."""
    p = subprocess.run([sys.executable, "bench.py", "--layers", "2", "--steps", "4", "--warmup", "2"], cwd=ROOT,
                       capture_output=True, text=True, timeout=600)
    assert p.returncode == 0, p.stderr[-2000:]
    lines = [l for l in p.stdout.splitlines() if l.startswith("{")]
    assert len(lines) == 1
    d = json.loads(lines[0])
    for k in ("metric", "value", "unit", "n_gpus", "steps", "warmup", "ms_per_step", "higher_is_better", "scaling",
              "vs_baseline", "dtype", "data", "config", "prefill", "roofline", "points"):
        assert k in d, k
    assert d["n_gpus"] == 1 and d["steps"] == 4 and d["warmup"] == 2 and d["higher_is_better"] is True and d["dtype"] == "bf16"
    assert d["value"] > 0 and abs(d["value"] - 8 * 1e3 / d["ms_per_step"]) < 0.01 * d["value"]
    c = d["config"]
    assert len(c) <= 20 and all(not isinstance(v, (dict, list)) for v in c.values())
    assert c["layers"] == 2 and c["layers_full"] == 26 and c["global_batch"] == 8 and c["hidden"] == 2304
    assert set(d["prefill"]) >= {"value", "tokens", "ms", "frac"} and d["prefill"]["tokens"] == 2048
    r = d["roofline"]
    assert r["bound"] == "hbm" and r["unit"] == "GB/s" and r["peak"] == 8000.0 and abs(r["frac"] - r["achieved"] / r["peak"]) < 1e-3
    assert set(d["points"]) >= {"decode_b1", "decode_b64", "generate_b8", "decode_b8_ctx7900", "decode_b8_9b", "decode_b8_27b",
                                "prefill_2048_9b", "prefill_2048_27b"}
    assert all(isinstance(v, float) and v > 0 for v in d["points"].values())
    assert set(d["points_frac"]) == set(d["points"]) - {"generate_b8"} and all(0 < v < 1 for v in d["points_frac"].values())
    k = d["kernels"]
    assert {"decode_b8.gate_up", "decode_b8.down", "decode_b8.qkv", "decode_b8.o", "decode_b8.add_rms_norm", "prefill_2048.gate_up",
            "prefill_2048.attention"} <= set(k) and any(n.startswith("decode_b8.attention_ctx") for n in k)
    for name, row in k.items():
        assert row["us"] > 0 and 0 < row["frac"] < 1 and ("GB/s" in row) != ("TFLOP/s" in row), name
    p = subprocess.run([sys.executable, "bench.py", "--gpus", "2"], cwd=ROOT, capture_output=True, text=True, timeout=120)
    assert p.returncode == 2 and len((p.stdout + p.stderr).strip().splitlines()) == 1
