"""Command line: run | generate | replay | random | bench.

The reference's command line is positional, one binary per architecture: `gemma_run <model.cbk> <prompt.bin>`
with the prompt as little-endian int32 ids (runtime/src/bin/gemma_run.rs:1-19, runtime/src/lib.rs:4437-4441);
its request options are max_tokens, temperature, top_p, repetition_penalty (runtime/src/bin/serve.rs:1285-1292).

  python -m trapetum_amd run MODEL_DIR PROMPT.bin [--max-tokens 24] ...      one prompt, like gemma_run
  python -m trapetum_amd run MODEL_DIR --prompt "text" ...                   with the folder's tokenizer.json
  python -m trapetum_amd generate MODEL_DIR --prompts-file ids.txt ...       many prompts, one id list per line
  python -m trapetum_amd replay --model DIR --dtype D --out DIR --max-tokens N   (same as bin/trace_run)
  python -m trapetum_amd random --config CONFIG.json --out DIR --seed S     write a random model folder
  python -m trapetum_amd bench [--steps K] [--warmup W] [--sizes 2b|9b|27b] ...  (same as bench.py)

Instead of a model folder, `run` and `generate` take `--random CONFIG.json` (with --weights-seed, --sigma,
--sigma-norm): a model of that configuration with seeded random weights, written to a temporary folder first.
"""
import argparse
import json
import sys
import time


def _read_ids_bin(path):
    import numpy as np
    return [int(t) for t in np.fromfile(path, dtype="<i4")]


def _add_sampling(ap):
    ap.add_argument("--max-tokens", type=int, default=24, help="tokens to generate per prompt (gemma_run generates 24)")
    ap.add_argument("--temperature", type=float, default=0.0, help="0 = greedy")
    ap.add_argument("--top-p", type=float, default=0.95)
    ap.add_argument("--top-k", type=int, default=256, help="candidates kept (the reference keeps 256); 0: the whole vocabulary, with --top-p 1")
    ap.add_argument("--repetition-penalty", type=float, default=1.0)
    ap.add_argument("--seed", type=int, default=0, help="sampling seed")
    ap.add_argument("--stop-id", type=int, action="append", default=None,
                    help="stop token (repeatable); default: eos_token_id of the model folder")
    ap.add_argument("--no-stop", action="store_true", help="ignore stop tokens, like gemma_run")
    ap.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "float32"])
    ap.add_argument("--device", default="cuda:0")
    ap.add_argument("--max-context", type=int, default=None)
    ap.add_argument("--cache-tokens", type=int, default=16384, help="tokens the cache holds over all live sequences")
    ap.add_argument("--max-batch", type=int, default=64)
    ap.add_argument("--random", metavar="CONFIG.json", help="random weights of this configuration instead of a model folder")
    ap.add_argument("--weights-seed", type=int, default=0, help="seed of --random's weights")
    ap.add_argument("--sigma", type=float, default=0.02, help="standard deviation of --random's matrices")
    ap.add_argument("--sigma-norm", type=float, default=0.1, help="standard deviation of --random's norm weights")


def _config_of(path):
    from .config.base import architecture_name
    from .registry import architecture
    with open(path) as f:
        d = json.load(f)
    return architecture(architecture_name(d)).config_cls.from_dict(d)


def _generate(args, prompts):
    import tempfile

    from .engine import Engine
    from .weights import write_model_folder
    if (args.model is None) == (args.random is None):
        raise SystemExit("give a model folder or --random CONFIG.json (one of the two)")
    t0 = time.time()
    with tempfile.TemporaryDirectory() as tmp:
        folder = args.model
        if args.random is not None:
            folder = write_model_folder(_config_of(args.random), tmp, args.weights_seed, args.sigma, args.sigma_norm)
        engine = Engine.from_folder(folder, dtype=args.dtype, device=args.device, max_tokens_in_cache=args.cache_tokens,
                                    max_context=args.max_context, max_batch=args.max_batch)
    print(f"loaded in {time.time() - t0:.1f}s vocab={engine.config.vocab_size} prompts={len(prompts)}", file=sys.stderr)
    stops = () if args.no_stop else (tuple(args.stop_id) if args.stop_id else None)
    t0 = time.time()
    out = engine.generate(prompts, max_tokens=args.max_tokens, temperature=args.temperature, top_p=args.top_p,
                          top_k=args.top_k, repetition_penalty=args.repetition_penalty, seed=args.seed, stop_ids=stops)
    dt = time.time() - t0
    n = sum(len(o) for o in out)
    print(f"generated {n} tokens in {dt * 1e3:.1f} ms ({n / max(dt, 1e-9):.1f} tok/s, prefill included)", file=sys.stderr)
    return out


def main(argv=None):
    ap = argparse.ArgumentParser(prog="python -m trapetum_amd", description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    sub = ap.add_subparsers(dest="command", required=True)
    run = sub.add_parser("run", help="generate for one prompt")
    run.add_argument("model", nargs="?", help="folder with config.json and model.safetensors")
    run.add_argument("prompt", nargs="?", help="file of little-endian int32 token ids")
    run.add_argument("--prompt-ids", help="comma-separated token ids instead of a file")
    run.add_argument("--prompt-text", "--prompt", dest="prompt_text", metavar="TEXT",
                     help="a text prompt, encoded by the model folder's tokenizer.json (no special tokens added)")
    _add_sampling(run)
    gen = sub.add_parser("generate", help="generate for many prompts")
    gen.add_argument("model", nargs="?")
    gen.add_argument("--prompts-file", required=True, help="one prompt per line: token ids separated by commas or blanks")
    _add_sampling(gen)
    rep = sub.add_parser("replay", help="trace replay (bin/trace_run)")
    rep.add_argument("rest", nargs=argparse.REMAINDER)
    rnd = sub.add_parser("random", help="write a model folder with random weights")
    rnd.add_argument("--config", required=True, help="a config.json")
    rnd.add_argument("--out", required=True)
    rnd.add_argument("--seed", type=int, default=0)
    rnd.add_argument("--sigma", type=float, default=0.02)
    rnd.add_argument("--sigma-norm", type=float, default=0.1)
    rnd.add_argument("--store-dtype", default="bfloat16", choices=["bfloat16", "float32"],
                     help="width the tensors are stored in (float32: the drawn values unrounded)")
    ben = sub.add_parser("bench", help="the benchmark (bench.py)")
    ben.add_argument("rest", nargs=argparse.REMAINDER)
    args = ap.parse_args(argv)

    if args.command == "replay":
        from .engine.trace import main as trace_main
        return trace_main(args.rest)
    if args.command == "bench":
        from .measure import main as bench_main
        return bench_main(args.rest)
    if args.command == "random":
        from .weights import write_model_folder
        write_model_folder(_config_of(args.config), args.out, args.seed, args.sigma, args.sigma_norm, store_dtype=args.store_dtype)
        print(f"wrote {args.out}")
        return 0
    if args.command == "run":
        tok = None
        if args.prompt_text is not None:
            from .text import FolderTokenizer, TextError
            if args.model is None:
                ap.error("a text prompt needs a model folder with a tokenizer.json")
            if args.prompt is not None:
                ap.error("give a prompt file or --prompt, not both")
            try:
                tok = FolderTokenizer(args.model)
                prompt = tok.encode(args.prompt_text)
            except TextError as e:
                raise SystemExit(str(e))
        elif args.prompt_ids:
            prompt = [int(t) for t in args.prompt_ids.replace(",", " ").split()]
        elif args.prompt:
            prompt = _read_ids_bin(args.prompt)
        else:
            ap.error("run needs a prompt file or --prompt-ids")
        out = _generate(args, [prompt])
        print("continuation ids:", out[0])
        if tok is not None:
            print("continuation text:", tok.decode(out[0]))
        return 0
    if args.command == "generate":
        with open(args.prompts_file) as f:
            prompts = [[int(t) for t in line.replace(",", " ").split()] for line in f if line.strip()]
        for o in _generate(args, prompts):
            print(" ".join(str(t) for t in o))
        return 0


if __name__ == "__main__":
    sys.exit(main())
