"""Measurement: decode tokens per second of Gemma-2 layer sizes with random weights on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--layers L] [--dtype bfloat16|float32]
                    [--sizes 2b|9b|27b] [--prompt T] [--batch B] [--unequal] [--no-graph] [--no-points]
    python -m trapetum_amd bench ...                                   (the same)

A step is one decode step of the generation loop (`BatchRun.advance`, what `generate()` runs): every sequence of
the batch one token, chosen greedily on the device and fed to the next step, the host reading the ids one step
behind.  One JSON line is printed: decode tokens per second as `value`, the prefill of 2,048 tokens, the decode
step's share of the HBM roofline, and decode at batch 1 and 64 and a whole `generate()` call as `points`.
Fractions are given against the published peaks of the MI355X and (`frac_probe`) against what two probe kernels
measure on this GPU: a streaming read and a loop of matrix instructions.  Default sizes are those of the Gemma-2
2B configuration (26 layers, hidden 2304, 8 heads on 4 kv heads of 256, feed-forward 9216, vocabulary 256000,
window 4096, caps 50 / 30), context 8192, a batch of 8, prompts of 512 tokens; weights and token ids are seeded
random numbers.  `--unequal` draws the prompts' lengths uniformly from 64 to 2,048.  The reference times its own
loop the same way: warm-up, then the decode steps alone, a sync before the clock stops
(runtime/src/bin/gemma_run.rs:14-18).
"""
import argparse
import json
import sys
import time

PEAK_HBM_GBS = 8000.0
PEAK_FLOPS = {"bfloat16": 2.5e15, "float32": 157.3e12}

SIZES = dict(num_hidden_layers=26, hidden_size=2304, num_attention_heads=8, num_key_value_heads=4, head_dim=256,
             intermediate_size=9216, vocab_size=256000, rms_norm_eps=1e-6, rope_theta=10000.0, sliding_window=4096,
             query_pre_attn_scalar=256, attn_logit_softcapping=50.0, final_logit_softcapping=30.0,
             max_position_embeddings=8192)
# the other two Gemma-2 sizes, for `--sizes`: what differs from the 2B configuration
OTHER_SIZES = {
    "2b": {},
    "9b": dict(num_hidden_layers=42, hidden_size=3584, num_attention_heads=16, num_key_value_heads=8, intermediate_size=14336),
    "27b": dict(num_hidden_layers=46, hidden_size=4608, num_attention_heads=32, num_key_value_heads=16, head_dim=128,
                intermediate_size=36864, query_pre_attn_scalar=144),
}
CONTEXT, PROMPT, PREFILL_TOKENS, BATCH = 8192, 512, 2048, 8
UNEQUAL = (64, 2048)


def weight_bytes(c, itemsize):
    q, kv = c.num_attention_heads * c.head_dim, c.num_key_value_heads * c.head_dim
    per_layer = c.hidden_size * (q + 2 * kv) + q * c.hidden_size + 3 * c.hidden_size * c.intermediate_size
    return (c.num_hidden_layers * per_layer + c.vocab_size * c.hidden_size) * itemsize


def kv_bytes(c, context, itemsize):
    """Bytes of keys and values one sequence of `context` tokens reads in a decode step."""
    per_row = 2 * c.num_key_value_heads * c.head_dim * itemsize
    rows = sum(min(context, c.sliding_window) if c.layer_is_local(l) else context for l in range(c.num_hidden_layers))
    return rows * per_row


def prefill_flops(c, tokens):
    q, kv = c.num_attention_heads * c.head_dim, c.num_key_value_heads * c.head_dim
    per_layer = c.hidden_size * (q + 2 * kv) + q * c.hidden_size + 3 * c.hidden_size * c.intermediate_size
    linear = 2.0 * tokens * c.num_hidden_layers * per_layer
    attn = 0.0
    for l in range(c.num_hidden_layers):
        w = c.sliding_window if c.layer_is_local(l) else tokens
        pairs = sum(min(p + 1, w) for p in range(tokens))
        attn += 4.0 * pairs * q
    head = 2.0 * c.vocab_size * c.hidden_size
    return linear + attn + head


def main(argv=None):
    ap = argparse.ArgumentParser(prog="bench", description=__doc__.split("\n\n")[0])
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=64)
    ap.add_argument("--warmup", type=int, default=8)
    ap.add_argument("--sizes", default="2b", choices=sorted(OTHER_SIZES), help="layer sizes of which Gemma-2 (the metric is 2b)")
    ap.add_argument("--layers", type=int, default=0, help="fewer layers than the configuration's, if memory or time needs it")
    ap.add_argument("--batch", type=int, default=BATCH, help="sequences of the timed decode steps (the metric: 8)")
    ap.add_argument("--prompt", type=int, default=PROMPT, help="tokens of each prompt before decoding (the metric: 512)")
    ap.add_argument("--unequal", action="store_true", help=f"prompt lengths drawn uniformly from {UNEQUAL[0]} to {UNEQUAL[1]}")
    ap.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "float32"])
    ap.add_argument("--no-points", action="store_true", help="skip decode at batch 1 and 64 and the generate() call")
    ap.add_argument("--no-graph", action="store_true", help="launch decode steps kernel by kernel instead of replaying a HIP graph")
    args = ap.parse_args(argv)
    if args.gpus != 1:
        print(f"bench.py measures one GPU: this library runs on a single MI355X, --gpus {args.gpus} is not supported")
        return 2
    if args.steps < 1 or args.warmup < 0 or (args.warmup < 1 and not args.no_graph):
        print("bench.py: --steps must be at least 1, and --warmup at least 1 with HIP graphs (the first step of a batch "
              "size captures its graph, which is no decode step's time)")
        return 2

    import torch

    from .config import Gemma2Config
    from .engine import Engine
    from .engine.generate import BatchRun
    from .sampling import Sampler, SamplingParams

    sizes = dict(SIZES, **OTHER_SIZES[args.sizes])
    full_layers = sizes["num_hidden_layers"]
    cfg = Gemma2Config.from_kwargs(**dict(sizes, num_hidden_layers=args.layers or full_layers))
    itemsize = 2 if args.dtype == "bfloat16" else 4
    longest = UNEQUAL[1] if args.unequal else args.prompt
    if longest + args.steps + args.warmup + 2 > CONTEXT:
        print(f"bench.py: prompts of {longest} tokens and {args.steps + args.warmup} steps exceed the context of {CONTEXT}")
        return 2
    t0 = time.time()
    rows = args.batch if args.no_points else max(64, args.batch)
    room = args.steps + args.warmup + 128                       # what a sequence may grow by, whole pages and all
    most = max(PREFILL_TOKENS, args.batch * (longest + room), 0 if args.no_points else 64 * (args.prompt + room))
    engine = Engine.from_config(cfg, seed=2, sigma=0.02, dtype=args.dtype, draw_on_device=True,
                                max_tokens_in_cache=max(64 * 1024, most), max_context=CONTEXT, max_batch=rows,
                                use_graph=not args.no_graph)
    model, cache = engine.model, engine.cache
    torch.cuda.synchronize()
    print(f"[bench] model ready in {time.time() - t0:.1f}s", file=sys.stderr, flush=True)
    probe_gbs, probe_flops = model.rt.ops.measured_ceilings()
    print(f"[bench] probes: streaming read {probe_gbs:.0f} GB/s, bf16 matrix loop {probe_flops / 1e12:.0f} TFLOP/s", file=sys.stderr, flush=True)
    gen = torch.Generator().manual_seed(2)

    def prompts(lengths):
        return [torch.randint(0, cfg.vocab_size, (n,), generator=gen).tolist() for n in lengths]

    # ---- prefill: one sequence of 2,048 tokens ----------------------------------------------------------
    def prefill_once():
        s = cache.acquire()
        toks = prompts([PREFILL_TOKENS])[0]
        torch.cuda.synchronize()
        t = time.perf_counter()
        model.step(cache, [s], toks, counts=[PREFILL_TOKENS])
        torch.cuda.synchronize()
        dt = time.perf_counter() - t
        cache.release(s)
        return dt
    prefill_once()
    pre_s = min(prefill_once() for _ in range(3))
    pre_flops = prefill_flops(cfg, PREFILL_TOKENS)
    prefill = {"value": round(PREFILL_TOKENS / pre_s, 1), "tokens": PREFILL_TOKENS, "ms": round(pre_s * 1e3, 3),
               "frac": round(pre_flops / pre_s / PEAK_FLOPS[args.dtype], 4)}
    if args.dtype == "bfloat16":
        prefill["frac_probe"] = round(pre_flops / pre_s / probe_flops, 4)
    print(f"[bench] prefill {prefill}", file=sys.stderr, flush=True)

    # ---- decode: the generation loop's own steps ----------------------------------------------------------------
    sampler = Sampler(model.rt, SamplingParams())              # greedy

    def decode(lengths, steps, warmup):
        items = [(i, p, i) for i, p in enumerate(prompts(lengths))]
        run = BatchRun(model, cache, items, 1 << 30, sampler, 0, set(), graphs=engine.graphed)
        try:
            run.prefill()
            for _ in range(warmup):
                run.advance()
            torch.cuda.synchronize()
            t = time.perf_counter()
            for _ in range(steps):
                run.advance()
            torch.cuda.synchronize()
            dt = time.perf_counter() - t
        finally:
            run.close()
        return dt, [n + warmup + steps / 2.0 for n in lengths]

    if args.unequal:
        lengths = torch.randint(UNEQUAL[0], UNEQUAL[1] + 1, (args.batch,), generator=torch.Generator().manual_seed(3)).tolist()
    else:
        lengths = [args.prompt] * args.batch
    dt, contexts = decode(lengths, args.steps, args.warmup)
    ms_step = dt / args.steps * 1e3
    value = args.batch * args.steps / dt
    step_bytes = weight_bytes(cfg, itemsize) + sum(kv_bytes(cfg, int(c), itemsize) for c in contexts)
    achieved = step_bytes / (dt / args.steps) / 1e9
    roofline = {"bound": "hbm", "achieved": round(achieved, 1), "peak": PEAK_HBM_GBS, "unit": "GB/s",
                "frac": round(achieved / PEAK_HBM_GBS, 4), "peak_probe": round(probe_gbs, 1),
                "frac_probe": round(achieved / probe_gbs, 4)}
    points = {}
    if not args.no_points:
        for b in (1, 64):
            n = max(8, args.steps // 2)
            d, _ = decode([args.prompt] * b, n, max(2, args.warmup // 2))
            points[f"decode_b{b}"] = round(b * n / d, 1)
            print(f"[bench] decode batch {b}: {points[f'decode_b{b}']} tok/s", file=sys.stderr, flush=True)
        # a whole generate() call, prompts and all: what a user of the entry point gets
        ps, new = prompts([args.prompt] * 8), 128
        engine.generate(ps, max_tokens=4, stop_ids=())
        torch.cuda.synchronize()
        t = time.perf_counter()
        engine.generate(ps, max_tokens=new, stop_ids=())
        torch.cuda.synchronize()
        points["generate_b8"] = round(8 * new / (time.perf_counter() - t), 1)
        print(f"[bench] generate() of 8 prompts, {new} tokens each, prefill included: {points['generate_b8']} tok/s", file=sys.stderr, flush=True)

    line = {
        "metric": f"decode tok/s @ batch {args.batch}, Gemma-2-{args.sizes.upper()} layer sizes", "value": round(value, 1), "unit": "tok/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(ms_step, 4),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "bf16" if args.dtype == "bfloat16" else "fp32",
        "data": "synthetic: seeded random weights N(0, 0.02) and uniform-random token ids",
        "config": {"model": f"gemma-2-{args.sizes} sizes", "layers": cfg.num_hidden_layers, "layers_full": full_layers,
                   "hidden": cfg.hidden_size, "heads": cfg.num_attention_heads, "kv_heads": cfg.num_key_value_heads,
                   "head_dim": cfg.head_dim, "intermediate": cfg.intermediate_size, "vocab": cfg.vocab_size,
                   "window": cfg.sliding_window, "global_batch": args.batch, "seq_len": CONTEXT,
                   "prompt_len": round(sum(lengths) / len(lengths), 1), "prompts": "unequal" if args.unequal else "equal",
                   "decode_context": round(sum(contexts) / len(contexts), 1), "hip_graph": not args.no_graph,
                   "loop": "generate", "parallelism": "single GPU"},
        "prefill": prefill, "roofline": roofline, "points": points,
    }
    print(json.dumps(line), flush=True)
    return 0
