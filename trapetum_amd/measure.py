"""Measurement: decode tokens per second of Gemma-2 layer sizes with random weights on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--layers L] [--dtype bfloat16|float32]
                    [--sizes 2b|9b|27b] [--prompt T] [--batch B] [--unequal] [--no-graph] [--no-points]
    python -m trapetum_amd bench ...                                   (the same)

A step is one decode step of the generation loop (`BatchRun.advance`, what `generate()` runs): every sequence of
the batch one token, chosen greedily on the device and fed to the next step, the host reading the ids one step
behind.  One JSON line is printed: decode tokens per second as `value`, the prefill of 2,048 tokens, the decode
step's share of the HBM roofline, and as `points` decode at batch 1 and 64, a whole `generate()` call, decode at a
context of 7,900 tokens, and decode at batch 8 and the prefill of 2,048 tokens at the 9B and 27B layer sizes (all
their layers), each with its share of the published peak in `points_frac`; `kernels` times the kernels a decode step
of 8 sequences and a prefill of 2,048 tokens spend their time in, one by one, with HIP events at the same shapes
(the reference prints a per-operation breakdown from the program itself as well: runtime/src/lib.rs:3218-3245).
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
CONTEXT, PROMPT, PREFILL_TOKENS, BATCH, LONG_CONTEXT = 8192, 512, 2048, 8, 7900
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


def time_kernels(engine, cfg, batch, context, prefill_tokens):
    """Microseconds of the kernels that a decode step of `batch` sequences at `context` tokens and a prefill of
    `prefill_tokens` spend their time in, each called once per layer on that layer's own weights (so that no call
    finds its matrix in a cache), replayed from a HIP graph and timed with events.  {name: {"us", "GB/s" | "TFLOP/s", "frac"}}."""
    import torch
    model, ops, dev = engine.model, engine.model.rt.ops, engine.model.rt.device
    bf = torch.bfloat16
    layers = [l.block for l in model.layers]
    c = cfg
    H, KV, hd, D, I = c.num_attention_heads, c.num_key_value_heads, c.head_dim, c.hidden_size, c.intermediate_size
    out = {}

    def timed(name, calls, bytes_each=None, flops_each=None):
        calls = calls * max(1, -(-24 // len(calls)))       # enough calls a replay that its launch does not show
        calls[0]()                                         # outside the capture: first use of a kernel may compile or configure
        torch.cuda.synchronize()
        side = torch.cuda.Stream(device=dev)
        side.wait_stream(torch.cuda.current_stream(dev))
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.stream(side):
            with torch.cuda.graph(graph, stream=side):
                for f in calls:
                    f()
        torch.cuda.current_stream(dev).wait_stream(side)
        best = float("inf")
        for _ in range(4):
            a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            a.record()
            graph.replay()
            b.record()
            b.synchronize()
            best = min(best, a.elapsed_time(b) * 1e3 / len(calls))
        row = {"us": round(best, 2)}
        if bytes_each is not None:
            row["GB/s"] = round(bytes_each / best / 1e3, 1)
            row["frac"] = round(bytes_each / best / 1e3 / PEAK_HBM_GBS, 4)
        else:
            row["TFLOP/s"] = round(flops_each / best / 1e6, 1)
            row["frac"] = round(flops_each / (best * 1e-6) / PEAK_FLOPS["bfloat16"], 4)
        out[name] = row

    for rows, tag in ((batch, f"decode_b{batch}"), (prefill_tokens, f"prefill_{prefill_tokens}")):
        x = torch.randn((rows, D), device=dev).to(bf)
        xa = torch.randn((rows, H * hd), device=dev).to(bf)
        xi = torch.randn((rows, I), device=dev).to(bf)
        decode = rows == batch
        products = [("qkv", lambda b: ops.linear(x, b.mixer.w_qkv, bf, defer=decode), (H + 2 * KV) * hd * D),
                    ("o", lambda b: ops.linear(xa, b.mixer.w_o, bf, defer=True), D * H * hd),
                    ("gate_up", lambda b: ops.gated_linear(x, b.feed_forward.w_gate_up, I, b.feed_forward.activation, bf), 2 * I * D),
                    ("down", lambda b: ops.linear(xi, b.feed_forward.w_down, bf, defer=True), D * I)]
        for name, call, elems in products:
            calls = [(lambda b=b: call(b)) for b in layers]
            if decode:
                timed(f"{tag}.{name}", calls, bytes_each=2.0 * elems)
            else:
                timed(f"{tag}.{name}", calls, flops_each=2.0 * rows * elems)
    # attention: a prefill of `prefill_tokens` (all keys visible), and the decode step's fused rotation, cache write and
    # attention over `context` cached tokens
    q, k, v = (torch.randn((prefill_tokens, n * hd), device=dev).to(bf) for n in (H, KV, KV))
    cu = torch.tensor([0, prefill_tokens], dtype=torch.int32, device=dev)
    scale = c.query_pre_attn_scalar ** -0.5
    cap = c.attn_logit_softcapping or 0.0
    pairs = prefill_tokens * (prefill_tokens + 1) / 2.0
    timed(f"prefill_{prefill_tokens}.attention", [lambda: ops.attention_prefill(q, k, v, H, KV, hd, cu, prefill_tokens, scale, cap, 0, bf)] * 8,
          flops_each=4.0 * pairs * H * hd)
    cache = engine.cache
    slots = [cache.acquire() for _ in range(batch)]
    try:
        for s in slots:
            cache.grow(s, context)
        from .engine.batch import StepContext
        ctx = StepContext(model.rt, cache, slots, [1] * batch, [context - 1] * batch, list(range(batch)))
        sites = [cache.site(i) for i, e in enumerate(model.schedule) if cache.site(i) is not None and cache.site(i).rows_cap is None]
        site = sites[0]
        mixer = layers[1].mixer if len(layers) > 1 else layers[0].mixer
        qkv = torch.randn((batch, (H + 2 * KV) * hd), device=dev).to(bf)
        table = ctx.page_table(site.group_index)
        calls = [lambda: ops.attention_decode_step(qkv, H, KV, hd, mixer.inv_freq, mixer.position.rotary_dim, ctx.new_len, table,
                                                   site.tensor("k"), site.tensor("v"), 0, scale, cap, 0, bf, max_keys=context)] * 8
        timed(f"decode_b{batch}.attention_ctx{context}", calls, bytes_each=2.0 * batch * context * 2 * KV * hd)
    finally:
        for s in slots:
            cache.release(s)
    # the two launches between products: residual add with both norms
    stream = torch.randn((batch, D), device=dev)
    rows_b = torch.randn((batch, D), device=dev).to(bf)
    g = torch.ones(D, device=dev)
    timed(f"decode_b{batch}.add_rms_norm", [lambda: ops.add_rms_norm(stream, rows_b, g, 1e-6, g, 1e-6, bf)] * 16,
          bytes_each=batch * D * (4 + 4 + 2 + 2) + 8.0 * D)
    return out


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
    ap.add_argument("--no-points", action="store_true", help="skip the further points (other batches, contexts and sizes) and the kernels' times")
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

    itemsize = 2 if args.dtype == "bfloat16" else 4
    longest = UNEQUAL[1] if args.unequal else args.prompt
    if longest + args.steps + args.warmup + 2 > CONTEXT:
        print(f"bench.py: prompts of {longest} tokens and {args.steps + args.warmup} steps exceed the context of {CONTEXT}")
        return 2
    gen = torch.Generator().manual_seed(2)

    class Bench:
        """One size's engine and what is timed on it."""

        def __init__(self, which, rows, most_tokens):
            sizes = dict(SIZES, **OTHER_SIZES[which])
            self.full_layers = sizes["num_hidden_layers"]
            self.cfg = Gemma2Config.from_kwargs(**dict(sizes, num_hidden_layers=args.layers or self.full_layers))
            t0 = time.time()
            self.engine = Engine.from_config(self.cfg, seed=2, sigma=0.02, dtype=args.dtype, draw_on_device=True,
                                             max_tokens_in_cache=most_tokens, max_context=CONTEXT, max_batch=rows,
                                             use_graph=not args.no_graph)
            self.model, self.cache = self.engine.model, self.engine.cache
            self.sampler = Sampler(self.model.rt, SamplingParams())          # greedy
            torch.cuda.synchronize()
            print(f"[bench] {which} model ready in {time.time() - t0:.1f}s", file=sys.stderr, flush=True)

        def prompts(self, lengths):
            return [torch.randint(0, self.cfg.vocab_size, (n,), generator=gen).tolist() for n in lengths]

        def prefill(self):
            """Seconds of one sequence of 2,048 tokens in one step: the best of three after a first run."""
            def once():
                s = self.cache.acquire()
                toks = self.prompts([PREFILL_TOKENS])[0]
                torch.cuda.synchronize()
                t = time.perf_counter()
                self.model.step(self.cache, [s], toks, counts=[PREFILL_TOKENS])
                torch.cuda.synchronize()
                dt = time.perf_counter() - t
                self.cache.release(s)
                return dt
            once()
            return min(once() for _ in range(3))

        def decode(self, lengths, steps, warmup):
            """Seconds of `steps` steps of the generation loop after prompts of `lengths`, and each sequence's mean context."""
            items = [(i, p, i) for i, p in enumerate(self.prompts(lengths))]
            run = BatchRun(self.model, self.cache, items, 1 << 30, self.sampler, 0, set(), graphs=self.engine.graphed)
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

        def step_bytes(self, contexts):
            return weight_bytes(self.cfg, itemsize) + sum(kv_bytes(self.cfg, int(c), itemsize) for c in contexts)

        def close(self):
            del self.engine, self.model, self.cache, self.sampler
            torch.cuda.empty_cache()

    rows = args.batch if args.no_points else max(64, args.batch)
    room = args.steps + args.warmup + 128                       # what a sequence may grow by, whole pages and all
    most = max(PREFILL_TOKENS, args.batch * (longest + room), 0 if args.no_points else 64 * (args.prompt + room))
    bench = Bench(args.sizes, rows, max(64 * 1024 + 8 * 256, most))
    cfg, engine, model, full_layers = bench.cfg, bench.engine, bench.model, bench.full_layers
    probe_gbs, probe_flops = model.rt.ops.measured_ceilings()
    print(f"[bench] probes: streaming read {probe_gbs:.0f} GB/s, bf16 matrix loop {probe_flops / 1e12:.0f} TFLOP/s", file=sys.stderr, flush=True)

    # ---- prefill: one sequence of 2,048 tokens ----------------------------------------------------------
    pre_s = bench.prefill()
    pre_flops = prefill_flops(cfg, PREFILL_TOKENS)
    prefill = {"value": round(PREFILL_TOKENS / pre_s, 1), "tokens": PREFILL_TOKENS, "ms": round(pre_s * 1e3, 3),
               "frac": round(pre_flops / pre_s / PEAK_FLOPS[args.dtype], 4)}
    if args.dtype == "bfloat16":
        prefill["frac_probe"] = round(pre_flops / pre_s / probe_flops, 4)
    print(f"[bench] prefill {prefill}", file=sys.stderr, flush=True)

    # ---- decode: the generation loop's own steps ----------------------------------------------------------------
    if args.unequal:
        lengths = torch.randint(UNEQUAL[0], UNEQUAL[1] + 1, (args.batch,), generator=torch.Generator().manual_seed(3)).tolist()
    else:
        lengths = [args.prompt] * args.batch
    dt, contexts = bench.decode(lengths, args.steps, args.warmup)
    ms_step = dt / args.steps * 1e3
    value = args.batch * args.steps / dt
    achieved = bench.step_bytes(contexts) / (dt / args.steps) / 1e9
    roofline = {"bound": "hbm", "achieved": round(achieved, 1), "peak": PEAK_HBM_GBS, "unit": "GB/s",
                "frac": round(achieved / PEAK_HBM_GBS, 4), "peak_probe": round(probe_gbs, 1),
                "frac_probe": round(achieved / probe_gbs, 4)}
    points, points_frac, kernels = {}, {}, {}

    def decode_point(b, name, lens, steps, warmup):
        d, ctxs = b.decode(lens, steps, warmup)
        points[name] = round(len(lens) * steps / d, 1)
        points_frac[name] = round(b.step_bytes(ctxs) / (d / steps) / 1e9 / PEAK_HBM_GBS, 4)
        print(f"[bench] {name}: {points[name]} tok/s, {points_frac[name]} of {PEAK_HBM_GBS:.0f} GB/s", file=sys.stderr, flush=True)

    if not args.no_points:
        n = max(8, args.steps // 2)
        for b in (1, 64):
            decode_point(bench, f"decode_b{b}", [args.prompt] * b, n, max(2, args.warmup // 2))
        # a whole generate() call, prompts and all: what a user of the entry point gets
        ps, new = bench.prompts([args.prompt] * 8), 128
        engine.generate(ps, max_tokens=4, stop_ids=())
        torch.cuda.synchronize()
        t = time.perf_counter()
        engine.generate(ps, max_tokens=new, stop_ids=())
        torch.cuda.synchronize()
        points["generate_b8"] = round(8 * new / (time.perf_counter() - t), 1)
        print(f"[bench] generate() of 8 prompts, {new} tokens each, prefill included: {points['generate_b8']} tok/s", file=sys.stderr, flush=True)
        # a context near the configuration's end: the cache is most of what a step reads
        decode_point(bench, f"decode_b8_ctx{LONG_CONTEXT}", [LONG_CONTEXT] * 8, n, max(2, args.warmup // 2))
        if args.dtype == "bfloat16":
            kernels = time_kernels(engine, cfg, 8, args.prompt + 40, PREFILL_TOKENS)
            for name, row in kernels.items():
                print(f"[bench] kernel {name}: {row}", file=sys.stderr, flush=True)
        # the other sizes of the architecture, all their layers (or --layers of them)
        engine = model = None
        for which in ("9b", "27b") if args.sizes == "2b" else ():
            bench.close()
            bench = Bench(which, 8, max(PREFILL_TOKENS, 8 * (args.prompt + room)))
            s_pre = bench.prefill()
            points[f"prefill_2048_{which}"] = round(PREFILL_TOKENS / s_pre, 1)
            points_frac[f"prefill_2048_{which}"] = round(prefill_flops(bench.cfg, PREFILL_TOKENS) / s_pre / PEAK_FLOPS[args.dtype], 4)
            print(f"[bench] prefill_2048_{which}: {s_pre * 1e3:.1f} ms, {points_frac[f'prefill_2048_{which}']} of the matrix peak", file=sys.stderr, flush=True)
            decode_point(bench, f"decode_b8_{which}", [args.prompt] * 8, n, max(2, args.warmup // 2))
    bench.close()

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
        "prefill": prefill, "roofline": roofline, "points": points, "points_frac": points_frac, "kernels": kernels,
    }
    print(json.dumps(line), flush=True)
    return 0
