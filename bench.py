"""Decode and prefill throughput of the Llama-3.1-8B shape on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

A step is one decode step of a batch of 8 sequences (128-token random prompts, cache of
4,096 positions per sequence, random bfloat16 weights, greedy sampling on the device).
W untimed steps, then exactly K timed steps between device synchronisations.  Prints one
JSON line: ``value`` is decoded tokens per second; ``prefill`` is one 2,048-token prompt;
``roofline`` compares the bytes a decode step must read (every weight once, the cache of
the live sequences) per second with the HBM peak; ``points`` holds decode at batch 1 and 64;
``vs_baseline`` compares the batch-1 point with the reference's published batch-1 number.

Other workloads of the same program: ``--preset`` (another shape), ``--context`` (cache
positions per sequence), ``--prompt-lens LO:HI`` (prompts of unequal, seeded random lengths;
adds the ragged prefill's tokens per second), ``--prefill-only`` (just the timed prompt, for
profiling), ``--parts`` (no model: a layer's products at ``--batch`` rows and the prompt
attention at ``--prefill-tokens`` tokens, each timed alone).  The line also holds what this GPU reaches with a bare read stream and a bare
matrix-instruction loop (``measured_peaks``, and the step's fractions of them beside the
fractions of the datasheet peaks), the per-step time of each of the ``--runs`` timed regions
(``ms_per_step`` is their median) and the peak device memory in use.
"""
import argparse
import json
import os
import random
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0                 # MI355X HBM3E
MFMA_PEAK_TFLOPS = {"bf16": 2500.0, "fp32": 157.3}
BASELINE_TOK_S = 93.89                # reference README: Llama-3.1-8B bf16, batch 1, A100


def log(msg):
    print(msg, file=sys.stderr, flush=True)


def decode_run(engine, prompt_lens, warmup, steps, use_graph=True, warm_prefill=False, runs=3):
    """(seconds per step, bytes a step reads, seconds of the prefill, seconds per step of
    every run) for decode steps of sequences with the given prompt lengths: ``warmup``
    untimed steps, then ``runs`` timed regions of exactly ``steps`` steps each, one after
    the other in the same session; the first figure is the median region's."""
    import torch
    from gpt_fast_amd import Entry
    from gpt_fast_amd.engine.decode import DecodeSession
    from gpt_fast_amd.sampling import SamplingParams, sample
    batch = len(prompt_lens)
    g = torch.Generator().manual_seed(batch)
    V = engine.vocab_size
    slots = [engine.start_sequence() for _ in range(batch)]
    entries = [Entry(s, torch.randint(0, V, (n,), generator=g).tolist(), want=[n - 1], key=i)
               for i, (s, n) in enumerate(zip(slots, prompt_lens))]
    params = SamplingParams(temperature=0.0)

    def prefill(items):
        # in pieces of at most 8 prompts to bound activation memory
        out = []
        for i in range(0, len(items), 8):
            b = engine.prepare(items[i:i + 8])
            logits = engine.model.forward(b, engine.cache)
            out.append(sample(logits, params, b.row_keys, None))
        return torch.cat(out)

    if warm_prefill:
        # the same prompts once before, in slots of their own: the timed prefill then runs
        # with the libraries' first-use work (kernel selection, module loading) behind it
        spare = [engine.start_sequence() for _ in range(min(batch, 8))]
        prefill([Entry(s, e.tokens, want=[len(e.tokens) - 1], key=e.key) for s, e in zip(spare, entries)])
        torch.cuda.synchronize()
        for s in spare:
            engine.end_sequence(s)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    first = prefill(entries)
    torch.cuda.synchronize()
    prefill_seconds = time.perf_counter() - t0
    sess = DecodeSession(engine, slots, list(range(batch)), first, params, use_graph=use_graph,
                         max_new_tokens=warmup + runs * steps + 1)
    for _ in range(warmup):
        sess.advance()
    per_run = []
    for _ in range(runs):
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(steps):
            sess.advance()
        torch.cuda.synchronize()
        per_run.append((time.perf_counter() - t0) / steps)
    median_run = sorted(range(runs), key=lambda r: per_run[r])[runs // 2]
    dt = per_run[median_run]
    sess.close()
    # bytes of the median run's middle step: weights once + keys and values of every live token
    ctx = sum(n + warmup + median_run * steps + steps // 2 for n in prompt_lens)
    kv_bytes = sum(g.bytes_per_token() for _, g in engine.cache.kv_groups) * ctx
    step_bytes = engine.model.parameter_bytes() + kv_bytes
    for s in slots:
        engine.end_sequence(s)
    return dt, step_bytes, prefill_seconds, per_run


def prefill_run(engine, n_tokens, repeats=3):
    import torch
    from gpt_fast_amd import Entry
    g = torch.Generator().manual_seed(7)
    toks = torch.randint(0, engine.vocab_size, (n_tokens,), generator=g).tolist()
    times = []
    for r in range(repeats + 1):
        slot = engine.start_sequence()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        engine.step([Entry(slot, toks, want=[n_tokens - 1])])
        torch.cuda.synchronize()
        dt = time.perf_counter() - t0
        engine.end_sequence(slot)
        if r > 0:                                  # the first run is the warm-up
            times.append(dt)
    return sorted(times)[len(times) // 2]          # median


def parts_run(sizes, rows, prompt_tokens):
    """Microseconds of a layer's products at ``rows`` rows of x, each through the dispatch of
    ``ops.linear`` as a step calls it (weights cycled through enough copies that none stays in
    a cache; twenty calls recorded as one HIP graph, so launches do not count), and of the
    prompt attention over ``prompt_tokens`` tokens of one sequence (least of four rounds)."""
    import torch
    from gpt_fast_amd.ops import attention_bf16 as A
    from gpt_fast_amd.ops import linear as L
    dev = "cuda:0"
    D, H, G, hd = sizes["dim"], sizes["n_head"], sizes["n_kv_heads"], sizes["head_dim"]
    inner, V = sizes["intermediate_size"], sizes["vocab_size"]

    class Norm:
        def __init__(self, n):
            self.w = torch.ones(n, device=dev)

        def row_and_column_form(self):
            return self.w, 1e-5

    def timed(fn, n=20):
        fn(0)
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            for i in range(n):
                fn(i)
        graph.replay()
        torch.cuda.synchronize()
        best = None
        for _ in range(3):
            a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            a.record()
            graph.replay()
            b.record()
            torch.cuda.synchronize()
            t = a.elapsed_time(b) / n * 1e3
            best = t if best is None else min(best, t)
        return best

    products = {}
    shapes = {"wqkv": ((H + 2 * G) * hd, D), "wo": (D, H * hd), "w13": (2 * inner, D),
              "w2": (D, inner), "head": (V, D)}
    for name, (N, K_) in shapes.items():
        copies = max(2, int(700e6 // (N * K_ * 2)) + 1)
        ws = [(torch.randn(N, K_, device=dev) * 0.02).bfloat16() for _ in range(copies)]
        x = torch.randn(rows, K_, device=dev).bfloat16()
        res = torch.zeros(rows, N, device=dev) if name in ("wo", "w2") else None
        norm = Norm(N)
        if name == "wqkv":
            fn = lambda i: L.linear(x, ws[i % copies], may_stay_sliced=True)    # the rotation adds slices
        elif name == "w13":
            fn = lambda i: L.gated_linear(x, ws[i % copies])
        elif name == "head":
            fn = lambda i: L.linear(x, ws[i % copies], out_dtype=torch.float32)
        else:
            fn = lambda i: L.linear_into(x, ws[i % copies], res, norm)          # sum and next norm ride along
        for i in range(copies):
            fn(i)                                  # second copies of the weights are made outside the recording
        us = timed(fn)
        products[name] = {"us": round(us, 1), "tb_s": round(N * K_ * 2 / us / 1e6, 2)}
        log(f"[bench] {name:5s} {rows:3d} rows: {us:7.1f} us  {N * K_ * 2 / us / 1e6:5.2f} TB/s of weights")
        del ws

    T = prompt_tokens
    width = (T + 63) // 64
    k = torch.randn(width + 1, G, 64, hd, device=dev).bfloat16()
    v = torch.randn(width + 1, G, hd, 64, device=dev).bfloat16()
    q = torch.randn(T, H, hd, device=dev).bfloat16()

    class Step:
        n_seqs, max_q_len = 1, T
        q_start = torch.tensor([0, T], dtype=torch.int32, device=dev)
        start_pos = torch.zeros(1, dtype=torch.int32, device=dev)

    table = torch.arange(width, dtype=torch.int32, device=dev).view(1, width)
    best = None
    for _ in range(4):
        A.attention(q, k, v, Step, table, hd ** -0.5, 0)
        torch.cuda.synchronize()
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        a.record()
        for _ in range(10):
            A.attention(q, k, v, Step, table, hd ** -0.5, 0)
        b.record()
        torch.cuda.synchronize()
        t = a.elapsed_time(b) * 100
        best = t if best is None else min(best, t)
    flops = 4.0 * H * hd * T * (T + 1) / 2
    log(f"[bench] prompt attention {T} tokens: {best:.1f} us  {flops / best / 1e6:.0f} TFLOP/s of causal work")
    return {"products": products,
            "prompt_attention": {"tokens": T, "us": round(best, 1), "tflops": round(flops / best / 1e6, 1),
                                 "frac": round(flops / best / 1e6 / MFMA_PEAK_TFLOPS["bf16"], 4)}}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=256)
    ap.add_argument("--warmup", type=int, default=16)
    ap.add_argument("--layers", type=int, default=None, help="run fewer layers than the model has")
    ap.add_argument("--batch", type=int, default=8, help="sequences decoded together (headline: 8)")
    ap.add_argument("--preset", default="llama-3.1-8b",
                    help="shape to run (headline: llama-3.1-8b; others: 7B, llama-3.1-70b, ...)")
    ap.add_argument("--architecture", default=None, help="architecture that knows the preset")
    ap.add_argument("--prompt-len", type=int, default=128)
    ap.add_argument("--prompt-lens", default=None, metavar="LO:HI",
                    help="prompts of unequal lengths, uniform in [LO, HI], seeded")
    ap.add_argument("--context", type=int, default=4096, help="cache positions per sequence")
    ap.add_argument("--prefill-tokens", type=int, default=2048, help="length of the timed prompt")
    ap.add_argument("--prefill-only", action="store_true", help="time the prompt and nothing else")
    ap.add_argument("--runs", type=int, default=3,
                    help="timed regions of --steps steps each; the median one is reported")
    ap.add_argument("--parts", action="store_true",
                    help="time a layer's products at --batch rows and the prompt attention at "
                         "--prefill-tokens alone, no model")
    ap.add_argument("--no-graph", action="store_true")
    ap.add_argument("--no-points", action="store_true", help="skip batch 1, batch 64 and prefill")
    args = ap.parse_args()
    if args.gpus != 1:
        print(f"bench.py measures one GPU; --gpus {args.gpus} is not supported by this library")
        sys.exit(2)

    import torch
    import gpt_fast_amd as gfa

    arch, cfg = gfa.find_preset(args.preset, args.architecture)
    raw = arch.config_dict(cfg)
    full_layers = raw[arch.layer_count_key]
    if args.layers:
        raw[arch.layer_count_key] = args.layers
        cfg = arch.read_config(raw)
    sizes = dict(arch.describe(cfg)) if arch.describe is not None else {}
    n_layers = raw[arch.layer_count_key]
    batch, context = args.batch, args.context
    if args.parts:
        print(json.dumps({"metric": f"kernels alone; {args.preset} bf16", "rows": batch,
                          **parts_run(sizes, batch, args.prefill_tokens)}), flush=True)
        return
    if args.prompt_lens:
        lo, hi = (int(v) for v in args.prompt_lens.split(":"))
        rng = random.Random(batch)
        prompt_lens = [rng.randint(lo, hi) for _ in range(batch)]
    else:
        prompt_lens = [args.prompt_len] * batch
    rows = batch if args.no_points or args.prefill_only else max(64, batch)
    if args.prompt_lens:
        rows += min(batch, 8)                       # slots for the untimed first pass of the prompts
    t0 = time.time()
    engine = gfa.Engine.from_random(arch.names[0], cfg, seed=0, dtype="bfloat16", device="cuda:0",
                                    max_tokens=max(rows * context, args.prefill_tokens + 64),
                                    max_sequences=rows)
    torch.cuda.synchronize()
    log(f"[bench] model ready in {time.time() - t0:.1f} s")

    model_name = "Llama-3.1-8B" if args.preset == "llama-3.1-8b" else args.preset
    # the reference's published number is for this shape only
    headline = args.preset == "llama-3.1-8b" and not args.layers
    use_graph = not args.no_graph
    T = args.prefill_tokens

    def prefill_point():
        pt = prefill_run(engine, T)
        flops = engine.model.step_flops([T], [0], n_want=1)      # what the parts count
        log(f"[bench] prefill {T}: {pt * 1e3:.2f} ms")
        return {"value": round(T / pt, 1), "tokens": T, "ms": round(pt * 1e3, 3),
                "frac": round(flops / pt / 1e12 / MFMA_PEAK_TFLOPS["bf16"], 4)}

    def with_measured(point, measured):
        point["frac_of_measured"] = round(point["frac"] * MFMA_PEAK_TFLOPS["bf16"]
                                          / measured["mfma_bf16_tflops"], 4)
        return point

    if args.prefill_only:
        print(json.dumps({"metric": f"prefill tok/s @ {T} tokens; {model_name} bf16",
                          "n_layer": n_layers, "prefill": prefill_point()}), flush=True)
        return

    runs = max(1, args.runs)
    if max(prompt_lens) + args.warmup + runs * args.steps + 1 > context:
        print(f"prompt ({max(prompt_lens)}) + {args.warmup + runs * args.steps + 1} decoded tokens "
              f"exceed --context {context}")
        sys.exit(2)
    from gpt_fast_amd.ops import ceilings
    measured = ceilings.measure("cuda:0")          # a few milliseconds of bare kernels
    log(f"[bench] this GPU: {measured}")
    dt, step_bytes, prefill_s, per_run = decode_run(engine, prompt_lens, args.warmup, args.steps,
                                                    use_graph, warm_prefill=bool(args.prompt_lens),
                                                    runs=runs)
    value = batch / dt
    log(f"[bench] decode b{batch}: {dt * 1e3:.3f} ms/step, {value:.1f} tok/s")
    out = {
        "metric": f"decode tok/s @ batch {batch}; {model_name} bf16", "value": round(value, 2),
        "unit": "tokens/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(dt * 1e3, 4), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": round(value / BASELINE_TOK_S, 3) if headline and batch == 1 else None,
        "dtype": "bf16", "data": "synthetic",
        "config": {
            "model": args.preset, **sizes, "n_layer_full": full_layers,
            "global_batch": batch, "seq_len": context,
            "prompt_len": args.prompt_lens or args.prompt_len,
            "new_tokens": args.warmup + runs * args.steps,
            "weights": "random N(0,0.02) bf16", "sampling": "greedy", "hip_graph": use_graph,
            "parallelism": "single GPU",
        },
        # ms_per_step is the median of these timed regions of `steps` steps each
        "runs_ms_per_step": [round(t * 1e3, 4) for t in per_run],
        "roofline": {"bound": "hbm", "achieved": round(step_bytes / dt / 1e9, 1),
                     "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(step_bytes / dt / 1e9 / HBM_PEAK_GBS, 4),
                     # what a bare read stream reaches on this GPU, and the step against that
                     "measured_peak": measured["hbm_read_gbs"],
                     "frac_of_measured": round(step_bytes / dt / 1e9 / measured["hbm_read_gbs"], 4)},
    }
    if args.prompt_lens:
        # the unequal prompts went through the engine in one step per eight of them (timed on
        # their second pass, in other slots than the first)
        out["ragged_prefill"] = {"value": round(sum(prompt_lens) / prefill_s, 1),
                                 "tokens": sum(prompt_lens), "ms": round(prefill_s * 1e3, 3),
                                 "lengths": " ".join(map(str, prompt_lens))}
    if not args.no_points:
        out["prefill"] = with_measured(prefill_point(), measured)
        points = {}
        for b in (1, 64):
            steps = min(args.steps, 128)
            d, _, _, _ = decode_run(engine, [args.prompt_len] * b, min(args.warmup, 8), steps, use_graph,
                                    runs=runs)
            points[f"decode_b{b}"] = round(b / d, 2)
            log(f"[bench] decode b{b}: {d * 1e3:.3f} ms/step, {b / d:.1f} tok/s")
        out["points"] = points
        if headline:
            # like for like: the reference's published number is its batch-1 decode speed
            out["vs_baseline"] = round(points["decode_b1"] / BASELINE_TOK_S, 3)
            out["vs_baseline_point"] = "decode_b1"
    out["measured_peaks"] = measured
    out["memory_gb"] = round(torch.cuda.max_memory_allocated() / 1e9, 2)
    print(json.dumps(out), flush=True)


if __name__ == "__main__":
    main()
