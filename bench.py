#!/usr/bin/env python3
"""Decode and prefill throughput of the engine on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--batch B] [--layers L]

The default run: a Llama-3.1-8B-shaped model (32 layers, width 4096, 32 heads on 8
KV heads of 128, feed-forward 14336, vocabulary 128256, llama3 rope scaling) with
random N(0, 0.02) weights in bfloat16, context window 8192, 8 requests with
1,024-token prompts of seeded uniform random ids.  A step is one decode step of
the scheduler (one new token for every request).  W untimed steps, then exactly K
timed steps between two synchronisations.  One JSON line is printed: decoded
tokens per second, the step's achieved fraction of the HBM roofline (every weight
read once plus the cache of the live requests), a 2,048-token prefill with its
fraction of the bf16 matrix peak, and under `points` decode at batch 1 and 64, the
same measurements at the 1B and 13B shapes of the architecture, and prefill and
decode at a context of 8,192 tokens.  Beside the published peaks the line gives what
the simplest kernels reach on the GPU it ran on (`measured_peak`: a read-only stream
over 4 GiB, a loop of nothing but matrix instructions; `--yardsticks` prints them alone).
"""
import argparse
import json
import sys
import time

HBM_PEAK = 8.0e12          # bytes/s, MI355X HBM3E
BF16_PEAK = 2.5e15         # dense MFMA flop/s
BASE_8B = dict(num_hidden_layers=32, hidden_size=4096, num_attention_heads=32, num_key_value_heads=8,
               head_dim=128, intermediate_size=14336, vocab_size=128256, max_position_embeddings=131072,
               rope_theta=500000.0, rms_norm_eps=1e-5, tie_word_embeddings=False,
               rope_scaling={"rope_type": "llama3", "factor": 8.0, "low_freq_factor": 1.0,
                             "high_freq_factor": 4.0, "original_max_position_embeddings": 8192})
# other shapes of the same architecture, for looking at kernels away from the default sizes
SHAPES = {
    "llama-3.1-8b": BASE_8B,
    "llama-3.2-1b": dict(BASE_8B, num_hidden_layers=16, hidden_size=2048, head_dim=64, intermediate_size=8192,
                         tie_word_embeddings=True,
                         rope_scaling=dict(BASE_8B["rope_scaling"], factor=32.0)),
    "llama-2-13b": dict(BASE_8B, num_hidden_layers=40, hidden_size=5120, num_attention_heads=40,
                        num_key_value_heads=40, intermediate_size=13824, vocab_size=32000,
                        max_position_embeddings=4096, rope_theta=10000.0, rope_scaling=None),
    "llama-3.2-3b": dict(BASE_8B, num_hidden_layers=28, hidden_size=3072, num_attention_heads=24,
                         intermediate_size=8192, tie_word_embeddings=True,
                         rope_scaling=dict(BASE_8B["rope_scaling"], factor=32.0)),
    "llama-2-7b": dict(BASE_8B, num_hidden_layers=32, num_key_value_heads=32, intermediate_size=11008,
                       vocab_size=32000, max_position_embeddings=4096, rope_theta=10000.0, rope_scaling=None),
    # (141 GB of weights: the layers bound last do without their second copy in tiles)
    "llama-3.1-70b": dict(BASE_8B, num_hidden_layers=80, hidden_size=8192, num_attention_heads=64,
                          intermediate_size=28672),
}
SHAPE_NAMES = {"llama-3.1-8b": "Llama-3.1-8B", "llama-3.2-1b": "Llama-3.2-1B", "llama-2-13b": "Llama-2-13B",
               "llama-3.2-3b": "Llama-3.2-3B", "llama-2-7b": "Llama-2-7B", "llama-3.1-70b": "Llama-3.1-70B"}
CONTEXT = 8192
PROMPT = 1024
PREFILL = 2048


def parse(argv=None):
    ap = argparse.ArgumentParser(prog="bench.py")
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=64)
    ap.add_argument("--warmup", type=int, default=8)
    ap.add_argument("--batch", type=int, default=8)
    ap.add_argument("--shape", choices=sorted(SHAPES), default="llama-3.1-8b")
    ap.add_argument("--layers", type=int, default=0, help="fewer layers than the shape has (0: all)")
    ap.add_argument("--no-points", action="store_true", help="skip the batch 1 / 64 and prefill measurements")
    ap.add_argument("--sampling", choices=["greedy", "default"], default="greedy",
                    help="decode with greedy sampling (the default run) or with the reference's default options "
                         "(temperature 0.8, top-k 40, top-p 0.9, repeat penalty 1.1 over 64 tokens)")
    ap.add_argument("--serving", type=int, default=0, metavar="R",
                    help="instead of the default run: R requests at once under continuous batching, prompts of "
                         "64 to 2,048 tokens, 128 new tokens each, context 4,096; prints its own line")
    ap.add_argument("--context", type=int, default=0, metavar="T",
                    help="instead of the default run: a prompt of T tokens in portions of 2,048, then decode "
                         "steps at that context with --batch requests; prints its own line")
    ap.add_argument("--prefill-only", action="store_true",
                    help="run only the 2,048-token prefill (for profiling); prints its own short line")
    ap.add_argument("--prefill-tokens", type=int, default=0, metavar="T",
                    help="with --prefill-only: a prompt of T tokens (65 to 2,048) in place of 2,048")
    ap.add_argument("--yardsticks", action="store_true",
                    help="only measure what the simplest kernels get from this GPU: a read-only stream over 4 GiB "
                         "and a loop of nothing but bfloat16 matrix instructions; prints its own line")
    ap.add_argument("--attention-alone", action="store_true",
                    help="only time the prefill attention kernel by itself: the last 2,048 rows of one sequence of "
                         "2,048, 8,192 and 32,768 tokens (heads and head size of --shape); prints its own line")
    ap.add_argument("--no-extra-points", action="store_true",
                    help="skip the other shapes and the longer context that the default run adds under `points`")
    return ap.parse_args(argv)


def yardsticks():
    """What the simplest possible kernels reach on this GPU: (GB/s of a read-only stream over
    4 GiB of device memory, TFLOP/s of a loop of nothing but bfloat16 matrix instructions)."""
    import torch
    from hfee_amd.kernels import ops
    buf = torch.empty(4 << 30, dtype=torch.uint8, device="cuda:0")
    buf.fill_(1)
    start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)

    def best(fn, reps=5):
        fn()
        torch.cuda.synchronize()
        times = []
        for _ in range(reps):
            start.record()
            fn()
            stop.record()
            torch.cuda.synchronize()
            times.append(start.elapsed_time(stop) * 1e-3)
        return min(times)
    read_s = best(lambda: ops.read_stream(buf, 2048, True))
    flops = ops.mfma_loop(1, 1)
    mfma_s = best(lambda: ops.mfma_loop(1000, 2048))
    flops = flops * 1000 * 2048
    del buf
    torch.cuda.empty_cache()
    return (4 << 30) / read_s / 1e9, flops / mfma_s / 1e12


def attention_alone(shape: dict) -> dict:
    """The prefill attention kernel by itself, as a yardstick for changes to it: one sequence of T
    tokens in the cache, its last 2,048 rows attending: {T: (microseconds, TFLOP/s)}."""
    import torch
    from hfee_amd.kernels import ops
    dev, page_size, rows = "cuda:0", 16, 2048
    heads, kv_heads = shape["num_attention_heads"], shape["num_key_value_heads"]
    head_dim = shape.get("head_dim") or shape["hidden_size"] // heads
    start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    out = {}
    for tokens in (2048, 8192, 32768):
        pages = (tokens + page_size - 1) // page_size
        cache = (torch.randn(pages, 2, kv_heads, page_size * head_dim, device=dev) * 0.5).to(torch.bfloat16)
        q = (torch.randn(rows, heads * head_dim, device=dev) * 0.5).to(torch.bfloat16)
        o = torch.zeros_like(q)
        tables = torch.arange(pages, dtype=torch.int32, device=dev).view(1, -1)
        tiles = torch.tensor([(r, 32, tokens - rows + r, 0) for r in range(0, rows, 32)], dtype=torch.int32, device=dev)
        runs = None
        if heads == kv_heads:      # heads that share no keys: row tiles that follow one another share them, four at a time
            runs = torch.tensor([(i, min(4, rows // 32 - i)) for i in range(0, rows // 32, 4)], dtype=torch.int32, device=dev)
        kernel = ops.prefill_attention_kernel(tiles.tolist(), 0, kv_heads, heads // kv_heads, head_dim)     # (as the engine chooses)
        call = lambda: ops.attention_bf16_prefill(o, q, cache, tiles, tables, heads, kv_heads, head_dim, page_size,
                                                  head_dim ** -0.5, runs=runs, kernel=kernel)
        call()
        torch.cuda.synchronize()
        best = float("inf")
        for _ in range(20):
            start.record()
            call()
            stop.record()
            torch.cuda.synchronize()
            best = min(best, start.elapsed_time(stop) * 1e3)
        visible = sum(tokens - rows + r + 1 for r in range(rows))          # keys that the rows see, causal
        out[tokens] = (round(best, 1), round(4.0 * visible * head_dim * heads / best / 1e6, 1))
        del cache
    return out


def main(argv=None) -> int:
    args = parse(argv)
    if args.gpus != 1:
        print(f"bench.py: this engine runs on one GPU; --gpus {args.gpus} is not supported")
        return 2
    if args.yardsticks:
        import hfee_amd  # noqa: F401
        gbs, tflops = yardsticks()
        print(json.dumps({"read_stream_gb_per_s": round(gbs, 1), "hbm_published_gb_per_s": HBM_PEAK / 1e9,
                          "mfma_loop_tflop_per_s": round(tflops, 1), "bf16_published_tflop_per_s": BF16_PEAK / 1e12}),
              flush=True)
        return 0
    if args.attention_alone:
        import hfee_amd  # noqa: F401
        timed = attention_alone(SHAPES[args.shape])
        print(json.dumps({"kernel": "prefill attention alone, the last 2,048 rows of a sequence", "shape": args.shape,
                          "microseconds": {str(t): v[0] for t, v in timed.items()},
                          "tflop_per_s": {str(t): v[1] for t, v in timed.items()}}), flush=True)
        return 0
    line = run(args)
    if isinstance(line, int):
        return line
    if "points" in line and not args.no_extra_points and args.shape == "llama-3.1-8b" and not args.layers:
        import copy
        import torch
        torch.cuda.empty_cache()
        # the same measurements at the other shapes of the architecture and at a longer context
        for shape in ("llama-3.2-1b", "llama-2-13b"):
            other = copy.copy(args)
            other.shape, other.no_points, other.steps, other.warmup = shape, False, min(args.steps, 32), min(args.warmup, 4)
            other.point_batches = (1, 64)
            got = run(other)
            torch.cuda.empty_cache()
            line["points"][f"decode_b8_{shape}"] = got["value"]
            line["points"][f"decode_b8_hbm_frac_{shape}"] = got["roofline"]["frac"]
            for key, value in got["points"].items():
                line["points"][f"{key}_{shape}"] = value
            line["points"][f"prefill_2048_{shape}"] = got["prefill"]["value"]
            line["points"][f"prefill_2048_frac_{shape}"] = got["prefill"]["frac"]
        # continuous batching at the small shape: 128 requests at once, prompts of 64 to 2,048
        # tokens, 128 new tokens each
        serving = copy.copy(args)
        serving.shape, serving.serving = "llama-3.2-1b", 128
        got = run(serving)
        torch.cuda.empty_cache()
        line["points"]["serving_128_generated_tok_s_llama-3.2-1b"] = got["value"]
        line["points"]["serving_128_all_tok_s_llama-3.2-1b"] = got["all_tokens_per_s"]
        if got.get("gpu_ms_from_first_step_to_last"):
            line["points"]["serving_128_gpu_inside_steps_frac_llama-3.2-1b"] = round(
                got["gpu_ms_inside_steps"] / got["gpu_ms_from_first_step_to_last"], 4)
        longer = copy.copy(args)
        longer.context, longer.steps, longer.warmup = 8192, min(args.steps, 16), 2
        got = run(longer)
        torch.cuda.empty_cache()
        line["points"]["prefill_8192"] = got["prefill"]["value"]
        line["points"]["prefill_8192_frac"] = got["prefill"]["frac"]
        line["points"]["decode_b8_ctx8192"] = got["decode"]["value"]
        line["points"]["decode_b8_ctx8192_hbm_frac"] = got["decode"]["hbm_frac"]
        gbs, tflops = yardsticks()
        line["roofline"]["measured_peak"] = round(gbs, 1)
        line["roofline"]["frac_of_measured"] = round(line["roofline"]["achieved"] / gbs, 4)
        line["prefill"]["measured_peak_tflops"] = round(tflops, 1)
    print(json.dumps(line), flush=True)
    return 0


def run(args):
    """One measurement as the arguments say; returns the record to print (or an exit code)."""
    import torch

    import hfee_amd  # noqa: F401
    from hfee_amd.config import config_from_dict
    from hfee_amd.engine import Engine, Request, Scheduler, random_model
    from hfee_amd.sampling import Sampler, SamplingParams

    base = SHAPES[args.shape]
    context = min(CONTEXT, base["max_position_embeddings"])
    cj = dict(base, architectures=["LlamaForCausalLM"], num_hidden_layers=args.layers or base["num_hidden_layers"])
    cfg = config_from_dict(cj)
    t0 = time.perf_counter()
    model = random_model(cfg, seed=0, dtype="bfloat16", device="cuda:0", std=0.02)
    torch.cuda.synchronize()
    print(f"[bench] random weights made in {time.perf_counter() - t0:.1f} s", file=sys.stderr, flush=True)

    L, d, H, K, hd = cfg.num_hidden_layers, cfg.hidden_size, cfg.num_attention_heads, cfg.num_key_value_heads, cfg.head_dim
    F, V = cfg.intermediate_size, cfg.vocab_size
    layer_params = d * (H + 2 * K) * hd + H * hd * d + 3 * d * F
    weight_bytes = 2 * (L * layer_params + V * d)              # every matrix a decode step reads, once
    kv_bytes_per_token = L * 2 * K * hd * 2
    max_batch = max(64 if args.no_points else 128, args.batch, args.serving)
    steps_total = args.steps + args.warmup

    page_size = 16
    # (while the later prompts are read, the earlier requests already decode: a token a step)
    tokens_cached = max_batch * (PROMPT + steps_total + page_size + max_batch * PROMPT // PREFILL) + PREFILL + page_size
    if args.serving:
        context = min(context, 4096)
        tokens_cached = args.serving * (2048 + 128 + page_size)
    if args.context:
        # the first requests go on decoding while the later ones run their prompts
        context = args.context + args.batch * (args.context // PREFILL + 2) + steps_total + page_size
        if context > base["max_position_embeddings"]:
            print(f"bench.py: --context {args.context} is beyond what the shape allows")
            return 2
        tokens_cached = args.batch * (context + page_size)
    engine = Engine(model, cache_tokens=tokens_cached, page_size=page_size, max_requests=max_batch,
                    max_batch_tokens=PREFILL, num_positions=context)
    sampler = Sampler(V, engine.device, max_rows=max_batch)
    gen = torch.Generator().manual_seed(0)

    def decode_run(batch: int, steps: int, warmup: int):
        sched = Scheduler(engine, sampler, max_num_seqs=batch, max_batch_tokens=PREFILL, num_ctx=context)
        params = (SamplingParams.greedy(num_predict=-1, ignore_eos=True) if args.sampling == "greedy"
                  else SamplingParams(num_predict=-1, ignore_eos=True, seed=1))
        for i in range(batch):
            prompt = torch.randint(0, V, (PROMPT,), generator=gen).tolist()
            sched.add(Request(("bench", batch, i), prompt, params, seed=i))
        while any(not r.decoding for r in list(sched.running) + list(sched.waiting)):
            sched.step()
        for _ in range(warmup):
            sched.step()
        lengths = [engine.cached_length(r.request_id) for r in sched.running]
        before = sum(len(r.generated) for r in sched.running)
        torch.cuda.synchronize()
        t = time.perf_counter()
        for _ in range(steps):
            sched.step()
        torch.cuda.synchronize()
        dt = time.perf_counter() - t
        made = sum(len(r.generated) for r in sched.running) - before
        assert made == batch * steps, f"{made} tokens decoded in {steps} steps of batch {batch}"
        mean_ctx = sum(lengths) / batch + steps / 2
        for r in list(sched.running):
            sched.cancel(r.request_id)
        while sched.has_work():          # (a step launched ahead is read first; the one after frees them)
            sched.step()
        return dt, mean_ctx

    def prefill_run(tokens: int = PREFILL):
        best = None
        for i in range(3):
            prompt = torch.randint(0, V, (tokens,), generator=gen).tolist()
            from hfee_amd.engine import StepEntry
            rid = ("prefill", i)
            engine.admit(rid)
            torch.cuda.synchronize()
            t = time.perf_counter()
            logits = engine.step([StepEntry(rid, prompt, [tokens - 1])])
            del logits
            torch.cuda.synchronize()
            dt = time.perf_counter() - t
            engine.release(rid)
            best = dt if best is None else min(best, dt)
        return best

    def serving_run(count: int):
        """All requests arrive at once; portions of prompts run beside decoded tokens until
        the last request has its 128 tokens."""
        sched = Scheduler(engine, sampler, max_num_seqs=count, max_batch_tokens=PREFILL, num_ctx=context)
        params = SamplingParams.greedy(num_predict=128, ignore_eos=True)
        lengths = torch.randint(64, 2049, (count,), generator=gen).tolist()
        for i, n in enumerate(lengths):
            sched.add(Request(("serving", i), torch.randint(0, V, (n,), generator=gen).tolist(), params, seed=i))
        # an event in front of and behind every step's launches: what lies between a step's two events is
        # the GPU's time inside steps, whatever it waits for there; the rest of the span it waits for the host
        marks = []
        run_step = engine.step

        def marked_step(entries, tokens_from=None):
            a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            a.record()
            out = run_step(entries, tokens_from)
            b.record()
            marks.append((a, b))
            return out
        engine.step = marked_step
        torch.cuda.synchronize()
        t = time.perf_counter()
        steps = made = 0
        try:
            while sched.has_work():
                for fin in sched.step():
                    made += len(fin.request.generated)
                steps += 1
        finally:
            del engine.step
        torch.cuda.synchronize()
        dt = time.perf_counter() - t
        serving_run.inside_ms = sum(a.elapsed_time(b) for a, b in marks)
        serving_run.span_ms = marks[0][0].elapsed_time(marks[-1][1]) if marks else 0.0
        return dt, sum(lengths), made, steps

    if args.serving:
        serving_run(min(args.serving, 8))        # (compiles nothing, but captures graphs and sizes buffers)
        dt, prompt_tokens, made, steps = serving_run(args.serving)
        return ({
            "metric": "continuous batching, generated tok/s (%s bf16)" % SHAPE_NAMES[args.shape],
            "value": round(made / dt, 1), "unit": "tokens/s", "n_gpus": 1, "steps": steps, "seconds": round(dt, 3),
            "all_tokens_per_s": round((prompt_tokens + made) / dt, 1), "dtype": "bf16",
            "gpu_ms_from_first_step_to_last": round(serving_run.span_ms, 1),
            "gpu_ms_inside_steps": round(serving_run.inside_ms, 1),
            "data": "synthetic (seeded uniform random token ids, random N(0,0.02) weights)",
            "config": {"model": SHAPE_NAMES[args.shape] + "-shaped", "layers": L, "requests": args.serving,
                       "prompt_tokens_total": prompt_tokens, "generated_total": made, "seq_len": context,
                       "max_batch_tokens": PREFILL, "page_size": page_size}})

    def context_run(batch: int, tokens: int, steps: int, warmup: int):
        """Prompts of `tokens` tokens, the first one timed alone (portions of 2,048 tokens
        each attend to all that came before), then decode steps at that context."""
        sched = Scheduler(engine, sampler, max_num_seqs=batch, max_batch_tokens=PREFILL, num_ctx=context)
        params = SamplingParams.greedy(num_predict=-1, ignore_eos=True)
        sched.add(Request(("context", 0), torch.randint(0, V, (tokens,), generator=gen).tolist(), params, seed=0))
        sched.look_ahead = False         # (the prompt's time is not to hold a decode step launched behind it)
        torch.cuda.synchronize()
        t = time.perf_counter()
        while not sched.running or not sched.running[0].decoding:
            sched.step()
        torch.cuda.synchronize()
        prefill_s = time.perf_counter() - t
        sched.look_ahead = True
        for i in range(1, batch):
            sched.add(Request(("context", i), torch.randint(0, V, (tokens,), generator=gen).tolist(), params, seed=i))
        while any(not r.decoding for r in list(sched.running) + list(sched.waiting)):
            sched.step()
        for _ in range(warmup):
            sched.step()
        before = sum(len(r.generated) for r in sched.running)
        torch.cuda.synchronize()
        t = time.perf_counter()
        for _ in range(steps):
            sched.step()
        torch.cuda.synchronize()
        dt = time.perf_counter() - t
        made = sum(len(r.generated) for r in sched.running) - before
        lengths = [engine.cached_length(r.request_id) for r in sched.running]
        assert made == batch * steps and len(lengths) == batch and min(lengths) >= tokens, (made, lengths)
        for r in list(sched.running):
            sched.cancel(r.request_id)
        while sched.has_work():          # (a step launched ahead is read first; the one after frees them)
            sched.step()
        return prefill_s, dt

    if args.context:
        prefill_s, dt = context_run(args.batch, args.context, args.steps, args.warmup)
        T = args.context
        flops = 2.0 * T * (L * layer_params) + 2.0 * V * d + L * 4.0 * hd * H * T * (T + 1) / 2
        step_bytes = weight_bytes + args.batch * (T + args.warmup + args.steps / 2) * kv_bytes_per_token
        return ({
            "metric": "prefill and decode at a context of %d tokens (%s bf16)" % (T, SHAPE_NAMES[args.shape]),
            "prefill": {"value": round(T / prefill_s, 1), "tokens": T, "ms": round(prefill_s * 1e3, 2),
                        "frac": round(flops / prefill_s / BF16_PEAK, 4)},
            "decode": {"value": round(args.batch * args.steps / dt, 1), "batch": args.batch,
                       "ms_per_step": round(dt / args.steps * 1e3, 3),
                       "hbm_frac": round(step_bytes / (dt / args.steps) / HBM_PEAK, 4)},
            "unit": "tokens/s", "n_gpus": 1, "dtype": "bf16", "layers": L})

    if args.prefill_only:
        tokens = args.prefill_tokens or PREFILL
        if not 1 <= tokens <= PREFILL:
            print(f"bench.py: --prefill-tokens takes 1 to {PREFILL}")
            return 2
        pt = prefill_run(tokens)
        return {"prefill_ms": round(pt * 1e3, 3), "tokens": tokens, "layers": L, "us_per_layer": round(pt * 1e6 / L, 1)}

    dt, mean_ctx = decode_run(args.batch, args.steps, args.warmup)
    ms_per_step = dt / args.steps * 1e3
    value = args.batch * args.steps / dt
    step_bytes = weight_bytes + args.batch * mean_ctx * kv_bytes_per_token
    achieved = step_bytes / (dt / args.steps)
    line = {
        "metric": "decode tok/s @ batch 1/8/64; prefill tok/s @ 2,048 tokens (%s bf16)" % SHAPE_NAMES[args.shape],
        "value": round(value, 2), "unit": "tokens/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16", "data": "synthetic (seeded uniform random token ids, random N(0,0.02) weights)",
        "config": {"model": SHAPE_NAMES[args.shape] + "-shaped", "layers": L, "layers_of_config": base["num_hidden_layers"],
                   "hidden": d, "heads": H, "kv_heads": K, "head_dim": hd, "intermediate": F, "vocab": V,
                   "global_batch": args.batch, "seq_len": context, "prompt_tokens": PROMPT,
                   "mean_context_in_timed_steps": round(mean_ctx, 1), "page_size": page_size,
                   "max_batch_tokens": PREFILL, "parallelism": "single GPU"},
        "roofline": {"bound": "hbm", "achieved": round(achieved / 1e9, 1), "peak": HBM_PEAK / 1e9, "unit": "GB/s",
                     "frac": round(achieved / HBM_PEAK, 4)},
    }
    if not args.no_points:
        pt = prefill_run()
        gemm_flops = 2.0 * PREFILL * (L * layer_params) + 2.0 * V * d
        attn_flops = L * 4.0 * hd * H * PREFILL * (PREFILL + 1) / 2
        flops = gemm_flops + attn_flops
        line["prefill"] = {"value": round(PREFILL / pt, 1), "tokens": PREFILL, "ms": round(pt * 1e3, 3),
                           "frac": round(flops / pt / BF16_PEAK, 4)}
        points = {}
        for b in getattr(args, "point_batches", (1, 64, 128)):
            steps = max(8, min(args.steps, 64))
            dtb, ctx_b = decode_run(b, steps, min(args.warmup, 4))
            points[f"decode_b{b}"] = round(b * steps / dtb, 2)
            points[f"decode_b{b}_hbm_frac"] = round((weight_bytes + b * ctx_b * kv_bytes_per_token) / (dtb / steps) / HBM_PEAK, 4)
        if not hasattr(args, "point_batches"):        # (the line's own shape: shorter prompts, ms until they are in the cache)
            for tokens in (128, 512, 1024):
                points[f"prefill_{tokens}_ms"] = round(prefill_run(tokens) * 1e3, 3)
        line["points"] = points
    return line


if __name__ == "__main__":
    sys.exit(main())
