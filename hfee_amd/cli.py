"""The command line, in the reference's manner: `hfee run <model> [prompt]`
(/root/reference/cmd/hfee/main.go:28, /root/reference/cmd/hfee/run.go:23-67).
<model> is a model folder; the prompt is the remaining arguments joined by spaces,
with piped standard input in front of it; --verbose prints the counts and rates
that the reference prints (/root/reference/cmd/hfee/run.go:210-223).  The context
window and the number of requests served at once default to $HFEE_NUM_CTX and
$HFEE_NUM_PARALLEL (/root/reference/internal/server/server.go:46-57).  Sampling
options carry the names of the reference's request options
(/root/reference/internal/llm/sampler.go:10-21).
"""
from __future__ import annotations

import argparse
import os
import sys
import time

USAGE = """HFee runs large language models on one MI355X.

Usage:
  hfee <command> [arguments]

Commands:
  run <model> [prompt]   Generate from a model folder (config.json + model.safetensors)
  replay ...             Feed token ids step by step and write logits (see bin/trace_run)
  bench ...              Decode and prefill throughput (the options of bench.py)
  version                Print the version

Environment:
  HFEE_NUM_CTX          context window per request (default 4096)
  HFEE_NUM_PARALLEL     requests answered at once (default 4)
"""

VERSION = "0.1.0"


def _env_int(name, default):
    try:
        return int(os.environ.get(name, default))
    except ValueError:
        return default


def run(argv) -> int:
    ap = argparse.ArgumentParser(prog="hfee run", usage="hfee run <model> [prompt] [options]")
    ap.add_argument("model")
    ap.add_argument("prompt", nargs="*")
    ap.add_argument("--verbose", action="store_true")
    ap.add_argument("--tokens", help="comma-separated token ids instead of a text prompt")
    ap.add_argument("--random-weights", action="store_true", help="ignore the folder's tensors; seeded random weights")
    ap.add_argument("--seed", type=int, default=0, help="seed of the random weights")
    ap.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "bf16", "float32", "fp32"])
    ap.add_argument("--num-predict", type=int, default=-1)
    ap.add_argument("--temperature", type=float, default=0.8)
    ap.add_argument("--top-k", type=int, default=40)
    ap.add_argument("--top-p", type=float, default=0.9)
    ap.add_argument("--min-p", type=float, default=0.0)
    ap.add_argument("--repeat-penalty", type=float, default=1.1)
    ap.add_argument("--repeat-last-n", type=int, default=64)
    ap.add_argument("--sample-seed", type=int, default=-1)
    ap.add_argument("--stop", action="append", default=[])
    ap.add_argument("--ignore-eos", action="store_true")
    ap.add_argument("--num-ctx", type=int, default=_env_int("HFEE_NUM_CTX", 4096))
    ap.add_argument("--num-parallel", type=int, default=_env_int("HFEE_NUM_PARALLEL", 4))
    ap.add_argument("--max-batch-tokens", type=int, default=2048)
    ap.add_argument("--page-size", type=int, default=16)
    ap.add_argument("--num-pages", type=int, default=None)
    args = ap.parse_args(argv)

    from .api import LLM

    t0 = time.perf_counter()
    llm = LLM(args.model, random_weights=args.random_weights, seed=args.seed, dtype=args.dtype,
              num_ctx=args.num_ctx, num_parallel=args.num_parallel, max_batch_tokens=args.max_batch_tokens,
              page_size=args.page_size, num_pages=args.num_pages)
    load = time.perf_counter() - t0

    if args.tokens:
        prompt = [int(t) for t in args.tokens.replace(" ", "").split(",") if t]
    else:
        text = " ".join(args.prompt)
        if not sys.stdin.isatty():
            text = (sys.stdin.read().strip() + "\n\n" + text).strip()      # run.go:46-53
        if not text and sys.stdin.isatty() and llm.tokenizer is not None:
            return interactive(llm, make_params(args), args.verbose, load)
        if not text:
            print("usage: hfee run <model> [prompt]   (or --tokens 1,2,3)", file=sys.stderr)
            return 1
        if llm.tokenizer is None:
            print("this model folder has no tokenizer.json: pass the prompt as --tokens 1,2,3", file=sys.stderr)
            return 1
        prompt = text

    answer(llm, prompt, make_params(args), args.verbose, load, t0)
    return 0


def make_params(args):
    from .sampling import SamplingParams
    return SamplingParams(temperature=args.temperature, top_k=args.top_k, top_p=args.top_p, min_p=args.min_p,
                          repeat_penalty=args.repeat_penalty, repeat_last_n=args.repeat_last_n,
                          seed=args.sample_seed, num_predict=args.num_predict, stop=tuple(args.stop),
                          ignore_eos=args.ignore_eos)


def answer(llm, prompt, params, verbose: bool, load: float, t0: float):
    """Generates from one prompt, printing the pieces as they come, and with --verbose the
    counts and rates of /root/reference/cmd/hfee/run.go:210-223."""
    def show(index, token, text):
        if llm.tokenizer is not None:
            if text:
                print(text, end="", flush=True)
        else:
            print(token, end=" ", flush=True)

    out = llm.generate([prompt], params, on_token=show)[0]
    print("\n")
    if verbose:
        s = out.stats
        total = time.perf_counter() - t0

        def rate(n, d):
            return "-" if d <= 0 else f"{n / d:.2f} tokens/s"
        print(f"total duration:       {total:.3f}s")
        print(f"load duration:        {load:.3f}s")
        print(f"prompt eval count:    {s.prompt_tokens} token(s)")
        print(f"prompt eval rate:     {rate(s.prompt_tokens, s.prompt_duration)}")
        print(f"eval count:           {s.eval_tokens} token(s)")
        print(f"eval rate:            {rate(s.eval_tokens, s.eval_duration)}")
        print(f"done reason:          {out.done_reason}\n")
    return out


def read_message(readline, prompt_more=lambda: print("... ", end="", flush=True)):
    """One line, or several between \"\"\" markers (/root/reference/cmd/hfee/run.go:154-175).
    None at the end of the input."""
    line = readline()
    if not line:
        return None
    line = line.strip()
    if not line.startswith('"""'):
        return line
    body = line[3:]
    while not body.strip().endswith('"""') or not body:
        prompt_more()
        more = readline()
        if not more:
            return None
        body += "\n" + more.rstrip("\r\n")
    return body.strip()[:-3].strip()


def interactive(llm, params, verbose: bool, load: float) -> int:
    """`hfee run <model>` without a prompt on a terminal: messages are read one after the
    other (/root/reference/cmd/hfee/run.go:69-152).  Every message is a prompt of its
    own: the reference keeps a conversation through its server's chat template, and the
    server is no part of this engine, so /clear and /system have nothing to act on."""
    print('Type a message, or /? for help. Use """ to begin a multi-line message.')
    while True:
        print(">>> ", end="", flush=True)
        try:
            line = read_message(sys.stdin.readline)
        except KeyboardInterrupt:
            print("\nUse Ctrl + d or /bye to exit.")
            continue
        if line is None:
            print()
            return 0
        if line == "":
            continue
        if line in ("/bye", "/exit"):
            return 0
        if line in ("/?", "/help"):
            print('  /bye            Exit\n  """             Start or end a multi-line message')
            continue
        if line.startswith("/"):
            print(f"Unknown command {line.split()[0]}. Type /? for help.")
            continue
        try:
            answer(llm, line, params, verbose, load, time.perf_counter())
        except KeyboardInterrupt:
            print()


def bench(argv) -> int:
    """`hfee bench ...`: the measurement program that lies beside the package, with its own options."""
    import importlib.util
    path = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "bench.py")
    if not os.path.isfile(path):
        print(f"hfee bench: {path} is not there (the measurement program ships with the source tree)", file=sys.stderr)
        return 1
    spec = importlib.util.spec_from_file_location("hfee_bench", path)
    module = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(module)
    return module.main(argv)


def main(argv=None) -> int:
    argv = list(sys.argv[1:] if argv is None else argv)
    if not argv:
        print(USAGE, end="")
        return 1
    cmd, rest = argv[0], argv[1:]
    if cmd == "run":
        return run(rest)
    if cmd == "replay":
        from .trace_replay import main as replay_main
        return replay_main(rest)
    if cmd == "bench":
        return bench(rest)
    if cmd in ("version", "--version", "-v"):
        print(f"hfee version {VERSION}")
        return 0
    print(f"unknown command {cmd!r}\n\n{USAGE}", file=sys.stderr, end="")
    return 1
