"""Command line in the manner of kappai-cli (src/cli/main.c, option table and usage text
src/config.c:84-154, 403-447): the same option names and meanings where kappai has them.
Prompts and output are token ids, because text and tokenizers lie outside this engine.

    python -m kappai_amd -m DIR -p "1,2,3" -n 16 -t 0
"""
from __future__ import annotations

import argparse
import json
import re
import sys
import tempfile
import time
from pathlib import Path

_TRUE, _FALSE = {"yes", "on", "true", "1"}, {"no", "off", "false", "0"}


def parse_bool(text: str) -> bool:
    """kappai's boolean words (src/config.c:37-42)."""
    t = text.strip().lower()
    if t in _TRUE:
        return True
    if t in _FALSE:
        return False
    raise argparse.ArgumentTypeError(f"expected yes/on/true/1 or no/off/false/0, got {text!r}")


def parse_ids(text: str):
    ids = [int(x) for x in re.split(r"[,\s]+", text.strip()) if x]
    if not ids:
        raise argparse.ArgumentTypeError("a prompt needs at least one token id")
    return ids


def build_parser() -> argparse.ArgumentParser:
    ap = argparse.ArgumentParser(
        prog="kappai-amd", formatter_class=argparse.RawDescriptionHelpFormatter,
        description="Generates token ids from prompt token ids with an LFM2 model on one MI355X.",
        usage="kappai-amd --model <dir> [options] [prompt ids]")
    e = ap.add_argument_group("Engine")
    e.add_argument("-m", "--model", help="model folder: config.json and model.safetensors (required "
                   "unless --random-weights)")
    e.add_argument("-c", "--ctx-size", type=int, default=0, help="context size (0 = from model)")
    e.add_argument("--metrics", default="pp,tg", help="comma-separated metrics to print after "
                   "generation, in any order: pp,tg,ttft (default: pp,tg)")
    e.add_argument("--stream", nargs="?", const=True, default=True, type=parse_bool,
                   help="print token ids as they are generated (default: on)")
    e.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "float32", "bf16", "fp32"],
                   help="compute type; float32 is true 32-bit arithmetic throughout")
    e.add_argument("--page-size", type=int, default=16, help="tokens per cache page")
    e.add_argument("--num-pages", type=int, default=0, help="cache pages (0 = from free memory)")
    e.add_argument("--max-batch", type=int, default=64, help="requests live at the same time")
    e.add_argument("--token-budget", type=int, default=2048, help="tokens per step at most")
    e.add_argument("--chunk", type=int, default=2048, help="longest prompt portion in a step")
    e.add_argument("--random-weights", metavar="SHAPE|CONFIG.json", help="make a model folder "
                   "with random weights and run it: the name of a shape (tiny-a, tiny-b, "
                   "lfm2-350m, lfm2-1.2b, lfm2-2.6b) or a config.json; with --model the folder is "
                   "written there")
    e.add_argument("--weight-seed", type=int, default=0, help="seed of --random-weights")
    e.add_argument("--weight-std", type=float, default=0.02,
                   help="--random-weights: matrices and tables are N(0, std) (default 0.02)")
    e.add_argument("--norm-jitter", type=float, default=0.0,
                   help="--random-weights: norm weights are 1 + N(0, jitter) (default 0: all 1)")
    g = ap.add_argument_group("LLM behavior")
    g.add_argument("-p", "--prompt", action="append", type=parse_ids, default=[],
                   help="prompt as token ids, comma or space separated; may be given several "
                   "times for several requests (or as the last positional argument)")
    g.add_argument("--prompt-file", help="file with one prompt of token ids per line")
    g.add_argument("-n", "--n-predict", type=int, default=-1,
                   help="max tokens to generate (-1 = unlimited)")
    g.add_argument("-t", "--temperature", type=float, default=0.80,
                   help="sampling temperature (default 0.80, 0.0 = greedy)")
    g.add_argument("-k", "--top-k", type=int, default=40, help="top-k sampling (default 40, "
                   "0 = disabled)")
    g.add_argument("-P", "--top-p", type=float, default=0.90, help="top-p sampling (default 0.90, "
                   "1.0 = disabled)")
    g.add_argument("-M", "--min-p", type=float, default=0.10, help="min-p sampling (default 0.10, "
                   "0.0 = disabled)")
    g.add_argument("--repeat-penalty", type=float, default=1.0,
                   help="repetition penalty (default 1.0 = disabled)")
    g.add_argument("--repeat-last-n", type=int, default=64,
                   help="last-n tokens considered by repeat penalty (default 64)")
    g.add_argument("-s", "--seed", type=int, default=0, help="RNG seed (0 = random)")
    d = ap.add_argument_group("Tools / debug")
    d.add_argument("--time", action="store_true",
                   help="print the time of every step, and after the run the time by stage of "
                        "the forward pass for steps with prompt portions and for decode steps")
    d.add_argument("--debug-forward", action="store_true",
                   help="print the top logits of every sampled row")
    d.add_argument("--debug", action="store_true", help="print the engine's decisions")
    d.add_argument("--dump-logits", metavar="FILE", help="append the float32 logits of every "
                   "sampled row to FILE")
    ap.add_argument("positional_prompt", nargs="?", type=parse_ids, help=argparse.SUPPRESS)
    return ap


def main(argv=None) -> int:
    ap = build_parser()
    args = ap.parse_args(argv)
    prompts = list(args.prompt)
    if args.positional_prompt:
        prompts.append(args.positional_prompt)
    if args.prompt_file:
        for line in Path(args.prompt_file).read_text().splitlines():
            if line.strip():
                prompts.append(parse_ids(line))
    if not prompts:
        ap.error("no prompt: give -p/--prompt, --prompt-file or a positional prompt of token ids")
    if not args.model and not args.random_weights:
        ap.error("--model is required")

    from .engine import Engine, EngineConfig
    from .sampling import SamplingParams

    model_dir = args.model
    tmp = None
    if args.random_weights:
        from .config import SHAPES, config_from_dict, named_shape
        from .weights import write_random_model
        spec = args.random_weights
        if spec.strip().lower() in SHAPES:
            raw = named_shape(spec)
        elif Path(spec).is_file():
            raw = json.loads(Path(spec).read_text())
        else:
            ap.error(f"--random-weights: {spec!r} is neither a file nor one of the shapes "
                     f"{', '.join(sorted(SHAPES))}")
        cfg = config_from_dict(raw)
        if not model_dir:
            tmp = tempfile.TemporaryDirectory(prefix="kappai_amd_model_")
            model_dir = tmp.name
        write_random_model(model_dir, cfg, args.weight_seed, std=args.weight_std,
                           norm_jitter=args.norm_jitter)
        print(f"wrote random weights (seed {args.weight_seed}, std {args.weight_std}, norm jitter "
              f"{args.norm_jitter}) to {model_dir}", file=sys.stderr)

    engine = Engine(EngineConfig(
        model=model_dir, dtype=args.dtype, ctx_size=args.ctx_size, page_size=args.page_size,
        num_pages=args.num_pages, max_batch=args.max_batch, token_budget=args.token_budget,
        chunk=args.chunk,
        # per-step output (logits, timing) needs every step waited for, and the times by stage
        # need steps that are launched kernel by kernel
        decode_run=1 if (args.debug_forward or args.dump_logits or args.time) else 8,
        pipeline=not (args.debug_forward or args.dump_logits or args.time),
        decode_graphs=not args.time))
    stage_records = {"prefill": [], "decode": []}
    if args.time:
        from .kernels import profile
        profile.STAGE_TIMES.start()
    params = SamplingParams(
        temperature=args.temperature, top_k=args.top_k, top_p=args.top_p, min_p=args.min_p,
        repeat_penalty=args.repeat_penalty, repeat_last_n=args.repeat_last_n, seed=args.seed,
        n_predict=args.n_predict)
    ids = [engine.add_request(p, params) for p in prompts]
    outputs = {rid: [] for rid in ids}
    dump = open(args.dump_logits, "ab") if args.dump_logits else None
    status = 0
    try:
        while engine.has_unfinished():
            t0 = time.perf_counter()
            prefilled = engine.metrics.prefill_tokens
            outs = engine.step()
            if args.time:
                print(f"step {engine.metrics.steps}: {(time.perf_counter() - t0) * 1e3:.3f} ms, "
                      f"{len(outs)} tokens", file=sys.stderr)
                kind = "prefill" if engine.metrics.prefill_tokens > prefilled else "decode"
                stage_records[kind] += profile.STAGE_TIMES.take()
            if (args.debug_forward or dump) and engine.last_logits is not None and outs:
                lg = engine.last_logits.float().cpu()
                if dump:
                    dump.write(lg.numpy().astype("<f4").tobytes())
                if args.debug_forward:
                    for row in lg:
                        top = row.topk(min(8, row.numel()))
                        print("top logits:" + "".join(
                            f" [{int(i)}]={float(v):.4f}" for v, i in zip(top.values, top.indices)),
                            file=sys.stderr)
            for o in outs:
                if o.token is not None:
                    outputs[o.request_id].append(o.token)
                    if args.stream and len(ids) == 1:
                        print(o.token, end=" ", flush=True)
                if o.finished and args.debug:
                    print(f"request {o.request_id} ended: {o.finish_reason}", file=sys.stderr)
                if o.finished and o.token is None:
                    print(f"request {o.request_id} failed: {o.finish_reason}", file=sys.stderr)
                    status = 1
        if args.stream and len(ids) == 1:
            print()
        else:
            for rid in ids:
                print(" ".join(str(t) for t in outputs[rid]))
        line = engine.metrics.line(args.metrics)
        if line:
            print(line, file=sys.stderr)
        if args.time:
            # kappai prints its table after prefill and after decoding (src/context.c:1597-1625)
            m = engine.metrics
            # (a step with prompt portions beside decoded tokens is booked under prefill whole;
            # the engine's clock shares such a step's time out by tokens)
            walls = {"prefill": m.prefill_seconds * 1e6, "decode": m.decode_seconds * 1e6}
            for kind in ("prefill", "decode"):
                if stage_records[kind]:
                    print(profile.STAGE_TIMES.report(kind, walls[kind], stage_records[kind]),
                          file=sys.stderr)
            profile.STAGE_TIMES.stop()
    except KeyboardInterrupt:
        print("\ninterrupted", file=sys.stderr)
        status = 130
    finally:
        if dump:
            dump.close()
        engine.shutdown()
        if tmp is not None:
            tmp.cleanup()
    return status


if __name__ == "__main__":
    sys.exit(main())
