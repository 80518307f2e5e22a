#!/usr/bin/env python3
"""Decode and prefill throughput of kappai_amd on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

The default run has the layer sizes of the LFM2-1.2B shape with random bfloat16 weights:
W untimed and K timed decode steps at batch 8 with every request holding a context of 4,096
tokens at the last step (one step = one token for every request: row tables, model,
sampling on the GPU, token ids back on the host), a prefill of 2,048 tokens (a step among eight
such prompts queued one behind the other, as the decode steps are queued; "alone_ms" is one such
step with the GPU idle before it), and further points: decode at batch 1 and 64, decode at the
headline batch with contexts of 32,768 tokens, prompt steps of 128 and 512 tokens ("points":
tokens a second; "points_frac": each point's share of the peak that bounds it, HBM for decode
steps and the matrix cores for prompt steps).  It prints ONE JSON line.  The model is a folder that the framework's own
random-weights mode writes (config.json, model.safetensors) and its own loader reads; token ids
are uniform random with a fixed seed, and every request's context is computed by real prompt
steps before its decoding is timed: no dataset is involved ("data": "synthetic").  kappai
publishes no numbers for this architecture, so "vs_baseline" is null; the roofline fractions are
against MI355X's published peaks, and beside them against what a kernel that only reads and a
kernel that only multiplies reach on the same box ("kernels": the engine's own products and
attention kernels at the shapes of the run, timed one by one outside the timed step).
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0          # MI355X HBM3E, GB/s
MFMA_PEAK_TFLOPS = {"bfloat16": 2500.0, "float32": 157.3}      # dense

def _shape(name):
    from kappai_amd.config import named_shape
    return named_shape(name)


LFM2_1_2B, LFM2_350M, LFM2_2_6B = _shape("lfm2-1.2b"), _shape("lfm2-350m"), _shape("lfm2-2.6b")

# Serving workloads (through Engine: scheduler, prompt portions beside decoded tokens, sampling)
WORKLOADS = {
    # 64 requests at once, prompts of 128..2048 tokens cut into portions of 512, 256 tokens each
    "serve-350m": dict(raw=LFM2_350M, name="LFM2-350M shape", requests=64, prompt=(128, 2048),
                       n_predict=256, chunk=512, token_budget=576, ctx=4096),
    # 16 requests with 32,768-token contexts, 512 tokens each
    "long-2.6b": dict(raw=LFM2_2_6B, name="LFM2-2.6B shape", requests=16, prompt=(32768 - 512, 32768 - 512),
                      n_predict=512, chunk=2048, token_budget=2048, ctx=32768),
}


def run_workload(key, dtype, device, repeat_penalty=1.0):
    """One serving workload from start to end through ``Engine.generate`` with greedy sampling
    (after a repeat penalty over the last 64 tokens, if one is asked for): all requests arrive
    together.  Prints one JSON line: generated tokens a second over the
    whole run (prompts included in the time), and the engine's own prefill / decode rates."""
    import torch

    from kappai_amd.engine import Engine, EngineConfig
    from kappai_amd.sampling import SamplingParams
    w = WORKLOADS[key]
    model = random_model(dict(w["raw"]), dtype, device)
    n = w["requests"]
    page = 16
    eng = Engine(EngineConfig(dtype=dtype, ctx_size=w["ctx"], max_batch=n, page_size=page,
                              num_pages=n * (w["ctx"] // page), token_budget=w["token_budget"],
                              chunk=w["chunk"]), model=model)
    g = torch.Generator().manual_seed(3)
    lo, hi = w["prompt"]
    lengths = [int(t) for t in torch.randint(lo, hi + 1, (n,), generator=g)]
    prompts = [[int(t) for t in torch.randint(0, model.vocab_size, (L,), generator=g)]
               for L in lengths]
    sync()
    t0 = time.perf_counter()
    import dataclasses
    params = dataclasses.replace(SamplingParams.greedy(n_predict=w["n_predict"]),
                                 repeat_penalty=float(repeat_penalty))
    out = eng.generate(prompts, params)
    sync()
    dt = time.perf_counter() - t0
    m = eng.metrics
    generated = sum(len(o) for o in out)
    cfg = model.config
    print(json.dumps({
        "metric": f"generated tok/s, {key} workload ({w['name']})", "value": round(generated / dt, 1),
        "unit": "tok/s", "n_gpus": 1, "seconds": round(dt, 3), "dtype": dtype, "data": "synthetic",
        "config": {"model": w["name"] + ", random weights", "hidden_size": cfg.hidden_size,
                   "num_layers": cfg.num_hidden_layers, "attention_layers": len(cfg.attention_layers),
                   "ff_dim": cfg.ff_dim, "requests": n, "prompt_tokens": sum(lengths),
                   "generated_tokens": generated, "chunk": w["chunk"],
                   "token_budget": w["token_budget"], "ctx_size": w["ctx"],
                   "repeat_penalty": float(repeat_penalty)},
        "engine": {"steps": m.steps, "prefill_tok_s": round(m.pp, 1), "decode_tok_s": round(m.tg, 1),
                   "ttft_ms": round(m.first_token_ms, 2), "graph_replays": eng.runner.graph_replays,
                   "preemptions": eng.scheduler.preempted_total},
    }))
    return 0


def random_model(raw, dtype, device, seed=0, std=0.02):
    """The model of ``raw`` with N(0, std) weights (norm weights 1), through the framework's own
    random-weights mode and loader: the folder is written once (under the temp folder, named by
    the configuration and the seed) and loaded like any checkpoint."""
    import hashlib
    import tempfile

    from kappai_amd.config import config_from_dict
    from kappai_amd.models import load_model
    from kappai_amd.weights import write_random_model

    cfg = config_from_dict(raw)
    tag = hashlib.sha256(json.dumps([cfg.to_dict(), seed, std], sort_keys=True).encode())
    folder = os.path.join(tempfile.gettempdir(),
                          f"kappai_amd_bench_{os.getuid()}_{tag.hexdigest()[:16]}")
    done = os.path.join(folder, ".complete")
    if not os.path.exists(done):
        t0 = time.perf_counter()
        os.makedirs(folder, mode=0o700, exist_ok=True)
        write_random_model(folder, cfg, seed=seed, std=std)
        open(done, "w").close()
        print(f"bench.py: wrote {folder} in {time.perf_counter() - t0:.1f} s", file=sys.stderr,
              flush=True)
    return load_model(folder, dtype, device)


def sync():
    import torch
    torch.cuda.synchronize()


class DecodeBench:
    """``batch`` requests whose contexts of ``start`` random tokens are computed by prompt steps
    (portions of at most 2,048 tokens, one request a step), then decoded greedily one token a
    step."""

    def __init__(self, model, batch, start, total, page_size, device, seed=1, graphs=True):
        import torch

        from kappai_amd.cache import CacheManager
        from kappai_amd.engine import StepEntry, StepRunner
        self.torch, self.StepEntry = torch, StepEntry
        pages = batch * ((total + page_size - 1) // page_size)
        self.cache = CacheManager(model.cache_specs(), page_size, pages, batch)
        self.cache.allocate_storage(model.dtype, device)
        self.runner = StepRunner(model, self.cache, device, decode_graphs=graphs)
        self.requests = [self.cache.open(i) for i in range(batch)]
        gen = torch.Generator().manual_seed(seed)
        for rc in self.requests:
            prompt = torch.randint(0, model.vocab_size, (start,), generator=gen).tolist()
            for at in range(0, start, 2048):
                self.runner.step([StepEntry(rc, prompt[at:at + 2048], [])])
        sync()
        self.tokens = [int(t) for t in torch.randint(0, model.vocab_size, (batch,), generator=gen)]
        self.temp = torch.zeros(batch, dtype=torch.float32, device=device)
        self.uni = torch.zeros(batch, dtype=torch.float32, device=device)
        self.model = model

    def step(self):
        from kappai_amd.kernels import ops
        entries = [self.StepEntry(rc, [tok], [0]) for rc, tok in zip(self.requests, self.tokens)]
        logits = self.runner.step(entries)
        self.tokens = ops.sample_rows(logits, self.temp, self.uni).tolist()

    def _choose(self, logits, step, out_row, also):
        from kappai_amd.kernels import ops
        ops.sample_rows(logits, self.temp, self.uni, out=out_row, also=also)

    def run(self, warmup, steps, run_len=8, ahead=True):
        """``steps`` decode steps, taken the way the engine takes them when nothing but decoding
        is going on: up to ``run_len`` steps queued back to back, each step's token handed to the
        next on the GPU, and a run queued before the host has read the tokens of the run before
        it (they travel to pinned memory behind the run's last kernel)."""
        from kappai_amd.kernels import ops
        torch = self.torch
        B = len(self.requests)
        hosts = [torch.empty((run_len, B), dtype=torch.int32, pin_memory=True) for _ in range(2)]
        state = {"before": None, "runs": 0}   # before: (tokens of the last run on the GPU, host
                                               # copy, event behind the copy)

        def read(rec):
            rec[2].synchronize()
            self.tokens = rec[1][rec[0].shape[0] - 1].tolist()

        def take(steps):
            left = steps
            while left > 0:
                n = min(run_len, left)
                before = state["before"]
                out = None
                if n > 1:
                    placed = None
                    if before is not None:
                        last = (before[0].shape[0] - 1) * B
                        placed = (before[0].view(-1), [(i, last + i) for i in range(B)])
                    out = self.runner.decode_run(self.requests, self.tokens, n, self._choose,
                                                 placed=placed)
                if out is None:
                    if before is not None:
                        read(before)
                        state["before"] = None
                    self.step()
                    left -= 1
                    continue
                host = hosts[state["runs"] % 2]
                ops.tokens_to_host(out, host)
                done = torch.cuda.Event()
                done.record()
                if before is not None:
                    read(before)
                state["before"] = (out, host, done)
                if not ahead:            # every run read before the next is queued
                    read(state["before"])
                    state["before"] = None
                state["runs"] += 1
                left -= n
            if state["before"] is not None:
                read(state["before"])
                state["before"] = None

        # warm-up: single steps first (the second of a shape captures its graph), then, when
        # there are steps enough, two short runs, so that everything a run needs has run once
        singles = warmup - 4 if warmup >= 6 else warmup
        for _ in range(singles):
            self.step()
        if warmup > singles:
            full = run_len
            run_len = 2
            take(warmup - singles)
            run_len = full
        sync()
        t0 = time.perf_counter()
        take(steps)
        sync()
        return time.perf_counter() - t0

    def close(self):
        for rc in self.requests:
            self.cache.close(rc)


def measured_read_bandwidth(device, mb=256, buffers=8, reps=24):
    """GB/s of a kernel that only reads: buffers of ``mb`` MB taken in turn (2 GB together, eight
    times what the memory-side cache holds), ``reps`` reads between two synchronisations; the best
    of several numbers of blocks sharing a read, so that the figure is what reading reaches on
    this box and not what one launch shape reaches."""
    import torch

    from kappai_amd.kernels import ops
    bufs = [torch.empty(mb * 1000 * 1000 // 4, dtype=torch.int32, device=device).random_()
            for _ in range(buffers)]
    best = 0.0
    for blocks in (512, 1024, 2048, 4096):
        for b in bufs:
            ops.stream_read(b, blocks)
        sync()
        t0 = time.perf_counter()
        total = 0
        for i in range(reps):
            total += ops.stream_read(bufs[i % buffers], blocks)
        sync()
        best = max(best, total / (time.perf_counter() - t0) / 1e9)
    return best


def measured_mfma_tflops(device, iters=20000):
    """TFLOP/s of a kernel that only issues bfloat16 matrix instructions from registers."""
    from kappai_amd.kernels import ops
    ops.mfma_probe(200, device)
    sync()
    t0 = time.perf_counter()
    flops = ops.mfma_probe(iters, device)
    sync()
    return flops / (time.perf_counter() - t0) / 1e12


def graph_time(fn, reps):
    """Seconds per call of ``fn(i)``, from a captured graph of ``reps`` calls replayed twice
    (kernels one after the other as in a step, no host in between)."""
    import torch
    fn(0)
    sync()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g):
        for i in range(reps):
            fn(i)
    g.replay()
    sync()
    t0 = time.perf_counter()
    g.replay()
    g.replay()
    sync()
    return (time.perf_counter() - t0) / (2 * reps)


def kernel_rates(model, cfg, batch, context, prefill_tokens, page_size, device, read_gbs,
                 mfma_tflops, dtype):
    """The engine's own kernels by class, one by one at the shapes of this run, each over
    distinct matrices in turn that together exceed the memory-side cache several times (the
    model's own layers, and copies where those are too few: 2 GB for the head and for the cache
    of the decode attention), so that every call reads from memory as in a step: the products of
    a decode step (K3),
    decode attention over the cache (K10) and the output head (K11) in GB/s of what they have to
    read, the products of a prompt step (K4) and its attention (K9) in TFLOP/s.  Every figure
    also as a fraction of the published peak and of what the read-only / multiply-only kernels
    reach on this box."""
    import math

    import torch

    from kappai_amd.kernels import ops
    if dtype != "bfloat16":
        return {}
    BF = torch.bfloat16
    D, F = cfg.hidden_size, cfg.ff_dim
    H, G, d = cfg.num_attention_heads, cfg.num_key_value_heads, cfg.head_dim
    ffs = [blk.feed_forward for blk in model.layers]
    convs = [blk.mixer for blk in model.layers if hasattr(blk.mixer, "in_proj")]
    out = {}

    def rate_gbs(name, seconds, nbytes):
        gbs = nbytes / seconds / 1e9
        out[name] = {"us": round(seconds * 1e6, 2), "gbs": round(gbs, 1),
                     "frac": round(gbs / HBM_PEAK_GBS, 4), "frac_measured": round(gbs / read_gbs, 4)}

    def rate_tflops(name, seconds, flops):
        tf = flops / seconds / 1e12
        out[name] = {"us": round(seconds * 1e6, 2), "tflops": round(tf, 1),
                     "frac": round(tf / MFMA_PEAK_TFLOPS["bfloat16"], 4),
                     "frac_measured": round(tf / mfma_tflops, 4)}

    g = torch.Generator(device=device).manual_seed(5)
    x = torch.randn(batch, D, generator=g, device=device).to(BF)
    act = torch.randn(batch, F, generator=g, device=device).to(BF)
    resid = torch.randn(batch, D, generator=g, device=device)
    n = len(ffs)
    # K3: products of a decode step
    gu = [f.gate_up for f in ffs]
    if all(f.fused for f in ffs):
        t = graph_time(lambda i: ops.linear_swiglu(x, gu[i % n].weight), 2 * n)
        rate_gbs("k3_decode_gate_up", t, gu[0].weight_bytes())
    dn = [f.down for f in ffs]
    t = graph_time(lambda i: dn[i % n].forward(act, add_into=ops.AddInto(resid)), 2 * n)
    rate_gbs("k3_decode_down", t, dn[0].weight_bytes())
    def copies(weight, total_bytes):
        """The matrix and copies of it, ``total_bytes`` together."""
        nbytes = weight.numel() * weight.element_size()
        k = max(1, -(-total_bytes // nbytes) - 1)
        clone = (lambda w: ops.InFragments(w.data.clone())) if isinstance(
            weight, ops.InFragments) else (lambda w: w.clone())
        return [weight] + [clone(weight) for _ in range(k)]

    if convs:
        ip = [c.in_proj.weight for c in convs]
        while sum(w.numel() * 2 for w in ip) < 1 << 30:
            ip = ip + copies(ip[0], 0)[1:]
        t = graph_time(lambda i: ops.linear(x, ip[i % len(ip)]), len(ip))
        rate_gbs("k3_decode_in_proj", t, convs[0].in_proj.weight_bytes())
    # K11: the output head on `batch` rows
    head = model.head.linear
    heads = copies(head.weight, 2 << 30)
    t = graph_time(lambda i: ops.linear(x, heads[i % len(heads)], head.bias,
                                        out_dtype=torch.float32), len(heads))
    rate_gbs("k11_head", t, head.weight_bytes())
    del heads
    # K10: decode attention of `batch` requests over `context` keys
    if cfg.attention_layers and d % 16 == 0:
        per = (context + page_size - 1) // page_size
        n_pool = max(3, -(-(2 << 30) // (batch * per * G * page_size * d * 2 * 2)))
        kp = [torch.randn(batch * per + 1, G, page_size, d, generator=g, device=device).to(BF)
              for _ in range(n_pool)]
        vp = [torch.randn(batch * per + 1, G, d, page_size, generator=g, device=device).to(BF)
              for _ in range(n_pool)]
        q = torch.randn(batch, (H + 2 * G) * d, generator=g, device=device).to(BF)
        bt = torch.arange(batch * per, dtype=torch.int32, device=device).view(batch, per)
        pos = torch.full((batch,), context - 1, dtype=torch.int32, device=device)
        seg = torch.arange(batch, dtype=torch.int32, device=device)
        t = graph_time(lambda i: ops.paged_attention(
            q, H, G, d, kp[i % n_pool], vp[i % n_pool], pos, seg, bt, page_size,
            1.0 / math.sqrt(d), single_rows=True, max_position=context - 1), n_pool)
        rate_gbs("k10_decode_attention", t, batch * context * G * d * 2 * 2)
        del kp, vp
    # K4: products of a prompt step of `prefill_tokens` rows
    T = prefill_tokens
    xp = torch.randn(T, D, generator=g, device=device).to(BF)
    actp = torch.randn(T, F, generator=g, device=device).to(BF)
    if all(f.fused for f in ffs):
        t = graph_time(lambda i: ops.linear_swiglu(xp, gu[i % n].weight), n)
        rate_tflops("k4_prefill_gate_up", t, 2.0 * T * D * 2 * F)
    t = graph_time(lambda i: dn[i % n].forward(actp, partial_sums=True), n)
    rate_tflops("k4_prefill_down", t, 2.0 * T * F * D)
    if convs:
        t = graph_time(lambda i: ops.linear(xp, ip[i % len(ip)]), len(convs))
        rate_tflops("k4_prefill_in_proj", t, 2.0 * T * D * 3 * D)
    # K9: attention of one prompt of `prefill_tokens` tokens over itself
    if cfg.attention_layers and d % 16 == 0:
        per = (T + page_size - 1) // page_size
        kp = torch.randn(per + 1, G, page_size, d, generator=g, device=device).to(BF)
        vp = torch.randn(per + 1, G, d, page_size, generator=g, device=device).to(BF)
        qp = torch.randn(T, (H + 2 * G) * d, generator=g, device=device).to(BF)
        bt = torch.arange(per, dtype=torch.int32, device=device).view(1, per)
        pos = torch.arange(T, dtype=torch.int32, device=device)
        seg = torch.zeros(T, dtype=torch.int32, device=device)
        R = ops.ATTENTION_TILE_ROWS
        nt = (T + R - 1) // R
        tiles = torch.tensor([(0, r, min(R, T - r), j | (nt << 16) if nt <= 0x7fff else 0)
                              for j, r in enumerate(range(0, T, R))], dtype=torch.int32,
                             device=device)
        t = graph_time(lambda i: ops.paged_attention(
            qp, H, G, d, kp, vp, pos, seg, bt, page_size, 1.0 / math.sqrt(d), q_tiles=tiles,
            max_position=T - 1), 4)
        rate_tflops("k9_prefill_attention", t, 4.0 * d * H * (T * (T + 1) // 2))
    return out


def prefill_flops(cfg, n_tokens, n_layers_run):
    """Multiply-adds x 2 of a whole prompt of ``n_tokens``: every projection, attention over
    the causal half, and the head for the last row."""
    D, F, H, G, d = (cfg.hidden_size, cfg.ff_dim, cfg.num_attention_heads,
                     cfg.num_key_value_heads, cfg.head_dim)
    per_tok = 0
    att = 0
    for kind in cfg.layer_types[:n_layers_run]:
        per_tok += 2 * (3 * D * F)
        if kind == "conv":
            per_tok += 2 * (3 * D * D + D * D)
        else:
            per_tok += 2 * (D * (H + 2 * G) * d + H * d * D)
            att += 4 * d * H * (n_tokens * (n_tokens + 1) // 2)
    return per_tok * n_tokens + att + 2 * D * cfg.vocab_size


PREFILL_STEPS = 8      # prompt steps queued back to back for the prefill figure


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=64)
    ap.add_argument("--warmup", type=int, default=8)
    ap.add_argument("--batch", type=int, default=8)
    ap.add_argument("--context", type=int, default=4096)
    ap.add_argument("--prefill-tokens", type=int, default=2048)
    ap.add_argument("--layers", type=int, default=0, help="run only the first N layers (0 = all)")
    ap.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "float32"])
    ap.add_argument("--page-size", type=int, default=16)
    ap.add_argument("--skip-points", action="store_true", help="only the headline batch")
    ap.add_argument("--long-context", type=int, default=32768,
                    help="a further decode point at the headline batch with contexts of this many "
                         "tokens (0: none)")
    ap.add_argument("--short-prompts", type=lambda v: [int(x) for x in v.split(",") if x],
                    default=[128, 512],
                    help="further prompt-step points: tokens a prompt, comma separated")
    ap.add_argument("--skip-kernels", action="store_true",
                    help="leave out the kernel-by-kernel rates")
    ap.add_argument("--no-graphs", action="store_true",
                    help="launch decode steps kernel by kernel (for counter collection)")
    ap.add_argument("--workload", default="decode", choices=["decode"] + sorted(WORKLOADS),
                    help="decode: the headline run; the others are serving workloads through "
                         "the engine's scheduler")
    ap.add_argument("--repeat-penalty", type=float, default=1.0,
                    help="serving workloads: a repeat penalty over the last 64 tokens before "
                         "the greedy choice (1: none)")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this engine runs on one GPU; --gpus must be 1 (nothing was measured)")
        return 2
    if args.workload != "decode":
        return run_workload(args.workload, args.dtype, "cuda:0", args.repeat_penalty)

    import torch

    from kappai_amd.engine import StepEntry, StepRunner
    from kappai_amd.cache import CacheManager

    device = "cuda:0"
    raw = dict(LFM2_1_2B)
    n_layers_full = raw["num_hidden_layers"]
    n_layers = args.layers or n_layers_full
    raw["num_hidden_layers"] = n_layers
    raw["layer_types"] = raw["layer_types"][:n_layers]
    model = random_model(raw, args.dtype, device)
    cfg = model.config
    elem = 2 if args.dtype == "bfloat16" else 4
    K, W = args.steps, args.warmup
    if args.context - (K + W) < 1:
        print("bench.py: --context must exceed --steps + --warmup")
        return 2

    def decode(batch, context=None):
        """(seconds of the K timed steps, tok/s, share of the HBM peak) of decoding at ``batch``
        with contexts of ``context`` tokens at the last step.  The bytes a decode step has to
        read: every weight once, and the cache of the live requests at their mean length."""
        context = context or args.context
        first = context - (K + W)
        b = DecodeBench(model, batch, first, context, args.page_size, device,
                        graphs=not args.no_graphs)
        dt = b.run(W, K)
        kv_bytes = b.cache.bytes_per_token(elem)
        b.close()
        del b
        torch.cuda.empty_cache()
        mean_ctx = first + W + (K - 1) / 2.0
        step_bytes = model.weight_bytes_per_step() + batch * mean_ctx * kv_bytes
        return dt, batch * K / dt, step_bytes / (dt / K) / 1e9

    dt, value, achieved = decode(args.batch)
    ms_per_step = dt / K * 1e3

    # further points: tokens a second, and beside each its share of the peak that bounds it (HBM
    # for decode steps, the matrix cores for prompt steps) in points_frac
    points, points_frac = {}, {}
    if not args.skip_points:
        for b in (1, 64):
            if b == args.batch:
                points[f"decode_b{b}"] = round(value, 1)
                points_frac[f"decode_b{b}"] = round(achieved / HBM_PEAK_GBS, 4)
                continue
            _, rate, gbs = decode(b)
            points[f"decode_b{b}"] = round(rate, 1)
            points_frac[f"decode_b{b}"] = round(gbs / HBM_PEAK_GBS, 4)
        if args.long_context > K + W and args.long_context != args.context:
            _, rate, gbs = decode(args.batch, args.long_context)
            points[f"decode_b{args.batch}_ctx{args.long_context}"] = round(rate, 1)
            points_frac[f"decode_b{args.batch}_ctx{args.long_context}"] = round(
                gbs / HBM_PEAK_GBS, 4)

    read_gbs = measured_read_bandwidth(device)
    # (the probe multiplies bfloat16; a float32 run has no matrix-core yardstick)
    mfma_tflops = measured_mfma_tflops(device) if args.dtype == "bfloat16" else None

    # prefill of one prompt, whole, logits at its last token
    peak = MFMA_PEAK_TFLOPS[args.dtype] * 1e12

    def prefill(T):
        """(seconds of a step alone, seconds of a step among PREFILL_STEPS queued one behind the
        other, flops of a step) for prompts of ``T`` tokens."""
        cm = CacheManager(model.cache_specs(), args.page_size,
                          (T + args.page_size - 1) // args.page_size + 1, 1)
        cm.allocate_storage(model.dtype, device)
        runner = StepRunner(model, cm, device)
        toks = [int(t) for t in torch.randint(0, cfg.vocab_size, (T,),
                                              generator=torch.Generator().manual_seed(2))]

        def prompt_steps(n):
            """n prompts of T tokens, one step each, queued one behind the other; seconds a step."""
            sync()
            t0 = time.perf_counter()
            for i in range(n):
                rc = cm.open(f"p{i}")
                runner.step([StepEntry(rc, toks, [T - 1])])
                cm.close(rc)                 # (its pages go to the next prompt: one stream, in order)
            sync()
            return (time.perf_counter() - t0) / n

        # one step by itself (the GPU idle before and after it), and PREFILL_STEPS of them back to
        # back, which is how an engine with work waiting runs them and how the decode steps above
        # are timed: the host's launches then run ahead of the kernels and the chip keeps its clocks
        alone = min(prompt_steps(1) for _ in range(3))
        queued = min(prompt_steps(PREFILL_STEPS) for _ in range(2))
        del runner, cm
        torch.cuda.empty_cache()
        return alone, queued, prefill_flops(cfg, T, n_layers)

    T = args.prefill_tokens
    alone_s, pre_s, flops = prefill(T)
    if not args.skip_points:
        for t_short in args.short_prompts:
            if t_short != T:
                _, queued, fl = prefill(t_short)
                points[f"prefill_t{t_short}"] = round(t_short / queued, 1)
                points_frac[f"prefill_t{t_short}"] = round(fl / queued / peak, 4)
    kernels = {} if args.skip_kernels else kernel_rates(
        model, cfg, args.batch, args.context, T, args.page_size, device, read_gbs, mfma_tflops,
        args.dtype)

    out = {
        "metric": f"decode tok/s at batch {args.batch} (LFM2-1.2B shape, context {args.context})",
        "value": round(value, 1), "unit": "tok/s", "n_gpus": 1, "steps": K, "warmup": W,
        "ms_per_step": round(ms_per_step, 4), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "bf16" if args.dtype == "bfloat16" else "fp32",
        "data": "synthetic",
        "config": {
            "model": "LFM2-1.2B shape, random weights", "hidden_size": cfg.hidden_size,
            "num_layers": n_layers_full, "num_layers_run": n_layers,
            "attention_layers": len(cfg.attention_layers), "conv_layers": len(cfg.conv_layers),
            "heads": cfg.num_attention_heads, "kv_heads": cfg.num_key_value_heads,
            "head_dim": cfg.head_dim, "ff_dim": cfg.ff_dim, "vocab_size": cfg.vocab_size,
            "conv_L_cache": cfg.conv_L_cache, "global_batch": args.batch,
            "seq_len": args.context, "prefill_tokens": T, "page_size": args.page_size,
            "parallelism": "single GPU",
        },
        "prefill": {"value": round(T / pre_s, 1), "tokens": T, "ms": round(pre_s * 1e3, 3),
                    "frac": round(flops / pre_s / peak, 5),
                    # ms is a step among PREFILL_STEPS queued back to back; alone_ms one step
                    # with the GPU idle before it
                    "steps": PREFILL_STEPS, "alone_ms": round(alone_s * 1e3, 3),
                    # what a kernel that only multiplies gets on this box, and the step against it
                    "measured_mfma_tflops": mfma_tflops and round(mfma_tflops, 1),
                    "frac_of_measured_mfma": mfma_tflops and round(
                        flops / pre_s / (mfma_tflops * 1e12), 5)},
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS,
                     "unit": "GB/s", "frac": round(achieved / HBM_PEAK_GBS, 5),
                     # what a kernel that only reads gets on this box, and the step against that
                     "measured_read": round(read_gbs, 1),
                     "frac_of_measured_read": round(achieved / read_gbs, 5)},
        "points": points,
        "points_frac": points_frac,
        "kernels": kernels,
    }
    print(json.dumps(out))
    return 0


if __name__ == "__main__":
    sys.exit(main())
