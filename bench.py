#!/usr/bin/env python3
"""Decode and prefill throughput of kappai_amd on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

The default run has the layer sizes of the LFM2-1.2B shape with random bfloat16 weights:
W untimed and K timed decode steps at batch 8 with every request holding a context of 4,096
tokens at the last step (one step = one token for every request: row tables, model,
sampling on the GPU, token ids back on the host), a prefill of 2,048 tokens, and decode at
batch 1 and 64.  It prints ONE JSON line.  Token ids are uniform random with a fixed seed
and the cache contents that stand for the earlier context are random numbers: no dataset
is involved ("data": "synthetic").  kappai publishes no numbers for this architecture, so
"vs_baseline" is null; the roofline fractions are against MI355X's published peaks.
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

LFM2_1_2B = {
    "architectures": ["Lfm2ForCausalLM"], "model_type": "lfm2", "hidden_size": 2048,
    "num_hidden_layers": 16,
    "layer_types": ["conv", "conv", "full_attention", "conv", "conv", "full_attention", "conv",
                    "conv", "full_attention", "conv", "full_attention", "conv", "full_attention",
                    "conv", "full_attention", "conv"],
    "num_attention_heads": 32, "num_key_value_heads": 8, "head_dim": 64,
    "intermediate_size": 12288, "block_auto_adjust_ff_dim": True, "block_multiple_of": 256,
    "block_ffn_dim_multiplier": 1.0, "vocab_size": 65536, "norm_eps": 1e-5,
    "rope_theta": 1000000.0, "conv_L_cache": 3, "conv_bias": False, "tie_embedding": True,
    "max_position_embeddings": 128000,
}


def lfm2_shape(hidden, layers, attention_at, heads, kv_heads, intermediate):
    raw = dict(LFM2_1_2B)
    raw.update(hidden_size=hidden, num_hidden_layers=layers, num_attention_heads=heads,
               num_key_value_heads=kv_heads, intermediate_size=intermediate,
               layer_types=["full_attention" if i in attention_at else "conv"
                            for i in range(layers)])
    return raw


LFM2_350M = lfm2_shape(1024, 16, (2, 5, 8, 10, 12, 14), 16, 8, 6656)
LFM2_2_6B = lfm2_shape(2048, 30, (2, 6, 10, 14, 18, 21, 24, 27), 32, 8, 10752)

# Serving workloads (through Engine: scheduler, prompt portions beside decoded tokens, sampling)
WORKLOADS = {
    # 64 requests at once, prompts of 128..2048 tokens cut into portions of 512, 256 tokens each
    "serve-350m": dict(raw=LFM2_350M, name="LFM2-350M shape", requests=64, prompt=(128, 2048),
                       n_predict=256, chunk=512, token_budget=576, ctx=4096),
    # 16 requests with 32,768-token contexts, 512 tokens each
    "long-2.6b": dict(raw=LFM2_2_6B, name="LFM2-2.6B shape", requests=16, prompt=(32768 - 512, 32768 - 512),
                      n_predict=512, chunk=2048, token_budget=2048, ctx=32768),
}


def run_workload(key, dtype, device):
    """One serving workload from start to end through ``Engine.generate`` with greedy sampling:
    all requests arrive together.  Prints one JSON line: generated tokens a second over the
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
    out = eng.generate(prompts, SamplingParams.greedy(n_predict=w["n_predict"]))
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
                   "token_budget": w["token_budget"], "ctx_size": w["ctx"]},
        "engine": {"steps": m.steps, "prefill_tok_s": round(m.pp, 1), "decode_tok_s": round(m.tg, 1),
                   "ttft_ms": round(m.first_token_ms, 2), "graph_replays": eng.runner.graph_replays,
                   "preemptions": eng.scheduler.preempted_total},
    }))
    return 0


def random_model(raw, dtype, device, seed=0, std=0.02):
    """The model of ``raw`` with N(0, std) weights made on the GPU (norm weights 1)."""
    import torch

    from kappai_amd.config import config_from_dict
    from kappai_amd.models import build_model
    from kappai_amd.weights import parse_dtype

    cfg = config_from_dict(raw)
    tdt = parse_dtype(dtype)
    model = build_model(cfg, tdt)
    gen = torch.Generator(device=device).manual_seed(seed)
    tensors = {}
    for spec in model.tensor_specs():
        if spec.init == "ones":
            t = torch.ones(spec.shape, dtype=torch.float32, device=device)
        else:
            t = torch.randn(spec.shape, generator=gen, dtype=torch.float32, device=device) * std
        tensors[spec.name] = t.to(tdt)
    model.bind(tensors)
    return model


def sync():
    import torch
    torch.cuda.synchronize()


class DecodeBench:
    """``batch`` requests whose caches hold ``start`` tokens of random keys and values, then
    decoded greedily one token a step."""

    def __init__(self, model, batch, start, total, page_size, device, seed=1, graphs=True):
        import torch

        from kappai_amd.cache import CacheManager
        from kappai_amd.engine import StepEntry, StepRunner
        self.torch, self.StepEntry = torch, StepEntry
        pages = batch * ((total + page_size - 1) // page_size)
        self.cache = CacheManager(model.cache_specs(), page_size, pages, batch)
        self.cache.allocate_storage(model.dtype, device)
        gen = torch.Generator(device=device).manual_seed(seed)
        for g in self.cache.paged_groups:
            for pools in g.pools.values():
                for t in pools.values():
                    t.copy_(torch.randn(t.shape, generator=gen, device=device,
                                        dtype=torch.float32) * 0.5)
        self.runner = StepRunner(model, self.cache, device, decode_graphs=graphs)
        self.requests = [self.cache.open(i) for i in range(batch)]
        for rc in self.requests:
            self.cache.extend(rc, start)
            self.cache.commit(rc, start)
        self.tokens = [int(t) for t in torch.randint(0, model.vocab_size, (batch,), generator=torch.Generator().manual_seed(seed))]
        self.temp = torch.zeros(batch, dtype=torch.float32, device=device)
        self.uni = torch.zeros(batch, dtype=torch.float32, device=device)
        self.model = model

    def step(self):
        from kappai_amd.kernels import ops
        entries = [self.StepEntry(rc, [tok], [0]) for rc, tok in zip(self.requests, self.tokens)]
        logits = self.runner.step(entries)
        self.tokens = ops.sample_rows(logits, self.temp, self.uni).tolist()

    def _choose(self, logits, step, out_row):
        from kappai_amd.kernels import ops
        ops.sample_rows(logits, self.temp, self.uni, out=out_row)

    def run(self, warmup, steps, run_len=8):
        """``steps`` decode steps, taken the way the engine takes them when nothing but decoding
        is going on: up to ``run_len`` steps queued back to back, each step's token handed to the
        next on the GPU, the host reading the tokens at the end of the run."""
        for _ in range(warmup):
            self.step()
        sync()
        t0 = time.perf_counter()
        left = steps
        while left > 0:
            n = min(run_len, left)
            out = None
            if n > 1:
                out = self.runner.decode_run(self.requests, self.tokens, n, self._choose)
            if out is None:
                self.step()
                left -= 1
            else:
                self.tokens = out[-1].tolist()
                left -= n
        sync()
        return time.perf_counter() - t0

    def close(self):
        for rc in self.requests:
            self.cache.close(rc)


def measured_read_bandwidth(device, mb=256, buffers=5, reps=20):
    """GB/s of a kernel that only reads: buffers of ``mb`` MB taken in turn (more than the
    memory-side cache holds), ``reps`` reads between two synchronisations."""
    import torch

    from kappai_amd.kernels import ops
    bufs = [torch.empty(mb * 1000 * 1000 // 4, dtype=torch.int32, device=device).random_()
            for _ in range(buffers)]
    for b in bufs:
        ops.stream_read(b)
    sync()
    t0 = time.perf_counter()
    total = 0
    for i in range(reps):
        total += ops.stream_read(bufs[i % buffers])
    sync()
    return total / (time.perf_counter() - t0) / 1e9


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
    ap.add_argument("--no-graphs", action="store_true",
                    help="launch decode steps kernel by kernel (for counter collection)")
    ap.add_argument("--workload", default="decode", choices=["decode"] + sorted(WORKLOADS),
                    help="decode: the headline run; the others are serving workloads through "
                         "the engine's scheduler")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this engine runs on one GPU; --gpus must be 1 (nothing was measured)")
        return 2
    if args.workload != "decode":
        return run_workload(args.workload, args.dtype, "cuda:0")

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
    start = args.context - (K + W)
    if start < 1:
        print("bench.py: --context must exceed --steps + --warmup")
        return 2

    def decode(batch):
        b = DecodeBench(model, batch, start, args.context, args.page_size, device,
                        graphs=not args.no_graphs)
        dt = b.run(W, K)
        kv_bytes = b.cache.bytes_per_token(elem)
        b.close()
        del b
        torch.cuda.empty_cache()
        return dt, kv_bytes

    dt, kv_bytes_per_token = decode(args.batch)
    ms_per_step = dt / K * 1e3
    value = args.batch * K / dt
    # bytes a decode step has to read: every weight once, the cache of the live requests
    mean_ctx = start + W + (K - 1) / 2.0
    step_bytes = model.weight_bytes_per_step() + args.batch * mean_ctx * kv_bytes_per_token
    achieved = step_bytes / (dt / K) / 1e9

    points = {}
    if not args.skip_points:
        for b in (1, 64):
            if b == args.batch:
                points[f"decode_b{b}"] = round(value, 1)
                continue
            dtb, _ = decode(b)
            points[f"decode_b{b}"] = round(b * K / dtb, 1)

    read_gbs = measured_read_bandwidth(device)

    # prefill of one prompt, whole, logits at its last token
    T = args.prefill_tokens
    cm = CacheManager(model.cache_specs(), args.page_size, (T + args.page_size - 1) // args.page_size + 1, 1)
    cm.allocate_storage(model.dtype, device)
    runner = StepRunner(model, cm, device)
    toks = [int(t) for t in torch.randint(0, cfg.vocab_size, (T,), generator=torch.Generator().manual_seed(2))]
    times = []
    for it in range(3):
        rc = cm.open("p")
        sync()
        t0 = time.perf_counter()
        runner.step([StepEntry(rc, toks, [T - 1])])
        sync()
        times.append(time.perf_counter() - t0)
        cm.close(rc)
    pre_s = min(times[1:])
    flops = prefill_flops(cfg, T, n_layers)
    peak = MFMA_PEAK_TFLOPS[args.dtype] * 1e12

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
                    "frac": round(flops / pre_s / peak, 5)},
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS,
                     "unit": "GB/s", "frac": round(achieved / HBM_PEAK_GBS, 5),
                     # what a kernel that only reads gets on this box, and the step against that
                     "measured_read": round(read_gbs, 1),
                     "frac_of_measured_read": round(achieved / read_gbs, 5)},
        "points": points,
    }
    print(json.dumps(out))
    return 0


if __name__ == "__main__":
    sys.exit(main())
