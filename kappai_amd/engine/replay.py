"""Trace replay: feed given token ids through a model step by step and write logits.

Nothing is sampled.  The program drives the framework's own model, step function, cache
manager and kernels, the ones that generation uses.  kappai has no such program; its
nearest relatives are the parity runs of its tests (src/test/test_plan.c:888-925,
src/test/test_hybrid.c:164-386).

Input, one JSON object a line:
    {"step": 0, "entries": [{"id": "a", "tokens": [5, 17, 3], "want": [0, 2]}], "end": []}
For a step in which something is wanted, ``<out>/<step>.f32`` holds the logits at the wanted
places as little-endian float32 [wanted, vocab], and ``<out>/index.jsonl`` gets a line that says
which rows these are: ``{"step": 0, "file": "0.f32", "vocab": V, "rows": [[id, position], ...]}``
(the position of the token in its request).  After every step a line ``done <step>``.
"""
from __future__ import annotations

import argparse
import json
import sys
from pathlib import Path
from typing import Callable, Dict, Iterable, Optional

import numpy as np

from ..cache.manager import CacheManager, RequestCache
from .batch import StepEntry

MAX_LIVE_REQUESTS = 8          # state slots of the replay pool (a trace has up to four live)
REPLAY_PAGE_SIZE = 16          # divides the 64 that a request's token count is rounded up to


def make_replay_cache(model, max_tokens: int, page_size: int = REPLAY_PAGE_SIZE,
                      num_slots: int = MAX_LIVE_REQUESTS) -> CacheManager:
    """A pool for ``max_tokens`` tokens: the most that live requests hold at any time, each
    request's count rounded up to a multiple of 64, hence to whole pages."""
    if 64 % page_size:
        raise ValueError(f"the replay pool needs a page size that divides 64, got {page_size}")
    pages = (max_tokens + page_size - 1) // page_size
    return CacheManager(model.cache_specs(), page_size, pages, num_slots)


class TraceReplayer:
    def __init__(self, runner, out_dir, log: Callable[[str], None] = None):
        self.runner = runner
        self.cache: CacheManager = runner.cache
        self.out_dir = Path(out_dir)
        self.out_dir.mkdir(parents=True, exist_ok=True)
        self.live: Dict[str, RequestCache] = {}
        self.log = log or (lambda s: None)
        self.index_path = self.out_dir / "index.jsonl"
        self.index_path.write_text("")

    def run_step(self, obj: dict) -> Optional[np.ndarray]:
        step = obj["step"]
        entries, rows = [], []
        for e in obj.get("entries", []):
            rid = e["id"]
            if rid not in self.live:
                self.live[rid] = self.cache.open(rid)
            want = list(e.get("want", []))
            rows += [[rid, self.live[rid].length + int(w)] for w in want]
            entries.append(StepEntry(self.live[rid], list(e["tokens"]), want))
        result = None
        if entries:
            logits = self.runner.step(entries)
            if logits.shape[0] > 0:
                result = logits.detach().to("cpu").numpy().astype("<f4", copy=False)
                result.tofile(self.out_dir / f"{step}.f32")
                with open(self.index_path, "a") as f:
                    f.write(json.dumps({"step": step, "file": f"{step}.f32",
                                        "vocab": int(result.shape[1]), "rows": rows}) + "\n")
        for rid in obj.get("end", []):
            if rid in self.live:
                self.cache.close(self.live.pop(rid))
        return result

    def run(self, lines: Iterable[str], done: Callable[[int], None]) -> None:
        for line in lines:
            line = line.strip()
            if not line:
                continue
            obj = json.loads(line)
            self.run_step(obj)
            done(obj["step"])


def main(argv=None) -> int:
    ap = argparse.ArgumentParser(prog="trace_run", description=__doc__.split("\n\n")[0])
    ap.add_argument("--model", required=True, help="folder with config.json and model.safetensors")
    ap.add_argument("--dtype", required=True, choices=["bfloat16", "float32"])
    ap.add_argument("--out", required=True, help="folder for <step>.f32")
    ap.add_argument("--max-tokens", type=int, required=True,
                    help="most tokens that live requests hold at any time")
    ap.add_argument("--page-size", type=int, default=REPLAY_PAGE_SIZE)
    ap.add_argument("--device", default="cuda:0")
    args = ap.parse_args(argv)

    import torch

    from ..models import load_model
    from .step import StepRunner

    if not torch.cuda.is_available():
        print("trace_run: no GPU is visible; kappai_amd runs on the GPU only", file=sys.stderr)
        return 1
    model = load_model(args.model, args.dtype, args.device)
    cache = make_replay_cache(model, args.max_tokens, args.page_size)
    cache.allocate_storage(model.dtype, args.device)
    runner = StepRunner(model, cache, args.device)
    rep = TraceReplayer(runner, args.out)

    def done(step):
        sys.stdout.write(f"done {step}\n")
        sys.stdout.flush()

    rep.run(sys.stdin, done)
    return 0
