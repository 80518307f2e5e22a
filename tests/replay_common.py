"""Shared by the replay tests: random requests, the plain implementation's logits for
them, and the comparison of a replay's output with those."""
from __future__ import annotations

import json
import math
from pathlib import Path

import numpy as np

from plain import lfm2 as plain


def make_requests(vocab: int, lengths, seed: int):
    rng = np.random.default_rng(seed)
    return {f"r{i}": [int(t) for t in rng.integers(0, vocab, size=n)]
            for i, n in enumerate(lengths)}


_plain_cache = {}


def plain_logits(model_dir, requests, rnd=None):
    """{id: float64 [len, vocab]} from the plain implementation (cached per folder)."""
    key = (str(model_dir), json.dumps(requests, sort_keys=True), rnd is not None)
    if key not in _plain_cache:
        cfg, w = plain.read_model_dir(model_dir)
        kw = {} if rnd is None else {"rnd": rnd}
        _plain_cache[key] = {rid: plain.forward(cfg, w, toks, **kw)
                             for rid, toks in requests.items()}
    return _plain_cache[key]


def collect(index, outputs, vocab):
    """outputs: {step: float32 [wanted, vocab]} -> {(id, pos): logits row}."""
    got = {}
    for step, idx in enumerate(index):
        if not idx:
            continue
        arr = outputs[step]
        assert arr.shape == (len(idx), vocab), (step, arr.shape, len(idx))
        for row, key in zip(arr, idx):
            assert key not in got, f"{key} was asked for twice"
            got[key] = row
    return got


def worst_error(got, ref):
    """Largest |difference| over all wanted rows, relative to the largest |logit| of the
    reference, and where it is: (error, (id, pos))."""
    scale = max(float(np.abs(v).max()) for v in ref.values())
    worst, where = 0.0, None
    for (rid, pos), row in got.items():
        assert np.isfinite(row).all(), f"non-finite logits at {rid} position {pos}"
        err = float(np.abs(row.astype(np.float64) - ref[rid][pos]).max()) / scale
        if err > worst:
            worst, where = err, (rid, pos)
    return worst, where


FP32_TOL = 2e-5         # of the largest |logit|: float32 arithmetic against float64
# bfloat16 is measured against what rounding the same intermediate values to bfloat16 costs the
# plain implementation itself on the same requests (``rnd=plain.round_bf16``): the engine's
# largest error may be 1.5 times the plain implementation's largest, and its root mean square
# error 1.15 times (measured over the tiny configurations: 0.72-1.30 and 0.85-1.02).
BF16_MAX_FACTOR = 1.5
BF16_RMS_FACTOR = 1.15


def bf16_bounds(model_dir, requests, keys):
    """(largest error, rms error) of the plain implementation with bfloat16 rounding against
    itself without, over the rows ``keys`` = [(id, pos)], both relative to the largest |logit|."""
    ref = plain_logits(model_dir, requests)
    rounded = plain_logits(model_dir, requests, rnd=plain.round_bf16)
    scale = max(float(np.abs(v).max()) for v in ref.values())
    worst, sq, n = 0.0, 0.0, 0
    for rid, pos in keys:
        e = rounded[rid][pos] - ref[rid][pos]
        worst = max(worst, float(np.abs(e).max()))
        sq += float((e * e).sum())
        n += e.size
    return worst / scale, math.sqrt(sq / max(n, 1)) / scale


def assert_matches_plain(got, model_dir, requests, dtype, what=""):
    """``got``: {(id, pos): logits row} of the engine.  float32: every row within FP32_TOL;
    bfloat16: largest and rms error within their factors of the plain implementation's own."""
    ref = plain_logits(model_dir, requests)
    err, where = worst_error(got, ref)
    if dtype == "float32":
        assert err < FP32_TOL, (what, err, where, first_bad(got, ref, FP32_TOL))
        return err
    scale = max(float(np.abs(v).max()) for v in ref.values())
    sq, n = 0.0, 0
    for (rid, pos), row in got.items():
        e = row.astype(np.float64) - ref[rid][pos]
        sq += float((e * e).sum())
        n += e.size
    rms = math.sqrt(sq / max(n, 1)) / scale
    max_own, rms_own = bf16_bounds(model_dir, requests, list(got))
    tol = BF16_MAX_FACTOR * max_own
    assert err < tol, (what, "largest error", err, tol, where, first_bad(got, ref, tol))
    assert rms < BF16_RMS_FACTOR * rms_own, (what, "rms error", rms, rms_own)
    return err


def first_bad(got, ref, tol):
    """The first (id, position) whose error exceeds ``tol`` (for the failure message)."""
    scale = max(float(np.abs(v).max()) for v in ref.values())
    for (rid, pos) in sorted(got):
        err = float(np.abs(got[(rid, pos)].astype(np.float64) - ref[rid][pos]).max()) / scale
        if err > tol:
            return rid, pos, err
    return None


def read_outputs(out_dir, index, vocab):
    out = {}
    for step, idx in enumerate(index):
        if idx:
            out[step] = np.fromfile(Path(out_dir) / f"{step}.f32", dtype="<f4").reshape(-1, vocab)
    return out
