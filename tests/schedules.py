"""Ways of cutting the same requests into steps.  Every builder returns
(steps, index, peak_tokens): the step objects that trace replay reads, for each step the
(request id, position) of every wanted row in output order, and the most tokens that live
requests hold at any time, each request's count rounded up to a multiple of 64."""
from __future__ import annotations

import itertools
from typing import Dict, List, Sequence, Tuple


def _round64(n: int) -> int:
    return (n + 63) // 64 * 64


def build(requests: Dict[str, Sequence[int]], plans: Dict[str, Tuple[int, List[int]]],
          want: str = "all"):
    """``plans[id] = (first step, portion sizes)``; the portions must add up to the request's
    length.  ``want``: "all" asks for every row, "last" for each portion's last row."""
    for rid, (_, portions) in plans.items():
        assert sum(portions) == len(requests[rid]), (rid, sum(portions), len(requests[rid]))
        assert all(p >= 1 for p in portions)
    done_tokens = {rid: 0 for rid in requests}
    next_portion = {rid: 0 for rid in requests}
    steps, index, peak = [], [], 0
    step = 0
    last_step = max(s + len(p) for s, p in plans.values())
    while step < last_step:
        entries, ended, idx = [], [], []
        for rid in requests:
            start, portions = plans[rid]
            k = next_portion[rid]
            if step < start or k >= len(portions):
                continue
            n = portions[k]
            p0 = done_tokens[rid]
            toks = [int(t) for t in requests[rid][p0:p0 + n]]
            wanted = list(range(n)) if want == "all" else [n - 1]
            entries.append({"id": rid, "tokens": toks, "want": wanted})
            idx.extend((rid, p0 + w) for w in wanted)
            done_tokens[rid] += n
            next_portion[rid] += 1
            if next_portion[rid] == len(portions):
                ended.append(rid)
        live = sum(_round64(done_tokens[r]) for r in requests
                   if 0 < done_tokens[r] and (next_portion[r] < len(plans[r][1]) or r in ended))
        peak = max(peak, live)
        assert len(entries) <= 4, "a trace has at most four live requests"
        steps.append({"step": step, "entries": entries, "end": ended})
        index.append(idx)
        step += 1
    return steps, index, peak


def whole(requests):
    """Each request alone, its whole token list in one step."""
    plans, step = {}, 0
    for rid, toks in requests.items():
        plans[rid] = (step, [len(toks)])
        step += 1
    return build(requests, plans)


def prefill_then_decode(requests, tail: int = 32):
    """Each request alone: all but the last ``tail`` tokens in one step, then one by one."""
    plans, step = {}, 0
    for rid, toks in requests.items():
        t = min(tail, len(toks) - 1)
        portions = [len(toks) - t] + [1] * t
        plans[rid] = (step, portions)
        step += len(portions)
    return build(requests, plans)


def cut(length: int, sizes: Sequence[int]) -> List[int]:
    out, it = [], itertools.cycle(sizes)
    while length > 0:
        n = min(next(it), length)
        out.append(n)
        length -= n
    return out


def changing_portions(requests, sizes=(7, 1, 2, 5, 3, 2, 16, 2, 1, 9, 2, 4)):
    """Each request alone, in portions of changing size, down to two tokens and one."""
    plans, step = {}, 0
    for i, (rid, toks) in enumerate(requests.items()):
        rot = list(sizes[i % len(sizes):]) + list(sizes[:i % len(sizes)])
        portions = cut(len(toks), rot)
        plans[rid] = (step, portions)
        step += len(portions)
    return build(requests, plans)


def mixed(requests, tail: int = 8, sizes=(5, 2, 9, 3, 2, 7), stagger: int = 3, max_live: int = 4):
    """Up to ``max_live`` requests live at a time: portions of the prompts of some beside
    single decoded tokens of others; a new request starts when an earlier one has ended, so
    that with a small pool its pages are those the earlier one gave back."""
    plans = {}
    ends: List[int] = []          # step after which each planned request has ended
    for i, (rid, toks) in enumerate(requests.items()):
        t = min(tail, len(toks) - 1)
        rot = list(sizes[i % len(sizes):]) + list(sizes[:i % len(sizes)])
        portions = cut(len(toks) - t, rot) + [1] * t
        start = i * stagger
        if len(ends) >= max_live:
            start = max(start, sorted(ends)[len(ends) - max_live] + 1)
        plans[rid] = (start, portions)
        ends.append(start + len(portions) - 1)
    return build(requests, plans)
