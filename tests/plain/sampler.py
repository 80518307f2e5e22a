"""Plain host sampler after src/sampler.c of System64fumo/kappai, one token at a time."""
from __future__ import annotations

import numpy as np

MASK = (1 << 64) - 1


def splitmix64(state: int):
    """src/common.h:243-248.  Returns (new_state, value)."""
    state = (state + 0x9E3779B97F4A7C15) & MASK
    z = state
    z = ((z ^ (z >> 30)) * 0xBF58476D1CE4E5B9) & MASK
    z = ((z ^ (z >> 27)) * 0x94D049BB133111EB) & MASK
    return state, z ^ (z >> 31)


def _rotl(x, k):
    return ((x << k) | (x >> (64 - k))) & MASK


class Rng:
    """src/sampler.c:13-32: four words from splitmix64(seed); a xoshiro256-style step
    whose output is rotl(s0+s3, 23)+s0; a uniform is the top 24 bits times 2^-24."""

    def __init__(self, seed: int):
        if seed == 0:
            seed = 0xDEADBEEFCAFEBABE
        z = seed & MASK
        self.s = []
        for _ in range(4):
            z, v = splitmix64(z)
            self.s.append(v)

    def uniform(self) -> float:
        s = self.s
        result = (_rotl((s[0] + s[3]) & MASK, 23) + s[0]) & MASK
        t = (s[1] << 17) & MASK
        s[2] ^= s[0]
        s[3] ^= s[1]
        s[1] ^= s[2]
        s[0] ^= s[3]
        s[2] ^= t
        s[3] = _rotl(s[3], 45)
        return float(np.float32(result >> 40) * np.float32(2.0 ** -24))


def argmax_lowest(logits) -> int:
    """ties go to the lowest index (src/sampler.c:125-136)."""
    best, bestv = 0, logits[0]
    for i in range(1, len(logits)):
        if logits[i] > bestv:
            bestv, best = logits[i], i
    return best


def apply_repeat_penalty(logits, recent, penalty):
    """positive logits divided, others multiplied, once per occurrence in the window
    (src/sampler.c:205-216)."""
    out = np.array(logits, dtype=np.float32, copy=True)
    for tok in recent:
        if 0 <= tok < len(out):
            if out[tok] > 0:
                out[tok] = out[tok] / np.float32(penalty)
            else:
                out[tok] = out[tok] * np.float32(penalty)
    return out


def sample_full_vocab(logits, temperature, u):
    """softmax of logit/T over the whole vocabulary and an inverse-CDF draw with one
    uniform (src/sampler.c:234-258)."""
    lg = np.asarray(logits, dtype=np.float32)
    inv = np.float32(1.0) / np.float32(temperature)
    scaled = lg * inv
    mx = scaled.max()
    e = np.exp((scaled - mx).astype(np.float32)).astype(np.float32)
    total = float(np.sum(e.astype(np.float64)))
    rnd = float(u) * total
    acc = np.cumsum(e.astype(np.float64))
    idx = int(np.searchsorted(acc, rnd, side="right"))
    return min(idx, len(lg) - 1)


def sample_filtered(logits, temperature, top_k, top_p, min_p, u, cap=1024):
    """candidates sorted by logit, top-k (or the best ``cap`` when only top-p/min-p are
    set, src/sampler.c:218-232), softmax of logit/T, top-p keeps the crossing token
    (:271-281), min-p is relative to the best (:283-291), then a draw (:293-314)."""
    lg = np.asarray(logits, dtype=np.float32)
    vocab = len(lg)
    if 0 < top_k < vocab:
        keep = top_k
    elif top_p < 1.0 or min_p > 0.0:
        keep = min(vocab, cap)
    else:
        keep = vocab
    order = np.argsort(-lg, kind="stable")[:keep]
    vals = lg[order]
    inv = np.float32(1.0) / np.float32(temperature)
    e = np.exp((vals * inv - vals[0] * inv).astype(np.float32)).astype(np.float32)
    total = np.float32(0)
    for x in e:
        total = np.float32(total + x)
    kept = len(e)
    if top_p < 1.0:
        cum = np.float32(0)
        for i in range(len(e)):
            cum = np.float32(cum + e[i] / total)
            if cum > np.float32(top_p):
                kept = i + 1
                break
    if min_p > 0.0:
        floor = np.float32(min_p) * (e[0] / total)
        n = 0
        while n < kept and (e[n] / total) >= floor:
            n += 1
        kept = n if n > 0 else 1
    psum = np.float32(0)
    for x in e[:kept]:
        psum = np.float32(psum + x)
    rnd = np.float32(u) * psum
    acc = np.float32(0)
    for i in range(kept):
        acc = np.float32(acc + e[i])
        if rnd < acc:
            return int(order[i])
    return int(order[kept - 1])


class PlainSampler:
    """src/sampler.c:334-352 with the defaults' meanings of src/config.c:156-172."""

    def __init__(self, seed, temperature=0.8, top_k=40, top_p=0.9, min_p=0.1,
                 repeat_penalty=1.0, repeat_last_n=64):
        self.rng = Rng(seed)
        self.temperature, self.top_k, self.top_p, self.min_p = temperature, top_k, top_p, min_p
        self.repeat_penalty, self.repeat_last_n = repeat_penalty, repeat_last_n
        self.recent = []

    def observe(self, tok):
        self.recent.append(int(tok))

    def sample(self, logits) -> int:
        lg = np.asarray(logits, dtype=np.float32)
        vocab = len(lg)
        if self.repeat_penalty != 1.0 and self.recent:
            n = min(self.repeat_last_n, len(self.recent))
            lg = apply_repeat_penalty(lg, self.recent[len(self.recent) - n:], self.repeat_penalty)
        if self.temperature <= 0.0 or self.top_k == 1:
            return argmax_lowest(lg)
        if (self.top_k <= 0 or self.top_k >= vocab) and self.top_p >= 1.0 and self.min_p <= 0.0:
            return sample_full_vocab(lg, self.temperature, self.rng.uniform())
        return sample_filtered(lg, self.temperature, self.top_k, self.top_p, self.min_p,
                               self.rng.uniform())
