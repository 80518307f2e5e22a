"""kappai's random stream (src/sampler.c:13-32): four words from splitmix64(seed)
(src/common.h:243-248), a xoshiro256-style step whose output is rotl(s0 + s3, 23) + s0,
and uniforms made of the top 24 bits."""
from __future__ import annotations

import os

_MASK = (1 << 64) - 1


def _rotl(x: int, k: int) -> int:
    return ((x << k) | (x >> (64 - k))) & _MASK


def _splitmix64(state: int):
    state = (state + 0x9E3779B97F4A7C15) & _MASK
    z = state
    z = ((z ^ (z >> 30)) * 0xBF58476D1CE4E5B9) & _MASK
    z = ((z ^ (z >> 27)) * 0x94D049BB133111EB) & _MASK
    return state, z ^ (z >> 31)


class RandomStream:
    def __init__(self, seed: int):
        """Seed 0 asks the operating system (src/sampler.c:34-43)."""
        seed = int(seed) & _MASK
        if seed == 0:
            seed = int.from_bytes(os.urandom(8), "little") or 0xDEADBEEFCAFEBABE
        z = seed
        self.s = [0, 0, 0, 0]
        for i in range(4):
            z, self.s[i] = _splitmix64(z)

    def uniform(self) -> float:
        """A float32 value in [0, 1): (next >> 40) * 2^-24."""
        s = self.s
        result = (_rotl((s[0] + s[3]) & _MASK, 23) + s[0]) & _MASK
        t = (s[1] << 17) & _MASK
        s[2] ^= s[0]
        s[3] ^= s[1]
        s[1] ^= s[2]
        s[0] ^= s[3]
        s[2] ^= t
        s[3] = _rotl(s[3], 45)
        return (result >> 40) * (2.0 ** -24)
