"""Generation options with kappai's names, meanings and defaults (``cli_args``,
src/config.c:156-172; usage text :84-154)."""
from __future__ import annotations

from dataclasses import dataclass


@dataclass
class SamplingParams:
    temperature: float = 0.80     # <= 0: greedy argmax
    top_k: int = 40               # 0: disabled; 1: greedy
    top_p: float = 0.90           # 1.0: disabled
    min_p: float = 0.10           # 0.0: disabled
    repeat_penalty: float = 1.0   # 1.0: disabled
    repeat_last_n: int = 64
    seed: int = 0                 # 0: from the operating system's entropy
    n_predict: int = -1           # most tokens to generate; -1: until the context ends

    @classmethod
    def greedy(cls, n_predict: int = -1) -> "SamplingParams":
        return cls(temperature=0.0, top_k=0, top_p=1.0, min_p=0.0, n_predict=n_predict)

    def is_greedy(self) -> bool:
        return self.temperature <= 0.0 or self.top_k == 1

    def is_filtered(self, vocab: int) -> bool:
        """True when top-k, top-p or min-p narrows the candidates (src/sampler.c:345-351)."""
        if self.is_greedy():
            return False
        return not ((self.top_k <= 0 or self.top_k >= vocab) and self.top_p >= 1.0
                    and self.min_p <= 0.0)

    def validate(self) -> None:
        if self.repeat_penalty <= 0:
            raise ValueError("repeat_penalty must be positive")
        if self.repeat_last_n < 0:
            raise ValueError("repeat_last_n must not be negative")
        if not 0.0 <= self.min_p <= 1.0:
            raise ValueError("min_p must lie in [0, 1]")
        if self.top_p <= 0.0:
            raise ValueError("top_p must be positive")
