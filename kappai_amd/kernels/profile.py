"""Time by stage of the forward pass, for ``--time``.

kappai keeps a table of stages (embedding, norms, the products by role, rotation, cache store,
attention, logits; src/profile.h:9-92) that its executor fills with the time of every call
(src/recipe/exec.c:224-249) and prints after prefill and after decoding
(src/context.c:1597-1625, profile_print in src/profile.c:65-117).  Here a stage is a pair of
events on the GPU's stream around the kernels of a call: when the table is switched on, every
``scope`` records one before and one after, and ``report`` reads the differences once the
stream has drained.  Switched off (the default) a scope costs one attribute test.  Steps that
are replayed from a captured graph record nothing: the command line runs steps kernel by
kernel when it is asked for times.
"""
from __future__ import annotations

from typing import Dict, List, Tuple

import torch

# the order in which stages are printed (kappai's, as far as this engine has them)
STAGES = ["embd", "rmsnorm", "matmul", "matmul_qkv", "matmul_attn_out", "matmul_in_proj",
          "matmul_out_proj", "matmul_ffn_gate_up", "matmul_ffn_down", "short_conv", "rope_kvput",
          "attn", "ffn_act", "add", "logits_norm", "logits_matmul", "sample"]


class _Nothing:
    def __enter__(self):
        return self

    def __exit__(self, *exc):
        return False


_NOTHING = _Nothing()


class _Scope:
    def __init__(self, table, stage, weight_bytes):
        self.table, self.stage, self.weight_bytes = table, stage, weight_bytes

    def __enter__(self):
        self.e0 = torch.cuda.Event(enable_timing=True)
        self.e1 = torch.cuda.Event(enable_timing=True)
        self.table._depth += 1
        self.e0.record()
        return self

    def __exit__(self, *exc):
        self.e1.record()
        self.table._depth -= 1
        self.table._open.append((self.stage, self.e0, self.e1, self.weight_bytes))
        return False


class StageTimes:
    def __init__(self):
        self.enabled = False
        self._open: List[Tuple[str, torch.cuda.Event, torch.cuda.Event, int]] = []
        self._depth = 0

    def start(self) -> None:
        self.reset()
        self.enabled = True

    def stop(self) -> None:
        self.enabled = False

    def reset(self) -> None:
        self._open = []

    def scope(self, stage: str, weight_bytes: int = 0):
        """A context that times what is launched inside on the current stream under ``stage``.
        Scopes inside a scope are not recorded (a product that casts its input is still one
        product).  Switched off, this hands out one shared context that does nothing."""
        if not self.enabled or self._depth > 0:
            return _NOTHING
        return _Scope(self, stage, int(weight_bytes))

    def take(self) -> list:
        """The records made since the last ``take`` or ``reset``, which are then forgotten here:
        for a caller that keeps several tables (one for steps with prompt portions, one for
        decode steps) and hands each to ``report``."""
        recs, self._open = self._open, []
        return recs

    def totals(self, records=None) -> Dict[str, Tuple[float, int, int]]:
        """{stage: (microseconds, calls, weight bytes)}; waits for the GPU."""
        records = self._open if records is None else records
        if records:
            torch.cuda.synchronize()
        out: Dict[str, List[float]] = {}
        for stage, e0, e1, nbytes in records:
            t = out.setdefault(stage, [0.0, 0, 0])
            t[0] += e0.elapsed_time(e1) * 1e3
            t[1] += 1
            t[2] += nbytes
        return {k: (v[0], int(v[1]), int(v[2])) for k, v in out.items()}

    def report(self, label: str, wall_us: float = 0.0, records=None) -> str:
        """The table kappai prints (src/profile.c:86-112): stage, us, calls, us/call, share,
        weights read in MB and the rate in MB/s they were streamed at."""
        tot = self.totals(records)
        total = sum(v[0] for v in tot.values())
        head = f"[profile] {label}  accounted={total:.0f} us"
        if wall_us:
            head += f"  wall={wall_us:.0f} us  ({100.0 * total / wall_us:.1f}% attributed)"
        lines = [head]
        if not tot:
            return head + "\n  (no stages recorded)"
        lines.append(f"  {'stage':<18s} {'us':>12s} {'calls':>8s} {'us/call':>10s} {'share':>8s} "
                     f"{'wtMB':>9s} {'MB/s':>10s}")
        names = [s for s in STAGES if s in tot] + sorted(s for s in tot if s not in STAGES)
        for s in names:
            us, calls, nbytes = tot[s]
            lines.append(f"  {s:<18s} {us:12.0f} {calls:8d} {us / max(calls, 1):10.2f} "
                         f"{100.0 * us / max(total, 1e-9):7.2f}% {nbytes / 1e6:9.1f} "
                         f"{(nbytes / us if us else 0.0):10.2f}")
        if wall_us > total:
            lines.append(f"  {'  (unattributed)':<18s} {wall_us - total:12.0f} {'-':>8s} {'-':>10s} "
                         f"{100.0 * (wall_us - total) / wall_us:7.2f}%")
        return "\n".join(lines)


# the one table of the process (kappai keeps one per context; an engine here is one context)
STAGE_TIMES = StageTimes()
scope = STAGE_TIMES.scope
