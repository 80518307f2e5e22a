"""How a part describes itself to the C side of a step (``csrc/engine.h``).

The C walk runs a model as a list of calls, each a function (a "runner", registered in C under
a name) and a description that only that function reads.  A part that wants its steps launched
from C gives itself one more method, which builds its description and names its runner:

* a mixer or a feed-forward: ``c_part(plan, view, shared_cache) -> PartDesc or None``,
* a norm: ``c_norm(plan) -> NormPartDesc or None``,
* a block: ``c_call(plan, view, shared_cache) -> CallDesc or None``,
* a position encoding that changes the embedded rows: ``c_embedded(plan) -> EmbeddedPartDesc or
  None``

(``None``: not from C in this configuration; the model then runs from the parts' ``forward``
methods).  ``plan`` is a ``CPlan``: it looks runners up by name, checks that the description has
the size the runner expects, keeps alive what the descriptions point into, and lets a part ask to
be called before every step (``on_step``: the rotation tables grow with the context).

The structures here mirror those of ``csrc/engine.h`` that parts are made of; the descriptions of
the framework's own parts (``csrc/engine_parts.h``) are mirrored where those parts live.
kappai: operations register their handlers themselves (RECIPE_REGISTER, src/recipe.h:577-580).
"""
from __future__ import annotations

import ctypes
from ctypes import POINTER, Structure, c_float, c_int, c_void_p
from typing import Callable, List, Optional

import torch

RUNNER_PART, RUNNER_NORM, RUNNER_BLOCK, RUNNER_EMBEDDED = 0, 1, 2, 3
TAKES_DEFERRED_ROWS, ADDS_RESIDUAL = 1, 2


class LinearDesc(Structure):
    _fields_ = [("w", c_void_p), ("w_frag", c_void_p), ("bias", c_void_p), ("n", c_int),
                ("k", c_int), ("w_is_f32", c_int)]


class FoldDesc(Structure):
    _fields_ = [("w", c_void_p), ("eps", c_float)]


class RowsDesc(Structure):
    _fields_ = [("data", c_void_p), ("is_bf16", c_int), ("M", c_int), ("D", c_int), ("ld", c_int),
                ("frag", c_int), ("ss", c_void_p), ("ss_parts", c_int), ("eps", c_float),
                ("norm", POINTER(FoldDesc))]


class CarryDesc(Structure):
    _fields_ = [("kind", c_int), ("data", c_void_p), ("is_f32", c_int), ("parts", c_int),
                ("scaled", RowsDesc)]


class PartDesc(Structure):
    _fields_ = [("run", c_void_p), ("desc", c_void_p), ("flags", c_int),
                ("first", POINTER(LinearDesc))]


class NormPartDesc(Structure):
    _fields_ = [("run", c_void_p), ("desc", c_void_p), ("fold", POINTER(FoldDesc))]


class CallDesc(Structure):
    _fields_ = [("run", c_void_p), ("desc", c_void_p), ("first_norm", POINTER(NormPartDesc)),
                ("first_consumer", POINTER(PartDesc))]


class EmbeddedPartDesc(Structure):
    _fields_ = [("run", c_void_p), ("desc", c_void_p)]


class AttentionKernels(Structure):
    _fields_ = [(n, c_void_p) for n in
                ("keys_per_wave", "decode_block_waves", "attn_prefill", "attn_decode",
                 "attn_decode_block", "attn_decode_rows", "decode_takes_qk", "attn_decode_qk")]


def address_of(fn) -> int:
    return ctypes.cast(fn, c_void_p).value


def tensor_ptr(t: Optional[torch.Tensor]):
    return None if t is None else t.data_ptr()


def defined_together(part, method: str, c_method: str) -> bool:
    """True if the class that gave ``part`` its ``method`` also gave it ``c_method``: a subclass
    that changes what ``forward`` does without saying how that looks from C does not inherit the
    description of its parent's behaviour."""
    def origin(name):
        for k in type(part).__mro__:
            if name in k.__dict__:
                return k
        return None
    return origin(c_method) is not None and origin(method) is origin(c_method)


class CPlan:
    """What parts build their descriptions with; one per model and cache."""

    def __init__(self, engine_lib, model, cache, device):
        self.lib, self.model, self.cache, self.device = engine_lib, model, cache, device
        self.bf16 = model.dtype == torch.bfloat16
        self._keep: List[object] = []
        self._before_step: List[Callable] = []
        self._mfma = {}
        self.tables: List[str] = []       # names of the parts' own step tables, by their place
        self.numbers: List[str] = []      # in kappai_batch::tables / numbers
        engine_lib.kappai_runner.restype = c_void_p
        engine_lib.kappai_runner.argtypes = [ctypes.c_char_p, c_int, POINTER(c_int)]
        engine_lib.kappai_register_runner.argtypes = [ctypes.c_char_p, c_int, c_void_p, c_int]

    # -- lifetime --------------------------------------------------------------------------------
    def keep(self, obj):
        """Hold ``obj`` (a ctypes structure, a tensor) for as long as the plan lives."""
        self._keep.append(obj)
        return obj

    def on_step(self, fn: Callable) -> None:
        """``fn(batch)`` runs before every step's call into C (to refresh a description)."""
        self._before_step.append(fn)

    def before_step(self, batch) -> None:
        for fn in self._before_step:
            fn(batch)

    # -- the parts' own tables of a step -----------------------------------------------------------
    MAX_TABLES = 8

    def table(self, name: str) -> int:
        """The place in ``kappai_batch::tables`` where the runner finds ``RowBatch.extra[name]``
        (what the part's ``StepTables`` lays out under that name)."""
        return self._place(self.tables, name)

    def number(self, name: str) -> int:
        """The place in ``kappai_batch::numbers`` of ``RowBatch.numbers[name]``."""
        return self._place(self.numbers, name)

    def _place(self, names: List[str], name: str) -> int:
        if name not in names:
            if len(names) >= self.MAX_TABLES:
                from ..kernels.lib import KernelLaunchError
                raise KernelLaunchError(f"a step carries at most {self.MAX_TABLES} tables and "
                                        f"numbers of the parts' own")
            names.append(name)
        return names.index(name)

    # -- runners ---------------------------------------------------------------------------------
    def register_runner(self, name: str, kind: int, fn, desc_type) -> None:
        """Register a runner of a library of the caller's own (``fn``: the ctypes function)."""
        from ..kernels.lib import KernelLaunchError
        rc = self.lib.kappai_register_runner(name.encode(), kind, address_of(fn),
                                             ctypes.sizeof(desc_type))
        if rc != 0:
            raise KernelLaunchError(self.lib.kappai_forward_error().decode())

    def runner(self, name: str, kind: int, desc_type) -> int:
        from ..kernels.lib import KernelLaunchError
        size = c_int(-1)
        fn = self.lib.kappai_runner(name.encode(), kind, ctypes.byref(size))
        if not fn:
            raise KernelLaunchError(f"no runner is registered in C under the name {name!r}")
        if size.value != ctypes.sizeof(desc_type):
            raise KernelLaunchError(
                f"the runner {name!r} reads a description of {size.value} bytes, the host's "
                f"{desc_type.__name__} has {ctypes.sizeof(desc_type)}")
        return fn

    # -- building blocks -------------------------------------------------------------------------
    def linear(self, lin) -> LinearDesc:
        """The description of a ``parts.linear.Linear`` (kept alive by the plan)."""
        from ..kernels import ops
        w = lin.weight
        in_fragments = isinstance(w, ops.InFragments)
        return self.keep(LinearDesc(
            None if in_fragments else w.data_ptr(), w.data_ptr() if in_fragments else None,
            tensor_ptr(lin.bias), w.shape[0], w.shape[1], 1 if w.dtype == torch.float32 else 0))

    def part(self, runner: str, desc, takes_deferred_rows: bool = False,
             adds_residual: bool = False, first: Optional[LinearDesc] = None) -> PartDesc:
        self.keep(desc)
        flags = (TAKES_DEFERRED_ROWS if takes_deferred_rows else 0) | (
            ADDS_RESIDUAL if adds_residual else 0)
        return self.keep(PartDesc(self.runner(runner, RUNNER_PART, type(desc)),
                                  ctypes.addressof(desc), flags,
                                  ctypes.pointer(first) if first is not None else None))

    def norm(self, runner: str, desc, fold: Optional[FoldDesc] = None) -> NormPartDesc:
        self.keep(desc)
        return self.keep(NormPartDesc(self.runner(runner, RUNNER_NORM, type(desc)),
                                      ctypes.addressof(desc),
                                      ctypes.pointer(fold) if fold is not None else None))

    def call(self, runner: str, desc, first_norm: Optional[NormPartDesc] = None,
             first_consumer: Optional[PartDesc] = None) -> CallDesc:
        self.keep(desc)
        return self.keep(CallDesc(
            self.runner(runner, RUNNER_BLOCK, type(desc)), ctypes.addressof(desc),
            ctypes.pointer(first_norm) if first_norm is not None else None,
            ctypes.pointer(first_consumer) if first_consumer is not None else None))

    def embedded(self, runner: str, desc) -> EmbeddedPartDesc:
        """What changes the embedded rows before the first call (an encoding of positions)."""
        self.keep(desc)
        return self.keep(EmbeddedPartDesc(self.runner(runner, RUNNER_EMBEDDED, type(desc)),
                                          ctypes.addressof(desc)))

    def attention_kernels(self, head_dim: int) -> AttentionKernels:
        """The launchers of the matrix-core attention library of one head size."""
        from ..kernels.lib import library
        if head_dim not in self._mfma:
            lib = library("attention_mfma", HEAD_DIM=head_dim)
            a = AttentionKernels()
            for field, symbol in (("keys_per_wave", "kappai_attn_keys_per_wave"),
                                  ("decode_block_waves", "kappai_attn_decode_block_waves"),
                                  ("attn_prefill", "kappai_attn_prefill"),
                                  ("attn_decode", "kappai_attn_decode"),
                                  ("attn_decode_block", "kappai_attn_decode_block"),
                                  ("attn_decode_rows", "kappai_attn_decode_rows"),
                                  ("decode_takes_qk", "kappai_attn_decode_takes_qk"),
                                  ("attn_decode_qk", "kappai_attn_decode_qk")):
                setattr(a, field, address_of(getattr(lib, symbol)))
            self._mfma[head_dim] = self.keep(a)
        return self._mfma[head_dim]
