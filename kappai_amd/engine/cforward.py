"""The model and a step's rows as the C side takes them (``csrc/engine.h``), and the call that
runs a whole step from C: ``kappai_forward``.

kappai's forward call is C over a row description (compute_forward_rows, src/compute.h:120-149);
its entry points are C as well (src/engine.h:12-17).  Here the host builds, once per model and
cache, a flat list of the schedule's calls, each described by its own block and that block's
parts (``parts/cdesc.py``: a runner's name and the description it reads), and per step a small
struct with the addresses of the row tables; the C function then launches every kernel of the
step without coming back to Python in between.  Nothing here names a kind of part: a model whose
parts all describe themselves runs from C, any other model runs its steps from the parts' own
``forward`` methods, which give the same logits bit for bit for the models both can run.
"""
from __future__ import annotations

import ctypes
from ctypes import POINTER, Structure, c_float, c_int, c_size_t, c_void_p
from typing import List, Optional

import torch

from ..kernels import ops, tuning
from ..kernels.lib import KernelLaunchError, library
from ..parts.cdesc import (AttentionKernels, CallDesc, CarryDesc, CPlan, EmbeddedPartDesc,
                           FoldDesc, LinearDesc, NormPartDesc, PartDesc, RowsDesc, address_of,
                           defined_together)

ENGINE_ABI = 11
MAX_GROUPS = 8
MAX_TABLES = 8         # KAPPAI_MAX_TABLES


def _ptrs(names):
    return [(n, c_void_p) for n in names]


class Kernels(Structure):
    _fields_ = _ptrs(["embed_rows", "embed_rmsnorm", "add_rmsnorm", "swiglu", "cast",
                      "sum_partials", "gemm_f32", "gemm_bf16", "gemm_bf16_any", "gemm_bf16_swiglu",
                      "gemm_bf16_shortconv_step", "shortconv", "shortconv_parts",
                      "qk_norm_rope_store", "paged_attention_rows"])


class TuningDesc(Structure):
    _fields_ = [(n, c_int) for n in
                ("fused_step_min_width", "fused_step_narrow_width", "fused_step_narrow_rows",
                 "partial_sums_min_rows", "partial_sums_max_rows", "fragment_rows_min",
                 "fragment_rows_from", "fused_max_rows", "decode_waves", "decode_max_splits",
                 "decode_block_max_keys", "attention_tile_rows", "fused_qk")]


class ModelDesc(Structure):
    _fields_ = [
        ("abi", c_int), ("compute_bf16", c_int), ("width", c_int), ("vocab", c_int),
        ("page_size", c_int), ("embed_table", c_void_p), ("embed_is_bf16", c_int),
        ("n_calls", c_int), ("calls", POINTER(CallDesc)), ("final_norm", NormPartDesc),
        ("head", LinearDesc), ("kernels", POINTER(Kernels)), ("tuning", TuningDesc),
        ("on_embedding", EmbeddedPartDesc)]


class BatchDesc(Structure):
    _fields_ = [
        ("n_rows", c_int), ("n_segments", c_int), ("n_logit_rows", c_int), ("max_position", c_int),
        ("max_segment_rows", c_int), ("logits_of_every_row", c_int),
        ("tokens", c_void_p), ("row_pos", c_void_p),
        ("row_seg", c_void_p), ("seg_start", c_void_p), ("seg_pos0", c_void_p),
        ("seg_slot", c_void_p), ("logit_rows", c_void_p),
        ("tables", c_void_p * MAX_TABLES), ("table_rows", c_int * MAX_TABLES),
        ("numbers", c_int * MAX_TABLES), ("n_groups", c_int),
        ("block_tables", c_void_p * MAX_GROUPS),
        ("max_blocks", c_int * MAX_GROUPS)]


def engine_library():
    """The library of the C walk, its struct layouts checked against this module's."""
    lib = library("engine")
    if not getattr(lib, "_kappai_checked", False):
        mine = [ENGINE_ABI] + [ctypes.sizeof(t) for t in (
            Kernels, AttentionKernels, LinearDesc, FoldDesc, RowsDesc, CarryDesc, PartDesc,
            NormPartDesc, CallDesc, TuningDesc, ModelDesc, BatchDesc)]
        sizes = (c_int * len(mine))()
        n = lib.kappai_engine_layout(sizes, len(mine))
        if n != len(mine) or list(sizes) != mine:
            raise KernelLaunchError(f"csrc/engine.h and the host disagree about the layout of "
                                    f"their structs: {list(sizes)} ({n}) against {mine}")
        lib.kappai_forward_workspace_bytes.restype = c_size_t
        lib.kappai_forward_workspace_bytes.argtypes = [POINTER(ModelDesc), POINTER(BatchDesc)]
        lib.kappai_forward.argtypes = [POINTER(ModelDesc), POINTER(BatchDesc), c_void_p, c_size_t,
                                       c_void_p, c_void_p]
        lib.kappai_forward_error.restype = ctypes.c_char_p
        lib._kappai_checked = True
    return lib


class Workspace:
    """The memory a step's activations are cut from; grows to the largest step seen.  A captured
    graph keeps one of its own (its kernels hold addresses inside it)."""

    def __init__(self):
        self.buffer: Optional[torch.Tensor] = None

    def at_least(self, nbytes: int, device) -> torch.Tensor:
        if self.buffer is None or self.buffer.numel() < nbytes:
            self.buffer = None
            self.buffer = torch.empty(int(nbytes * 1.25) + 4096, dtype=torch.uint8, device=device)
        return self.buffer


class NotDescribed(Exception):
    """A part of the model has no description for the C side: its steps run from the host."""


class CForward:
    @staticmethod
    def plannable(model) -> bool:
        """Whether the model as a whole can be walked from C: it is bound, its embedding, final
        norm and head describe themselves, so does what changes the embedded rows (if anything
        does), and its ``forward`` is the one the C walk repeats.  Whether every block describes
        itself shows when the plan is built (``NotDescribed``)."""
        if not model.bound:
            return False
        if model.embedding_position is not None and not defined_together(
                model.embedding_position, "on_embedding", "c_embedded"):
            return False
        if model.dtype not in (torch.bfloat16, torch.float32):
            return False
        return (defined_together(model, "forward", "c_calls")
                and defined_together(model.embedding, "forward", "c_table")
                and defined_together(model.head, "forward", "c_linear")
                and defined_together(model.final_norm, "add_norm", "c_norm"))

    def __init__(self, model, cache, device):
        self.model, self.cache, self.device = model, cache, torch.device(device)
        self.lib = engine_library()
        self.plan = plan = CPlan(self.lib, model, cache, self.device)
        k = Kernels()
        el, gm, sc, at = (library("elementwise"), library("gemm"), library("shortconv"),
                          library("attention"))
        for name, fn in (("embed_rows", el.kappai_embed_rows),
                         ("embed_rmsnorm", el.kappai_embed_rmsnorm),
                         ("add_rmsnorm", el.kappai_add_rmsnorm),
                         ("swiglu", el.kappai_swiglu), ("cast", el.kappai_cast),
                         ("sum_partials", el.kappai_sum_partials),
                         ("gemm_f32", gm.kappai_gemm_f32), ("gemm_bf16", gm.kappai_gemm_bf16),
                         ("gemm_bf16_any", gm.kappai_gemm_bf16_any),
                         ("gemm_bf16_swiglu", gm.kappai_gemm_bf16_swiglu),
                         ("gemm_bf16_shortconv_step", gm.kappai_gemm_bf16_shortconv_step),
                         ("shortconv", sc.kappai_shortconv),
                         ("shortconv_parts", sc.kappai_shortconv_parts),
                         ("qk_norm_rope_store", at.kappai_qk_norm_rope_store),
                         ("paged_attention_rows", at.kappai_paged_attention_rows)):
            setattr(k, name, address_of(fn))
        self.kernels = k
        described = model.c_calls(plan)
        final_norm = model.final_norm.c_norm(plan)
        on_embedding = None
        if model.embedding_position is not None:
            on_embedding = model.embedding_position.c_embedded(plan)
        if described is None or final_norm is None or (
                model.embedding_position is not None and on_embedding is None):
            raise NotDescribed()
        calls = (CallDesc * max(len(described), 1))()
        for ci, call in enumerate(described):
            calls[ci] = call
        self.calls = calls
        m = ModelDesc()
        m.abi, m.compute_bf16 = ENGINE_ABI, 1 if plan.bf16 else 0
        m.width, m.vocab, m.page_size = model.embedding.width, model.vocab_size, cache.page_size
        table = model.embedding.c_table()
        m.embed_table = table.data_ptr()
        m.embed_is_bf16 = (2 if isinstance(table, ops.InFragments)
                           else 1 if table.dtype == torch.bfloat16 else 0)
        m.n_calls, m.calls = len(described), calls
        m.final_norm = final_norm
        if on_embedding is not None:
            m.on_embedding = on_embedding
        m.head = plan.linear(model.head.c_linear())
        m.kernels = ctypes.pointer(self.kernels)
        t = m.tuning
        t.fused_step_min_width = tuning.FUSED_STEP_MIN_WIDTH
        t.fused_step_narrow_width = tuning.FUSED_STEP_NARROW_WIDTH
        t.fused_step_narrow_rows = tuning.FUSED_STEP_NARROW_ROWS
        t.partial_sums_min_rows = tuning.PARTIAL_SUMS_MIN_ROWS
        t.partial_sums_max_rows = tuning.PARTIAL_SUMS_MAX_ROWS
        t.fragment_rows_min = tuning.FRAGMENT_ROWS_MIN if tuning.FRAGMENT_ROWS else 1 << 30
        t.fragment_rows_from = ops.FRAGMENT_ROWS_FROM
        t.fused_max_rows = ops.FUSED_MAX_ROWS
        t.decode_waves, t.decode_max_splits = ops.DECODE_WAVES, ops.DECODE_MAX_SPLITS
        t.decode_block_max_keys = ops.DECODE_BLOCK_MAX_KEYS
        t.attention_tile_rows = ops.ATTENTION_TILE_ROWS
        t.fused_qk = tuning.FUSED_QK_MAX_ROWS if tuning.FUSED_QK else 0
        self.desc = m
        self.workspace = Workspace()

    def batch_desc(self, batch) -> BatchDesc:
        b = BatchDesc()
        b.n_rows, b.n_segments, b.n_logit_rows = batch.n_rows, batch.n_segments, batch.n_logit_rows
        b.max_position, b.max_segment_rows = batch.max_position, batch.max_segment_rows
        b.logits_of_every_row = 1 if batch.logits_of_every_row else 0
        b.tokens, b.row_pos, b.row_seg = (batch.tokens.data_ptr(), batch.row_pos.data_ptr(),
                                          batch.row_seg.data_ptr())
        b.seg_start, b.seg_pos0, b.seg_slot = (batch.seg_start.data_ptr(), batch.seg_pos0.data_ptr(),
                                               batch.seg_slot.data_ptr())
        b.logit_rows = batch.logit_rows.data_ptr()
        for at, name in enumerate(self.plan.tables):
            t = batch.extra.get(name)
            if t is not None:
                b.tables[at], b.table_rows[at] = t.data_ptr(), t.shape[0]
        for at in range(MAX_TABLES):
            b.numbers[at] = -1
        for at, name in enumerate(self.plan.numbers):
            b.numbers[at] = batch.numbers.get(name, -1)
        if len(batch.block_tables) > MAX_GROUPS:
            raise ValueError(f"a step carries block tables for at most {MAX_GROUPS} groups")
        b.n_groups = len(batch.block_tables)
        for g, t in enumerate(batch.block_tables):
            b.block_tables[g] = t.data_ptr()
            b.max_blocks[g] = t.shape[1]
        return b

    def forward(self, batch, workspace: Optional[Workspace] = None) -> torch.Tensor:
        """float32 logits [wanted rows, vocab] of the step, every kernel queued on torch's
        current stream."""
        self.plan.before_step(batch)
        b = self.batch_desc(batch)
        need = self.lib.kappai_forward_workspace_bytes(ctypes.byref(self.desc), ctypes.byref(b))
        if need == 0:
            raise KernelLaunchError(self.lib.kappai_forward_error().decode() or
                                    "kappai_forward refuses this step")
        ws = (workspace or self.workspace).at_least(need, self.device)
        logits = torch.empty((batch.n_logit_rows, self.model.vocab_size), dtype=torch.float32,
                             device=self.device)
        rc = self.lib.kappai_forward(ctypes.byref(self.desc), ctypes.byref(b), ws.data_ptr(),
                                     ws.numel(), logits.data_ptr(), ops._stream())
        if rc != 0:
            msg = self.lib.kappai_forward_error().decode()
            raise KernelLaunchError(f"kappai_forward: HIP error {rc}" + (f" ({msg})" if msg else ""))
        return logits
