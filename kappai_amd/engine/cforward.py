"""The model and a step's rows as the C side takes them (``csrc/engine.h``), and the call that
runs a whole step from C: ``kappai_forward``.

kappai's forward call is C over a row description (compute_forward_rows, src/compute.h:120-149);
its entry points are C as well (src/engine.h:12-17).  Here the host builds, once per model and
cache, a flat description of the layer calls with the addresses of their tensors, and per step a
small struct with the addresses of the row tables; the C function then launches every kernel of
the step without coming back to Python in between.  ``CForward.plannable`` says whether a model
is made of the parts that the C side knows (the framework's own); any other model runs its steps
from the parts' own ``forward`` methods, which give the same logits bit for bit for the models
both can run.
"""
from __future__ import annotations

import ctypes
from ctypes import POINTER, Structure, c_float, c_int, c_size_t, c_void_p
from typing import List, Optional

import torch

from ..cache.specs import PagedKV
from ..kernels import ops, profile, tuning
from ..kernels.lib import KernelLaunchError, library
from ..parts import attention as attention_part
from ..parts import norm as norm_part
from ..parts import shortconv as shortconv_part
from ..parts.block import PreNormBlock
from ..parts.embedding import OutputHead, TokenEmbedding
from ..parts.feed_forward import SwiGLU
from ..parts.rotary import RotaryEncoding

ENGINE_ABI = 8
MAX_GROUPS = 8


def _ptrs(names):
    return [(n, c_void_p) for n in names]


class Kernels(Structure):
    _fields_ = _ptrs(["embed_rows", "embed_rmsnorm", "add_rmsnorm", "swiglu", "cast", "gemm_f32", "gemm_bf16",
                      "gemm_bf16_any", "gemm_bf16_swiglu", "gemm_bf16_shortconv_step", "shortconv",
                      "shortconv_parts", "qk_norm_rope_store", "paged_attention_rows"])


class AttentionKernels(Structure):
    _fields_ = _ptrs(["keys_per_wave", "decode_block_waves", "attn_prefill", "attn_decode",
                      "attn_decode_block", "attn_decode_rows", "decode_takes_qk",
                      "attn_decode_qk"])


class LinearDesc(Structure):
    _fields_ = [("w", c_void_p), ("w_frag", c_void_p), ("bias", c_void_p), ("n", c_int),
                ("k", c_int), ("w_is_f32", c_int)]


class NormDesc(Structure):
    _fields_ = [("w", c_void_p), ("eps", c_float)]


class LayerCallDesc(Structure):
    _fields_ = [
        ("mixer", c_int), ("mixer_norm", NormDesc), ("ffn_norm", NormDesc),
        ("in_proj", LinearDesc), ("out_proj", LinearDesc), ("taps", c_void_p),
        ("conv_bias", c_void_p), ("taps_per_channel", c_int), ("state", c_void_p),
        ("qkv", LinearDesc), ("attn_out", LinearDesc), ("q_norm_w", c_void_p),
        ("k_norm_w", c_void_p), ("qk_eps", c_float), ("heads", c_int), ("kv_heads", c_int),
        ("head_dim", c_int), ("window", c_int), ("scale", c_float), ("cos_table", c_void_p),
        ("sin_table", c_void_p), ("rot_dim", c_int), ("rot_mode", c_int), ("rot_positions", c_int),
        ("k_pool", c_void_p), ("v_pool", c_void_p), ("group", c_int), ("shared_cache", c_int),
        ("mfma", POINTER(AttentionKernels)),
        ("gate_up", LinearDesc), ("down", LinearDesc), ("hidden", c_int), ("ffn_fused", c_int)]


class ModelDesc(Structure):
    _fields_ = [
        ("abi", c_int), ("compute_bf16", c_int), ("width", c_int), ("vocab", c_int),
        ("page_size", c_int), ("embed_table", c_void_p), ("embed_is_bf16", c_int),
        ("n_calls", c_int), ("calls", POINTER(LayerCallDesc)), ("final_norm", NormDesc),
        ("head", LinearDesc), ("kernels", POINTER(Kernels)),
        ("fused_step_min_width", c_int), ("fused_step_narrow_width", c_int),
        ("fused_step_narrow_rows", c_int), ("partial_sums_min_rows", c_int),
        ("partial_sums_max_rows", c_int),
        ("fragment_rows_min", c_int), ("fragment_rows_from", c_int), ("fused_max_rows", c_int),
        ("decode_waves", c_int), ("decode_max_splits", c_int), ("decode_block_max_keys", c_int),
        ("attention_tile_rows", c_int), ("fused_qk", c_int)]


class BatchDesc(Structure):
    _fields_ = [
        ("n_rows", c_int), ("n_segments", c_int), ("n_logit_rows", c_int), ("max_position", c_int),
        ("max_segment_rows", c_int), ("logits_of_every_row", c_int),
        ("tokens", c_void_p), ("row_pos", c_void_p),
        ("row_seg", c_void_p), ("seg_start", c_void_p), ("seg_pos0", c_void_p),
        ("seg_slot", c_void_p), ("logit_rows", c_void_p), ("q_tiles", c_void_p),
        ("n_tiles", c_int), ("lone_rows", c_void_p), ("n_lone_rows", c_int),
        ("max_lone_position", c_int), ("n_groups", c_int),
        ("block_tables", c_void_p * MAX_GROUPS),
        ("max_blocks", c_int * MAX_GROUPS)]


def _engine():
    lib = library("engine")
    if not getattr(lib, "_kappai_checked", False):
        sizes = (c_int * 8)()
        lib.kappai_engine_layout(sizes, 8)
        mine = [ENGINE_ABI] + [ctypes.sizeof(t) for t in (Kernels, AttentionKernels, LinearDesc,
                                                          NormDesc, LayerCallDesc, ModelDesc,
                                                          BatchDesc)]
        if list(sizes) != mine:
            raise KernelLaunchError(f"csrc/engine.h and engine/cforward.py disagree about the "
                                    f"layout of their structs: {list(sizes)} against {mine}")
        lib.kappai_forward_workspace_bytes.restype = c_size_t
        lib.kappai_forward_workspace_bytes.argtypes = [POINTER(ModelDesc), POINTER(BatchDesc)]
        lib.kappai_forward.argtypes = [POINTER(ModelDesc), POINTER(BatchDesc), c_void_p, c_size_t,
                                       c_void_p, c_void_p]
        lib.kappai_forward_error.restype = ctypes.c_char_p
        lib._kappai_checked = True
    return lib


def _address(fn) -> int:
    return ctypes.cast(fn, c_void_p).value


def _tensor_ptr(t: Optional[torch.Tensor]):
    return None if t is None else t.data_ptr()


def _linear(lin) -> LinearDesc:
    w = lin.weight
    in_fragments = isinstance(w, ops.InFragments)
    return LinearDesc(None if in_fragments else w.data_ptr(), w.data_ptr() if in_fragments else None,
                      _tensor_ptr(lin.bias), w.shape[0], w.shape[1],
                      1 if w.dtype == torch.float32 else 0)


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


class CForward:
    @staticmethod
    def plannable(model) -> bool:
        """True if every part of the model is one the C side knows, exactly (a subclass may have
        changed what ``forward`` does)."""
        if model.embedding_position is not None or not model.bound:
            return False
        if type(model.embedding) is not TokenEmbedding or type(model.head) is not OutputHead:
            return False
        if type(model.final_norm) is not norm_part.RMSNorm:
            return False
        if model.dtype not in (torch.bfloat16, torch.float32):
            return False
        for blk in model.layers:
            if type(blk) is not PreNormBlock:
                return False
            if (type(blk.mixer_norm) is not norm_part.RMSNorm
                    or type(blk.ffn_norm) is not norm_part.RMSNorm
                    or type(blk.feed_forward) is not SwiGLU):
                return False
            mx = blk.mixer
            if type(mx) is shortconv_part.GatedShortConv:
                continue
            if type(mx) is not attention_part.GroupedQueryAttention:
                return False
            if mx.position is not None and type(mx.position) is not RotaryEncoding:
                return False
            if type(mx.cache_spec()) is not PagedKV:
                return False
        return True

    def __init__(self, model, cache, device):
        self.model, self.cache, self.device = model, cache, torch.device(device)
        self.lib = _engine()
        self._keep: List[object] = []                # everything the descriptions point into
        k = Kernels()
        el, gm, sc, at = (library("elementwise"), library("gemm"), library("shortconv"),
                          library("attention"))
        for name, fn in (("embed_rows", el.kappai_embed_rows),
                         ("embed_rmsnorm", el.kappai_embed_rmsnorm),
                         ("add_rmsnorm", el.kappai_add_rmsnorm),
                         ("swiglu", el.kappai_swiglu), ("cast", el.kappai_cast),
                         ("gemm_f32", gm.kappai_gemm_f32), ("gemm_bf16", gm.kappai_gemm_bf16),
                         ("gemm_bf16_any", gm.kappai_gemm_bf16_any),
                         ("gemm_bf16_swiglu", gm.kappai_gemm_bf16_swiglu),
                         ("gemm_bf16_shortconv_step", gm.kappai_gemm_bf16_shortconv_step),
                         ("shortconv", sc.kappai_shortconv),
                         ("shortconv_parts", sc.kappai_shortconv_parts),
                         ("qk_norm_rope_store", at.kappai_qk_norm_rope_store),
                         ("paged_attention_rows", at.kappai_paged_attention_rows)):
            setattr(k, name, _address(fn))
        self.kernels = k
        self._mfma = {}
        bf16 = model.dtype == torch.bfloat16
        calls = (LayerCallDesc * max(len(model.schedule), 1))()
        self._rotary = []            # (call index, RotaryEncoding)
        for ci, call in enumerate(model.schedule):
            blk = model.layers[call.layer]
            d = calls[ci]
            d.mixer_norm = NormDesc(blk.mixer_norm.weight.data_ptr(), blk.mixer_norm.eps)
            d.ffn_norm = NormDesc(blk.ffn_norm.weight.data_ptr(), blk.ffn_norm.eps)
            view = cache.view(model.cache_id(ci))
            mx = blk.mixer
            if type(mx) is shortconv_part.GatedShortConv:
                d.mixer = 0
                d.in_proj, d.out_proj = _linear(mx.in_proj), _linear(mx.out_proj)
                d.taps, d.conv_bias = mx.taps.data_ptr(), _tensor_ptr(mx.conv_bias)
                d.taps_per_channel = mx.L
                d.state = view.state.data_ptr()
            else:
                d.mixer = 1
                d.qkv, d.attn_out = _linear(mx.qkv), _linear(mx.out)
                d.q_norm_w, d.k_norm_w = _tensor_ptr(mx.q_norm_w), _tensor_ptr(mx.k_norm_w)
                d.qk_eps = mx.qk_norm_eps or 0.0
                d.heads, d.kv_heads, d.head_dim = mx.H, mx.G, mx.d
                d.window, d.scale = mx.window or 0, mx.scale
                d.k_pool, d.v_pool = view.pool("k").data_ptr(), view.pool("v").data_ptr()
                d.group = view.group
                d.shared_cache = 1 if call.reads_cache_of is not None else 0
                d.rot_mode = ops.ROT_NONE
                if mx.position is not None:
                    self._rotary.append((ci, mx.position))
                if bf16 and mx.d % 16 == 0 and mx.d <= 256:
                    d.mfma = ctypes.pointer(self._attention_kernels(mx.d))
            ff = blk.feed_forward
            d.gate_up, d.down = _linear(ff.gate_up), _linear(ff.down)
            d.hidden, d.ffn_fused = ff.hidden, 1 if ff.fused else 0
        self.calls = calls
        m = ModelDesc()
        m.abi, m.compute_bf16 = ENGINE_ABI, 1 if bf16 else 0
        m.width, m.vocab, m.page_size = model.embedding.width, model.vocab_size, cache.page_size
        table = model.embedding.table
        m.embed_table = table.data_ptr()
        m.embed_is_bf16 = (2 if isinstance(table, ops.InFragments)
                           else 1 if table.dtype == torch.bfloat16 else 0)
        m.n_calls, m.calls = len(model.schedule), calls
        m.final_norm = NormDesc(model.final_norm.weight.data_ptr(), model.final_norm.eps)
        m.head = _linear(model.head.linear)
        m.kernels = ctypes.pointer(self.kernels)
        m.fused_step_min_width = tuning.FUSED_STEP_MIN_WIDTH
        m.fused_step_narrow_width = tuning.FUSED_STEP_NARROW_WIDTH
        m.fused_step_narrow_rows = tuning.FUSED_STEP_NARROW_ROWS
        m.partial_sums_min_rows = tuning.PARTIAL_SUMS_MIN_ROWS
        m.partial_sums_max_rows = tuning.PARTIAL_SUMS_MAX_ROWS
        m.fragment_rows_min = tuning.FRAGMENT_ROWS_MIN if tuning.FRAGMENT_ROWS else 1 << 30
        m.fragment_rows_from = ops.FRAGMENT_ROWS_FROM
        m.fused_max_rows = ops.FUSED_MAX_ROWS
        m.decode_waves, m.decode_max_splits = ops.DECODE_WAVES, ops.DECODE_MAX_SPLITS
        m.decode_block_max_keys = ops.DECODE_BLOCK_MAX_KEYS
        m.attention_tile_rows = ops.ATTENTION_TILE_ROWS
        m.fused_qk = tuning.FUSED_QK_MAX_ROWS if tuning.FUSED_QK else 0
        self.desc = m
        self.workspace = Workspace()

    def _attention_kernels(self, head_dim: int) -> AttentionKernels:
        if head_dim not in self._mfma:
            lib = library("attention_mfma", HEAD_DIM=head_dim)
            a = AttentionKernels()
            a.keys_per_wave = _address(lib.kappai_attn_keys_per_wave)
            a.decode_block_waves = _address(lib.kappai_attn_decode_block_waves)
            a.attn_prefill = _address(lib.kappai_attn_prefill)
            a.attn_decode = _address(lib.kappai_attn_decode)
            a.attn_decode_block = _address(lib.kappai_attn_decode_block)
            a.attn_decode_rows = _address(lib.kappai_attn_decode_rows)
            a.decode_takes_qk = _address(lib.kappai_attn_decode_takes_qk)
            a.attn_decode_qk = _address(lib.kappai_attn_decode_qk)
            self._mfma[head_dim] = a
        return self._mfma[head_dim]

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
        if batch.q_tiles is not None:
            b.q_tiles, b.n_tiles = batch.q_tiles.data_ptr(), batch.q_tiles.shape[0]
        if batch.lone_rows is not None:
            b.lone_rows, b.n_lone_rows = batch.lone_rows.data_ptr(), batch.lone_rows.shape[0]
            b.max_lone_position = batch.max_lone_position
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
        for ci, pos in self._rotary:
            rot = pos.rotation(self.device, batch.max_position)
            d = self.calls[ci]
            d.cos_table, d.sin_table = rot.cos.data_ptr(), rot.sin.data_ptr()
            d.rot_dim, d.rot_mode, d.rot_positions = rot.rot_dim, rot.mode, rot.cos.shape[0]
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
