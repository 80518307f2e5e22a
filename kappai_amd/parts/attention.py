"""Grouped-query attention over the paged cache.

Order as kappai's attention block (src/models/lfm.c:32-51): q, k, v projections (one
product over the stacked matrices); optional per-head RMSNorm of q and k with one shared
weight per head size (src/backend/cpu/scalar/quants.c:1521-1531); rotation at the row's
absolute position; k and v stored before attention so that a portion's own keys are
visible (src/recipe/ops_basic.c:567-632); softmax(q k / sqrt(d)) v over keys 0..p, head h
reading kv head h // (H/G) (src/backend/cpu/scalar/core.c:383-433, 623-666); output
projection.
"""
from __future__ import annotations

import math
from dataclasses import dataclass
from typing import Dict, List, Optional

import numpy as np
import torch

from ..cache.specs import PagedKV
from ..kernels import ops, profile, tuning
from ..weights.spec import INIT_ONES, VECTOR, TensorSpec
import ctypes
from ctypes import POINTER, Structure, c_float, c_int, c_void_p

from .base import Mixer, PositionEncoding, StepTables, register_part
from .cdesc import AttentionKernels, LinearDesc, tensor_ptr
from .linear import Linear


class AttentionMixerDesc(Structure):
    """``kappai_attention_mixer`` of csrc/engine_parts.h."""
    _fields_ = [
        ("qkv", LinearDesc), ("out", LinearDesc), ("q_norm_w", c_void_p), ("k_norm_w", c_void_p),
        ("qk_eps", c_float), ("heads", c_int), ("kv_heads", c_int), ("head_dim", c_int),
        ("window", c_int), ("scale", c_float), ("cos_table", c_void_p), ("sin_table", c_void_p),
        ("rot_dim", c_int), ("rot_mode", c_int), ("rot_positions", c_int), ("k_pool", c_void_p),
        ("v_pool", c_void_p), ("group", c_int), ("shared_cache", c_int),
        ("mfma", POINTER(AttentionKernels)), ("tiles_table", c_int), ("lone_table", c_int),
        ("lone_number", c_int)]


@dataclass(frozen=True)
class AttentionTiles(StepTables):
    """What the tiled attention kernel walks: ``q_tiles`` [tiles, 4], the segments cut into runs
    of at most ``rows`` rows, tile j of a segment as (segment, first row, rows, place); the
    fourth number tells a kernel where the tile stands in its segment (index | tiles of the
    segment << 16, or 0 when the segment has more tiles than 15 bits hold), so that it can pair
    tiles of one segment.  ``lone_from``: in a step that holds segments of several rows, the
    segments of a single row are left out of the tiles and listed in ``lone_rows`` (with the
    number ``max_lone_position``) when the longest of their contexts has at least that many
    keys: the block that got such a row as a tile would walk all its keys alone, so these rows
    go to the decode kernel."""
    rows: int
    lone_from: Optional[int] = None

    family = "attention_tiles"
    decode_constant = True

    def combine(self, others):
        rows = {self.rows} | {o.rows for o in others}
        if len(rows) > 1:
            raise ValueError(f"the layers ask for tiles of different sizes: {sorted(rows)}")
        lone = {self.lone_from} | {o.lone_from for o in others}
        return AttentionTiles(self.rows, lone.pop() if len(lone) == 1 else None)

    def build(self, step):
        seg_start = step.arrays["seg_start"].astype(np.int64)
        p0 = step.arrays["seg_pos0"].astype(np.int64)
        n = seg_start[1:] - seg_start[:-1]
        S = n.shape[0]
        arrays, numbers = {}, {"max_lone_position": -1}
        nt = (n + self.rows - 1) // self.rows
        lone = n == 1
        if (self.lone_from and lone.any() and not lone.all() and step.page_size % 16 == 0
                and int(p0[lone].max()) + 1 >= self.lone_from):
            arrays["lone_rows"] = seg_start[:-1][lone].astype(np.int32)
            numbers["max_lone_position"] = int(p0[lone].max())
            nt = np.where(lone, 0, nt)
        tile_seg = np.repeat(np.arange(S, dtype=np.int64), nt)
        first_tile = np.cumsum(nt) - nt
        idx = np.arange(int(nt.sum()), dtype=np.int64) - np.repeat(first_tile, nt)
        rows = np.minimum(self.rows, n[tile_seg] - idx * self.rows)
        nts = nt[tile_seg]
        place = np.where(nts > 0x7fff, 0, idx | (nts << 16))
        arrays["q_tiles"] = np.stack(
            [tile_seg, seg_start[tile_seg] + idx * self.rows, rows, place],
            axis=1).astype(np.int32)
        return arrays, numbers


class GroupedQueryAttention(Mixer):
    takes_deferred_rows = True     # its first product takes what ops.linear takes
    adds_residual = True           # its last product can add into the residual stream

    def __init__(self, prefix: str, width: int, num_heads: int, num_kv_heads: int, head_dim: int,
                 dtype: torch.dtype, position: Optional[PositionEncoding] = None,
                 qk_norm_eps: Optional[float] = None, window: Optional[int] = None,
                 bias: bool = False, scale: Optional[float] = None, names=None):
        n = {"q": "q_proj", "k": "k_proj", "v": "v_proj", "o": "out_proj",
             "q_norm": "q_layernorm", "k_norm": "k_layernorm"}
        n.update(names or {})
        if num_heads % num_kv_heads:
            raise ValueError(f"{num_heads} heads cannot be shared out over {num_kv_heads} kv heads")
        self.prefix, self.width, self.dtype = prefix, width, dtype
        self.H, self.G, self.d = num_heads, num_kv_heads, head_dim
        self.window = window
        self.position = position
        self.qk_norm_eps = qk_norm_eps
        self.scale = float(scale) if scale is not None else 1.0 / math.sqrt(head_dim)
        self.qkv = Linear([prefix + n["q"], prefix + n["k"], prefix + n["v"]], width,
                          [num_heads * head_dim, num_kv_heads * head_dim, num_kv_heads * head_dim],
                          bias=bias, stage="matmul_qkv", cut_rows_at=[num_heads * head_dim])
        self.q_only: Optional[Linear] = None      # the q rows alone (bind)
        self.out = Linear([prefix + n["o"]], num_heads * head_dim, [width], bias=bias,
                          stage="matmul_attn_out")
        self._qn, self._kn = prefix + n["q_norm"], prefix + n["k_norm"]
        self.q_norm_w: Optional[torch.Tensor] = None
        self.k_norm_w: Optional[torch.Tensor] = None

    @property
    def step_tables(self) -> AttentionTiles:
        # single rows beside portions: what the decode kernel needs (the page size is checked
        # where the table is laid out)
        ok = (self.dtype == torch.bfloat16 and self.H // self.G <= 16 and self.d % 16 == 0
              and self.d <= 256)
        return AttentionTiles(ops.ATTENTION_TILE_ROWS,
                              tuning.LONE_ROWS_FROM if ok and tuning.LONE_ROWS_FROM else None)

    def cache_spec(self):
        return PagedKV(self.G, self.d, self.window)

    def tensor_specs(self) -> List[TensorSpec]:
        specs = self.qkv.tensor_specs() + self.out.tensor_specs()
        if self.qk_norm_eps is not None:
            specs.append(TensorSpec(self._qn + ".weight", (self.d,), VECTOR, INIT_ONES))
            specs.append(TensorSpec(self._kn + ".weight", (self.d,), VECTOR, INIT_ONES))
        return specs

    def bind(self, tensors: Dict[str, torch.Tensor]) -> None:
        self.qkv.bind(tensors)
        self.out.bind(tensors)
        # the q rows of the stacked matrix, for a layer that reads another layer's keys
        self.q_only = self.qkv.first_rows(self.H * self.d)
        if self.qk_norm_eps is not None:
            self.q_norm_w = tensors[self._qn + ".weight"].to(torch.float32).contiguous()
            self.k_norm_w = tensors[self._kn + ".weight"].to(torch.float32).contiguous()

    def forward(self, x, batch, cache, shared_cache: bool = False, into=None):
        H, G, d = self.H, self.G, self.d
        # more than 16 rows (decode, short prompt portions): the projection may come as sums over
        # ranges of its input dimension (more blocks stream the matrix), which the next kernel adds up
        proj = (self.q_only if shared_cache else self.qkv).forward(
            x, partial_sums=tuning.takes_partial_sums(x.shape[0], batch.max_segment_rows == 1))
        rot = self.position.rotation(x.device, batch.max_position) if self.position else None
        tables = batch.block_tables[cache.group]
        k_pool, v_pool = cache.pool("k"), cache.pool("v")
        single = batch.max_segment_rows == 1
        if self._prologue_in_kernel(proj, rot, single, cache.page_size, batch.max_position):
            # decode: norm, rotation and store inside the attention kernel
            with profile.scope("attn"):
                ctx = ops.paged_attention(
                    proj, H, G, d, k_pool, v_pool, batch.row_pos, batch.row_seg, tables,
                    cache.page_size, self.scale, window=self.window or 0, single_rows=True,
                    max_position=batch.max_position, kernel="decode",
                    qk=ops.QkPrologue(self.q_norm_w, self.k_norm_w, self.qk_norm_eps or 0.0,
                                      rot.cos if rot else None, rot.sin if rot else None,
                                      store_kv=not shared_cache))
            return self.out.forward(ctx, partial_sums=True, add_into=into)
        with profile.scope("rope_kvput"):
            q = ops.qk_norm_rope_store(
                proj, H, G, d, self.q_norm_w, self.k_norm_w, self.qk_norm_eps or 0.0,
                rot.cos if rot else None, rot.sin if rot else None, rot.rot_dim if rot else 0,
                rot.mode if rot else ops.ROT_NONE, k_pool, v_pool, batch.row_pos,
                batch.row_seg, tables, cache.page_size, store_kv=not shared_cache)
        with profile.scope("attn"):
            ctx = ops.paged_attention(q, H, G, d, k_pool, v_pool, batch.row_pos,
                                      batch.row_seg, tables, cache.page_size, self.scale,
                                      window=self.window or 0,
                                      q_tiles=batch.extra.get("q_tiles"), single_rows=single,
                                      max_position=batch.max_position,
                                      lone_rows=batch.extra.get("lone_rows"),
                                      max_lone_position=batch.numbers.get("max_lone_position",
                                                                          -1))
        return self.out.forward(ctx, partial_sums=True, add_into=into)

    def c_part(self, plan, view, shared_cache: bool = False):
        """The runner "mixer.attention" (csrc/engine_parts.hip) makes the same choices as
        ``forward``.  The rotation tables grow with the context, so the description is brought
        up to date before every step."""
        first = plan.linear(self.qkv)
        d = AttentionMixerDesc()
        d.qkv, d.out = first, plan.linear(self.out)
        d.q_norm_w, d.k_norm_w = tensor_ptr(self.q_norm_w), tensor_ptr(self.k_norm_w)
        d.qk_eps = self.qk_norm_eps or 0.0
        d.heads, d.kv_heads, d.head_dim = self.H, self.G, self.d
        d.window, d.scale = self.window or 0, self.scale
        d.k_pool, d.v_pool = view.pool("k").data_ptr(), view.pool("v").data_ptr()
        d.group = view.group
        d.shared_cache = 1 if shared_cache else 0
        d.rot_mode = ops.ROT_NONE
        d.tiles_table, d.lone_table = plan.table("q_tiles"), plan.table("lone_rows")
        d.lone_number = plan.number("max_lone_position")
        if plan.bf16 and self.d % 16 == 0 and self.d <= 256:
            d.mfma = ctypes.pointer(plan.attention_kernels(self.d))
        if self.position is not None:
            def rotation_tables(batch, d=d, position=self.position, device=plan.device):
                rot = position.rotation(device, batch.max_position)
                if rot is None:
                    d.rot_mode = ops.ROT_NONE
                    return
                d.cos_table, d.sin_table = rot.cos.data_ptr(), rot.sin.data_ptr()
                d.rot_dim, d.rot_mode, d.rot_positions = rot.rot_dim, rot.mode, rot.cos.shape[0]
            plan.on_step(rotation_tables)
        return plan.part("mixer.attention", d, takes_deferred_rows=True, adds_residual=True,
                         first=first)

    def _prologue_in_kernel(self, proj, rot, single_rows: bool, page_size: int,
                            max_position: int) -> bool:
        """Whether the decode attention kernels take the projection as it is (see
        ``ops.QkPrologue``): a step of a few single rows whose projection came as bfloat16 rows, few
        enough query heads a kv head for the decode kernels, a head size they do it for, no
        rotation or rotate-half over the whole head, and keys enough for the kernel that splits
        them over blocks (where a block is one wave; in the other every wave of a block would do
        the prologue again, which costs what the kernel saved)."""
        if not (tuning.FUSED_QK and single_rows and isinstance(proj, torch.Tensor)
                and proj.dim() == 2 and proj.shape[0] <= tuning.FUSED_QK_MAX_ROWS
                and proj.dtype == torch.bfloat16 and proj.is_cuda
                and self.H // self.G <= 16 and proj.stride(0) % 8 == 0
                and proj.data_ptr() % 16 == 0):
            return False
        if rot is not None and not (rot.mode == ops.ROT_HALF and rot.rot_dim == self.d):
            return False
        return (ops.decode_takes_qk(self.d, page_size)
                and ops.decode_form(self.H, self.G, self.d, max_position,
                                    self.window or 0) == "decode-split")

    def weight_bytes(self) -> int:
        return self.qkv.weight_bytes() + self.out.weight_bytes() + 2 * self.d * 4


register_part("mixer", "attention", GroupedQueryAttention)
