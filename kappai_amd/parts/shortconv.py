"""Gated short convolution (the LFM2 conv layer's mixer).

kappai: src/models/lfm.c:13-19 and src/backend/cpu/common.c:2393-2431.  p = W_in x is cut
into B, C, x in this order; bx = B*x; a causal depthwise FIR of ``kernel_size`` taps runs
over bx, its history before the portion coming from the request's state slot
([width, kernel_size-1] float32, oldest first); y = C * s; out = W_out y.  With ``bias`` the
three linear maps (in_proj, the FIR, out_proj) have one each.
"""
from __future__ import annotations

from typing import Dict, List, Optional

import torch

from ..cache.specs import FixedState
from ..kernels import ops, profile, tuning
from ..weights.spec import INIT_NORMAL, INIT_SMALL, VECTOR, TensorSpec
from ctypes import Structure, c_int, c_void_p

from .base import Mixer, register_part
from .cdesc import LinearDesc, tensor_ptr
from .linear import Linear


class ConvMixerDesc(Structure):
    """``kappai_conv_mixer`` of csrc/engine_parts.h."""
    _fields_ = [("in_proj", LinearDesc), ("out_proj", LinearDesc), ("taps", c_void_p),
                ("conv_bias", c_void_p), ("taps_per_channel", c_int), ("state", c_void_p)]


class GatedShortConv(Mixer):
    takes_deferred_rows = True     # its first product takes what ops.linear takes
    adds_residual = True           # its last product can add into the residual stream

    def __init__(self, prefix: str, width: int, kernel_size: int, dtype: torch.dtype,
                 bias: bool = False, names=None):
        n = {"in": "in_proj", "conv": "conv", "out": "out_proj"}
        n.update(names or {})
        if kernel_size < 2:
            raise ValueError(f"a short convolution needs at least 2 taps, got {kernel_size}")
        self.prefix, self.width, self.L, self.dtype, self.has_bias = (
            prefix, width, kernel_size, dtype, bias)
        self.in_proj = Linear([prefix + n["in"]], width, [3 * width], bias=bias,
                              stage="matmul_in_proj")
        self.out_proj = Linear([prefix + n["out"]], width, [width], bias=bias,
                               stage="matmul_out_proj")
        self._conv = prefix + n["conv"]
        self.taps: Optional[torch.Tensor] = None
        self.conv_bias: Optional[torch.Tensor] = None

    def cache_spec(self):
        return FixedState((self.width, self.L - 1), "float32")

    def tensor_specs(self) -> List[TensorSpec]:
        specs = self.in_proj.tensor_specs() + self.out_proj.tensor_specs()
        # depthwise taps in the checkpoint's layout [channels, 1, taps]
        specs.append(TensorSpec(self._conv + ".weight", (self.width, 1, self.L), VECTOR,
                                INIT_NORMAL))
        if self.has_bias:
            specs.append(TensorSpec(self._conv + ".bias", (self.width,), VECTOR, INIT_SMALL))
        return specs

    def bind(self, tensors: Dict[str, torch.Tensor]) -> None:
        self.in_proj.bind(tensors)
        self.out_proj.bind(tensors)
        self.taps = tensors[self._conv + ".weight"].to(torch.float32).reshape(
            self.width, self.L).contiguous()
        if self.has_bias:
            self.conv_bias = tensors[self._conv + ".bias"].to(torch.float32).contiguous()

    def forward(self, x, batch, cache, shared_cache: bool = False, into=None):
        if shared_cache:
            raise ValueError("a short convolution's state cannot be read by another layer")
        w = self.in_proj.weight
        rows = x.shape[0]
        wide_enough = self.width >= tuning.FUSED_STEP_MIN_WIDTH or (
            self.width >= tuning.FUSED_STEP_NARROW_WIDTH
            and rows <= tuning.FUSED_STEP_NARROW_ROWS)
        if (batch.max_segment_rows == 1 and rows <= 64
                and x.dtype == torch.bfloat16
                and w.dtype == torch.bfloat16 and self.width % 16 == 0 and wide_enough):
            # decode: projection, convolution and state shift in one kernel
            with profile.scope("matmul_in_proj", self.in_proj.weight_bytes()):
                y = ops.linear_shortconv_step(x, w, self.in_proj.bias, self.taps, self.conv_bias,
                                              cache.state, batch.seg_pos0, batch.seg_slot,
                                              out_fragment=True)
            return self.out_proj.forward(y, partial_sums=True, add_into=into)
        # more than 16 rows (decode, short prompt portions): the projection may come as sums over
        # ranges of its input dimension (more blocks stream the matrix), which the conv kernel
        # adds up; with fewer rows the unsplit product and the plain step are as fast or faster
        proj = self.in_proj.forward(
            x, partial_sums=tuning.takes_partial_sums(x.shape[0], batch.max_segment_rows == 1))
        with profile.scope("short_conv"):
            y = ops.shortconv(proj, self.taps, self.conv_bias, cache.state, batch.row_seg,
                              batch.seg_start, batch.seg_pos0, batch.seg_slot)
        return self.out_proj.forward(y, partial_sums=True, add_into=into)

    def c_part(self, plan, view, shared_cache: bool = False):
        """The runner "mixer.conv" (csrc/engine_parts.hip) makes the same choices as ``forward``."""
        if shared_cache:
            return None
        first = plan.linear(self.in_proj)
        desc = ConvMixerDesc(first, plan.linear(self.out_proj), self.taps.data_ptr(),
                             tensor_ptr(self.conv_bias), self.L, view.state.data_ptr())
        return plan.part("mixer.conv", desc, takes_deferred_rows=True, adds_residual=True,
                         first=first)

    def weight_bytes(self) -> int:
        return self.in_proj.weight_bytes() + self.out_proj.weight_bytes() + self.width * self.L * 4


register_part("mixer", "conv", GatedShortConv)
