"""Drop-in for sharktank's FFN (sharktank/sharktank/layers/ffn_block.py:21-51): the dense feed-forward network of a
transformer block, `ffn_down(act(ffn_gate(h)) * ffn_up(h))` (gated) or `ffn_down(act(ffn_up(h)))` (un-gated), with
quantized or dense weights.

The gated form with plain weights runs as the MoE kernels with a single expert: one fused gate/up launch (activation
and product in its epilogue) and one down launch, every intermediate rounded where the reference's three linears and
two element-wise ops round.  Everything else (a bias, an input quantizer, the un-gated form, an activation without a
kernel epilogue) composes LinearLayers and `ops.elementwise` exactly as the reference does; those still run on the
packed matrix kernels through `ops.linear`.
"""

from __future__ import annotations

from typing import Callable

import torch
import torch.nn.functional as F

from .. import _hip, ops
from ..ops.hip_impls import cached_device_weight
from .base import Theta, ThetaLayer
from .ffn_moe_block import activation_enum
from .linear import LinearLayer

__all__ = ["FFN"]


class FFN(ThetaLayer):
    def __init__(self, theta: Theta, is_gated: bool = True, activation_fn: Callable = F.silu):
        super().__init__(theta)
        self.is_gated = is_gated
        self.activation_fn = activation_fn
        if self.is_gated:
            self.add_module("ffn_gate", LinearLayer(theta("ffn_gate")))
        self.add_module("ffn_up", LinearLayer(theta("ffn_up")))
        self.add_module("ffn_down", LinearLayer(theta("ffn_down")))
        try:
            self._act = activation_enum(activation_fn)
        except NotImplementedError:
            self._act = None

    def _fusable(self, h: torch.Tensor) -> bool:
        if not self.is_gated or self._act is None or h.dtype not in (torch.float16, torch.bfloat16, torch.float32):
            return False
        layers = (self.ffn_gate, self.ffn_up, self.ffn_down)
        return all(l.bias is None and l.q_input is None and not l.fake_quant for l in layers)

    def forward(self, h: torch.Tensor) -> torch.Tensor:
        if self._fusable(h):
            wg, wu, wd = (cached_device_weight(l.weight, stacked=False, cast_to=h.dtype)
                          for l in (self.ffn_gate, self.ffn_up, self.ffn_down))
            x = h.reshape(-1, h.shape[-1])
            T = x.shape[0]
            if T == 0:
                return h.new_empty(*h.shape[:-1], wd.rows)
            y = _hip.grouped_ffn(x, wg, wu, wd, self._act, None, None, 1)  # one expert owns every row: no offsets array
            return y.reshape(*h.shape[:-1], y.shape[-1])
        if self.is_gated:
            ffn_gate = ops.elementwise(self.activation_fn, self.ffn_gate(h))
            ffn_up = self.ffn_up(h)
            return self.ffn_down(ffn_gate * ffn_up)
        h = self.ffn_up(h)
        h = ops.elementwise(self.activation_fn, h)
        return self.ffn_down(h)
