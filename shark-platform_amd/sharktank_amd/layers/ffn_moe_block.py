"""Drop-in for sharktank's PreGatherFFNMOE (sharktank/sharktank/layers/ffn_moe_block.py:23-74).

Same constructor, attributes and `forward(h, experts, expert_gate)` contract.  Instead of gathering a
[T,k,N,K] copy of the expert weights per token and running T batched M=1 products, the rows are grouped by
expert (stable counting sort of the (token, slot) pairs) and the three projections run as grouped kernels over
the stacked, still-quantized weights; the slot-weighted sum is the combine kernel.
"""

from __future__ import annotations

import torch
import torch.nn.functional as F

from .. import _hip
from .. import ops
from ..ops import device_weight, gather_experts
from ..types import StaticScaledQuantizer, Theta
from .base import ThetaLayer

__all__ = ["PreGatherFFNMOE", "activation_enum"]


def activation_enum(activation) -> int:
    """Maps the reference's activation callables to kernel enums: F.silu (default, ffn_moe_block.py:27) and
    F.gelu in its exact erf form (Grok, sharktank/sharktank/models/grok/grok.py:108)."""
    if activation is F.silu or isinstance(activation, torch.nn.SiLU):
        return _hip.ACT_SILU
    if activation is F.gelu or (isinstance(activation, torch.nn.GELU) and activation.approximate == "none"):
        return _hip.ACT_GELU_ERF
    raise NotImplementedError(f"PreGatherFFNMOE: no kernel epilogue for activation {activation!r} (have F.silu, F.gelu)")


class PreGatherFFNMOE(ThetaLayer):
    def __init__(self, theta: Theta, activation=F.silu):
        super().__init__(theta)
        self.ffn_gate = theta.tensor("ffn_gate_exps", "weight")
        self.ffn_up = theta.tensor("ffn_up_exps", "weight")
        self.ffn_down = theta.tensor("ffn_down_exps", "weight")
        # Optional static per-tensor fp8 quantizers of the activations, named as LinearLayer names its input quantizer
        # (sharktank/sharktank/layers/linear.py:57): `ffn_gate_exps.q_input` quantises h for the gate and up
        # projections, `ffn_down_exps.q_input` the gated intermediate for the down projection.  The values are the
        # reference's quantise-then-dequantise ones (linear.py:72-78).
        self.q_input = theta.optional_tensor("ffn_gate_exps", "q_input")
        self.q_intermediate = theta.optional_tensor("ffn_down_exps", "q_input")
        for q in (self.q_input, self.q_intermediate):
            if q is not None and not isinstance(q, StaticScaledQuantizer):
                raise NotImplementedError(f"PreGatherFFNMOE: activation quantizer {type(q).__name__} has no kernel")
        self.activation = activation
        self._act = activation_enum(activation)
        self._dw = None
        self.kernel_variant = _hip.VARIANT_AUTO
        # Re-order the quantized planes once into the kernels' streaming order (a second copy of the weights in
        # HBM; the planar tensors stay owned by `theta` and can be released by the caller).
        self.prepack_weights = True

    def device_weights(self):
        """C-ABI descriptors of the three stacked weights, built once (planes made contiguous once)."""
        if self._dw is None:
            self._dw = (
                device_weight(self.ffn_gate, stacked=True, prepack=self.prepack_weights),
                device_weight(self.ffn_up, stacked=True, prepack=self.prepack_weights),
                device_weight(self.ffn_down, stacked=True, prepack=self.prepack_weights),
            )
        return self._dw

    def pre_matmul_gather(self, inputs, weights, experts, einstring="mk,menk->men"):
        """`einsum_2args(inputs, weights[experts, :, :], einstring)` as in the reference
        (sharktank/sharktank/layers/ffn_moe_block.py:37-41); the gather stays lazy and the product is grouped by expert."""
        return ops.einsum_2args(inputs, gather_experts(weights, experts), einstring)

    def forward_unfused(self, h: torch.Tensor, experts: torch.Tensor, expert_gate: torch.Tensor):
        """The reference's forward written with the same `ops` calls, one kernel per einsum (ffn_moe_block.py:60-74).
        `forward` computes the same values with fused kernels; this path exists for callers that compose the ops."""
        act = {_hip.ACT_SILU: F.silu, _hip.ACT_GELU_ERF: F.gelu}[self._act]
        if self.q_input is not None or self.q_intermediate is not None:
            raise NotImplementedError("forward_unfused: activation quantizers are handled by forward only")
        ffn_gate = ops.elementwise(act, self.pre_matmul_gather(h, self.ffn_gate, experts))
        ffn_up = self.pre_matmul_gather(h, self.ffn_up, experts)
        ffn_down = self.pre_matmul_gather(ffn_gate * ffn_up, self.ffn_down, experts, einstring="mek,menk->men")
        ffn_down = ops.einsum_2args(expert_gate, ffn_down, "me,men->men")
        return torch.sum(ffn_down, dim=1)

    def activation_scales(self):
        """(reciprocal scale of the input quantizer, of the intermediate quantizer); None where there is none."""
        xs = self.q_input.reciprocal_scale if self.q_input is not None else None
        zs = self.q_intermediate.reciprocal_scale if self.q_intermediate is not None else None
        return xs, zs

    @property
    def expert_count(self) -> int:
        return int(self.ffn_gate.shape[0])

    def forward(self, h: torch.Tensor, experts: torch.Tensor, expert_gate: torch.Tensor):
        wg, wu, wd = self.device_weights()
        T, k = experts.shape
        _, offsets, perm, inv = _hip.dispatch_build(experts, wg.experts)
        xs, zs = self.activation_scales()
        y = _hip.grouped_ffn(h, wg, wu, wd, self._act, offsets, perm, k, variant=self.kernel_variant, x_scale=xs, z_scale=zs)
        return _hip.combine(y, expert_gate.to(h.dtype), inv, T, k)
