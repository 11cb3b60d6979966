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
from ..ops import device_weight, expert_dispatch, gather_experts
from ..utils import debugging
from ..types import (DefaultPrimitiveTensor, DynamicScaledQuantizer, PlanarQuantizedTensor, QuantizedTensor,
                     StaticScaledQuantizer, Theta)
from .base import ThetaLayer
from .linear import LinearLayer

__all__ = ["FFNMOE", "PreGatherFFNMOE", "activation_enum", "extract_ffn_layer"]


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
            if q is not None and not isinstance(q, (StaticScaledQuantizer, DynamicScaledQuantizer)):
                raise NotImplementedError(f"PreGatherFFNMOE: activation quantizer {type(q).__name__} has no kernel")
        # Inside the fused call the intermediate goes from one projection to the next without the host seeing it, so its
        # quantizer must be known before the launch: static and per tensor.  A dynamic one (its scale is the maximum of the
        # whole intermediate) or a per-axis one over the features runs between the two projections as calls of their own
        # (see forward); the scale it computes stays on the device.
        qz = self.q_intermediate
        if isinstance(qz, StaticScaledQuantizer) and qz.axis is not None and qz.axis not in (-1, 2):
            raise NotImplementedError("PreGatherFFNMOE: a per-axis quantizer of the gated intermediate [tokens, slots, features] "
                                      "(ffn_down_exps.q_input) must scale along the features (axis -1)")
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

    def pre_matmul_gather(self, inputs, weights, experts, einstring="mk,menk->men", dispatch=None):
        """`einsum_2args(inputs, weights[experts, :, :], einstring)` as in the reference
        (sharktank/sharktank/layers/ffn_moe_block.py:37-41); the gather stays lazy and the product is grouped by expert.
        `dispatch` (not in the reference): the grouping of `experts`, if the caller has it already."""
        return ops.einsum_2args(inputs, gather_experts(weights, experts, dispatch), einstring)

    def forward_unfused(self, h: torch.Tensor, experts: torch.Tensor, expert_gate: torch.Tensor):
        """The reference's forward written with the same `ops` calls, one kernel per einsum (ffn_moe_block.py:60-74).
        `forward` computes the same values with fused kernels; this path exists for callers that compose the ops."""
        act = {_hip.ACT_SILU: F.silu, _hip.ACT_GELU_ERF: F.gelu}[self._act]
        if self.q_input is not None or self.q_intermediate is not None:
            raise NotImplementedError("forward_unfused: activation quantizers are handled by forward only")
        dispatch = expert_dispatch(experts, self.expert_count)  # one grouping for the three products of this forward
        ffn_gate = ops.elementwise(act, self.pre_matmul_gather(h, self.ffn_gate, experts, dispatch=dispatch))
        ffn_up = self.pre_matmul_gather(h, self.ffn_up, experts, dispatch=dispatch)
        ffn_down = self.pre_matmul_gather(ffn_gate * ffn_up, self.ffn_down, experts, einstring="mek,menk->men", dispatch=dispatch)
        ffn_down = ops.einsum_2args(expert_gate, ffn_down, "me,men->men")
        return torch.sum(ffn_down, dim=1)

    def activation_scales(self):
        """(reciprocal scale of the input quantizer, of the intermediate quantizer) as the fused kernels take them: one
        device float each; None where there is no quantizer or where the quantizer has to run as a pass of its own."""
        q, qz = self.q_input, self.q_intermediate
        xs = q.reciprocal_scale if isinstance(q, StaticScaledQuantizer) and q.axis is None else None
        zs = qz.reciprocal_scale if isinstance(qz, StaticScaledQuantizer) and qz.axis is None else None
        return xs, zs

    @property
    def fusable(self) -> bool:
        """Whether one fused call can run the whole FFN: every activation quantizer is static and per tensor (or absent)."""
        return all(q is None or (isinstance(q, StaticScaledQuantizer) and q.axis is None) for q in (self.q_input, self.q_intermediate))

    def quantized_input(self, h: torch.Tensor):
        """(h', x_scale): how the input quantizer reaches the kernels.  Static per tensor: the kernels quantise themselves
        (h, reciprocal scale).  Per axis or dynamic: h is quantised and dequantised here with the quantizer's own
        arithmetic (x * scale, not x / reciprocal scale), as LinearLayer does with a q_input
        (sharktank/sharktank/layers/linear.py:72-78), and the kernels see plain activations."""
        q = self.q_input
        if q is None:
            return h, None
        if isinstance(q, StaticScaledQuantizer) and q.axis is None:
            return h, q.reciprocal_scale
        return q.quantize(h).unpack().dequant(h.dtype), None

    @property
    def expert_count(self) -> int:
        return int(self.ffn_gate.shape[0])

    def bigger_mmg(self, inputs, weights, experts):
        """`einsum_2args(inputs, weights[experts, :, :], "mek,menk->men")` (ffn_moe_block.py:43-47): every (token, slot)
        pair's own input row [T, k, cols] times its expert's matrix; pre_matmul_gather with the per-pair einsum."""
        return ops.einsum_2args(inputs, gather_experts(weights, experts), "mek,menk->men")

    def one_hot_matmul(self, inputs, weights, experts):
        """The reference's experiment that multiplies by every expert and mixes the results with a one-hot matrix of a
        fixed 8 classes (ffn_moe_block.py:49-58): never called by its forward; it has no kernel here."""
        raise NotImplementedError("PreGatherFFNMOE.one_hot_matmul: unused by forward in the reference; not built")

    def grouped(self, h: torch.Tensor, experts: torch.Tensor):
        """The expert FFN of every (token, slot) pair, rows grouped by expert: (y [T*k, K] in dispatch order, inv [T*k] with
        the row of pair t*k + j).  `forward` weights and sums these rows; MoeBlock does the same together with its output
        norm and residual."""
        wg, wu, wd = self.device_weights()
        T, k = experts.shape
        if debugging.flags.enable_nan_checks:
            # The dispatch kernel clamps expert ids into range instead of faulting; the reference's weights[experts] would
            # raise IndexError.  With the checks switched on (TURBINE_LLM_DEBUG=enable_nan_checks) so does this (one host read).
            if bool(((experts < 0) | (experts >= wg.experts)).any()):
                raise IndexError(f"PreGatherFFNMOE: expert index outside 0..{wg.experts - 1}")
        _, offsets, perm, inv = _hip.dispatch_build(experts, wg.experts)
        xs, zs = self.activation_scales()
        h, xs = self.quantized_input(h)
        qz = self.q_intermediate
        if qz is None or zs is not None:
            y = _hip.grouped_ffn(h, wg, wu, wd, self._act, offsets, perm, k, variant=self.kernel_variant, x_scale=xs, z_scale=zs)
        else:
            # A dynamic or per-axis quantizer of the intermediate: gate/up projection, the quantizer's own quantise and
            # dequantise on the whole intermediate (as LinearLayer applies a q_input, linear.py:72-78; the rows' order does not
            # matter to a maximum over all of them nor to a scale per feature), down projection.
            z = _hip.grouped_gate_up(h, wg, wu, self._act, offsets, perm, k, x_scale=xs)
            if isinstance(qz, StaticScaledQuantizer):  # per axis, along the features: axis 1 of the [T*k, N] rows
                qz = StaticScaledQuantizer(name=qz.name, scale=qz.scale, reciprocal_scale=qz.reciprocal_scale, dtype=qz.dtype, axis=1)
            z = qz.quantize(z).unpack().dequant(z.dtype)
            y = _hip.grouped_down(z, wd, offsets, T, k)
        return y, inv

    def forward(self, h: torch.Tensor, experts: torch.Tensor, expert_gate: torch.Tensor):
        T, k = experts.shape
        y, inv = self.grouped(h, experts)
        return _hip.combine(y, expert_gate.to(h.dtype), inv, T, k)


def extract_ffn_layer(merged_tensor, layer_name: str, expert_idx: int):
    """One expert's matrix out of an expert-stacked weight, named as the reference names it
    (sharktank/sharktank/layers/ffn_moe_block.py:130-140: `blk.<block>.<layer_name>.<expert>.weight`).  The reference
    slices plain tensors only; planar quantized tensors are sliced plane by plane here (a view, no copy)."""
    parts = merged_tensor.name.split(".")
    block = parts[1] if len(parts) > 1 else "0"
    name = f"blk.{block}.{layer_name}.{expert_idx}.weight"
    if isinstance(merged_tensor, QuantizedTensor):
        planar = merged_tensor.to_planar()
        layout = planar.unpack()
        planes = {k: (v[expert_idx] if v.dim() > 0 and v.shape[0] == merged_tensor.shape[0] else v) for k, v in layout.planes.items()}
        shape = list(merged_tensor.shape[1:])
        return PlanarQuantizedTensor(name=name, shape=shape, layout=type(layout).create(shape, getattr(layout, "metadata", None), planes))
    return DefaultPrimitiveTensor(name=name, data=merged_tensor.as_torch()[expert_idx])


class FFNMOE(ThetaLayer):
    """One expert's feed-forward network, `ffn_down(silu(ffn_gate(h)) * ffn_up(h))`: the mirror of the reference's
    FFNMOE (sharktank/sharktank/layers/ffn_moe_block.py:77-127), built from expert-stacked weights
    (`ffn_{gate,up,down}_exps.weight[expert_idx]`) or from per-expert thetas (`ffn_gate.<expert_idx>` ...).  The three
    projections are LinearLayers, as in the reference; `forward` runs them as one fused gate/up kernel and one down
    kernel (the grouped kernels with a single expert), with every intermediate rounded where the reference's three
    linears and two element-wise ops round."""

    def __init__(self, theta: Theta, expert_idx=None):
        super().__init__(theta)
        if theta.optional_tensor("ffn_gate_exps") is not None or "ffn_gate_exps" in theta.keys:
            for layer_name in ("ffn_gate", "ffn_up", "ffn_down"):
                merged = theta.tensor(f"{layer_name}_exps", "weight")
                expert = extract_ffn_layer(merged_tensor=merged, layer_name=layer_name, expert_idx=expert_idx)
                self.add_module(layer_name, LinearLayer(Theta({"weight": expert})))
        else:
            self.add_module("ffn_gate", LinearLayer(theta("ffn_gate", expert_idx)))
            self.add_module("ffn_up", LinearLayer(theta("ffn_up", expert_idx)))
            self.add_module("ffn_down", LinearLayer(theta("ffn_down", expert_idx)))
        self._dw = None

    def forward(self, h: torch.Tensor):
        if self._dw is None:
            self._dw = tuple(device_weight(layer.weight, stacked=False, prepack=True)
                             for layer in (self.ffn_gate, self.ffn_up, self.ffn_down))
        wg, wu, wd = self._dw
        x = h.reshape(-1, h.shape[-1])
        y = _hip.grouped_ffn(x, wg, wu, wd, _hip.ACT_SILU, None, None, 1)  # one expert owns every row: no offsets array
        return y.reshape(*h.shape[:-1], y.shape[-1])
