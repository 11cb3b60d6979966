"""Drop-in for sharktank's MoeBlock (sharktank/sharktank/layers/mixture_of_experts_block.py:23-90): same
constructor arguments, sub-module names and `forward(h [B,S,K]) -> [B,S,K]`.

forward = ffn_norm -> router (logits, fp32 softmax, top-k, renormalise) -> PreGatherFFNMOE ->
layer_output_norm -> residual, run as one C-ABI call that enqueues the HIP kernels back to back on the current
stream with one caller-owned workspace.
"""

from __future__ import annotations

from typing import Optional

import torch
import torch.nn.functional as F

from .. import _hip
from ..ops.hip_impls import _tensor_version
from ..types import Theta, unbox_tensor
from ..utils import debugging
from .base import ThetaLayer
from .ffn_moe_block import PreGatherFFNMOE
from .linear import LinearLayer
from .norm import RMSNormLayer

__all__ = ["MoeBlock"]


class MoeBlock(ThetaLayer):
    def __init__(self, theta: Theta, expert_count: int, expert_used_count: int, rms_epsilon: float, moe_activation=F.silu):
        super().__init__(theta)
        self.expert_count = expert_count
        self.expert_used_count = expert_used_count
        self.rms_epsilon = rms_epsilon

        self.add_module("ffn_gate_inp", LinearLayer(theta("ffn_gate_inp")))
        # The fused forward multiplies by the router matrix itself; what else a LinearLayer may carry would be dropped
        # silently, so it is refused here (the reference's router is a plain matrix: mixtral.py / grok.py theta trees).
        if self.ffn_gate_inp.bias is not None or self.ffn_gate_inp.q_input is not None:
            raise NotImplementedError("MoeBlock: ffn_gate_inp with a bias or an input quantizer has no fused kernel")
        self.add_module("ffn_norm", RMSNormLayer(theta("ffn_norm"), epsilon=rms_epsilon))
        if theta.optional_tensor("layer_output_norm") is not None:
            self.add_module("layer_output_norm", RMSNormLayer(theta("layer_output_norm"), epsilon=rms_epsilon))
        else:
            self.add_module("layer_output_norm", torch.nn.Identity())
        self.experts = PreGatherFFNMOE(theta, activation=moe_activation)

        self._router_w = {}  # activation dtype -> router matrix cast to it (the reference casts on every call)
        self._workspace: Optional[torch.Tensor] = None
        self.last_routing = None

    def _router_weight(self, dtype: torch.dtype) -> torch.Tensor:
        """The router matrix in the activation dtype.  The cast copy is keyed by the source tensor's storage, so a theta
        whose router tensor is replaced or resized gets a fresh copy (an in-place update of the same storage needs
        `reset_caches()`)."""
        src = unbox_tensor(self.ffn_gate_inp.weight)
        key = (dtype, src.data_ptr(), tuple(src.shape), src.dtype, _tensor_version(src))
        hit = self._router_w.get(dtype)
        if hit is None or hit[0] != key:
            hit = (key, src.to(dtype).contiguous())
            self._router_w[dtype] = hit
        return hit[1]

    def reset_caches(self):
        """Drops the cast router matrix, the packed expert weights and the workspace: call after changing theta tensors
        in place.  A HIP graph captured from an earlier forward replays into the old workspace and must be re-captured."""
        self._router_w.clear()
        self.experts._dw = None
        self._workspace = None

    def reserve_workspace(self, max_tokens: int, dtype: torch.dtype, device) -> None:
        """Allocates the workspace for forwards of up to `max_tokens` tokens ahead of time (for HIP graph capture)."""
        wg = self.experts.device_weights()[0]
        need = _hip.moe_forward_workspace_bytes(max_tokens, self.expert_used_count, self.expert_count, wg.cols, wg.rows, dtype)
        if self._workspace is None or self._workspace.numel() < need or self._workspace.device != torch.device(device):
            self._workspace = torch.empty(max(need, 1), dtype=torch.uint8, device=device)

    def forward(self, h: torch.Tensor, *, return_routing: bool = False):
        batch_size, sequence_length, feature_dim = h.shape
        x = h.reshape(-1, feature_dim)
        T = x.shape[0]
        wg, wu, wd = self.experts.device_weights()
        if wg.experts != self.expert_count:
            raise ValueError(f"expert_count {self.expert_count} != stacked weight experts {wg.experts}")
        out_norm = self.layer_output_norm
        out_norm_w = unbox_tensor(out_norm.weight) if isinstance(out_norm, RMSNormLayer) else None
        ffn_norm_w = unbox_tensor(self.ffn_norm.weight)
        if out_norm_w is not None and out_norm_w.dtype != ffn_norm_w.dtype:
            out_norm_w = out_norm_w.to(ffn_norm_w.dtype)  # the C ABI takes one dtype for both norm weights
        need = _hip.moe_forward_workspace_bytes(T, self.expert_used_count, self.expert_count, feature_dim, wg.rows, h.dtype)
        # The workspace grows to the largest forward seen and is then reused.  A HIP graph captured from a forward
        # replays into the workspace of that moment: capture after a warm-up call with the largest token count (or call
        # reserve_workspace first), so that no later, larger forward replaces the buffer under the graph.
        if self._workspace is None or self._workspace.numel() < need or self._workspace.device != h.device:
            self._workspace = torch.empty(max(need, 1), dtype=torch.uint8, device=h.device)
        if not self.experts.fusable:
            return self._forward_staged(h, x, ffn_norm_w, out_norm_w, return_routing)
        xs, zs = self.experts.activation_scales()
        # With tracing or golden dumps switched on, the routing is fetched as well and recorded beside the output (the
        # kernels and the results are the same either way).
        tracing = debugging.flags.enable_tensor_trace or debugging.flags.save_goldens_path is not None
        res = _hip.moe_forward(
            x, ffn_norm_w, out_norm_w, self.rms_epsilon, self._router_weight(h.dtype),
            wg, wu, wd, self.experts._act, self.expert_used_count,
            variant=self.experts.kernel_variant, workspace=self._workspace, want_routing=return_routing or tracing,
            x_scale=xs, z_scale=zs,
        )
        if return_routing or tracing:
            out, idx, gate = res
        else:
            out, idx, gate = res, None, None
        return self._finish(out, idx, gate, h.shape, return_routing)

    def _forward_staged(self, h, x, ffn_norm_w, out_norm_w, return_routing: bool):
        """The same forward as separate calls, for expert FFNs whose activation quantizers cannot ride inside the fused
        call (a dynamic or per-axis quantizer of the input or of the intermediate): norm, router, the experts' grouped FFN
        with its quantizer passes, then the weighted sum with the output norm and the residual."""
        T, k = x.shape[0], self.expert_used_count
        xn = _hip.rms_norm(x, ffn_norm_w, self.rms_epsilon)
        idx, gate, _ = _hip.router_topk(xn, self._router_weight(h.dtype), k)
        y, inv = self.experts.grouped(xn, idx)
        out = _hip.combine(y, gate, inv, T, k, out_norm_w=out_norm_w, eps=self.rms_epsilon, residual=x)
        return self._finish(out, idx, gate, h.shape, return_routing)

    def _finish(self, out, idx, gate, shape, return_routing: bool):
        batch_size, sequence_length, feature_dim = shape
        tracing = debugging.flags.enable_tensor_trace or debugging.flags.save_goldens_path is not None
        out = out.reshape(batch_size, sequence_length, feature_dim)
        if tracing:
            record = {"top_k_experts": idx, "expert_gate": gate, "output": out}
            self.trace_tensors("moe_block", record)
            self.trace_goldens("moe_block", record)
        self.assert_not_nan(out)
        if return_routing:
            return out, idx, gate
        return out
