"""The MoE side of the reference's model loops (sharktank/sharktank/models/mixtral/mixtral.py:86-233,
models/grok/grok.py:86-234): one MoeBlock per transformer block, built from the `blk.<n>.*` sub-trees of one Theta, run
block after block in `prefill` and `decode` with the reference's trace points around every block.

Attention, the KV cache, the embeddings and the output head are outside this path: where the reference's loop calls
`attn_block(h, ...)` between two MoE blocks, this loop calls `token_mixer(block_index, h)` if one is given (any callable
on the hidden states, standing in for whatever mixes tokens) and nothing otherwise.

A decode step is a handful of short launches per block, so its launch overhead matters: `capture_decode` records the
whole step (all blocks) once as a HIP graph and `decode` then replays it.
"""

from __future__ import annotations

from typing import Callable, Optional

import torch
import torch.nn as nn
import torch.nn.functional as F

from ..layers.base import ThetaLayer
from ..layers.mixture_of_experts_block import MoeBlock
from ..types import Theta

__all__ = ["MoeStack"]


class MoeStack(ThetaLayer):
    def __init__(self, theta: Theta, *, block_count: int, expert_count: int, expert_used_count: int, rms_epsilon: float,
                 moe_activation=F.silu, token_mixer: Optional[Callable[[int, torch.Tensor], torch.Tensor]] = None,
                 trace_prefix: str = "mixtral"):
        super().__init__(theta)
        self.block_count = block_count
        self.token_mixer = token_mixer
        self.trace_prefix = trace_prefix
        self.moe_blocks = nn.ModuleList()
        for n in range(block_count):
            self.moe_blocks.append(MoeBlock(theta("blk", n), expert_count=expert_count, expert_used_count=expert_used_count,
                                            rms_epsilon=rms_epsilon, moe_activation=moe_activation))
        self._graph = None  # (torch.cuda.CUDAGraph, static input, static output)

    # ---- the loop ----------------------------------------------------------------------------------------------
    def _run(self, h: torch.Tensor, trace: bool) -> torch.Tensor:
        for block_idx, moe_block in enumerate(self.moe_blocks):
            if self.token_mixer is not None:
                h = self.token_mixer(block_idx, h)
            if trace:
                self.trace_tensor(f"{self.trace_prefix}.attn_block.{block_idx}.output", h)
                self.trace_golden(f"{self.trace_prefix}.attn_block.{block_idx}.output", h)
            h = moe_block(h)
            if trace:
                self.trace_tensor(f"{self.trace_prefix}.moe_block.{block_idx}.output", h)
                self.trace_golden(f"{self.trace_prefix}.moe_block.{block_idx}.output", h)
        return h

    def prefill(self, h: torch.Tensor) -> torch.Tensor:
        """h [bs, seq_len, K]: the hidden states that enter block 0's MoE block.  Returns those that leave the last one."""
        return self._run(h, trace=True)

    def decode(self, h: torch.Tensor) -> torch.Tensor:
        """h [bs, 1, K].  Replays the captured graph when one was captured for this shape and dtype; runs eagerly otherwise."""
        g = self._graph
        if g is not None and tuple(g[1].shape) == tuple(h.shape) and g[1].dtype == h.dtype and g[1].device == h.device:
            g[1].copy_(h)
            g[0].replay()
            return g[2].clone()
        return self._run(h, trace=True)

    # ---- HIP graph of one decode step ---------------------------------------------------------------------------
    def capture_decode(self, bs: int, dtype: torch.dtype, device) -> None:
        """Records one decode step of `bs` sequences as a HIP graph.  The step runs eagerly first (twice, on the capture
        stream): that sizes every block's workspace, builds the packed weights and raises the LDS reservations of the
        kernels, none of which may happen under capture.  Tracing is off inside the graph (a dump would need the host).
        The graph replays into the buffers of this moment: `MoeBlock.reset_caches` or a larger forward through the same
        blocks invalidates it (capture again)."""
        K = self.moe_blocks[0].experts.ffn_gate.shape[2]
        static_in = torch.zeros(bs, 1, K, dtype=dtype, device=device)
        for blk in self.moe_blocks:
            blk.reserve_workspace(bs, dtype, device)
        stream = torch.cuda.Stream(device=device)
        stream.wait_stream(torch.cuda.current_stream(device))
        with torch.cuda.stream(stream):
            for _ in range(2):
                self._run(static_in, trace=False)
        torch.cuda.current_stream(device).wait_stream(stream)
        torch.cuda.synchronize(device)
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=stream):
            static_out = self._run(static_in, trace=False)
        self._graph = (graph, static_in, static_out)

    def release_decode_graph(self) -> None:
        self._graph = None
