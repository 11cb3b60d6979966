"""Raw ggml block tensors (mirror of sharktank/sharktank/types/gguf_interop/layouts.py:31-67, :260-307).

`Q8_0` holds 34-byte blocks {f16 d; i8 qs[32]}, `Q4_1` 20-byte blocks {f16 d; f16 m; u8 qs[16]} with ggml's
nibble order.  `unpack()` yields the planar layouts as views (Q8_0) or after the nibble re-order (Q4_1);
no arithmetic happens here.  For raw blocks that live on the GPU, `to_planar()` fills contiguous planes with one
kernel pass (`stmoe_gguf_ingest`), bit for bit what `unpack()` describes.
"""

from __future__ import annotations

import torch

from .layout_utils import linearize_interleaved_i4_block
from .layouts import BlockScaledI4Layout, BlockScaledLayout
from .tensors import PlanarQuantizedTensor, QuantizedTensor, UnnamedTensorName

__all__ = ["Q4_1", "Q8_0"]


def _device_planes(t, gguf_type: int):
    from .. import _hip

    lead = [int(s) for s in t.shape[:-2]]
    experts = 1
    for s in lead:
        experts *= s
    rows, cols = (int(t.shape[-2]), int(t.shape[-1])) if len(t.shape) >= 2 else (1, int(t.shape[-1]))
    dw = _hip.gguf_ingest(t.raw, gguf_type, experts, rows, cols, packed=False)
    qs, d, m = dw.keep
    plane_shape = list(t.shape[:-1]) + [cols // 32]
    return qs.reshape(plane_shape + [-1]), d.reshape(plane_shape + [1]), None if m is None else m.reshape(plane_shape + [1])


class Q8_0(QuantizedTensor):
    def __init__(self, *, raw: torch.Tensor, shape, name: str = UnnamedTensorName):
        super().__init__(name=name, shape=shape, layout_type=BlockScaledLayout)
        assert raw.dtype == torch.uint8
        self.raw = raw

    def unpack(self) -> BlockScaledLayout:
        blocks = self.raw.view(torch.int16).reshape(-1, 17).reshape(list(self.shape[:-1]) + [-1, 17])
        return BlockScaledLayout(self.shape, blocks[..., 0:1].view(torch.float16), blocks[..., 1:].view(torch.int8))

    def to_planar(self) -> PlanarQuantizedTensor:
        if not self.raw.is_cuda:
            return super().to_planar()
        qs, d, _ = _device_planes(self, 0)
        return PlanarQuantizedTensor(name=self.name, shape=self.shape, layout=BlockScaledLayout(self.shape, d, qs))

    @property
    def globals(self):
        return {self.name: self.raw}

    def _clone_with_globals(self, new_globals):
        return Q8_0(raw=new_globals[self.name], shape=self.shape, name=self.name)

    def __repr__(self):
        return f"Q8_0({self.name}, {self.shape})"


class Q4_1(QuantizedTensor):
    def __init__(self, *, raw: torch.Tensor, shape, name: str = UnnamedTensorName):
        super().__init__(name=name, shape=shape, layout_type=BlockScaledI4Layout)
        self.raw = raw

    def unpack(self) -> BlockScaledI4Layout:
        blocks = self.raw.view(torch.int16).reshape(-1, 10).reshape(list(self.shape[:-1]) + [-1, 10])
        d = blocks[..., 0:1].view(torch.float16)
        m = blocks[..., 1:2].view(torch.float16)
        qs = linearize_interleaved_i4_block(blocks[..., 2:].view(torch.int8))
        return BlockScaledI4Layout(self.shape, d, qs, m=m, signed=False)

    def to_planar(self) -> PlanarQuantizedTensor:
        if not self.raw.is_cuda:
            return super().to_planar()
        qs, d, m = _device_planes(self, 1)
        return PlanarQuantizedTensor(name=self.name, shape=self.shape, layout=BlockScaledI4Layout(self.shape, d, qs, m=m, signed=False))

    @property
    def globals(self):
        return {self.name: self.raw}

    def _clone_with_globals(self, new_globals):
        return Q4_1(raw=new_globals[self.name], shape=self.shape, name=self.name)

    def __repr__(self):
        return f"Q4_1({self.name}, {self.shape})"
