"""Raw ggml block tensors (mirror of sharktank/sharktank/types/gguf_interop/layouts.py:31-67, :260-307).

`Q8_0` holds 34-byte blocks {f16 d; i8 qs[32]}, `Q4_1` 20-byte blocks {f16 d; f16 m; u8 qs[16]} with ggml's
nibble order.  `unpack()` yields the planar layouts as views (Q8_0) or after the nibble re-order (Q4_1);
no arithmetic happens here.
"""

from __future__ import annotations

import torch

from .layout_utils import linearize_interleaved_i4_block
from .layouts import BlockScaledI4Layout, BlockScaledLayout
from .tensors import QuantizedTensor, UnnamedTensorName

__all__ = ["Q4_1", "Q8_0"]


class Q8_0(QuantizedTensor):
    def __init__(self, *, raw: torch.Tensor, shape, name: str = UnnamedTensorName):
        super().__init__(name=name, shape=shape, layout_type=BlockScaledLayout)
        assert raw.dtype == torch.uint8
        self.raw = raw

    def unpack(self) -> BlockScaledLayout:
        blocks = self.raw.view(torch.int16).reshape(-1, 17).reshape(list(self.shape[:-1]) + [-1, 17])
        return BlockScaledLayout(self.shape, blocks[..., 0:1].view(torch.float16), blocks[..., 1:].view(torch.int8))

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

    @property
    def globals(self):
        return {self.name: self.raw}

    def _clone_with_globals(self, new_globals):
        return Q4_1(raw=new_globals[self.name], shape=self.shape, name=self.name)

    def __repr__(self):
        return f"Q4_1({self.name}, {self.shape})"
