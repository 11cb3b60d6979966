"""Sub-byte layout helpers on device tensors (mirror of sharktank/sharktank/types/layout_utils.py).

Only what the MoE path touches is provided: i4 promotion (`promote_linear_i4_block_to_i8`, :67-86), the
ggml <-> linear nibble orders (:20-64, pure byte shuffles done with torch integer ops on the device that
holds the data) and `saturate_cast` (:150-176).
"""

from __future__ import annotations

import torch

__all__ = [
    "interleave_linear_i4_block",
    "linearize_interleaved_i4_block",
    "promote_linear_i4_block_to_i8",
]


def _view_uint8_tensor(data: torch.Tensor) -> torch.Tensor:
    if data.dtype == torch.uint8:
        return data
    if data.dtype == torch.int8:
        return data.view(torch.uint8)
    raise AssertionError(f"Expected tensor to by uint8 or int8. Got: {data.dtype}")


def linearize_interleaved_i4_block(i8_data: torch.Tensor) -> torch.Tensor:
    """ggml order (byte i = elements i and i+n) -> linear order (byte i = elements 2i and 2i+1)."""
    b = _view_uint8_tensor(i8_data)
    lo, hi = b & 0xF, b >> 4
    return torch.cat([(lo[..., 1::2] << 4) | lo[..., ::2], (hi[..., 1::2] << 4) | hi[..., ::2]], dim=-1)


def interleave_linear_i4_block(i8_data: torch.Tensor) -> torch.Tensor:
    b = _view_uint8_tensor(i8_data)
    t1, t2 = torch.tensor_split(b, 2, dim=-1)
    assert t1.size(-1) == t2.size(-1), "interleave_linear_i4_block: must have even inner-most dim"
    i0 = ((t2 & 0xF) << 4) | (t1 & 0xF)
    i1 = ((t2 >> 4) << 4) | (t1 >> 4)
    return torch.stack([i0, i1], dim=-1).flatten(start_dim=-2)


def promote_linear_i4_block_to_i8(linear_i4_data: torch.Tensor, *, signed: bool = False) -> torch.Tensor:
    from .. import _hip

    return _hip.promote_i4_block(linear_i4_data, signed)
