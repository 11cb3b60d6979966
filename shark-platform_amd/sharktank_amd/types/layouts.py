"""The three weight layouts the MoE path consumes.

Same constructor arguments, property names and plane shapes as the reference
(sharktank/sharktank/types/layouts.py:42 TensorScaledLayout, :194
BlockScaledLayout, :302 BlockScaledI4Layout).  The classes only hold planes;
`dequant()` runs the HIP dequantization kernels on the device that owns the
planes and raises for host tensors: this package has no CPU arithmetic path.
"""

from __future__ import annotations

from typing import Dict, Optional

import torch

from .tensors import QuantizedLayout, register_quantized_layout

__all__ = [
    "BlockScaledI4Layout",
    "BlockScaledLayout",
    "TensorScaledLayout",
]


def _hip():
    from .. import _hip as hip

    return hip


@register_quantized_layout
class TensorScaledLayout(QuantizedLayout):
    """`d` (scalar or broadcastable scale), `qs` samples, optional offset `m`.

    dequant = ((qs.to(d.dtype) - m) * d).to(dtype); dtype defaults to d.dtype
    (sharktank/sharktank/types/layouts.py:163-181).
    """

    def __init__(self, *, shape, d, qs, m=None, dtype: Optional[torch.dtype] = None):
        self._shape = list(shape)
        self._d = d
        self._qs = qs
        self._m = m
        self._dtype = dtype if dtype is not None else d.dtype

    @classmethod
    def serialized_name(cls) -> str:
        return "TensorScaledLayout"

    @classmethod
    def create(cls, shape, metadata, planes):
        dtype = None
        if metadata and metadata.get("dtype") is not None:
            dtype = metadata["dtype"]
            if isinstance(dtype, str):
                dtype = getattr(torch, dtype)
        return cls(shape=shape, d=planes["d"], qs=planes["qs"], m=planes.get("m"), dtype=dtype)

    @property
    def metadata(self):
        return {"dtype": str(self._dtype).replace("torch.", "")}

    @property
    def planes(self) -> Dict[str, torch.Tensor]:
        p = {"d": self._d, "qs": self._qs}
        if self._m is not None:
            p["m"] = self._m
        return p

    @property
    def shape(self):
        return self._shape

    @property
    def dtype(self) -> torch.dtype:
        return self._dtype

    @property
    def d(self):
        return self._d

    @property
    def m(self):
        return self._m

    @property
    def qs(self):
        return self._qs

    def _like(self, qs):
        return TensorScaledLayout(shape=qs.shape, d=self.d, qs=qs, m=self.m, dtype=self.dtype)

    def view(self, *args, **kwargs):
        return self._like(self.qs.view(*args, **kwargs))

    def flatten(self, *args, **kwargs):
        return self._like(self.qs.flatten(*args, **kwargs))

    def transpose(self, *args, **kwargs):
        return self._like(self.qs.transpose(*args, **kwargs))

    def dequant(self, dtype: Optional[torch.dtype] = None) -> torch.Tensor:
        return self.dequant_blocked(dtype)

    def dequant_blocked(self, dtype: Optional[torch.dtype] = None) -> torch.Tensor:
        return _hip().dequant_tensor_scaled(
            self._qs, self._d, self._m, self._dtype if dtype is None else dtype
        )

    def __repr__(self):
        r = (
            f"{type(self).__name__}(d({list(self.d.shape)}, dtype={self.d.dtype}), "
            f"qs({list(self.qs.shape)}, dtype={self.qs.dtype}))"
        )
        if self.m is not None:
            r += f", m({list(self.m.shape)}, dtype={self.m.dtype})"
        return r + f" -> {self.dtype}"


@register_quantized_layout
class BlockScaledLayout(QuantizedLayout):
    """Per-block scale `d [.., K/B, 1]`, samples `qs [.., K/B, B]`, optional
    pre-scaled offset `m [.., K/B, 1]`; dequant = d*qs (+ m) in d's dtype
    (sharktank/sharktank/types/layouts.py:274-290).  Q8_0 is B=32, int8 qs,
    fp16 d, no m.
    """

    def __init__(self, shape, d, qs, *, m=None):
        self._shape = list(shape)
        self._d = d
        self._m = m
        self._qs = qs

    @classmethod
    def serialized_name(cls) -> str:
        return "BlockScaledLayout"

    @classmethod
    def create(cls, shape, metadata, planes):
        return cls(shape, planes["d"], planes["qs"], m=planes.get("m"))

    @property
    def planes(self) -> Dict[str, torch.Tensor]:
        p = {"d": self._d, "qs": self._qs}
        if self._m is not None:
            p["m"] = self._m
        return p

    @property
    def shape(self):
        return self._shape

    @property
    def d(self):
        return self._d

    @property
    def m(self):
        return self._m

    @property
    def qs(self):
        return self._qs

    def dequant(self, dtype: Optional[torch.dtype] = None) -> torch.Tensor:
        return self.dequant_blocked(dtype).reshape(self.shape)

    def dequant_blocked(self, dtype: Optional[torch.dtype] = None) -> torch.Tensor:
        if dtype is None:
            assert self._m is None or self._m.dtype == self._d.dtype
        return _hip().dequant_block_scaled(self._d, self._qs, self._m, dtype)

    def __repr__(self):
        r = (
            f"{type(self).__name__}(d({list(self.d.shape)}, dtype={self.d.dtype}), "
            f"qs({list(self.qs.shape)}, dtype={self.qs.dtype}))"
        )
        if self.m is not None:
            r += f", m({list(self.m.shape)}, dtype={self.m.dtype})"
        return r


@register_quantized_layout
class BlockScaledI4Layout(BlockScaledLayout):
    """BlockScaledLayout whose samples are packed two per byte, linear order:
    element 2i is the low nibble of byte i, element 2i+1 the high nibble
    (sharktank/sharktank/types/layouts.py:302-357,
    sharktank/sharktank/types/layout_utils.py:67-86).  Q4_1 is B=32 (16 bytes),
    unsigned, fp16 d and m.
    """

    def __init__(self, shape, d, qs, *, m=None, signed: bool = False):
        super().__init__(shape, d, qs, m=m)
        self.signed = signed

    @classmethod
    def serialized_name(cls) -> str:
        return "BlockScaledI4Layout"

    @classmethod
    def create(cls, shape, metadata, planes):
        return cls(shape, planes["d"], planes["qs"], m=planes.get("m"), signed=metadata["signed"])

    @property
    def metadata(self):
        return {"signed": self.signed}

    @property
    def qs(self) -> torch.Tensor:
        """Samples promoted to one (u)int8 per element."""
        return _hip().promote_i4_block(self._qs, self.signed)

    @property
    def qs_bit_packed(self) -> torch.Tensor:
        return self._qs

    def dequant_blocked(self, dtype: Optional[torch.dtype] = None) -> torch.Tensor:
        if dtype is None:
            assert self._m is None or self._m.dtype == self._d.dtype
        return _hip().dequant_block_scaled_i4(self._d, self._qs, self._m, self.signed, dtype)
