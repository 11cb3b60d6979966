"""Activation quantizers that produce `TensorScaledLayout` tensors (mirror of
sharktank/sharktank/types/quantizers.py:87-183 StaticScaledQuantizer, per-tensor fp8 case, which is the one the
fp8 MoE configuration uses).  The cast runs in a HIP kernel."""

from __future__ import annotations

from typing import Optional

import torch

from .layouts import TensorScaledLayout
from .tensors import InferenceTensor, PlanarQuantizedTensor, QuantizedTensor, UnnamedTensorName, unbox_tensor

__all__ = ["DynamicScaledQuantizer", "QuantizerTensor", "StaticScaledQuantizer"]


class QuantizerTensor(InferenceTensor):
    def quantize(self, t, *, name: str = UnnamedTensorName) -> QuantizedTensor:
        return self._quantize_raw_tensor(unbox_tensor(t), name=name)

    def _quantize_raw_tensor(self, t: torch.Tensor, *, name: str) -> QuantizedTensor:
        raise NotImplementedError


class StaticScaledQuantizer(QuantizerTensor):
    """Mirror of sharktank/sharktank/types/quantizers.py:83-260 for float8_e4m3fn without offsets: per tensor (0-d scale:
    `saturate_cast(t / reciprocal_scale)`) or per axis (1-d scale: `saturate_cast(t * scale)` with the scale broadcast
    along `axis`), both producing a TensorScaledLayout whose `d` is the reciprocal scale."""

    def __init__(self, *, scale: torch.Tensor, dtype: torch.dtype, axis: Optional[int] = None,
                 reciprocal_scale: Optional[torch.Tensor] = None, offset: Optional[torch.Tensor] = None,
                 disable_saturate: bool = False, name: str = UnnamedTensorName):
        super().__init__(shape=scale.shape, name=name)
        if offset is not None or disable_saturate:
            raise NotImplementedError("StaticScaledQuantizer: only the offset-free, saturating forms have kernels")
        if dtype != torch.float8_e4m3fn:
            raise NotImplementedError(f"StaticScaledQuantizer: target dtype {dtype} has no kernel (gfx950 MFMA consumes float8_e4m3fn)")
        if axis is None:
            assert len(scale.shape) == 0, "Expected per-tensor scale to be 0D"
        else:
            assert len(scale.shape) == 1, "Expected per-axis scale to be 1D"
        self._axis = axis
        self._scale = scale
        self._reciprocal_scale = reciprocal_scale if reciprocal_scale is not None else 1.0 / scale
        self._dtype = dtype

    @property
    def axis(self):
        return self._axis

    @property
    def offset(self):
        return None

    @property
    def scale(self):
        return self._scale

    @property
    def reciprocal_scale(self):
        return self._reciprocal_scale

    @property
    def dtype(self):
        return self._dtype

    @property
    def globals(self):
        return {f"{self.name}:d": self._scale, f"{self.name}:rscale": self._reciprocal_scale}

    def _clone_with_globals(self, new_globals):
        return StaticScaledQuantizer(name=self.name, scale=new_globals[f"{self.name}:d"], axis=self._axis,
                                     reciprocal_scale=new_globals[f"{self.name}:rscale"], dtype=self._dtype)

    def _quantize_raw_tensor(self, t: torch.Tensor, *, name: str) -> QuantizedTensor:
        from .. import _hip

        shape = list(t.shape)
        if self._axis is None:
            qs = _hip.quantize_fp8(t, self._reciprocal_scale)
            d = self._reciprocal_scale
        else:
            axis = self._axis
            assert 0 <= axis < len(shape), f"Per-axis scale {axis} out of bounds of shape {shape}"
            qs = _hip.quantize_fp8_per_axis(t, self._scale, axis)
            scale_shape = [1] * len(shape)
            scale_shape[axis] = self._scale.shape[0]
            d = self._reciprocal_scale.reshape(scale_shape)
        return PlanarQuantizedTensor(
            shape=shape, name=name,
            layout=TensorScaledLayout(shape=shape, d=d, qs=qs, m=None, dtype=t.dtype),
        )


class DynamicScaledQuantizer(QuantizerTensor):
    """Per-tensor quantizer whose scale comes from the tensor itself: `scale = finfo.max / amax.clamp(finfo.eps)`
    (mirror of sharktank/sharktank/types/quantizers.py:338-389 for float8_e4m3fn, the fp8 format gfx950's matrix cores
    consume).  Produces a `TensorScaledLayout` with `d = 1 / scale` and `dtype` = the source dtype, like the reference."""

    def __init__(self, *, dtype: torch.dtype, name: str = UnnamedTensorName):
        super().__init__(name=name, shape=())
        if dtype != torch.float8_e4m3fn:
            raise NotImplementedError(f"DynamicScaledQuantizer: target dtype {dtype} has no kernel (have float8_e4m3fn)")
        self._dtype = dtype

    @property
    def dtype(self) -> torch.dtype:
        return self._dtype

    @property
    def globals(self):
        return {}

    def _clone_with_globals(self, new_globals):
        return DynamicScaledQuantizer(dtype=self._dtype, name=self.name)

    def _quantize_raw_tensor(self, t: torch.Tensor, *, name: str) -> QuantizedTensor:
        from .. import _hip

        qs, _, rscale = _hip.dynamic_quantize_fp8(t)
        shape = list(t.shape)
        return PlanarQuantizedTensor(
            shape=shape, name=name,
            layout=TensorScaledLayout(shape=shape, d=rscale, qs=qs, m=None, dtype=t.dtype),
        )
