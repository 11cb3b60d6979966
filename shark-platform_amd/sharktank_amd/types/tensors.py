"""Tensor wrappers that the MoE path receives from its callers.

Mirrors the part of the reference type hierarchy that reaches `MoeBlock`
(sharktank/sharktank/types/tensors.py:189 InferenceTensor, :480 PrimitiveTensor,
:508 DefaultPrimitiveTensor, :585 QuantizedTensor, :622 PlanarQuantizedTensor,
:1276 unbox_tensor).  Serialization (IRPA archives), sharded tensors and the
export hooks are not part of the hot path and are not provided.
"""

from __future__ import annotations

from abc import ABC, abstractmethod
from typing import Any, Dict, Optional, Type, Union

import torch

__all__ = [
    "AnyTensor",
    "DefaultPrimitiveTensor",
    "GatheredExpertsTensor",
    "InferenceTensor",
    "PlanarQuantizedTensor",
    "PrimitiveTensor",
    "QuantizedLayout",
    "QuantizedTensor",
    "REGISTERED_LAYOUT_CLASSES",
    "UnnamedTensorName",
    "register_quantized_layout",
    "unbox_tensor",
]

UnnamedTensorName = "<unnamed>"

REGISTERED_LAYOUT_CLASSES: Dict[str, Type["QuantizedLayout"]] = {}


class QuantizedLayout(ABC):
    """A physical arrangement of planes that dequantizes to a logical tensor."""

    @abstractmethod
    def dequant(self, dtype: Optional[torch.dtype] = None) -> torch.Tensor:
        ...

    @classmethod
    @abstractmethod
    def serialized_name(cls) -> str:
        ...

    @property
    @abstractmethod
    def planes(self) -> Dict[str, torch.Tensor]:
        ...

    @property
    def metadata(self) -> Optional[dict]:
        return None


def register_quantized_layout(ty):
    REGISTERED_LAYOUT_CLASSES[ty.serialized_name()] = ty
    return ty


class InferenceTensor(ABC):
    """A named, shaped tensor-like value owned by a parameter tree."""

    def __init__(self, *, shape, name: str = UnnamedTensorName):
        self._name = name
        self.shape = list(shape)

    @property
    def name(self) -> str:
        return self._name

    @name.setter
    def name(self, value: str):
        self._name = value

    @property
    @abstractmethod
    def globals(self) -> Dict[str, torch.Tensor]:
        """The torch tensors backing this value, keyed by global name."""

    @abstractmethod
    def _clone_with_globals(self, new_globals: Dict[str, torch.Tensor]):
        ...

    def transform_globals(self, *transforms):
        prev = self.globals
        for fn in transforms:
            nxt = fn(prev)
            if nxt is not None:
                prev = nxt
        return self._clone_with_globals(prev)

    def to(self, *, device=None) -> "InferenceTensor":
        return self.transform_globals(
            lambda d: {k: t.to(device=device) for k, t in d.items()}
        )

    def size(self, dim: Optional[int] = None):
        return tuple(self.shape) if dim is None else self.shape[dim]

    def __getitem__(self, key):
        from ..ops import get_index

        return get_index(self, key)


class PrimitiveTensor(InferenceTensor):
    """An InferenceTensor isomorphic to one torch.Tensor."""

    @abstractmethod
    def as_torch(self, *, dtype: Optional[torch.dtype] = None) -> torch.Tensor:
        ...

    @property
    def dtype(self) -> torch.dtype:
        return self.as_torch().dtype


class DefaultPrimitiveTensor(PrimitiveTensor):
    """Plain row-major torch.Tensor under a name."""

    def __init__(self, *, data: torch.Tensor, name: str = UnnamedTensorName):
        super().__init__(name=name, shape=list(data.shape))
        self._data = data

    def as_torch(self, *, dtype: Optional[torch.dtype] = None) -> torch.Tensor:
        if dtype is not None:
            return self._data.to(dtype)
        return self._data

    @property
    def globals(self) -> Dict[str, torch.Tensor]:
        return {self.name: self._data}

    def _clone_with_globals(self, new_globals):
        return DefaultPrimitiveTensor(name=self.name, data=new_globals[self.name])

    def __getitem__(self, key):
        if not isinstance(key, (list, tuple)):
            key = (key,)
        key = tuple(unbox_tensor(k) if isinstance(k, PrimitiveTensor) else k for k in key)
        return self._data[key]

    def __repr__(self):
        return f"PrimitiveTensor({self.name}, {self.shape}, {self._data.dtype})"


class QuantizedTensor(InferenceTensor):
    """An InferenceTensor whose storage is packed; `unpack()` gives its layout."""

    def __init__(self, *, shape, layout_type: Type[QuantizedLayout], name=UnnamedTensorName):
        super().__init__(name=name, shape=shape)
        self.layout_type = layout_type

    @abstractmethod
    def unpack(self) -> QuantizedLayout:
        ...

    def to_planar(self) -> "PlanarQuantizedTensor":
        return PlanarQuantizedTensor(name=self.name, shape=self.shape, layout=self.unpack())


class PlanarQuantizedTensor(QuantizedTensor):
    """Quantized tensor whose planes are already materialised (no unpacking)."""

    def __init__(self, *, shape, layout: QuantizedLayout, name=UnnamedTensorName):
        super().__init__(name=name, shape=shape, layout_type=type(layout))
        self.layout = layout

    def to_planar(self):
        return self

    def unpack(self) -> QuantizedLayout:
        return self.layout

    @property
    def globals(self) -> Dict[str, torch.Tensor]:
        return {f"{self.name}:{k}": v for k, v in self.layout.planes.items()}

    def _clone_with_globals(self, new_globals):
        prefix = f"{self.name}:"
        planes = {k: new_globals[prefix + k] for k in self.layout.planes.keys()}
        cls = REGISTERED_LAYOUT_CLASSES[self.layout.serialized_name()]
        layout = cls.create(self.shape, self.layout.metadata, planes)
        return PlanarQuantizedTensor(name=self.name, shape=self.shape, layout=layout)

    def __repr__(self):
        return f"PlanarQuantized({self.name}, {self.shape}, layout={self.layout})"


class GatheredExpertsTensor(InferenceTensor):
    """`weights[experts, :, :]` of an expert-stacked weight, kept lazy.

    The reference materialises this gather as a [T, k, rows, cols] copy of expert weights per token
    (sharktank/sharktank/layers/ffn_moe_block.py:39, ops/default_impls.py:204-218) and then runs T batched M=1
    products.  Here the indexing result only records the stacked weight and the index tensor; `einsum_2args` on it
    groups the (token, slot) pairs by expert and multiplies each group with its expert's matrix once.
    """

    def __init__(self, *, weights: InferenceTensor, experts: torch.Tensor, name: str = UnnamedTensorName):
        T, k = experts.shape
        super().__init__(name=name, shape=[T, k] + list(weights.shape[1:]))
        self.weights = weights
        self.experts = experts
        self._dispatch = None  # (offsets, perm) of `experts`, built on first use
        self._device_weight = None

    @property
    def globals(self) -> Dict[str, torch.Tensor]:
        g = dict(self.weights.globals)
        g[f"{self.name}:experts"] = self.experts
        return g

    def _clone_with_globals(self, new_globals):
        experts = new_globals[f"{self.name}:experts"]
        weights = self.weights._clone_with_globals({k: v for k, v in new_globals.items() if k in self.weights.globals})
        return GatheredExpertsTensor(weights=weights, experts=experts, name=self.name)

    def __repr__(self):
        return f"GatheredExperts({self.weights!r}[{list(self.experts.shape)}])"


AnyTensor = Union[torch.Tensor, InferenceTensor]


def unbox_tensor(t: Any) -> torch.Tensor:
    """torch.Tensor view of `t`; a QuantizedTensor is dequantized in full."""
    if isinstance(t, torch.Tensor):
        return t
    if isinstance(t, PrimitiveTensor):
        return t.as_torch()
    if isinstance(t, QuantizedTensor):
        return t.unpack().dequant()
    raise TypeError(f"cannot unbox {type(t)}")
