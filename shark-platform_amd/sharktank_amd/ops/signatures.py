"""Signatures of the `sharktank.ops` operators that the MoE layer path calls, with the reference's argument
lists (sharktank/sharktank/ops/signatures.py: einsum_2args :178-206, elementwise :209-228, get_index :317-336,
linear :615-655, matmul :659-688, rms_norm :761-776, softmax :974-993, to, view)."""

from __future__ import annotations

from typing import Optional

import torch
from torch import Tensor

from ..types.tensors import AnyTensor, InferenceTensor
from ._registry import SignatureDispatcher, overridable

__all__ = [
    "einsum_2args",
    "elementwise",
    "get_index",
    "linear",
    "matmul",
    "rms_norm",
    "softmax",
    "to",
    "view",
]


def _run(d: SignatureDispatcher, tensors, call):
    for override in d.find_overrides(tensors):
        result = call(override)
        if result is not NotImplemented:
            return override, result
    d.fail(tensors)


@overridable
def einsum_2args(input0: AnyTensor, input1: AnyTensor, einsum_str: str, *, accum_dtype: Optional[torch.dtype] = None) -> torch.Tensor:
    """y = torch.einsum(einsum_str, input0, input1)"""
    raise NotImplementedError


@einsum_2args.trampoline
def _einsum_trampoline(d, input0, input1, einsum_str: str):
    return _run(d, (input0, input1), lambda f: f(input0, input1, einsum_str))


@overridable
def elementwise(operator, *args, **kwargs) -> AnyTensor:
    """Applies an elementwise operator against arguments."""
    raise NotImplementedError


@elementwise.trampoline
def _elementwise_trampoline(d, operator, *args, **kwargs):
    tensors = []
    for a in args:
        if isinstance(a, (Tensor, InferenceTensor)):
            tensors.append(a)
        else:
            break
    return _run(d, tensors, lambda f: f(operator, *args, **kwargs))


@overridable
def get_index(tensor: AnyTensor, key) -> torch.Tensor:
    """out = tensor[key]"""
    raise NotImplementedError


@get_index.trampoline
def _get_index_trampoline(d, tensor, key):
    return _run(d, (tensor,), lambda f: f(tensor, key))


@overridable
def linear(input: AnyTensor, weight: AnyTensor, bias: Optional[AnyTensor] = None, *, accum_dtype: Optional[torch.dtype] = None) -> torch.Tensor:
    """y = torch.matmul(input, weight.T) + bias"""
    raise NotImplementedError


@linear.trampoline
def _linear_trampoline(d, input, weight, bias=None, *, accum_dtype=None):
    tensors = (input, weight) if bias is None else (input, weight, bias)
    return _run(d, tensors, lambda f: f(input, weight, bias, accum_dtype=accum_dtype))


@overridable
def matmul(lhs: AnyTensor, rhs: AnyTensor, *, transpose_rhs: bool = False):
    """lhs @ rhs, or lhs @ rhs^T when transpose_rhs (the storage order of inference weights)."""
    raise NotImplementedError


@matmul.trampoline
def _matmul_trampoline(d, lhs, rhs, *, transpose_rhs: bool = False):
    return _run(d, (lhs, rhs), lambda f: f(lhs, rhs, transpose_rhs=transpose_rhs))


@overridable
def rms_norm(x: AnyTensor, weight: AnyTensor, *, epsilon: float) -> AnyTensor:
    """Full, unbiased RMS normalisation of x along its last dim, times weight."""
    raise NotImplementedError


@rms_norm.trampoline
def _rms_norm_trampoline(d, x, weight, *, epsilon: float):
    return _run(d, (x, weight), lambda f: f(x, weight, epsilon=epsilon))


@overridable
def softmax(tensor: AnyTensor, dim: Optional[int] = None, dtype: Optional[torch.dtype] = None) -> AnyTensor:
    """See torch.nn.functional.softmax"""
    ...


@softmax.trampoline
def _softmax_trampoline(d, tensor, dim=None, dtype=None):
    return _run(d, [tensor], lambda f: f(tensor, dim=dim, dtype=dtype))


@overridable
def to(tensor: AnyTensor, *args, **kwargs) -> AnyTensor:
    """See torch.Tensor.to"""
    ...


@to.trampoline
def _to_trampoline(d, tensor, *args, **kwargs):
    return _run(d, (tensor,), lambda f: f(tensor, *args, **kwargs))


@overridable
def view(tensor: AnyTensor, shape) -> AnyTensor:
    """See torch.Tensor.view"""
    ...


@view.trampoline
def _view_trampoline(d, tensor, shape):
    return _run(d, (tensor,), lambda f: f(tensor, shape))
