"""GPU implementations of the `sharktank.ops` operators on the MoE path, registered through the same
`@op.override(...)` protocol the reference uses for its own kernels
(sharktank/sharktank/ops/custom_impls.py:54-103, default_impls.py:108-128,204-218,328-359,402-408).
Arithmetic runs in the HIP library; torch is used for allocation, views and dtype/device moves.
Anything not implemented returns `NotImplemented`, which surfaces as the reference's NotImplementedError.
"""

from __future__ import annotations

import torch
from torch import Tensor

from .. import _hip
from ..types.gguf_interop import Q4_1, Q8_0
from ..types.layouts import BlockScaledI4Layout, BlockScaledLayout, TensorScaledLayout
from ..types.tensors import GatheredExpertsTensor, InferenceTensor, PrimitiveTensor, QuantizedTensor, unbox_tensor
from ._registry import AllOfType
from .signatures import *

__all__ = ["device_weight", "expert_dispatch", "gather_experts"]

_FLOAT_DTYPES = (torch.float32, torch.float16, torch.bfloat16)


def device_weight(w, *, stacked: bool, prepack: bool = False) -> _hip.DeviceWeight:
    """C-ABI descriptor of a weight tensor.  `stacked`: [E, rows, cols]; otherwise a single [rows, cols] matrix.
    Planes are made contiguous once here (GGUF-derived planes are strided views of the raw blocks).  With
    `prepack`, quantized planes whose shape allows it are re-ordered once into the kernels' streaming order."""
    if isinstance(w, (Q8_0, Q4_1)) and w.raw.is_cuda:
        # raw ggml blocks go to planes (planar or streaming order) in one kernel pass
        shape = list(w.shape)
        experts, rows, cols = shape if stacked else [1] + shape
        packed = prepack and rows % 16 == 0 and cols % 256 == 0
        return _hip.gguf_ingest(w.raw, _hip.GGUF_Q8_0 if isinstance(w, Q8_0) else _hip.GGUF_Q4_1, experts, rows, cols, packed=packed)
    dw = _device_weight_planar(w, stacked=stacked)
    if prepack and dw.can_prepack():
        dw = dw.prepack()
    return dw


def _tensor_version(t: torch.Tensor) -> int:
    """The tensor's in-place modification counter.  Tensors created under torch.inference_mode() do not track one (reading
    it raises); they cannot be modified in place outside inference mode either, so they count as unchanged."""
    try:
        return t._version
    except RuntimeError:
        return -1


def _planes_key(w):
    """What a cached descriptor of `w` depends on: the identity, shape and version of every plane.  (The version counts
    in-place changes made through torch; a plane rewritten through a raw pointer needs a fresh tensor object.)"""
    if isinstance(w, torch.Tensor):
        ts = (w,)
    elif isinstance(w, (Q8_0, Q4_1)):
        ts = (w.raw,)
    else:
        ts = tuple(w.globals.values())
    return tuple((t.data_ptr(), tuple(t.shape), t.dtype, _tensor_version(t)) for t in ts)


_TENSOR_CACHE = {}  # id(torch.Tensor) -> (weakref to it, {(stacked, prepack, dtype): (planes key, descriptor)})


def cached_device_weight(w, *, stacked: bool, prepack: bool = True, cast_to: torch.dtype = None) -> _hip.DeviceWeight:
    """device_weight(w) built once per weight and kept with it: the planes are made contiguous and (where the shape allows)
    re-ordered into the kernels' streaming order on the first call; later calls with unchanged planes reuse the result.
    InferenceTensors carry their descriptors themselves; plain torch tensors are tracked through weak references.  `cast_to`
    (dense weights only) is the dtype the kernels need, cast once as well."""
    if isinstance(w, torch.Tensor):
        ent = _TENSOR_CACHE.get(id(w))
        if ent is None or ent[0]() is not w:
            import weakref

            wid = id(w)
            ent = (weakref.ref(w, lambda _, wid=wid: _TENSOR_CACHE.pop(wid, None)), {})
            _TENSOR_CACHE[wid] = ent
        store = ent[1]
    else:
        store = w.__dict__.setdefault("_stmoe_descriptors", {})
    slot, key = (stacked, prepack, cast_to), _planes_key(w)
    hit = store.get(slot)
    if hit is None or hit[0] != key:
        src = w
        if cast_to is not None and not isinstance(w, QuantizedTensor):
            src = unbox_tensor(w).to(cast_to)
        hit = (key, device_weight(src, stacked=stacked, prepack=prepack))
        store[slot] = hit
    return hit[1]


def _device_weight_planar(w, *, stacked: bool) -> _hip.DeviceWeight:
    shape = list(w.shape)
    if stacked:
        assert len(shape) == 3, f"expert-stacked weight must be [E, rows, cols], got {shape}"
        experts, rows, cols = shape
    else:
        assert len(shape) == 2, f"weight must be [rows, cols], got {shape}"
        experts, (rows, cols) = 1, shape
    if isinstance(w, QuantizedTensor):
        layout = w.unpack()
        if type(layout) is BlockScaledLayout:
            assert layout.m is None, "NYI: Q8 block scaled with offset"
            if layout.qs.shape[-1] != 32 or layout.d.dtype != torch.float16:
                raise NotImplementedError("BlockScaledLayout kernels exist for block 32 with fp16 scales (Q8_0) only")
            return _hip.DeviceWeight(_hip.W_Q8_0, experts, rows, cols, layout.qs.contiguous(), layout.d.contiguous())
        if type(layout) is BlockScaledI4Layout:
            assert layout.m is not None, "NYI: Q4 without offset not"
            assert not layout.signed, "NYI: Q4 signed"
            if layout.qs_bit_packed.shape[-1] != 16 or layout.d.dtype != torch.float16:
                raise NotImplementedError("BlockScaledI4Layout kernels exist for block 32 with fp16 d/m (Q4_1) only")
            return _hip.DeviceWeight(_hip.W_Q4_1, experts, rows, cols, layout.qs_bit_packed.contiguous(),
                                     layout.d.contiguous(), layout.m.contiguous())
        if type(layout) is TensorScaledLayout:
            if layout.m is not None or layout.qs.dtype != torch.float8_e4m3fn:
                raise NotImplementedError("TensorScaledLayout kernels exist for offset-free float8_e4m3fn samples only")
            d = layout.d.contiguous().reshape(-1)
            if d.numel() not in (1, experts) or d.dtype not in (torch.float32, torch.float16):
                raise NotImplementedError("TensorScaledLayout kernels take one f32/f16 scale per tensor or per expert")
            if layout.dtype != d.dtype:
                raise NotImplementedError("TensorScaledLayout kernels produce the scale's dtype before the activation cast")
            return _hip.DeviceWeight(_hip.W_FP8, experts, rows, cols, layout.qs.contiguous(), d, None, _hip.dtype_enum(d.dtype))
        raise NotImplementedError(f"no kernel for layout {type(layout).__name__}")
    t = unbox_tensor(w).contiguous()
    if t.dtype not in _FLOAT_DTYPES:
        raise NotImplementedError(f"no kernel for dense weights of dtype {t.dtype}")
    return _hip.DeviceWeight(_hip.W_DENSE, experts, rows, cols, t, None, None, _hip.dtype_enum(t.dtype))


# ---- plumbing ops ---------------------------------------------------------------------------------------


@to.override(Tensor)
def to_default(tensor, *args, **kwargs):
    return unbox_tensor(tensor).to(*args, **kwargs)


@view.override(Tensor)
def view_default(tensor, shape):
    return unbox_tensor(tensor).view(*shape)


@elementwise.override(Tensor)
def elementwise_unary(operator, x, *args, **kwargs):
    return operator(unbox_tensor(x), *args, **kwargs)


@elementwise.override(Tensor, Tensor)
def elementwise_binary(operator, x, y, *args, **kwargs):
    return operator(unbox_tensor(x), unbox_tensor(y), *args, **kwargs)


# ---- arithmetic ops -------------------------------------------------------------------------------------


@rms_norm.override(AllOfType(Tensor, InferenceTensor))
def rms_norm_hip(x, weight, *, epsilon: float):
    x = unbox_tensor(x)
    weight = unbox_tensor(weight)
    if x.dtype not in _FLOAT_DTYPES:
        return NotImplemented
    # the reference multiplies by the weight in the weight's dtype and returns that dtype
    # (sharktank/sharktank/ops/default_impls.py:402-408); RMSNormLayer casts x to fp32 before and back after.
    if x.dtype == torch.float32 and weight.dtype == torch.float32:
        return _hip.rms_norm(x, weight, epsilon)
    return NotImplemented


def _mmt_2d(lhs: torch.Tensor, dw: _hip.DeviceWeight):
    return _hip.mmt(lhs, dw)


@matmul.override(Tensor, QuantizedTensor)
def matmul_tensor_quantized(lhs, rhs: QuantizedTensor, *, transpose_rhs: bool):
    lhs = unbox_tensor(lhs)
    if not transpose_rhs or len(rhs.shape) != 2 or lhs.dtype not in _FLOAT_DTYPES:
        return NotImplemented
    # the descriptor (contiguous planes, streaming order) is built on the first product and kept with the weight
    return _mmt_2d(lhs, cached_device_weight(rhs, stacked=False))


@matmul.override(Tensor, Tensor)
def matmul_tensor_tensor(lhs, rhs, *, transpose_rhs: bool):
    lhs = unbox_tensor(lhs)
    holder = rhs  # the object the cast copy is kept with: the PrimitiveTensor, or the torch tensor itself
    rhs = unbox_tensor(rhs)
    if not transpose_rhs or rhs.dim() != 2 or lhs.dtype not in _FLOAT_DTYPES:
        return NotImplemented
    return _mmt_2d(lhs, cached_device_weight(holder, stacked=False, cast_to=lhs.dtype))


def _linear(input, weight, bias, *, accum_dtype=None):
    """matmul(input, weight^T) (+ bias), as linear_default composes it (sharktank/sharktank/ops/default_impls.py:328-341):
    the product is rounded to the input's dtype, the bias is added in the two tensors' promoted dtype."""
    input = unbox_tensor(input)
    result = matmul(input, weight, transpose_rhs=True)  # a dense weight is cast to the input's dtype once and kept
    if bias is not None:
        bias = unbox_tensor(bias)
        if bias.dim() != 1 or bias.dtype not in _FLOAT_DTYPES:
            return NotImplemented
        result = _hip.add_bias(result, bias)
    return result


linear.override(Tensor, Tensor)(_linear)
linear.override(Tensor, QuantizedTensor)(_linear)
linear.override(Tensor, Tensor, Tensor)(_linear)
linear.override(Tensor, QuantizedTensor, Tensor)(_linear)


@softmax.override(Tensor)
def softmax_hip(tensor, dim=None, dtype=None):
    """F.softmax (sharktank/sharktank/ops/default_impls.py:426-432) in fp32 on the device."""
    x = unbox_tensor(tensor)
    if x.dtype not in _FLOAT_DTYPES or (dtype is not None and dtype not in _FLOAT_DTYPES) or x.dim() == 0:
        return NotImplemented
    if dim is None:  # torch's legacy default: axis 0 for 0-, 1- and 3-dimensional inputs, else 1
        dim = 0 if x.dim() in (0, 1, 3) else 1
    return _hip.softmax(x, dim, dtype)


@get_index.override(AllOfType(Tensor, PrimitiveTensor))
def get_index_default(tensor, key):
    return unbox_tensor(tensor)[key]


# ---- the gathered-expert einsums of PreGatherFFNMOE -------------------------------------------------------------


def _is_expert_index(key):
    """`weights[experts, :, :]` / `weights[experts]` with an integer index tensor of shape [T, k]."""
    if isinstance(key, torch.Tensor):
        first, rest = key, ()
    elif isinstance(key, tuple) and key and isinstance(key[0], torch.Tensor):
        first, rest = key[0], key[1:]
    else:
        return None
    if first.dim() != 2 or first.dtype not in (torch.int32, torch.int64):
        return None
    if any(not (isinstance(r, slice) and r == slice(None)) for r in rest):
        return None
    return first


def gather_experts(weights, experts: torch.Tensor, dispatch=None) -> GatheredExpertsTensor:
    """Lazy `weights[experts, :, :]` for an expert-stacked weight [E, rows, cols] of any supported kind.  `dispatch`: the
    (offsets, perm) arrays of `experts` if the caller has built them already (the einsums of one forward index their
    weights with the same tensor); they are never kept beyond the gathered tensor itself."""
    if len(weights.shape) != 3:
        raise ValueError(f"gather_experts: expert-stacked weight must be [E, rows, cols], got {list(weights.shape)}")
    w = weights if isinstance(weights, InferenceTensor) else None
    if w is None:
        from ..types.tensors import DefaultPrimitiveTensor

        w = DefaultPrimitiveTensor(data=weights)
    g = GatheredExpertsTensor(weights=w, experts=experts)
    g._dispatch = dispatch
    return g


@get_index.override(QuantizedTensor)
def get_index_quantized_experts(tensor: QuantizedTensor, key):
    experts = _is_expert_index(key)
    if experts is None or len(tensor.shape) != 3:
        return NotImplemented
    return gather_experts(tensor, experts)


def expert_dispatch(experts: torch.Tensor, E: int):
    """(offsets, perm) of an index tensor [T, k]: rows grouped by expert.  Built from the tensor's present contents on
    every call: an index buffer may be refilled in place by a kernel (a fused forward, a graph replay) without torch
    noticing, so nothing here is remembered from call to call."""
    _, offsets, perm, _ = _hip.dispatch_build(experts, E)
    return offsets, perm


def _gathered_state(g: GatheredExpertsTensor):
    if g._device_weight is None:
        g._device_weight = cached_device_weight(g.weights, stacked=True)
    if g._dispatch is None:
        g._dispatch = expert_dispatch(g.experts, g._device_weight.experts)
    return g._device_weight, g._dispatch


@einsum_2args.override(Tensor, GatheredExpertsTensor)
def einsum_2args_gathered_experts(input0, input1: GatheredExpertsTensor, einsum_str: str):
    x = unbox_tensor(input0)
    T, k = input1.experts.shape
    if x.dtype not in _FLOAT_DTYPES:
        return NotImplemented
    if einsum_str == "mk,menk->men":
        if x.dim() != 2 or x.shape[0] != T:
            return NotImplemented
        dw, (offsets, perm) = _gathered_state(input1)
        return _hip.grouped_mmt(x, dw, offsets, perm, T, k, a_per_pair=False)
    if einsum_str == "mek,menk->men":
        if x.dim() != 3 or x.shape[0] != T or x.shape[1] != k:
            return NotImplemented
        dw, (offsets, perm) = _gathered_state(input1)
        return _hip.grouped_mmt(x.reshape(T * k, x.shape[2]), dw, offsets, perm, T, k, a_per_pair=True)
    return NotImplemented


@einsum_2args.override(Tensor, Tensor)
def einsum_2args_me_men(input0, input1, einsum_str: str):
    if einsum_str != "me,men->men":
        return NotImplemented
    g, y = unbox_tensor(input0), unbox_tensor(input1)
    if g.dim() != 2 or y.dim() != 3 or tuple(g.shape) != tuple(y.shape[:2]) or y.dtype not in _FLOAT_DTYPES:
        return NotImplemented
    return _hip.scale_rows(y, g)
