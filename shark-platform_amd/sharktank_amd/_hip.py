"""ctypes binding of libsharktank_moe_hip.so (the C ABI in include/sharktank_moe_hip.h).

torch is used for device memory and the current HIP stream only.  Every wrapper refuses host tensors and
raises if the shared library is missing: there is no CPU or eager-torch arithmetic path in this package.
"""

from __future__ import annotations

import ctypes
import os
from ctypes import POINTER, Structure, c_char_p, c_float, c_int, c_int32, c_int64, c_size_t, c_void_p
from typing import Optional

import torch

_LIB_NAME = "libsharktank_moe_hip.so"
_LIB_PATH = os.path.join(os.path.dirname(os.path.abspath(__file__)), _LIB_NAME)

# enum stmoe_dtype
F32, F16, BF16, F8E4M3FN, I8, U8 = 0, 1, 2, 3, 4, 5
# enum stmoe_act
ACT_SILU, ACT_GELU_ERF = 0, 1
# enum stmoe_wfmt
W_DENSE, W_Q8_0, W_Q4_1, W_FP8 = 0, 1, 2, 3
W_Q8_0_PACKED, W_Q4_1_PACKED, W_FP8_PACKED = 4, 5, 6
_PACKED_OF = {W_Q8_0: W_Q8_0_PACKED, W_Q4_1: W_Q4_1_PACKED, W_FP8: W_FP8_PACKED}
# grouped_ffn variants
VARIANT_AUTO, VARIANT_GENERIC, VARIANT_MFMA_TILE, VARIANT_SKINNY, VARIANT_MFMA_BIG, VARIANT_FP8_MFMA, VARIANT_MFMA_WS = 0, 1, 2, 3, 4, 5, 6
VARIANT_FP8_TILE = 7
VARIANT_STEP_BY_STEP = 8  # automatic choice among the kernels that round where the reference rounds (never the fp8 matrix cores)
VARIANT_MFMA_NARROW = 9  # 64 x 256 tiles: a single matrix with a few hundred rows (chosen automatically where it pays)

_DTYPE_ENUM = {
    torch.float32: F32,
    torch.float16: F16,
    torch.bfloat16: BF16,
    torch.float8_e4m3fn: F8E4M3FN,
    torch.int8: I8,
    torch.uint8: U8,
}

STATUS_NAMES = {
    0: "OK",
    1: "NULL pointer",
    2: "bad shape",
    3: "bad dtype",
    4: "misaligned pointer",
    5: "unsupported combination",
    6: "workspace too small",
    7: "kernel launch failed",
}


class StmoeWeight(Structure):
    _fields_ = [
        ("format", c_int32),
        ("dtype", c_int32),
        ("experts", c_int64),
        ("rows", c_int64),
        ("cols", c_int64),
        ("qs", c_void_p),
        ("d", c_void_p),
        ("m", c_void_p),
        ("d_count", c_int64),
    ]


# name -> (restype, argtypes); kept in one table so a test can check that the library exports them all.
SIGNATURES = {
    "stmoe_last_error": (c_char_p, []),
    "stmoe_abi_version": (c_int, []),
    "stmoe_dequant_block_scaled": (c_int, [c_void_p, c_void_p, c_int, c_void_p, c_int64, c_int, c_void_p, c_int, c_void_p]),
    "stmoe_dequant_block_scaled_i4": (c_int, [c_void_p, c_void_p, c_int, c_void_p, c_int64, c_int, c_int, c_void_p, c_int, c_void_p]),
    "stmoe_promote_i4": (c_int, [c_void_p, c_int64, c_int, c_void_p, c_void_p]),
    "stmoe_dequant_tensor_scaled": (c_int, [c_void_p, c_int, c_void_p, c_void_p, c_int, c_int64, c_int64, c_void_p, c_int, c_void_p]),
    "stmoe_prepack": (c_int, [POINTER(StmoeWeight), POINTER(StmoeWeight), c_void_p]),
    "stmoe_unpack": (c_int, [POINTER(StmoeWeight), POINTER(StmoeWeight), c_void_p]),
    "stmoe_gguf_ingest": (c_int, [c_void_p, c_int, POINTER(StmoeWeight), c_void_p]),
    "stmoe_quantize_fp8": (c_int, [c_void_p, c_int, c_void_p, c_int64, c_void_p, c_void_p]),
    "stmoe_quantize_fp8_per_axis": (c_int, [c_void_p, c_int, c_void_p, c_int, c_int64, c_int64, c_int64, c_void_p, c_void_p]),
    "stmoe_dequant_tensor_scaled_per_axis": (c_int, [c_void_p, c_int, c_void_p, c_void_p, c_int, c_int64, c_int64, c_int64, c_void_p,
                                                     c_int, c_void_p]),
    "stmoe_dynamic_quantize_fp8_scratch_bytes": (c_size_t, []),
    "stmoe_dynamic_quantize_fp8": (c_int, [c_void_p, c_int, c_int64, c_void_p, c_void_p, c_void_p, c_size_t, c_void_p]),
    "stmoe_fake_quant_fp8": (c_int, [c_void_p, c_int, c_void_p, c_int64, c_void_p, c_void_p]),
    "stmoe_rms_norm": (c_int, [c_void_p, c_int, c_void_p, c_int, c_int64, c_int64, c_float, c_void_p, c_void_p]),
    "stmoe_router_topk": (c_int, [c_void_p, c_void_p, c_int, c_int64, c_int64, c_int, c_int, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p]),
    "stmoe_dispatch_build": (c_int, [c_void_p, c_int64, c_int, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p]),
    "stmoe_grouped_ffn_workspace_bytes": (c_size_t, [c_int64, c_int, c_int64, c_int64, c_int]),
    "stmoe_moe_forward_workspace_bytes": (c_size_t, [c_int64, c_int, c_int, c_int64, c_int64, c_int]),
    "stmoe_grouped_ffn": (c_int, [c_void_p, c_int, c_int64, c_int64, c_int64, c_int, c_int, POINTER(StmoeWeight), POINTER(StmoeWeight),
                                  POINTER(StmoeWeight), c_int, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_size_t, c_int,
                                  c_void_p]),
    "stmoe_grouped_gate_up": (c_int, [c_void_p, c_int, c_int64, c_int64, c_int64, c_int, c_int, POINTER(StmoeWeight), POINTER(StmoeWeight),
                                      c_int, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_size_t, c_int, c_void_p]),
    "stmoe_grouped_down": (c_int, [c_void_p, c_int, c_int64, c_int64, c_int64, c_int, c_int, POINTER(StmoeWeight), c_void_p, c_void_p,
                                   c_void_p, c_size_t, c_int, c_void_p]),
    "stmoe_grouped_mmt": (c_int, [c_void_p, c_int, c_int64, c_int, c_int, POINTER(StmoeWeight), c_void_p, c_void_p, c_void_p, c_int, c_void_p]),
    "stmoe_add_bias": (c_int, [c_void_p, c_int, c_void_p, c_int, c_int64, c_int64, c_void_p, c_int, c_void_p]),
    "stmoe_softmax": (c_int, [c_void_p, c_int, c_int64, c_int64, c_void_p, c_int, c_void_p]),
    "stmoe_scale_rows": (c_int, [c_void_p, c_void_p, c_int, c_int64, c_int64, c_void_p, c_void_p]),
    "stmoe_combine": (c_int, [c_void_p, c_void_p, c_void_p, c_int, c_int64, c_int, c_int64, c_void_p, c_int, c_float, c_void_p, c_void_p, c_void_p]),
    "stmoe_moe_forward": (c_int, [c_void_p, c_int, c_int64, c_int64, c_int64, c_int, c_int, c_void_p, c_void_p, c_int, c_float, c_void_p,
                                  POINTER(StmoeWeight), POINTER(StmoeWeight), POINTER(StmoeWeight), c_int, c_void_p, c_void_p, c_void_p, c_void_p,
                                  c_void_p, c_void_p, c_size_t, c_int, c_void_p]),
    "stmoe_moe_forward_timed": (c_int, [c_void_p, c_int, c_int64, c_int64, c_int64, c_int, c_int, c_void_p, c_void_p, c_int, c_float, c_void_p,
                                        POINTER(StmoeWeight), POINTER(StmoeWeight), POINTER(StmoeWeight), c_int, c_void_p, c_void_p, c_void_p,
                                        c_void_p, c_void_p, c_void_p, c_size_t, c_int, c_void_p, POINTER(c_void_p)]),
    "stmoe_moe_forward_static": (c_int, [c_void_p, c_int, c_int64, c_int64, c_int64, c_int, c_int, c_void_p, c_void_p, c_int, c_float, c_void_p,
                                         POINTER(StmoeWeight), POINTER(StmoeWeight), POINTER(StmoeWeight), c_int, c_void_p, c_void_p, c_void_p,
                                         c_void_p, c_void_p, c_int, c_void_p]),
    "stmoe_mmt_workspace_bytes": (c_size_t, [c_int64]),
    "stmoe_mmt": (c_int, [c_void_p, c_int, c_int64, POINTER(StmoeWeight), c_void_p, c_void_p, c_size_t, c_int, c_int, c_void_p]),
    "stmoe_probe_mfma": (c_int, [c_int, c_int, c_int, c_void_p, POINTER(ctypes.c_double), c_void_p]),
}
STATIC_SCRATCH_BYTES = 16 << 20  # STMOE_STATIC_SCRATCH_BYTES

_lib = None


class StmoeError(RuntimeError):
    def __init__(self, status: int, message: str):
        super().__init__(f"sharktank_moe_hip: {STATUS_NAMES.get(status, status)}: {message}")
        self.status = status


def library_path() -> str:
    return _LIB_PATH


def load_library() -> ctypes.CDLL:
    """Loads the shared library; raises (never falls back) when it has not been built."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(_LIB_PATH):
        raise RuntimeError(
            f"{_LIB_PATH} is missing: build it with `make -C shark-platform_amd/csrc` "
            "(or __graft_entry__.build()). sharktank_amd has no other compute path."
        )
    lib = ctypes.CDLL(_LIB_PATH)
    for name, (restype, argtypes) in SIGNATURES.items():
        fn = getattr(lib, name)
        fn.restype = restype
        fn.argtypes = argtypes
    _lib = lib
    return lib


def _check(status: int):
    if status != 0:
        msg = load_library().stmoe_last_error()
        err = StmoeError(status, msg.decode() if msg else "")
        # The reference signals a missing kernel for a type combination with NotImplementedError.
        if status == 5:
            raise NotImplementedError(str(err))
        raise err


def dtype_enum(dt: torch.dtype) -> int:
    try:
        return _DTYPE_ENUM[dt]
    except KeyError:
        raise TypeError(f"sharktank_amd: dtype {dt} has no kernel support") from None


def _dev(*tensors: Optional[torch.Tensor]) -> torch.device:
    dev = None
    for t in tensors:
        if t is None:
            continue
        if not t.is_cuda:
            raise RuntimeError(
                "sharktank_amd computes on the GPU only: got a host tensor "
                f"({tuple(t.shape)}, {t.dtype}); move the parameters and inputs to the device first"
            )
        if dev is None:
            dev = t.device
        elif t.device != dev:
            raise RuntimeError(f"tensors on different devices: {dev} and {t.device}")
    return dev


def _ptr(t: Optional[torch.Tensor]) -> Optional[int]:
    return None if t is None else t.data_ptr()


def _stream(dev: torch.device) -> int:
    return torch.cuda.current_stream(dev).cuda_stream


def _contig(t: Optional[torch.Tensor]) -> Optional[torch.Tensor]:
    return None if t is None else t.contiguous()


# ---- dequantisation -------------------------------------------------------------------------------


def dequant_block_scaled(d, qs, m, dtype: Optional[torch.dtype]) -> torch.Tensor:
    """BlockScaledLayout.dequant_blocked: returns a tensor shaped like `qs`."""
    dev = _dev(d, qs, m)
    lib = load_library()
    out_dtype = d.dtype if dtype is None else dtype
    d_c, qs_c, m_c = _contig(d), _contig(qs), _contig(m)
    if qs_c.dtype != torch.int8:
        raise TypeError(f"BlockScaledLayout qs must be int8, got {qs_c.dtype}")
    block = qs_c.shape[-1]
    n_blocks = qs_c.numel() // block if block else 0
    out = torch.empty(qs_c.shape, dtype=out_dtype, device=dev)
    with torch.cuda.device(dev):
        _check(lib.stmoe_dequant_block_scaled(_ptr(d_c), _ptr(m_c), dtype_enum(d_c.dtype), _ptr(qs_c), n_blocks, block,
                                              _ptr(out), dtype_enum(out_dtype), _stream(dev)))
    return out


def dequant_block_scaled_i4(d, qs_packed, m, signed: bool, dtype: Optional[torch.dtype]) -> torch.Tensor:
    dev = _dev(d, qs_packed, m)
    lib = load_library()
    out_dtype = d.dtype if dtype is None else dtype
    d_c, qs_c, m_c = _contig(d), _contig(qs_packed), _contig(m)
    if qs_c.dtype not in (torch.uint8, torch.int8):
        raise AssertionError(f"Expected tensor to by uint8 or int8. Got: {qs_c.dtype}")
    block = qs_c.shape[-1] * 2
    n_blocks = qs_c.numel() * 2 // block if block else 0
    out = torch.empty(tuple(qs_c.shape[:-1]) + (block,), dtype=out_dtype, device=dev)
    with torch.cuda.device(dev):
        _check(lib.stmoe_dequant_block_scaled_i4(_ptr(d_c), _ptr(m_c), dtype_enum(d_c.dtype), _ptr(qs_c), n_blocks, block,
                                                 int(bool(signed)), _ptr(out), dtype_enum(out_dtype), _stream(dev)))
    return out


def promote_i4_block(qs_packed, signed: bool) -> torch.Tensor:
    dev = _dev(qs_packed)
    lib = load_library()
    qs_c = _contig(qs_packed)
    if qs_c.dtype not in (torch.uint8, torch.int8):
        raise AssertionError(f"Expected tensor to by uint8 or int8. Got: {qs_c.dtype}")
    out = torch.empty(tuple(qs_c.shape[:-1]) + (qs_c.shape[-1] * 2,), dtype=torch.int8 if signed else torch.uint8, device=dev)
    with torch.cuda.device(dev):
        _check(lib.stmoe_promote_i4(_ptr(qs_c), qs_c.numel(), int(bool(signed)), _ptr(out), _stream(dev)))
    return out


def dequant_tensor_scaled(qs, d, m, dtype: torch.dtype) -> torch.Tensor:
    dev = _dev(qs, d, m)
    lib = load_library()
    qs_c, d_c = _contig(qs), _contig(d)
    m_c = None if m is None else _contig(m).to(d_c.dtype)
    n = qs_c.numel()
    d_count = d_c.numel()
    if m_c is not None and m_c.numel() != d_count:
        raise NotImplementedError("TensorScaledLayout dequant: offset and scale must have the same shape")
    out = torch.empty(qs_c.shape, dtype=dtype, device=dev)
    axis = _broadcast_axis(d_c, qs_c) if d_count != 1 else None
    with torch.cuda.device(dev):
        if axis is None:
            _check(lib.stmoe_dequant_tensor_scaled(_ptr(qs_c), dtype_enum(qs_c.dtype), _ptr(d_c), _ptr(m_c), dtype_enum(d_c.dtype),
                                                   1, n, _ptr(out), dtype_enum(dtype), _stream(dev)))
        else:
            inner = 1
            for s_ in qs_c.shape[axis + 1:]:
                inner *= s_
            _check(lib.stmoe_dequant_tensor_scaled_per_axis(_ptr(qs_c), dtype_enum(qs_c.dtype), _ptr(d_c), _ptr(m_c),
                                                            dtype_enum(d_c.dtype), d_count, inner, n, _ptr(out),
                                                            dtype_enum(dtype), _stream(dev)))
    return out


def _broadcast_axis(d: torch.Tensor, qs: torch.Tensor) -> int:
    """The axis of `qs` along which the scales `d` vary: `d` is [A] (then the leading axis, the per-expert case) or has
    qs's rank with ones everywhere but on one axis (the per-axis quantizer's broadcast shape)."""
    if d.dim() == 1:
        if qs.dim() and qs.shape[0] == d.shape[0]:
            return 0
    elif d.dim() == qs.dim():
        axes = [i for i, s_ in enumerate(d.shape) if s_ != 1]
        if len(axes) == 1 and d.shape[axes[0]] == qs.shape[axes[0]]:
            return axes[0]
    raise NotImplementedError(f"TensorScaledLayout dequant: scale shape {tuple(d.shape)} for qs {tuple(qs.shape)}")


def quantize_fp8_per_axis(x: torch.Tensor, scale: torch.Tensor, axis: int) -> torch.Tensor:
    """StaticScaledQuantizer's per-axis branch: e4m3fn(clamp(x * scale broadcast along `axis`))."""
    dev = _dev(x, scale)
    lib = load_library()
    x_c, s_c = _contig(x), _contig(scale).reshape(-1)
    axis = axis % x_c.dim()
    if s_c.numel() != x_c.shape[axis]:
        raise ValueError(f"per-axis scale of {s_c.numel()} values for axis {axis} of {tuple(x_c.shape)}")
    if s_c.dtype != x_c.dtype and s_c.dtype != torch.float32:
        s_c = s_c.to(torch.float32)  # eager torch would promote the product of two 16-bit dtypes to fp32 as well
    inner = 1
    for s_ in x_c.shape[axis + 1:]:
        inner *= s_
    out = torch.empty(x_c.shape, dtype=torch.float8_e4m3fn, device=dev)
    with torch.cuda.device(dev):
        _check(lib.stmoe_quantize_fp8_per_axis(_ptr(x_c), dtype_enum(x_c.dtype), _ptr(s_c), dtype_enum(s_c.dtype), s_c.numel(),
                                               inner, x_c.numel(), _ptr(out), _stream(dev)))
    return out


def quantize_fp8(x: torch.Tensor, rscale: torch.Tensor) -> torch.Tensor:
    dev = _dev(x, rscale)
    lib = load_library()
    x_c = _contig(x)
    rs = _scale1(rscale)
    out = torch.empty(x_c.shape, dtype=torch.float8_e4m3fn, device=dev)
    with torch.cuda.device(dev):
        _check(lib.stmoe_quantize_fp8(_ptr(x_c), dtype_enum(x_c.dtype), _ptr(rs), x_c.numel(), _ptr(out), _stream(dev)))
    return out


def dynamic_quantize_fp8(x: torch.Tensor):
    """DynamicScaledQuantizer for float8_e4m3fn: (qs e4m3fn like x, scale, rscale), the two scales as 0-dim tensors of
    x's dtype holding the values eager torch computes."""
    dev = _dev(x)
    lib = load_library()
    x_c = _contig(x)
    out = torch.empty(x_c.shape, dtype=torch.float8_e4m3fn, device=dev)
    sr = torch.empty(2, dtype=torch.float32, device=dev)
    scratch = torch.empty(int(lib.stmoe_dynamic_quantize_fp8_scratch_bytes()), dtype=torch.uint8, device=dev)
    with torch.cuda.device(dev):
        _check(lib.stmoe_dynamic_quantize_fp8(_ptr(x_c), dtype_enum(x_c.dtype), x_c.numel(), _ptr(out), _ptr(sr), _ptr(scratch),
                                              scratch.numel(), _stream(dev)))
    sr_t = sr.to(x_c.dtype)  # exact: both values were rounded to x's dtype on the device
    return out, sr_t[0], sr_t[1]


def fake_quant_fp8(x: torch.Tensor, rscale: torch.Tensor) -> torch.Tensor:
    """quantize(x).unpack().dequant() of a static per-tensor e4m3fn quantizer, in x's dtype."""
    dev = _dev(x, rscale)
    lib = load_library()
    x_c = _contig(x)
    rs = _scale1(rscale)
    out = torch.empty_like(x_c)
    with torch.cuda.device(dev):
        _check(lib.stmoe_fake_quant_fp8(_ptr(x_c), dtype_enum(x_c.dtype), _ptr(rs), x_c.numel(), _ptr(out), _stream(dev)))
    return out


def _scale1(s: Optional[torch.Tensor]) -> Optional[torch.Tensor]:
    """A reciprocal scale as one contiguous device fp32 value (None stays None)."""
    if s is None:
        return None
    return s.to(torch.float32).reshape(1).contiguous()


# ---- layer pieces -----------------------------------------------------------------------------------


def rms_norm(x: torch.Tensor, weight: torch.Tensor, epsilon: float) -> torch.Tensor:
    dev = _dev(x, weight)
    lib = load_library()
    x_c, w_c = _contig(x), _contig(weight)
    K = x_c.shape[-1]
    T = x_c.numel() // K if K else 0
    out = torch.empty_like(x_c)
    with torch.cuda.device(dev):
        _check(lib.stmoe_rms_norm(_ptr(x_c), dtype_enum(x_c.dtype), _ptr(w_c), dtype_enum(w_c.dtype), T, K, float(epsilon),
                                  _ptr(out), _stream(dev)))
    return out


def router_topk(x: torch.Tensor, w_router: torch.Tensor, k: int, *, want_logits: bool = False, index_dtype=torch.int32):
    """x [T,K], w_router [E,K] (same dtype) -> (idx [T,k], gate [T,k], logits [T,E] | None)."""
    dev = _dev(x, w_router)
    lib = load_library()
    x_c, w_c = _contig(x), _contig(w_router)
    if w_c.dtype != x_c.dtype:
        raise TypeError("router weight must already be cast to the activation dtype")
    T, K = x_c.shape
    E = w_c.shape[0]
    idx = torch.empty((T, k), dtype=torch.int32, device=dev)
    idx64 = torch.empty((T, k), dtype=torch.int64, device=dev) if index_dtype == torch.int64 else None
    gate = torch.empty((T, k), dtype=x_c.dtype, device=dev)
    logits = torch.empty((T, E), dtype=x_c.dtype, device=dev) if want_logits else None
    with torch.cuda.device(dev):
        _check(lib.stmoe_router_topk(_ptr(x_c), _ptr(w_c), dtype_enum(x_c.dtype), T, K, E, k, _ptr(logits), _ptr(idx), _ptr(idx64),
                                     _ptr(gate), _stream(dev)))
    return (idx64 if idx64 is not None else idx), gate, logits


def dispatch_build(idx: torch.Tensor, E: int):
    """idx [T,k] int32 -> (counts [E], offsets [E+1], perm [T*k], inv [T*k]) int32."""
    dev = _dev(idx)
    lib = load_library()
    idx_c = _contig(idx.to(torch.int32))
    n = idx_c.numel()
    counts = torch.empty(E, dtype=torch.int32, device=dev)
    offsets = torch.empty(E + 1, dtype=torch.int32, device=dev)
    perm = torch.empty(n, dtype=torch.int32, device=dev)
    inv = torch.empty(n, dtype=torch.int32, device=dev)
    with torch.cuda.device(dev):
        _check(lib.stmoe_dispatch_build(_ptr(idx_c), n, E, _ptr(counts), _ptr(offsets), _ptr(perm), _ptr(inv), _stream(dev)))
    return counts, offsets, perm, inv


Q4_1_PACKED_MAX_SCALE = 64.0


class DeviceWeight:
    """An expert-stacked weight `[E, rows, cols]` as the C ABI sees it; keeps its planes alive."""

    def __init__(self, fmt: int, experts: int, rows: int, cols: int, qs, d=None, m=None, dtype_tag: int = 0):
        self.keep = (qs, d, m)
        self.device = _dev(qs, d, m)
        self.desc = StmoeWeight(
            format=fmt, dtype=dtype_tag, experts=experts, rows=rows, cols=cols,
            qs=_ptr(qs), d=_ptr(d), m=_ptr(m), d_count=(d.numel() if (d is not None and fmt in (W_FP8, W_FP8_PACKED)) else 1),
        )
        self.format = fmt
        self.experts, self.rows, self.cols = experts, rows, cols

    @property
    def ref(self):
        return ctypes.byref(self.desc)

    def nbytes(self) -> int:
        return sum(t.numel() * t.element_size() for t in self.keep if t is not None)

    @property
    def is_packed(self) -> bool:
        return self.format in (W_Q8_0_PACKED, W_Q4_1_PACKED, W_FP8_PACKED)

    def can_prepack(self) -> bool:
        return (self.format in _PACKED_OF and self.rows % 16 == 0 and self.cols % 256 == 0
                and (self.format != W_FP8 or self.desc.dtype == F32) and self.q4_scales_in_range())

    def q4_scales_in_range(self) -> bool:
        """The kernels that read Q4_1 weights in the streaming order fold the removal of their exponent bias into one fused
        multiply-add, which needs 1024 * |d| to stay finite in fp16: every block scale must be finite and below 64 in
        magnitude (block scales of real weights are orders of magnitude smaller).  A tensor that breaks the limit keeps the
        planar order, whose kernels have no such limit.  Checked once per tensor, at load time (one small reduction and a
        host read)."""
        if self.format not in (W_Q4_1, W_Q4_1_PACKED):
            return True
        d = self.keep[1]
        return bool(torch.isfinite(d).all()) and float(d.abs().max()) < Q4_1_PACKED_MAX_SCALE

    def prepack(self) -> "DeviceWeight":
        """The same weight in the streaming order of stmoe_prepack (new planes; this object is unchanged)."""
        qs, d, m = self.keep
        lib = load_library()
        new_qs = torch.empty_like(qs)
        fp8 = self.format == W_FP8
        new_d = d if fp8 else torch.empty_like(d)
        new_m = None if m is None else torch.empty_like(m)
        out = DeviceWeight(_PACKED_OF[self.format], self.experts, self.rows, self.cols, new_qs, new_d, new_m, self.desc.dtype)
        with torch.cuda.device(self.device):
            _check(lib.stmoe_prepack(self.ref, out.ref, _stream(self.device)))
        return out

    def unpack(self) -> "DeviceWeight":
        """Inverse of prepack()."""
        qs, d, m = self.keep
        lib = load_library()
        planar_fmt = {v: k for k, v in _PACKED_OF.items()}[self.format]
        fp8 = planar_fmt == W_FP8
        out = DeviceWeight(planar_fmt, self.experts, self.rows, self.cols, torch.empty_like(qs), d if fp8 else torch.empty_like(d),
                           None if m is None else torch.empty_like(m), self.desc.dtype)
        with torch.cuda.device(self.device):
            _check(lib.stmoe_unpack(self.ref, out.ref, _stream(self.device)))
        return out


GGUF_Q8_0, GGUF_Q4_1 = 0, 1


def gguf_ingest(raw: torch.Tensor, gguf_type: int, experts: int, rows: int, cols: int, *, packed: bool,
                check_scales: bool = True) -> DeviceWeight:
    """Raw ggml blocks (uint8, on the device) -> a DeviceWeight with freshly allocated planes, planar (the reference's
    planes bit for bit) or in the streaming order of stmoe_prepack.  With `check_scales` a Q4_1 tensor whose block scales
    the packed kernels cannot take (DeviceWeight.q4_scales_in_range) comes back planar even when `packed` is asked for."""
    dev = _dev(raw)
    lib = load_library()
    raw_c = _contig(raw)
    if raw_c.dtype != torch.uint8:
        raise TypeError(f"raw blocks must be uint8, got {raw_c.dtype}")
    nb = experts * rows * (cols // 32)
    block_bytes = {GGUF_Q8_0: 34, GGUF_Q4_1: 20}[gguf_type]
    if cols % 32 != 0 or raw_c.numel() != nb * block_bytes:
        raise ValueError(f"raw buffer of {raw_c.numel()} bytes does not hold [{experts},{rows},{cols}] in {block_bytes}-byte blocks")
    q4 = gguf_type == GGUF_Q4_1
    qs = torch.empty((experts, rows, cols // 32, 16 if q4 else 32), dtype=torch.uint8 if q4 else torch.int8, device=dev)
    d = torch.empty((experts, rows, cols // 32, 1), dtype=torch.float16, device=dev)
    m = torch.empty_like(d) if q4 else None
    fmt = W_Q4_1 if q4 else W_Q8_0
    out = DeviceWeight(_PACKED_OF[fmt] if packed else fmt, experts, rows, cols, qs, d, m)
    with torch.cuda.device(dev):
        _check(lib.stmoe_gguf_ingest(_ptr(raw_c), gguf_type, out.ref, _stream(dev)))
    if packed and check_scales and not out.q4_scales_in_range():
        return gguf_ingest(raw, gguf_type, experts, rows, cols, packed=False)  # see DeviceWeight.q4_scales_in_range
    return out


def grouped_ffn_workspace_bytes(T: int, k: int, K: int, N: int, dtype: torch.dtype) -> int:
    return int(load_library().stmoe_grouped_ffn_workspace_bytes(T, k, K, N, dtype_enum(dtype)))


def grouped_ffn(x, w_gate: DeviceWeight, w_up: DeviceWeight, w_down: DeviceWeight, act: int, offsets, perm, k: int,
                *, variant: int = VARIANT_AUTO, workspace: Optional[torch.Tensor] = None,
                x_scale: Optional[torch.Tensor] = None, z_scale: Optional[torch.Tensor] = None) -> torch.Tensor:
    """x [T,K] -> y_sorted [T*k, K] (rows in dispatch order).  x_scale / z_scale: reciprocal scales of the static
    e4m3fn quantizers of x and of the intermediate (None: not quantised)."""
    dev = _dev(x, offsets, perm)
    lib = load_library()
    x_c = _contig(x)
    T, K = x_c.shape
    N, E = w_gate.rows, w_gate.experts
    need = grouped_ffn_workspace_bytes(T, k, K, N, x_c.dtype)
    if workspace is None:
        if E == 1 and T * k <= 128:  # a single matrix of 33..128 rows: room for the split reductions of the prefill kernel
            need += int(lib.stmoe_mmt_workspace_bytes(T * k))
        workspace = torch.empty(max(need, 1), dtype=torch.uint8, device=dev)
    y = torch.empty((T * k, K), dtype=x_c.dtype, device=dev)
    xs, zs = _scale1(x_scale), _scale1(z_scale)
    with torch.cuda.device(dev):
        _check(lib.stmoe_grouped_ffn(_ptr(x_c), dtype_enum(x_c.dtype), T, K, N, E, k, w_gate.ref, w_up.ref, w_down.ref, act,
                                     _ptr(offsets), _ptr(perm), _ptr(xs), _ptr(zs), _ptr(y), _ptr(workspace), workspace.numel(), variant,
                                     _stream(dev)))
    return y


def grouped_gate_up(x, w_gate: DeviceWeight, w_up: DeviceWeight, act: int, offsets, perm, k: int, *, variant: int = VARIANT_AUTO,
                    x_scale: Optional[torch.Tensor] = None) -> torch.Tensor:
    """x [T,K] -> the gated intermediate z [T*k, N], rows in dispatch order (the first half of grouped_ffn)."""
    dev = _dev(x, offsets, perm)
    lib = load_library()
    x_c = _contig(x)
    T, K = x_c.shape
    N, E = w_gate.rows, w_gate.experts
    workspace = torch.empty(max(grouped_ffn_workspace_bytes(T, k, K, N, x_c.dtype), 1), dtype=torch.uint8, device=dev)
    z = torch.empty((T * k, N), dtype=x_c.dtype, device=dev)
    xs = _scale1(x_scale)
    with torch.cuda.device(dev):
        _check(lib.stmoe_grouped_gate_up(_ptr(x_c), dtype_enum(x_c.dtype), T, K, N, E, k, w_gate.ref, w_up.ref, act, _ptr(offsets),
                                         _ptr(perm), _ptr(xs), _ptr(z), _ptr(workspace), workspace.numel(), variant, _stream(dev)))
    return z


def grouped_down(z, w_down: DeviceWeight, offsets, T: int, k: int, *, variant: int = VARIANT_AUTO) -> torch.Tensor:
    """z [T*k, N] (dispatch order) -> y_sorted [T*k, K] (the second half of grouped_ffn; z is used as it is)."""
    dev = _dev(z, offsets)
    lib = load_library()
    z_c = _contig(z)
    N, K, E = w_down.cols, w_down.rows, w_down.experts
    workspace = torch.empty(max(grouped_ffn_workspace_bytes(T, k, K, N, z_c.dtype), 1), dtype=torch.uint8, device=dev)
    y = torch.empty((T * k, K), dtype=z_c.dtype, device=dev)
    with torch.cuda.device(dev):
        _check(lib.stmoe_grouped_down(_ptr(z_c), dtype_enum(z_c.dtype), T, K, N, E, k, w_down.ref, _ptr(offsets), _ptr(y),
                                      _ptr(workspace), workspace.numel(), variant, _stream(dev)))
    return y


def add_bias(y: torch.Tensor, bias: torch.Tensor) -> torch.Tensor:
    """y [..., cols] + bias [cols] in torch's promoted dtype (the bias add of `linear`)."""
    dev = _dev(y, bias)
    lib = load_library()
    y_c, b_c = _contig(y), _contig(bias)
    cols = y_c.shape[-1]
    if b_c.dim() != 1 or b_c.shape[0] != cols:
        raise ValueError(f"add_bias: bias {list(bias.shape)} does not match rows of {cols} elements")
    rows = y_c.numel() // cols if cols else 0
    out = torch.empty(y_c.shape, dtype=torch.promote_types(y_c.dtype, b_c.dtype), device=dev)
    with torch.cuda.device(dev):
        _check(lib.stmoe_add_bias(_ptr(y_c), dtype_enum(y_c.dtype), _ptr(b_c), dtype_enum(b_c.dtype), rows, cols, _ptr(out),
                                  dtype_enum(out.dtype), _stream(dev)))
    return out


def softmax(x: torch.Tensor, dim: int = -1, dtype: Optional[torch.dtype] = None) -> torch.Tensor:
    """torch.nn.functional.softmax(x, dim, dtype) computed in fp32 by the library; the result has dtype `dtype` (x's if None)."""
    dev = _dev(x)
    lib = load_library()
    out_dtype = dtype or x.dtype
    moved = x.movedim(dim, -1)
    x_c = _contig(moved)
    cols = x_c.shape[-1]
    rows = x_c.numel() // cols if cols else 0
    out = torch.empty(x_c.shape, dtype=out_dtype, device=dev)
    with torch.cuda.device(dev):
        _check(lib.stmoe_softmax(_ptr(x_c), dtype_enum(x_c.dtype), rows, cols, _ptr(out), dtype_enum(out_dtype), _stream(dev)))
    return out.movedim(-1, dim)


def grouped_mmt(a: torch.Tensor, w: "DeviceWeight", offsets, perm, T: int, k: int, *, a_per_pair: bool,
                variant: int = VARIANT_AUTO) -> torch.Tensor:
    """a [T, cols] (or [T*k, cols] when a_per_pair) -> out [T, k, rows]: every pair's row times its expert's matrix."""
    dev = _dev(a, offsets, perm)
    lib = load_library()
    a_c = _contig(a)
    out = torch.empty((T, k, w.rows), dtype=a_c.dtype, device=dev)
    with torch.cuda.device(dev):
        _check(lib.stmoe_grouped_mmt(_ptr(a_c), dtype_enum(a_c.dtype), T, k, int(bool(a_per_pair)), w.ref, _ptr(offsets),
                                     _ptr(perm), _ptr(out), variant, _stream(dev)))
    return out


def scale_rows(y: torch.Tensor, g: torch.Tensor) -> torch.Tensor:
    """y [..., K] * g [...] (one factor per row), rounded to y's dtype."""
    dev = _dev(y, g)
    lib = load_library()
    y_c, g_c = _contig(y), _contig(g.to(y.dtype))
    K = y_c.shape[-1]
    rows = y_c.numel() // K if K else 0
    out = torch.empty_like(y_c)
    with torch.cuda.device(dev):
        _check(lib.stmoe_scale_rows(_ptr(y_c), _ptr(g_c), dtype_enum(y_c.dtype), rows, K, _ptr(out), _stream(dev)))
    return out


def combine(y_sorted, gate, inv, T: int, k: int, *, out_norm_w=None, eps: float = 0.0, residual=None) -> torch.Tensor:
    dev = _dev(y_sorted, gate, inv, out_norm_w, residual)
    lib = load_library()
    K = y_sorted.shape[-1]
    y_c, g_c = _contig(y_sorted), _contig(gate)
    res_c = None if residual is None else _contig(residual)
    w_c = None if out_norm_w is None else _contig(out_norm_w)
    out = torch.empty((T, K), dtype=y_c.dtype, device=dev)
    with torch.cuda.device(dev):
        _check(lib.stmoe_combine(_ptr(y_c), _ptr(g_c), _ptr(inv), dtype_enum(y_c.dtype), T, k, K, _ptr(w_c),
                                 dtype_enum(w_c.dtype) if w_c is not None else F32, float(eps), _ptr(res_c), _ptr(out), _stream(dev)))
    return out


def moe_forward_workspace_bytes(T: int, k: int, E: int, K: int, N: int, dtype: torch.dtype) -> int:
    return int(load_library().stmoe_moe_forward_workspace_bytes(T, k, E, K, N, dtype_enum(dtype)))


def moe_forward(h, ffn_norm_w, out_norm_w, eps: float, w_router, w_gate: DeviceWeight, w_up: DeviceWeight, w_down: DeviceWeight,
                act: int, k: int, *, variant: int = VARIANT_AUTO, workspace: Optional[torch.Tensor] = None, want_routing: bool = False,
                out: Optional[torch.Tensor] = None, events=None, x_scale: Optional[torch.Tensor] = None,
                z_scale: Optional[torch.Tensor] = None):
    """h [T,K] -> out [T,K] (and, if asked, idx int32 [T,k] and gate [T,k]).  `events`: optional ctypes array of
    12 hipEvent_t handles that bracket the six stages (see stmoe_moe_forward_timed)."""
    dev = _dev(h, ffn_norm_w, out_norm_w, w_router)
    lib = load_library()
    h_c = _contig(h)
    T, K = h_c.shape
    N, E = w_gate.rows, w_gate.experts
    need = moe_forward_workspace_bytes(T, k, E, K, N, h_c.dtype)
    if workspace is None or workspace.numel() < need:
        workspace = torch.empty(max(need, 1), dtype=torch.uint8, device=dev)
    if out is None:
        out = torch.empty_like(h_c)
    idx = torch.empty((T, k), dtype=torch.int32, device=dev) if want_routing else None
    gate = torch.empty((T, k), dtype=h_c.dtype, device=dev) if want_routing else None
    xs, zs = _scale1(x_scale), _scale1(z_scale)
    args = (_ptr(h_c), dtype_enum(h_c.dtype), T, K, N, E, k, _ptr(ffn_norm_w), _ptr(out_norm_w),
            dtype_enum(ffn_norm_w.dtype), float(eps), _ptr(w_router), w_gate.ref, w_up.ref, w_down.ref, act,
            _ptr(xs), _ptr(zs), _ptr(out), _ptr(idx), _ptr(gate), _ptr(workspace), workspace.numel(), variant, _stream(dev))
    with torch.cuda.device(dev):
        if events is None:
            _check(lib.stmoe_moe_forward(*args))
        else:
            _check(lib.stmoe_moe_forward_timed(*args, events))
    if want_routing:
        return out, idx, gate
    return out


def moe_forward_static(h, ffn_norm_w, out_norm_w, eps: float, w_router, w_gate: DeviceWeight, w_up: DeviceWeight,
                       w_down: DeviceWeight, act: int, k: int, out: torch.Tensor, *, variant: int = VARIANT_AUTO,
                       idx: Optional[torch.Tensor] = None, gate: Optional[torch.Tensor] = None,
                       x_scale: Optional[torch.Tensor] = None, z_scale: Optional[torch.Tensor] = None) -> torch.Tensor:
    """moe_forward on the library's built-in workspace (stmoe_moe_forward_static): every buffer is the caller's (`h` contiguous
    [T,K], `out` like it, optional `idx` int32 / `gate` [T,k], scales as single fp32 device values), so the call allocates
    nothing.  Shapes beyond the built-in workspace raise StmoeError (status 6)."""
    dev = _dev(h, ffn_norm_w, out_norm_w, w_router, out, idx, gate, x_scale, z_scale)
    lib = load_library()
    if not h.is_contiguous() or not out.is_contiguous():
        raise ValueError("moe_forward_static: h and out must be contiguous")
    T, K = h.shape
    with torch.cuda.device(dev):
        _check(lib.stmoe_moe_forward_static(_ptr(h), dtype_enum(h.dtype), T, K, w_gate.rows, w_gate.experts, k, _ptr(ffn_norm_w),
                                            _ptr(out_norm_w), dtype_enum(ffn_norm_w.dtype), float(eps), _ptr(w_router), w_gate.ref,
                                            w_up.ref, w_down.ref, act, _ptr(x_scale), _ptr(z_scale), _ptr(out), _ptr(idx), _ptr(gate),
                                            variant, _stream(dev)))
    return out


_MMT_WORKSPACE = {}  # (device, stream) -> scratch of split reductions, allocated on the first product that can use it


def _mmt_workspace(dev: torch.device, stream: int, need: int) -> Optional[torch.Tensor]:
    """One scratch buffer per device and stream (launches on one stream run one after the other, so they can share it),
    zero-filled once: only stmoe_mmt writes to it afterwards, which lets every call skip the clearing of its counters."""
    if need == 0:
        return None
    key = (dev, stream)
    ws = _MMT_WORKSPACE.get(key)
    if ws is None or ws.numel() < need:
        ws = torch.zeros(need, dtype=torch.uint8, device=dev)
        _MMT_WORKSPACE[key] = ws
    return ws


def mmt(a: torch.Tensor, w: DeviceWeight, *, variant: int = VARIANT_AUTO, workspace: Optional[torch.Tensor] = None) -> torch.Tensor:
    """a [..., K] @ W[rows, K]^T -> [..., rows] in a's dtype.  `workspace`: scratch of stmoe_mmt_workspace_bytes(M) bytes;
    by default a buffer kept per device and stream (pass one of your own under HIP graph capture)."""
    dev = _dev(a)
    lib = load_library()
    a_c = _contig(a)
    K = a_c.shape[-1]
    M = a_c.numel() // K if K else 0
    out = torch.empty(tuple(a_c.shape[:-1]) + (w.rows,), dtype=a_c.dtype, device=dev)
    with torch.cuda.device(dev):
        stream = _stream(dev)
        ready = workspace is None  # a caller's buffer has an unknown history
        if workspace is None:
            need = int(lib.stmoe_mmt_workspace_bytes(M))
            if need and (dev, stream) not in _MMT_WORKSPACE and torch.cuda.is_current_stream_capturing():
                # the kept buffer is zero-filled by a launch of its own, which must not become part of somebody's graph
                # (it would run at replay time only): a buffer of this call's own, cleared by the library inside the graph
                workspace, ready = torch.empty(need, dtype=torch.uint8, device=dev), False
            else:
                workspace = _mmt_workspace(dev, stream, need)
        _check(lib.stmoe_mmt(_ptr(a_c), dtype_enum(a_c.dtype), M, w.ref, _ptr(out), _ptr(workspace),
                             workspace.numel() if workspace is not None else 0, int(ready), variant, stream))
    return out


def probe_mfma(device, kind: int = 0, random_operands: bool = True, iters: int = 20000, launches: int = 8,
               warm_launches: int = 12) -> float:
    """TFLOP/s of launches of nothing but independent matrix-core instructions (stmoe_probe_mfma; kind 0: fp16, 1: fp8),
    timed with events on the current stream.  The untimed launches in front (some tens of milliseconds) let the chip's
    power management settle: a short burst after idle runs at a clock the chip does not hold."""
    lib = load_library()
    dev = torch.device(device)
    sink = torch.zeros(1, dtype=torch.float32, device=dev)
    flop = ctypes.c_double(0.0)
    with torch.cuda.device(dev):
        for _ in range(warm_launches):
            _check(lib.stmoe_probe_mfma(kind, int(random_operands), iters, _ptr(sink), None, _stream(dev)))
        start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        start.record()
        for _ in range(launches):
            _check(lib.stmoe_probe_mfma(kind, int(random_operands), iters, _ptr(sink), ctypes.byref(flop), _stream(dev)))
        stop.record()
        stop.synchronize()
    return launches * flop.value / (start.elapsed_time(stop) * 1e-3) / 1e12
