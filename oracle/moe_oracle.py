"""CPU restatement of sharktank's quantized mixture-of-experts path.  TEST INFRASTRUCTURE ONLY.

This module is the checker for the HIP kernels: only tests/, __graft_entry__.smoke() and the
`cpu_baseline` leg of bench.py may import it.  Nothing in the product package imports or calls it.

It restates, in plain torch (CPU) and numpy, the algorithm of the reference's eager path.  All paths
below are relative to the reference checkout; `ST/` = sharktank/sharktank/.

Third-party arithmetic: the reference's floating-point work is done by PyTorch (pinned torch==2.3.0 CPU
in sharktank's pytorch-cpu-requirements.txt:3) -- matmul, softmax, topk, silu, gelu, rsqrt -- so this
restatement calls the same torch routines on the same rounding points.  The IREE-compiled kernels
(`mmt_block_scaled_q8` etc.) cannot be produced here; they agree with dequantize-then-matmul within the
tolerances of the reference's own kernel tests (tests/kernels/mmt_block_scaled_q8_test.py:24-41).

How each function is pinned (tests/test_oracle_*.py):
  nibble utilities ............ the reference's known-answer vectors (tests/types/layout_utils_test.py:15-65)
  dequant_tensor_scaled ....... the reference's known-answer vector (tests/types/layouts_test.py:107-125)
  dequant_block_scaled{,_i4} .. exact rational arithmetic (fractions.Fraction) + manual RNE on tiny inputs
  static/dynamic quantizers ... the reference's round-trip vectors (tests/types/quantizers_test.py:40-64,133-244)
  q8_0_unpack / q4_1_unpack ... hand-assembled ggml blocks (struct layouts quoted at
                                ST/types/gguf_interop/layouts.py:33-39,263-270)
  rms_norm .................... the formula of the reference's test (tests/ops/ops_test.py:228-232) in float64
  rms_norm_ordered ............ equals rms_norm bit for bit where every partial sum is exact, and within fp32 rounding of it
                                elsewhere; a pure-Python sequential restatement of the order on a tiny case
  router ...................... float64 brute force on tiny inputs incl. forced ties (tie rule: lower index)
  router_logits_ordered ....... equals an exact (float64) dot product wherever rounding is not in play, and
                                a pure-Python sequential restatement on a tiny case
  dispatch_permutation ........ brute-force Python loops; torch.sort(stable=True)
  pre_gather_ffn_moe .......... agrees with the independent per-expert formulation (`grouped_ffn_moe`, the
                                shape of the reference's FFNMOE, ST/layers/ffn_moe_block.py:77-140) and a
                                float64 per-token brute force on tiny inputs
  moe_block ................... composition of the above.  PARITY UNPINNED BY REFERENCE TESTS: the
                                reference's only MoE test (tests/models/llama/moe_block_test.py:17-30)
                                checks that the block exports and asserts no numbers.
"""

from __future__ import annotations

from typing import Callable, Optional, Tuple

import numpy as np
import torch
import torch.nn.functional as F

BLOCK = 32

# ---------------------------------------------------------------------------------------------------
# i4 nibble utilities -- ST/types/layout_utils.py:20-86
# ---------------------------------------------------------------------------------------------------


def _u8(t: torch.Tensor) -> torch.Tensor:
    if t.dtype == torch.uint8:
        return t
    if t.dtype == torch.int8:
        return t.view(torch.uint8)
    raise AssertionError(f"Expected tensor to by uint8 or int8. Got: {t.dtype}")


def linearize_interleaved_i4_block(i8_data: torch.Tensor) -> torch.Tensor:
    """ggml nibble order (byte i: low = element i, high = element i + n) -> linear order
    (byte i: low = element 2i, high = element 2i+1).  ST/types/layout_utils.py:20-44."""
    b = _u8(i8_data)
    lo, hi = b & 0xF, b >> 4
    t1 = (lo[..., 1::2] << 4) | lo[..., ::2]
    t2 = (hi[..., 1::2] << 4) | hi[..., ::2]
    return torch.cat([t1, t2], dim=-1)


def interleave_linear_i4_block(i8_data: torch.Tensor) -> torch.Tensor:
    """Inverse of linearize_interleaved_i4_block.  ST/types/layout_utils.py:47-64."""
    b = _u8(i8_data)
    t1, t2 = torch.tensor_split(b, 2, dim=-1)
    i0 = ((t2 & 0xF) << 4) | (t1 & 0xF)
    i1 = ((t2 >> 4) << 4) | (t1 >> 4)
    return torch.stack([i0, i1], dim=-1).flatten(start_dim=-2)


def promote_linear_i4_block_to_i8(linear_i4_data: torch.Tensor, *, signed: bool = False) -> torch.Tensor:
    """ST/types/layout_utils.py:67-86."""
    b = _u8(linear_i4_data)
    if signed:
        low = (b << 4).view(torch.int8) >> 4
        high = b.view(torch.int8) >> 4
    else:
        low = b & 0xF
        high = b >> 4
    return torch.stack([low, high], dim=-1).flatten(start_dim=-2)


# ---------------------------------------------------------------------------------------------------
# layouts: dequantisation -- ST/types/layouts.py
# ---------------------------------------------------------------------------------------------------


def dequant_block_scaled(d, qs, m=None, dtype: Optional[torch.dtype] = None) -> torch.Tensor:
    """BlockScaledLayout.dequant_blocked (ST/types/layouts.py:274-290).  d,m [...,1]; qs [...,B]."""
    if dtype is not None:
        d = d.to(dtype)
        if m is not None:
            m = m.to(dtype)
    else:
        dtype = d.dtype
        assert m is None or m.dtype == d.dtype
    scaled = d * qs.to(dtype)
    return scaled if m is None else scaled + m


def dequant_block_scaled_i4(d, qs_packed, m=None, *, signed: bool = False, dtype: Optional[torch.dtype] = None):
    """BlockScaledI4Layout: promote nibbles, then the block-scaled formula (ST/types/layouts.py:302-357)."""
    return dequant_block_scaled(d, promote_linear_i4_block_to_i8(qs_packed, signed=signed), m, dtype)


def dequant_tensor_scaled(d, qs, m=None, *, layout_dtype: Optional[torch.dtype] = None, dtype: Optional[torch.dtype] = None):
    """TensorScaledLayout.dequant_blocked (ST/types/layouts.py:163-181)."""
    if dtype is None:
        dtype = layout_dtype if layout_dtype is not None else d.dtype
    q = qs.to(dtype=d.dtype)
    result = (q - m.to(d.dtype)) * d if m is not None else q * d
    return result if result.dtype == dtype else result.to(dtype)


# ---------------------------------------------------------------------------------------------------
# quantizers -- ST/types/quantizers.py, ST/types/layout_utils.py:150-176
# ---------------------------------------------------------------------------------------------------


def saturate_cast(t: torch.Tensor, dtype: torch.dtype, round_int: bool = True, disable_saturate: bool = False):
    if dtype.is_floating_point:
        finfo = torch.finfo(dtype)
        if finfo.bits == 8 and not disable_saturate:
            t = t.clamp(finfo.min, finfo.max)
        return t.to(dtype=dtype)
    iinfo = torch.iinfo(dtype)
    if round_int:
        t = torch.round(t)
    if not disable_saturate:
        t = t.clamp(iinfo.min, iinfo.max)
    return t.to(dtype=dtype)


def static_quantize_per_tensor(t, reciprocal_scale, dtype, offset=None):
    """StaticScaledQuantizer._quantize_raw_tensor, per-tensor branch (ST/types/quantizers.py:153-183).
    Returns the planes of the TensorScaledLayout it builds: (qs, d = reciprocal_scale, m = offset)."""
    if offset is None:
        qs = saturate_cast(t / reciprocal_scale, dtype=dtype)
    else:
        qs = saturate_cast(t / reciprocal_scale + offset, dtype=dtype)
    return qs, reciprocal_scale, offset


def fake_quant_per_tensor(t, reciprocal_scale, dtype=torch.float8_e4m3fn):
    """`q_input.quantize(x).unpack().dequant()` of a static per-tensor quantizer (ST/layers/linear.py:72-78): the
    layout built by the quantizer has d = reciprocal_scale and dtype = t.dtype (ST/types/quantizers.py:176-183)."""
    qs, d, _ = static_quantize_per_tensor(t, reciprocal_scale, dtype)
    return dequant_tensor_scaled(d, qs, layout_dtype=t.dtype)


def static_quantize_per_axis(t, scale, axis: int, dtype, offset=None):
    """Per-axis branch (ST/types/quantizers.py:184-230): qs = saturate_cast(t * scale (+ offset)); d = 1/scale."""
    shape = [1] * t.dim()
    shape[axis] = scale.shape[0]
    bs = scale.reshape(shape)
    if offset is None:
        qs = saturate_cast(t * bs, dtype=dtype)
        bo = None
    else:
        bo = offset.reshape(shape)
        qs = saturate_cast(t * bs + bo, dtype=dtype)
    return qs, (1.0 / scale).reshape(shape), bo


def dynamic_quantize(t, dtype):
    """DynamicScaledQuantizer._quantize_raw_tensor (ST/types/quantizers.py:368-389)."""
    amax = torch.max(torch.abs(t))
    if dtype.is_floating_point:
        finfo = torch.finfo(dtype)
        scale = finfo.max / amax.clamp(finfo.eps)
    else:
        scale = torch.iinfo(dtype).max / amax.clamp(1e-6)
    return saturate_cast(t * scale, dtype, round_int=True), 1 / scale


# ---------------------------------------------------------------------------------------------------
# GGUF raw blocks -- ST/types/gguf_interop/layouts.py:31-67,260-307
# ---------------------------------------------------------------------------------------------------


def q8_0_unpack(raw: torch.Tensor, shape):
    """raw uint8 of ggml block_q8_0 {f16 d; i8 qs[32]} (34 B) -> planes (d [...,K/32,1] f16, qs [...,K/32,32] i8)."""
    assert raw.dtype == torch.uint8
    blocks = raw.view(torch.int16).reshape(-1, 17).reshape(list(shape[:-1]) + [-1, 17])
    return blocks[..., 0:1].view(torch.float16), blocks[..., 1:].view(torch.int8)


def q4_1_unpack(raw: torch.Tensor, shape):
    """raw uint8 of ggml block_q4_1 {f16 d; f16 m; u8 qs[16]} (20 B) -> (d, m, qs packed in linear order)."""
    blocks = raw.view(torch.int16).reshape(-1, 10).reshape(list(shape[:-1]) + [-1, 10])
    d = blocks[..., 0:1].view(torch.float16)
    m = blocks[..., 1:2].view(torch.float16)
    qs = linearize_interleaved_i4_block(blocks[..., 2:].view(torch.int8))
    return d, m, qs


# Synthetic quantisation (fp -> blocks).  Not in the reference (it only unpacks); follows ggml's
# quantize_row_q8_0 / quantize_row_q4_1 conventions.  Oracle and kernels consume the same planes, so the
# generator only has to be deterministic.
def quantize_q8_0(w: torch.Tensor):
    """w [..., K] float -> (d [..., K/32, 1] f16, qs [..., K/32, 32] i8)."""
    wb = w.float().reshape(*w.shape[:-1], -1, BLOCK)
    amax = wb.abs().amax(dim=-1, keepdim=True)
    d = amax / 127.0
    inv = torch.where(d > 0, 1.0 / d, torch.zeros_like(d))
    qs = torch.round(wb * inv).clamp(-127, 127).to(torch.int8)
    return d.to(torch.float16), qs


def quantize_q4_1(w: torch.Tensor):
    """w [..., K] float -> (d, m [..., K/32, 1] f16, qs packed [..., K/32, 16] u8, linear nibble order)."""
    wb = w.float().reshape(*w.shape[:-1], -1, BLOCK)
    mn = wb.amin(dim=-1, keepdim=True)
    mx = wb.amax(dim=-1, keepdim=True)
    d = (mx - mn) / 15.0
    inv = torch.where(d > 0, 1.0 / d, torch.zeros_like(d))
    q = torch.floor((wb - mn) * inv + 0.5).clamp(0, 15).to(torch.uint8)
    packed = q[..., 0::2] | (q[..., 1::2] << 4)
    return d.to(torch.float16), mn.to(torch.float16), packed


def quantize_fp8_per_tensor(w: torch.Tensor):
    """Per-tensor e4m3fn: d = amax/448 (f32 scalar), qs = saturate_cast(w / d)."""
    d = (w.float().abs().amax() / 448.0).to(torch.float32)
    qs = saturate_cast(w.float() / d, torch.float8_e4m3fn)
    return d, qs


# ---------------------------------------------------------------------------------------------------
# layer pieces
# ---------------------------------------------------------------------------------------------------


def rms_norm(x: torch.Tensor, weight: torch.Tensor, eps: float) -> torch.Tensor:
    """RMSNormLayer.forward (ST/layers/norm.py:34-41) + rms_norm_default (ST/ops/default_impls.py:402-408)."""
    orig = x.dtype
    x32 = x.to(torch.float32)
    variance = x32.pow(2).mean(-1, keepdim=True)
    out = x32 * torch.rsqrt(variance + eps)
    out = weight * out.to(weight.dtype)
    return out.to(orig)


def rms_norm_ordered(x: torch.Tensor, weight: torch.Tensor, eps: float) -> torch.Tensor:
    """rms_norm with the mean-of-squares summation order the HIP kernels document (the reference leaves the order to
    torch.mean): virtual thread j of 512 adds the fp32 squares of elements j, j+512, ... in order; the 64 sums of each of
    the 8 groups of 64 threads are combined by the xor butterfly 32..1; the 8 group sums as ((s0+s1)+(s2+s3))+((s4+s5)+
    (s6+s7)).  Everything else is the reference's arithmetic in fp32: sum / K, 1 / sqrt(. + eps), x * that, weight * ., cast."""
    assert weight.dtype == torch.float32
    T, K = x.shape
    x32 = x.float().numpy()
    C = (K + 511) // 512
    sq = np.zeros((T, C * 512), dtype=np.float32)
    sq[:, :K] = (x32 * x32).astype(np.float32)
    sq = sq.reshape(T, C, 512)
    acc = np.zeros((T, 512), dtype=np.float32)
    for c in range(C):
        acc = (acc + sq[:, c, :]).astype(np.float32)
    acc = acc.reshape(T, 8, 64)
    lanes = np.arange(64)
    for off in (32, 16, 8, 4, 2, 1):
        acc = (acc + acc[:, :, lanes ^ off]).astype(np.float32)
    s = acc[:, :, 0]
    f32 = np.float32
    total = ((s[:, 0] + s[:, 1]).astype(f32) + (s[:, 2] + s[:, 3]).astype(f32)).astype(f32) + \
            ((s[:, 4] + s[:, 5]).astype(f32) + (s[:, 6] + s[:, 7]).astype(f32)).astype(f32)
    total = total.astype(f32)
    var = (total / f32(K)).astype(f32)
    rs = (f32(1.0) / np.sqrt((var + f32(eps)).astype(f32)).astype(f32)).astype(f32)
    o = (x32 * rs[:, None]).astype(f32)
    o = (weight.numpy()[None, :] * o).astype(f32)
    return torch.from_numpy(o).to(x.dtype)


def router_logits(x: torch.Tensor, w_router: torch.Tensor) -> torch.Tensor:
    """linear_default -> matmul_default (ST/ops/default_impls.py:328-359): weight cast to x's dtype, result in x's
    dtype.  For 16-bit types the products are exact in fp32 and torch accumulates in fp32; computing the fp32
    matmul of the widened operands and rounding once states the same thing without depending on a CPU half GEMM."""
    w = w_router.to(x.dtype)
    if x.dtype == torch.float32:
        return torch.matmul(x, w.T)
    return torch.matmul(x.float(), w.float().T).to(x.dtype)


def router_logits_ordered(x: torch.Tensor, w_router: torch.Tensor) -> torch.Tensor:
    """Logits with the summation order the HIP router documents: lane l of 64 owns elements
    k = (c*64 + l)*8 + j (chunk c, j = 0..7), adds their fp32 products in increasing (c, j) order with
    separately rounded multiply and add, then the lanes are combined by the xor butterfly 32,16,...,1."""
    w = w_router.to(x.dtype)
    T, K = x.shape
    E = w.shape[0]
    assert K % 8 == 0
    C = (K + 511) // 512
    xp = np.zeros((T, C * 512), dtype=np.float32)
    wp = np.zeros((E, C * 512), dtype=np.float32)
    xp[:, :K] = x.float().numpy()
    wp[:, :K] = w.float().numpy()
    prod = (xp[:, None, :] * wp[None, :, :]).astype(np.float32)  # [T,E,C*512], each product rounded to fp32
    prod = prod.reshape(T, E, C, 64, 8)
    acc = np.zeros((T, E, 64), dtype=np.float32)
    for c in range(C):
        for j in range(8):
            acc = (acc + prod[:, :, c, :, j]).astype(np.float32)
    lanes = np.arange(64)
    for off in (32, 16, 8, 4, 2, 1):
        acc = (acc + acc[:, :, lanes ^ off]).astype(np.float32)
    return torch.from_numpy(acc[:, :, 0].copy()).to(x.dtype)


def topk_lower_index_first(values: torch.Tensor, k: int) -> Tuple[torch.Tensor, torch.Tensor]:
    """Top-k along the last dim, descending, equal values ordered by increasing index.  `torch.topk`
    (ST/layers/mixture_of_experts_block.py:78) leaves the order of ties unspecified; the contract fixes it."""
    order = torch.sort(values, dim=-1, descending=True, stable=True).indices[..., :k]
    return torch.gather(values, -1, order), order


def route(logits: torch.Tensor, k: int):
    """softmax in fp32, top-k, renormalise, cast (ST/layers/mixture_of_experts_block.py:75-83).
    Returns (idx int64 [T,k], gate [T,k] in logits.dtype, probs fp32 [T,E])."""
    probs = F.softmax(logits, dim=1, dtype=torch.float)
    gate, idx = topk_lower_index_first(probs, k)
    gate = gate / gate.sum(dim=-1, keepdim=True)
    return idx, gate.to(logits.dtype), probs


def dispatch_permutation(idx: torch.Tensor, E: int):
    """Stable counting sort of pairs p = t*k + j by expert: (counts [E], offsets [E+1], perm [T*k], inv [T*k])."""
    flat = idx.reshape(-1).to(torch.int64)
    counts = torch.bincount(flat, minlength=E)
    offsets = torch.zeros(E + 1, dtype=torch.int64)
    offsets[1:] = torch.cumsum(counts, 0)
    perm = torch.sort(flat, stable=True).indices
    inv = torch.empty_like(perm)
    inv[perm] = torch.arange(perm.numel())
    return counts.to(torch.int32), offsets.to(torch.int32), perm.to(torch.int32), inv.to(torch.int32)


def _mm_rt(a: torch.Tensor, b_t: torch.Tensor) -> torch.Tensor:
    """a @ b_t^T with fp32 accumulation, result in a's dtype (what torch.matmul gives for T tensors)."""
    if a.dtype == torch.float32:
        return torch.matmul(a, b_t.transpose(-1, -2))
    return torch.matmul(a.float(), b_t.float().transpose(-1, -2)).to(a.dtype)


def pre_gather_ffn_moe(h, experts, expert_gate, w_gate, w_up, w_down, activation: Callable = F.silu, chunk: int = 8,
                       x_rscale=None, z_rscale=None):
    """PreGatherFFNMOE.forward in the reference's own operation order (ST/layers/ffn_moe_block.py:37-41,60-74 with
    mk_menk_men / mek_menk_men / me_men_men, ST/ops/default_impls.py:72-105): per-token gathered weights,
    batched M=1 products, every intermediate materialised in h's dtype.  Weights are dense [E,N,K]/[E,K,N]
    tensors already in h's dtype (dequantize-then-cast).  Tokens are independent, so they are processed in
    chunks to bound the [chunk,k,N,K] gather.  x_rscale / z_rscale: reciprocal scales of fake-quantised activations
    (input of gate/up, input of down), None for none."""
    T = h.shape[0]
    if x_rscale is not None:
        h = fake_quant_per_tensor(h, x_rscale)
    out = torch.empty_like(h)
    for s in range(0, T, chunk):
        x = h[s : s + chunk]
        ex = experts[s : s + chunk]
        g = expert_gate[s : s + chunk]
        wg = w_gate[ex]  # [m,e,N,K]
        m_, e_, n_, k_ = wg.shape
        ffn_gate = _mm_rt(x.unsqueeze(1), wg.reshape(m_, e_ * n_, k_)).reshape(m_, e_, n_)
        ffn_gate = activation(ffn_gate)
        ffn_up = _mm_rt(x.unsqueeze(1), w_up[ex].reshape(m_, e_ * n_, k_)).reshape(m_, e_, n_)
        z = ffn_gate * ffn_up
        if z_rscale is not None:
            z = fake_quant_per_tensor(z, z_rscale)
        wd = w_down[ex]  # [m,e,K,N]
        down = _mm_rt(z.reshape(m_ * e_, 1, n_), wd.reshape(m_ * e_, k_, n_)).reshape(m_, e_, k_)
        down = (g.reshape(m_ * e_, 1, 1) * down.reshape(m_ * e_, k_, 1)).reshape(m_, e_, k_)  # "me,men->men"
        out[s : s + chunk] = torch.sum(down, dim=1)
    return out


def grouped_ffn_pairs(h, experts, w_gate, w_up, w_down, activation: Callable = F.silu, x_rscale=None, z_rscale=None):
    """Per (token, slot) pair the expert FFN output before the gate weighting, [T, k, K]: per expert, dense FFN on the
    rows routed to it (the shape of FFNMOE.forward, ST/layers/ffn_moe_block.py:120-127)."""
    T, K = h.shape
    k = experts.shape[1]
    E = w_gate.shape[0]
    down = torch.zeros(T, k, K, dtype=h.dtype)
    if x_rscale is not None:
        h = fake_quant_per_tensor(h, x_rscale)
    for e in range(E):
        t_idx, j_idx = torch.nonzero(experts == e, as_tuple=True)
        if t_idx.numel() == 0:
            continue
        x = h[t_idx]
        a = activation(_mm_rt(x, w_gate[e]))
        u = _mm_rt(x, w_up[e])
        z = a * u
        if z_rscale is not None:
            z = fake_quant_per_tensor(z, z_rscale)
        down[t_idx, j_idx] = _mm_rt(z, w_down[e])
    return down


def grouped_ffn_moe(h, experts, expert_gate, w_gate, w_up, w_down, activation: Callable = F.silu, x_rscale=None,
                    z_rscale=None):
    """PreGatherFFNMOE.forward, independent formulation: per-expert grouped FFN (grouped_ffn_pairs), then the gate
    weighting and the slot sum (ST/layers/ffn_moe_block.py:73-74)."""
    down = grouped_ffn_pairs(h, experts, w_gate, w_up, w_down, activation, x_rscale=x_rscale, z_rscale=z_rscale)
    down = expert_gate.unsqueeze(-1) * down
    return torch.sum(down, dim=1)


def moe_block(h, ffn_norm_w, w_router, w_gate, w_up, w_down, k: int, eps: float, activation: Callable = F.silu,
              out_norm_w: Optional[torch.Tensor] = None, formulation: str = "grouped", ordered_logits: bool = False,
              x_rscale=None, z_rscale=None):
    """MoeBlock.forward (ST/layers/mixture_of_experts_block.py:64-90).  h [B,S,K] or [T,K].
    Returns (y, idx, gate)."""
    shape = h.shape
    if ordered_logits:  # the kernels' documented summation orders: routing becomes reproducible bit for bit
        x = rms_norm_ordered(h.reshape(-1, shape[-1]), ffn_norm_w, eps)
        logits = router_logits_ordered(x, w_router)
    else:               # torch's own (unspecified) orders, as the reference runs
        x = rms_norm(h, ffn_norm_w, eps).reshape(-1, shape[-1])
        logits = router_logits(x, w_router)
    idx, gate, _ = route(logits, k)
    fn = grouped_ffn_moe if formulation == "grouped" else pre_gather_ffn_moe
    out = fn(x, idx, gate, w_gate, w_up, w_down, activation, x_rscale=x_rscale, z_rscale=z_rscale).reshape(shape)
    if out_norm_w is not None:
        out = rms_norm(out, out_norm_w, eps)
    return h + out, idx, gate


def mmt(a: torch.Tensor, w_dense: torch.Tensor) -> torch.Tensor:
    """matmul_default with transpose_rhs=True (ST/ops/default_impls.py:345-359): a @ w.to(a.dtype)^T."""
    return _mm_rt(a, w_dense.to(a.dtype))


def rel_l2(a: torch.Tensor, b: torch.Tensor) -> float:
    a64, b64 = a.double(), b.double()
    return float((a64 - b64).norm() / b64.norm().clamp_min(1e-30))
