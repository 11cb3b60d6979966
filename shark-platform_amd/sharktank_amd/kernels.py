"""The reference's three quantized-matmul custom ops as plain functions over planar planes, with the operand sets,
shapes and argument checks of `torch.ops.sharktank.*`:

* `mmt_block_scaled_q8(a, d, qs)`                      sharktank/sharktank/kernels/mmt_block_scaled_q8.py:20-75
* `mmt_block_scaled_offset_q4_unsigned(a, d, qs, m)`   sharktank/sharktank/kernels/mmt_block_scaled_offset_q4.py:25-100
* `einsum_2args_q4(a, d, qs, m, einsum_str)`           sharktank/sharktank/kernels/einsum_2args_q4.py:80-160

Each is `a @ dequant(b)^T` (or the einsum) on still-quantized planes, computed by the HIP library: weights dequantised in
fp16 as the layouts do, products accumulated in fp32, result in a's dtype.  Block size 32 with fp16 scales (GGUF Q8_0 /
Q4_1); other plane dtypes or block sizes raise NotImplementedError.  `einsum_2args_q4` takes the three einsum strings
of the mixture-of-experts layer; anything else raises NotImplementedError.  Shape mistakes raise RuntimeError with the
reference's messages (`torch._check`).
"""

from __future__ import annotations

import torch

from . import _hip

__all__ = ["einsum_2args_q4", "mmt_block_scaled_offset_q4_unsigned", "mmt_block_scaled_q8"]


def _need_fp16_planes(what: str, *planes):
    for p in planes:
        if p.dtype != torch.float16:
            raise NotImplementedError(f"{what}: the kernels take fp16 block scales / offsets (got {p.dtype})")


def mmt_block_scaled_q8(a: torch.Tensor, d: torch.Tensor, qs: torch.Tensor) -> torch.Tensor:
    *batch_dims, a_m, a_k = a.shape
    torch._check(a.dtype.is_floating_point, lambda: f"mmt_block_scaled_q8 arg 'a': Expected floating point (got {a.dtype})")
    torch._check(len(batch_dims) == 1, lambda: f"mmt_block_scaled_q8 arg 'a': Expected 3d tensor (got {a.shape})")
    torch._check(qs.dim() == 3 and qs.shape[1] * qs.shape[2] == a_k,
                 lambda: f"mmt_block_scaled_q8 arg 'qs': Incorrect shape (got {qs.shape})")
    qs_n, _, qs_bs = qs.shape
    torch._check(d.dim() == 3 and d.shape[1] * qs_bs == a_k and d.shape[2] == 1 and d.shape[0] == qs_n,
                 lambda: f"mmt_block_scaled_q8 arg 'd': Incorrect shape (got {d.shape})")
    if qs_bs != 32 or qs.dtype != torch.int8:
        raise NotImplementedError("mmt_block_scaled_q8: the kernels take int8 samples in blocks of 32")
    _need_fp16_planes("mmt_block_scaled_q8", d)
    w = _hip.DeviceWeight(_hip.W_Q8_0, 1, qs_n, a_k, qs.contiguous(), d.contiguous())
    return _hip.mmt(a, w)


def mmt_block_scaled_offset_q4_unsigned(a: torch.Tensor, d: torch.Tensor, qs: torch.Tensor, m: torch.Tensor) -> torch.Tensor:
    name = "mmt_block_scaled_offset_q4_unsigned"
    *a_batch, a_m, a_k = a.shape
    torch._check(a.dtype.is_floating_point, lambda: f"{name} arg 'a': Expected floating point (got {a.dtype})")
    torch._check(len(a_batch) == 1, lambda: f"{name} arg 'a': Expected 3d tensor (got {a.shape})")
    *qs_batch, qs_n, qs_group0, qs_bs_div_2 = qs.shape
    torch._check((len(qs_batch) == 0 or (len(qs_batch) == 1 and list(qs_batch) == list(a_batch))) and qs_group0 * qs_bs_div_2 * 2 == a_k,
                 lambda: f"{name} arg 'qs': Incorrect shape (got {qs.shape})")
    block_size = qs_bs_div_2 * 2
    *d_batch, d_n, d_group0, d_one = d.shape
    torch._check(list(d_batch) == list(qs_batch) and d_group0 * block_size == a_k and d_one == 1 and d_n == qs_n,
                 lambda: f"{name} arg 'd': Incorrect shape (got {d.shape})")
    *m_batch, m_n, m_group0, m_one = m.shape
    torch._check(list(m_batch) == list(qs_batch) and m_group0 * block_size == a_k and m_one == 1 and m_n == qs_n,
                 lambda: f"{name} arg 'm': Incorrect shape (got {m.shape})")
    if block_size != 32 or qs.dtype != torch.uint8:
        raise NotImplementedError(f"{name}: the kernels take packed uint8 nibbles in blocks of 32")
    _need_fp16_planes(name, d, m)
    if not qs_batch:
        w = _hip.DeviceWeight(_hip.W_Q4_1, 1, qs_n, a_k, qs.contiguous(), d.contiguous(), m.contiguous())
        return _hip.mmt(a, w)
    # one weight matrix per batch entry: a grouped product with the batch entries as "experts", a_m rows each
    b = a_batch[0]
    w = _hip.DeviceWeight(_hip.W_Q4_1, b, qs_n, a_k, qs.contiguous(), d.contiguous(), m.contiguous())
    offsets = (torch.arange(b + 1, dtype=torch.int32, device=a.device) * a_m).contiguous()
    perm = torch.arange(b * a_m, dtype=torch.int32, device=a.device)
    out = _hip.grouped_mmt(a.reshape(b * a_m, a_k), w, offsets, perm, b * a_m, 1, a_per_pair=True)
    return out.reshape(b, a_m, qs_n)


def einsum_2args_q4(a: torch.Tensor, d: torch.Tensor, qs: torch.Tensor, m: torch.Tensor, einsum_str: str) -> torch.Tensor:
    name = "einsum_2args_q4"
    torch._check(a.dtype.is_floating_point, lambda: f"{name} arg 'a': Expected floating point (got {a.dtype})")
    *qs_dims, qs_group0, qs_bs_div_2 = qs.shape
    *d_dims, d_group0, d_one = d.shape
    torch._check(d_group0 == qs_group0 and d_one == 1 and len(d_dims) == len(qs_dims),
                 lambda: f"{name} arg 'd': Incorrect shape (got {d.shape})")
    *m_dims, m_group0, m_one = m.shape
    torch._check(m.dtype == d.dtype and len(m_dims) == len(qs_dims), lambda: f"{name} arg 'm': Incorrect dtype (got {m.dtype})")
    torch._check(einsum_str.count(",") == 1 and einsum_str.count("->") == 1, lambda: f"{name} arg 'es': Incorrect einsum string (got {einsum_str})")
    if qs_bs_div_2 != 16 or qs.dtype != torch.uint8:
        raise NotImplementedError(f"{name}: the kernels take packed uint8 nibbles in blocks of 32")
    _need_fp16_planes(name, d, m)
    es = einsum_str.replace(" ", "")
    if es in ("mk,menk->men", "mek,menk->men"):
        # every (m, e) pair has its own [N, K] matrix: a grouped product with one row per "expert"
        M, E, N = (int(s) for s in qs_dims)
        K = qs_group0 * 32
        per_pair = es.startswith("mek")
        torch._check(tuple(a.shape) == ((M, E, K) if per_pair else (M, K)), lambda: f"{name} arg 'a': Incorrect shape (got {a.shape})")
        w = _hip.DeviceWeight(_hip.W_Q4_1, M * E, N, K, qs.contiguous(), d.contiguous(), m.contiguous())
        offsets = torch.arange(M * E + 1, dtype=torch.int32, device=a.device)
        perm = torch.arange(M * E, dtype=torch.int32, device=a.device)
        lhs = a.reshape(M * E, K) if per_pair else a
        return _hip.grouped_mmt(lhs, w, offsets, perm, M, E, a_per_pair=per_pair)
    if es == "me,men->men":
        M, E = (int(s) for s in qs_dims)
        N = qs_group0 * 32
        torch._check(tuple(a.shape) == (M, E), lambda: f"{name} arg 'a': Incorrect shape (got {a.shape})")
        # dequantised in the scales' dtype like the matmul kernels (and the layouts' default), then cast
        b = _hip.dequant_block_scaled_i4(d, qs, m, False, None).reshape(M, E, N).to(a.dtype)
        return _hip.scale_rows(b, a)
    raise NotImplementedError(f"{name}: einsum string {einsum_str!r} has no kernel (have mk,menk->men / mek,menk->men / me,men->men)")
