"""Parity of each HIP entry point against the CPU oracle (through the C ABI via the ctypes binding)."""

import pytest
import torch
import torch.nn.functional as F

from oracle import moe_oracle as O
import moe_cases as MC

pytestmark = pytest.mark.gpu


def _hip():
    from sharktank_amd import _hip

    return _hip


@pytest.mark.parametrize("out_dtype", [None, torch.float32, torch.bfloat16])
def test_dequant_q8_0_bit_exact(device, out_dtype):
    g = torch.Generator().manual_seed(1)
    w = torch.randn(64, 256, generator=g) * 0.02
    w[0, :32] = 0.0  # an all-zero block (d = 0)
    w[1, :32] *= 1e-4  # subnormal fp16 products
    d, qs = O.quantize_q8_0(w)
    want = O.dequant_block_scaled(d, qs, dtype=out_dtype)
    got = _hip().dequant_block_scaled(d.to(device), qs.to(device), None, out_dtype).cpu()
    assert got.dtype == want.dtype
    assert torch.equal(got.view(torch.int16 if got.element_size() == 2 else torch.int32),
                       want.view(torch.int16 if want.element_size() == 2 else torch.int32))


@pytest.mark.parametrize("out_dtype", [None, torch.float32, torch.bfloat16])
@pytest.mark.parametrize("signed", [False, True])
def test_dequant_q4_1_bit_exact(device, out_dtype, signed):
    g = torch.Generator().manual_seed(2)
    w = torch.randn(48, 128, generator=g) * 0.02
    d, m, qs = O.quantize_q4_1(w)
    want = O.dequant_block_scaled_i4(d, qs, m, signed=signed, dtype=out_dtype)
    got = _hip().dequant_block_scaled_i4(d.to(device), qs.to(device), m.to(device), signed, out_dtype).cpu()
    assert got.dtype == want.dtype
    view = torch.int16 if got.element_size() == 2 else torch.int32
    assert torch.equal(got.view(view), want.view(view))


def test_promote_i4_known_answer(device):
    packed = torch.tensor([[0x10, 0x32, 0x54, 0x76, 0x98, 0xBA, 0xDC, 0xFE]], dtype=torch.uint8)
    u = _hip().promote_i4_block(packed.to(device), False).cpu()
    s = _hip().promote_i4_block(packed.to(device), True).cpu()
    assert u.dtype == torch.uint8 and s.dtype == torch.int8
    assert u.tolist() == [list(range(16))]
    assert s.tolist() == [[0, 1, 2, 3, 4, 5, 6, 7, -8, -7, -6, -5, -4, -3, -2, -1]]


def test_dequant_tensor_scaled_known_answer(device):
    # the reference's own vector: sharktank/tests/types/layouts_test.py:107-125
    got = _hip().dequant_tensor_scaled(
        torch.tensor([2.0, 3.0, 4.0], dtype=torch.float16, device=device),
        torch.tensor(2.0, dtype=torch.float32, device=device),
        torch.tensor(5.0, dtype=torch.float32, device=device), torch.float32).cpu()
    assert got.tolist() == [-6.0, -4.0, -2.0]


def test_dequant_fp8_bit_exact(device):
    qs = torch.arange(256, dtype=torch.uint8).view(torch.float8_e4m3fn).repeat(4)
    d = torch.tensor(0.0118, dtype=torch.float32)
    for out_dtype in (torch.float32, torch.float16, torch.bfloat16):
        want = O.dequant_tensor_scaled(d, qs, dtype=out_dtype)
        got = _hip().dequant_tensor_scaled(qs.to(device), d.to(device), None, out_dtype).cpu()
        ok = (got == want) | (got.isnan() & want.isnan())
        assert bool(ok.all()), out_dtype


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16, torch.float32])
def test_quantize_fp8_bit_exact(device, dtype):
    g = torch.Generator().manual_seed(3)
    x = (torch.randn(4096, generator=g) * 3).to(dtype)
    x[:4] = torch.tensor([1000.0, -1000.0, 0.0, 448.0]).to(dtype)
    rscale = torch.tensor(0.0118, dtype=torch.float32)
    want, _, _ = O.static_quantize_per_tensor(x, rscale, torch.float8_e4m3fn)
    got = _hip().quantize_fp8(x.to(device), rscale.to(device)).cpu()
    assert torch.equal(got.view(torch.uint8), want.view(torch.uint8))


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16, torch.float32])
def test_fake_quant_fp8_bit_exact(device, dtype):
    g = torch.Generator().manual_seed(5)
    x = (torch.randn(4096, generator=g) * 3).to(dtype)
    x[:4] = torch.tensor([1000.0, -1000.0, 0.0, 448.0]).to(dtype)
    rscale = torch.tensor(0.0118, dtype=torch.float32)
    want = O.fake_quant_per_tensor(x, rscale)
    got = _hip().fake_quant_fp8(x.to(device), rscale.to(device)).cpu()
    assert torch.equal(got, want)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16, torch.float32])
def test_rms_norm(device, dtype):
    g = torch.Generator().manual_seed(4)
    x = torch.randn(37, 1024, generator=g).to(dtype)
    w = torch.ones(1024) + 0.1 * torch.randn(1024, generator=g)
    want = O.rms_norm(x, w, 1e-5)
    got = _hip().rms_norm(x.to(device), w.to(device), 1e-5).cpu()
    assert O.rel_l2(got, want) < (1e-6 if dtype == torch.float32 else 1e-3)
    # bit-exact against the restatement with the documented summation order (the router's input must be reproducible)
    ordered = O.rms_norm_ordered(x, w, 1e-5)
    view = torch.int32 if dtype == torch.float32 else torch.int16
    assert torch.equal(got.view(view), ordered.view(view))


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16, torch.float32])
@pytest.mark.parametrize("T,K,E,k", [(64, 512, 8, 2), (33, 4096, 8, 2), (5, 1000 * 8, 16, 4), (1, 64, 3, 3),
                                     # more than 512 tokens (launches that fill the chip several times over), rows longer
                                     # than the per-token LDS row of the one-workgroup-per-token kernel
                                     (700, 4096, 8, 2), (1100, 6144, 8, 2), (600, 1024, 16, 4), (512 * 66 + 5, 512, 8, 2),
                                     (520, 8192 + 512, 8, 2)])
def test_router_bit_exact(device, dtype, T, K, E, k):
    g = torch.Generator().manual_seed(5)
    x = torch.randn(T, K, generator=g).to(dtype)
    wr = (torch.randn(E, K, generator=g) * 0.02)
    idx, gate, logits = _hip().router_topk(x.to(device), wr.to(dtype).to(device), k, want_logits=True, index_dtype=torch.int64)
    want_logits = O.router_logits_ordered(x, wr)
    view = torch.int16 if dtype != torch.float32 else torch.int32
    assert torch.equal(logits.cpu().view(view), want_logits.view(view)), "logit bits differ from the documented order"
    want_idx, want_gate, _ = O.route(want_logits, k)
    assert idx.dtype == torch.int64
    assert torch.equal(idx.cpu(), want_idx)
    assert O.rel_l2(gate.cpu(), want_gate) < (1e-6 if dtype == torch.float32 else 2e-3)
    # against torch's own summation order: indices agree except where a logit sits on a rounding boundary
    ref_idx, _, _ = O.route(O.router_logits(x, wr), k)
    mism = int((ref_idx != want_idx).any(dim=1).sum())
    assert mism <= max(1, T // 100), f"{mism} of {T} tokens route differently from torch.matmul logits"


@pytest.mark.parametrize("T", [3, 700])
def test_router_fp16_subnormal_and_large_operands(device, T):
    """Subnormal, tiny and large fp16 operands: the logits' bits must still be the oracle's (exact conversions to fp32,
    products and sums rounded one by one in the documented order)."""
    g = torch.Generator().manual_seed(11)
    K, E, k = 1024, 8, 2
    def operands(rows, scale):
        v = torch.randn(rows, K, generator=g) * scale
        sub = torch.randint(1, 1024, (rows, K), generator=g).to(torch.int16).view(torch.float16).float()  # fp16 subnormals
        sub = sub * torch.where(torch.rand(rows, K, generator=g) < 0.5, -1.0, 1.0)
        kind = torch.randint(0, 4, (rows, K), generator=g)
        v = torch.where(kind == 0, sub, v)
        v = torch.where(kind == 1, v * 1e-4, v)
        v = torch.where(kind == 2, v * 30.0, v)
        return v.to(torch.float16)
    x, wr = operands(T, 1.0), operands(E, 0.02)
    assert bool((x.float().abs() < 6.2e-5).any()) and bool(torch.isfinite(x.float()).all())
    idx, gate, logits = _hip().router_topk(x.to(device), wr.to(device), k, want_logits=True, index_dtype=torch.int64)
    want_logits = O.router_logits_ordered(x, wr.float())
    assert bool(torch.isfinite(want_logits.float()).all())
    assert torch.equal(logits.cpu().view(torch.int16), want_logits.view(torch.int16))
    # Indices: logits of this size put some probabilities within an ulp of each other, where the exponential of the device
    # and the host's may order them differently (test_router_distinct_logits_with_equal_probabilities covers exact ties).
    # Every row whose k + 1 largest probabilities are at least 8 ulp apart from each other must route exactly as the oracle.
    want_idx, want_gate, probs = O.route(want_logits, k)
    top = torch.sort(probs, dim=1, descending=True).values[:, : k + 1]
    clear = ((top[:, :-1] - top[:, 1:]) > 8 * torch.finfo(torch.float32).eps * top[:, :-1]).all(dim=1)
    # (logits this large saturate the softmax of many rows: their lower probabilities are zero or equal)
    print(f"{int(clear.sum())} of {T} rows have separated probabilities")
    assert int(clear.sum()) >= max(1, T // 10), f"only {int(clear.sum())} of {T} rows have separated probabilities"
    assert torch.equal(idx.cpu()[clear], want_idx[clear])
    assert O.rel_l2(gate.cpu()[clear], want_gate[clear]) < 2e-3


def test_router_ties_lower_index_first(device):
    # identical router rows give identical logits: ties must resolve toward the lower expert index
    x = torch.randn(16, 64, generator=torch.Generator().manual_seed(6)).to(torch.float16)
    row = torch.randn(64, generator=torch.Generator().manual_seed(7)) * 0.02
    wr = torch.stack([row, row * 0.5, row, row * 0.5, row, -row, row * 0.25, row]).to(torch.float16)
    idx, gate, logits = _hip().router_topk(x.to(device), wr.to(device), 3, want_logits=True)
    want_idx, want_gate, _ = O.route(O.router_logits_ordered(x, wr), 3)
    assert torch.equal(idx.cpu().long(), want_idx)
    lg = logits.cpu().float()
    pos = lg[:, 0] > 0
    assert torch.equal(idx.cpu()[pos].long(), torch.tensor([[0, 2, 4]]).expand(int(pos.sum()), 3))


@pytest.mark.parametrize("K", [64, 16384])  # one workgroup per token / one wavefront per token (long rows)
def test_router_distinct_logits_with_equal_probabilities(device, K):
    """The reference ranks the fp32 softmax probabilities, not the logits (mixture_of_experts_block.py:75-78).  Two fp32
    logits one ulp apart, 2^-10 and the next number up, have the same probability: exp(-2^-33) rounds to 1.  For the
    reference that is a tie, which the contract resolves toward the lower expert index, although the higher index holds
    the larger logit.  The input row is a unit vector, so logit e is exactly the router's entry [e, 0]."""
    E, k = 8, 2
    a = torch.tensor(2.0 ** -10, dtype=torch.float32)
    b = torch.nextafter(a, torch.tensor(1.0))
    assert b > a and torch.exp(a - b) == 1.0
    x = torch.zeros(4, K, dtype=torch.float32)
    x[:, 0] = 1.0
    wr = torch.full((E, K), 0.0, dtype=torch.float32)
    wr[:, 0] = -1.0
    wr[3, 0], wr[5, 0] = a, b  # expert 5 has the larger logit, expert 3 the lower index
    wr[6, 0] = a - 0.25
    idx, gate, logits = _hip().router_topk(x.to(device), wr.to(device), k, want_logits=True)
    assert torch.equal(logits.cpu()[0], wr[:, 0]), "logits are not the router's first column"
    want_idx, want_gate, probs = O.route(O.router_logits_ordered(x, wr), k)
    assert probs[0, 3] == probs[0, 5]
    assert want_idx[0].tolist() == [3, 5]
    assert torch.equal(idx.cpu().long(), want_idx)
    assert torch.equal(gate.cpu(), torch.full((4, 2), 0.5))
    # a third slot takes the next probability down
    idx3, _, _ = _hip().router_topk(x.to(device), wr.to(device), 3, want_logits=True)
    assert idx3.cpu()[0].tolist() == [3, 5, 6]


@pytest.mark.parametrize("T,k,E", [(1, 2, 8), (32, 2, 8), (2048, 2, 8), (3000, 4, 64), (7, 1, 1),
                                   # either side of the limits of the kernel that keeps a launch's pairs in registers
                                   # (8192 pairs, 64 experts), partial last chunks, one pair per token
                                   (4096, 2, 8), (4097, 2, 8), (1023, 3, 64), (600, 2, 65), (8192, 1, 16), (513, 2, 3),
                                   # either side of the one-wavefront kernel's limits (64 pairs, 64 experts)
                                   (32, 2, 64), (16, 4, 64), (33, 2, 8), (8, 8, 8), (21, 3, 5), (64, 1, 65)])
def test_dispatch_bit_exact(device, T, k, E):
    g = torch.Generator().manual_seed(8)
    idx = torch.stack([torch.randperm(E, generator=g)[:k] for _ in range(T)]).to(torch.int32)
    counts, offsets, perm, inv = _hip().dispatch_build(idx.to(device), E)
    wc, wo, wp, wi = O.dispatch_permutation(idx, E)
    assert torch.equal(counts.cpu(), wc) and torch.equal(offsets.cpu(), wo)
    assert torch.equal(perm.cpu(), wp) and torch.equal(inv.cpu(), wi)


def test_dispatch_skewed_and_empty_experts(device):
    idx = torch.zeros(500, 2, dtype=torch.int32)
    idx[:, 1] = 5  # experts 1-4, 6, 7 receive nothing
    counts, offsets, perm, inv = _hip().dispatch_build(idx.to(device), 8)
    wc, wo, wp, wi = O.dispatch_permutation(idx, 8)
    assert torch.equal(counts.cpu(), wc) and torch.equal(offsets.cpu(), wo)
    assert torch.equal(perm.cpu(), wp) and torch.equal(inv.cpu(), wi)


def _ffn_parity(device, case, variant, tol):
    hip = _hip()
    from sharktank_amd.ops import device_weight

    case = MC.build(case)
    x = case.planes["h"]
    g = torch.Generator().manual_seed(case.seed + 100)
    idx = torch.stack([torch.randperm(case.E, generator=g)[: case.k] for _ in range(case.T)])
    gate = torch.rand(case.T, case.k, generator=g)
    gate = (gate / gate.sum(-1, keepdim=True)).to(case.dtype)
    wg, wu, wd = MC.dense_weights(case)
    want = O.grouped_ffn_moe(x, idx, gate, wg, wu, wd, case.activation)
    E, N, K = case.E, case.N, case.K
    dws = [device_weight(MC.to_inference_tensor(case.fmt, case.planes[n], shp, n, device), stacked=True)
           for n, shp in (("gate", [E, N, K]), ("up", [E, N, K]), ("down", [E, K, N]))]
    _, offsets, perm, inv = hip.dispatch_build(idx.to(torch.int32).to(device), E)
    act = hip.ACT_SILU if case.act == "silu" else hip.ACT_GELU_ERF
    y = hip.grouped_ffn(x.to(device), dws[0], dws[1], dws[2], act, offsets, perm, case.k, variant=variant)
    got = hip.combine(y, gate.to(device), inv, case.T, case.k).cpu()
    err = O.rel_l2(got, want)
    assert err < tol, f"rel-L2 {err:.3e} >= {tol}"
    return got


@pytest.mark.parametrize("fmt", ["dense", "q8_0", "q4_1", "fp8"])
@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16])
def test_ffn_generic_kernel(device, fmt, dtype):
    tol = 1e-5 if dtype == torch.float32 else (1e-3 if dtype == torch.float16 else 8e-3)
    _ffn_parity(device, MC.Case(T=24, K=128, N=256, fmt=fmt, dtype=dtype, seed=11), 1, tol)


@pytest.mark.parametrize("fmt", ["dense", "q8_0", "q4_1", "fp8"])
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("act", ["silu", "gelu"])
def test_ffn_mfma_tile_kernel(device, fmt, dtype, act):
    tol = 1e-3 if dtype == torch.float16 else 8e-3
    got = _ffn_parity(device, MC.Case(T=200, K=256, N=384, fmt=fmt, dtype=dtype, act=act, seed=12), 2, tol)
    # and against the independent vector-ALU kernel
    got2 = _ffn_parity(device, MC.Case(T=200, K=256, N=384, fmt=fmt, dtype=dtype, act=act, seed=12), 1, tol)
    assert O.rel_l2(got, got2) < tol


def test_combine_with_output_norm_and_residual(device):
    hip = _hip()
    g = torch.Generator().manual_seed(13)
    T, k, K = 19, 2, 512
    for dtype in (torch.float16, torch.bfloat16, torch.float32):
        y = torch.randn(T * k, K, generator=g).to(dtype)
        gate = torch.rand(T, k, generator=g).to(dtype)
        inv = torch.randperm(T * k, generator=g).to(torch.int32)
        h = torch.randn(T, K, generator=g).to(dtype)
        w = torch.ones(K) + 0.1 * torch.randn(K, generator=g)
        down = y[inv.long()].reshape(T, k, K)
        o = torch.sum(gate.unsqueeze(-1) * down, dim=1)
        want_plain = o
        want_full = h + O.rms_norm(o, w, 1e-5)
        got_plain = hip.combine(y.to(device), gate.to(device), inv.to(device), T, k).cpu()
        got_full = hip.combine(y.to(device), gate.to(device), inv.to(device), T, k, out_norm_w=w.to(device), eps=1e-5,
                               residual=h.to(device)).cpu()
        tol = 1e-6 if dtype == torch.float32 else 2e-3
        if dtype == torch.float16:
            assert torch.equal(got_plain, want_plain)  # products and the fp32 slot sum are exact: one rounding each
        assert O.rel_l2(got_plain, want_plain) < tol
        assert O.rel_l2(got_full, want_full) < tol


@pytest.mark.parametrize("fmt", ["q8_0", "q4_1", "fp8", "dense"])
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("T", [1, 7, 16, 32, 45])
def test_ffn_skinny_kernel(device, fmt, dtype, T):
    """The decode kernel: 1, <16, =16, 17..32 and >32 rows per expert (the last takes two passes)."""
    tol = 1e-3 if dtype == torch.float16 else 8e-3
    act = "gelu" if T == 7 else "silu"
    _ffn_parity(device, MC.Case(T=T, K=512, N=768, E=4 if T == 45 else 8, fmt=fmt, dtype=dtype, act=act, seed=40 + T), 3, tol)


@pytest.mark.parametrize("fmt", ["q8_0", "q4_1", "fp8"])
def test_prepack_round_trip_bit_exact(device, fmt):
    from sharktank_amd.ops import device_weight

    case = MC.build(MC.Case(T=4, K=512, N=256, E=3, fmt=fmt, seed=50))
    it = MC.to_inference_tensor(fmt, case.planes["gate"], [3, 256, 512], "w", device)
    planar = device_weight(it, stacked=True)
    packed = planar.prepack()
    assert packed.is_packed and packed.nbytes() == planar.nbytes()
    back = packed.unpack()
    for a, b in zip(planar.keep, back.keep):
        if a is not None:
            assert torch.equal(a.view(torch.uint8), b.view(torch.uint8))
    if fmt != "fp8":
        assert not torch.equal(planar.keep[0].view(torch.uint8), packed.keep[0].view(torch.uint8))


def test_prepack_layout_definition(device):
    """Spot-checks the documented order: lane 16*g + n of block (row tile rt, k block kb) holds row 16*rt+n,
    k = 64*kb + 16*g .. +15; scales of 8 consecutive blocks of a row are contiguous."""
    from sharktank_amd.ops import device_weight
    from sharktank_amd import types as ST

    E, N, K = 2, 32, 512
    qs = torch.arange(E * N * K, dtype=torch.int32).remainder(251).to(torch.int8).reshape(E, N, K // 32, 32)
    d = torch.arange(E * N * K // 32, dtype=torch.float32).reshape(E, N, K // 32, 1).to(torch.float16)
    it = ST.PlanarQuantizedTensor(shape=[E, N, K], layout=ST.BlockScaledLayout([E, N, K], d.to(device), qs.to(device)))
    packed = device_weight(it, stacked=True, prepack=True)
    pq = packed.keep[0].cpu().reshape(-1)
    pd = packed.keep[1].cpu().reshape(-1)
    flat = qs.reshape(E * N, K)
    dflat = d.reshape(E * N, K // 32)
    for rt, kb, g, n in [(0, 0, 0, 0), (1, 3, 2, 5), (3, 7, 3, 15), (2, 4, 1, 9)]:
        off = ((rt * (K // 64) + kb) * 64 + g * 16 + n) * 16
        assert torch.equal(pq[off : off + 16], flat[rt * 16 + n, kb * 64 + g * 16 : kb * 64 + g * 16 + 16])
    for rt, c, n in [(0, 0, 0), (3, 1, 7), (1, 1, 15)]:
        off = ((rt * (K // 256) + c) * 16 + n) * 8
        assert torch.equal(pd[off : off + 8], dflat[rt * 16 + n, c * 8 : c * 8 + 8])


@pytest.mark.parametrize("fmt", ["q8_0", "q4_1", "fp8"])
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("variant,T", [(1, 9), (2, 150), (3, 20)])
def test_packed_weights_match_planar(device, fmt, dtype, variant, T):
    """Every kernel family gives the same bits from packed planes as from planar planes."""
    hip = _hip()
    from sharktank_amd.ops import device_weight

    case = MC.build(MC.Case(T=T, K=512, N=256, fmt=fmt, dtype=dtype, seed=51))
    E, N, K = case.E, case.N, case.K
    g = torch.Generator().manual_seed(3)
    idx = torch.stack([torch.randperm(E, generator=g)[: case.k] for _ in range(T)]).to(torch.int32)
    _, offsets, perm, inv = hip.dispatch_build(idx.to(device), E)
    outs = []
    for prepack in (False, True):
        dws = [device_weight(MC.to_inference_tensor(fmt, case.planes[n], shp, n, device), stacked=True, prepack=prepack)
               for n, shp in (("gate", [E, N, K]), ("up", [E, N, K]), ("down", [E, K, N]))]
        assert dws[0].is_packed == prepack
        outs.append(hip.grouped_ffn(case.planes["h"].to(device), dws[0], dws[1], dws[2], hip.ACT_SILU, offsets, perm, case.k,
                                    variant=variant).cpu())
    assert torch.equal(outs[0].view(torch.int16), outs[1].view(torch.int16))


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("T,E,act", [(700, 8, "silu"), (700, 2, "gelu"), (130, 1, "silu")])
def test_ffn_mfma_big_kernel(device, dtype, T, E, act):
    """The 256 x 256 prefill kernels (packed Q8_0; one with every wavefront producing and consuming, one with
    specialised producer and consumer wavefronts): ragged tiles, several token tiles per expert, one expert."""
    hip = _hip()
    from sharktank_amd.ops import device_weight

    tol = 1e-3 if dtype == torch.float16 else 8e-3
    case = MC.build(MC.Case(T=T, K=512, N=512, E=E, k=min(2, E), fmt="q8_0", dtype=dtype, act=act, seed=60))
    K, N = case.K, case.N
    g = torch.Generator().manual_seed(61)
    idx = torch.stack([torch.randperm(E, generator=g)[: case.k] for _ in range(T)])
    gate = torch.rand(T, case.k, generator=g)
    gate = (gate / gate.sum(-1, keepdim=True)).to(dtype)
    wg, wu, wd = MC.dense_weights(case)
    want = O.grouped_ffn_moe(case.planes["h"], idx, gate, wg, wu, wd, case.activation)
    dws = [device_weight(MC.to_inference_tensor("q8_0", case.planes[n], shp, n, device), stacked=True, prepack=True)
           for n, shp in (("gate", [E, N, K]), ("up", [E, N, K]), ("down", [E, K, N]))]
    _, offsets, perm, inv = hip.dispatch_build(idx.to(torch.int32).to(device), E)
    act_e = hip.ACT_SILU if act == "silu" else hip.ACT_GELU_ERF
    outs = {}
    for variant in (hip.VARIANT_MFMA_BIG, hip.VARIANT_MFMA_WS, hip.VARIANT_MFMA_TILE):
        y = hip.grouped_ffn(case.planes["h"].to(device), dws[0], dws[1], dws[2], act_e, offsets, perm, case.k, variant=variant)
        outs[variant] = hip.combine(y, gate.to(device), inv, T, case.k).cpu()
        assert O.rel_l2(outs[variant], want) < tol
    assert O.rel_l2(outs[hip.VARIANT_MFMA_BIG], outs[hip.VARIANT_MFMA_TILE]) < tol
    # both 256 x 256 kernels accumulate every output in the same order, except that the specialised one splits the
    # reduction of the last units of a launch into fp32 partial sums (a different rounding of a few sums)
    assert O.rel_l2(outs[hip.VARIANT_MFMA_BIG], outs[hip.VARIANT_MFMA_WS]) < tol / 4


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("fmt", ["q4_1", "fp8"])
def test_ffn_mfma_ws_kernel_formats(device, dtype, fmt):
    """The specialised-wavefront prefill kernel on packed Q4_1 and fp8 weights: same values as the 128 x 128 tile
    kernel (both dequantise every weight to the activation dtype before the product) and the oracle."""
    hip = _hip()
    from sharktank_amd.ops import device_weight

    T, E = 600, 4
    tol = 1e-3 if dtype == torch.float16 else 8e-3
    case = MC.build(MC.Case(T=T, K=512, N=768, E=E, k=2, fmt=fmt, dtype=dtype, seed=62))
    K, N = case.K, case.N
    g = torch.Generator().manual_seed(63)
    idx = torch.stack([torch.randperm(E, generator=g)[: case.k] for _ in range(T)])
    gate = torch.rand(T, case.k, generator=g)
    gate = (gate / gate.sum(-1, keepdim=True)).to(dtype)
    wg, wu, wd = MC.dense_weights(case)
    want = O.grouped_ffn_moe(case.planes["h"], idx, gate, wg, wu, wd, case.activation)
    dws = [device_weight(MC.to_inference_tensor(fmt, case.planes[n], shp, n, device), stacked=True, prepack=True)
           for n, shp in (("gate", [E, N, K]), ("up", [E, N, K]), ("down", [E, K, N]))]
    assert all(w.is_packed for w in dws)
    _, offsets, perm, inv = hip.dispatch_build(idx.to(torch.int32).to(device), E)
    outs = {}
    for variant in (hip.VARIANT_MFMA_WS, hip.VARIANT_MFMA_TILE):
        y = hip.grouped_ffn(case.planes["h"].to(device), dws[0], dws[1], dws[2], hip.ACT_SILU, offsets, perm, case.k, variant=variant)
        outs[variant] = hip.combine(y, gate.to(device), inv, T, case.k).cpu()
        assert O.rel_l2(outs[variant], want) < tol
    assert O.rel_l2(outs[hip.VARIANT_MFMA_WS], outs[hip.VARIANT_MFMA_TILE]) < tol


def _raw_blocks(fmt: str, shape, seed: int):
    """Random bit patterns in ggml block structs: the scales are arbitrary fp16 bits (NaNs included), so a conversion
    anywhere on the way would show."""
    g = torch.Generator().manual_seed(seed)
    nb = shape[0] * shape[1] * shape[2] // 32
    return torch.randint(0, 256, (nb * (34 if fmt == "q8_0" else 20),), dtype=torch.uint8, generator=g)


@pytest.mark.parametrize("fmt", ["q8_0", "q4_1"])
@pytest.mark.parametrize("shape", [(3, 64, 512), (1, 16, 256), (2, 40, 96)])
def test_gguf_raw_blocks_to_planes(device, fmt, shape):
    """stmoe_gguf_ingest: raw ggml blocks -> the reference's planar planes, bit for bit, and -> the streaming order
    directly, identical to stmoe_prepack of the planar planes."""
    H = _hip()
    raw = _raw_blocks(fmt, shape, 90 + shape[1])
    E, rows, cols = shape
    gt = H.GGUF_Q8_0 if fmt == "q8_0" else H.GGUF_Q4_1
    planar = H.gguf_ingest(raw.to(device), gt, E, rows, cols, packed=False)
    qs, d, m = planar.keep
    if fmt == "q8_0":
        want_d, want_qs = O.q8_0_unpack(raw, list(shape))
        assert m is None
    else:
        want_d, want_m, want_qs = O.q4_1_unpack(raw, list(shape))
        assert torch.equal(m.cpu().view(torch.int16), want_m.contiguous().view(torch.int16))
    assert torch.equal(d.cpu().view(torch.int16), want_d.contiguous().view(torch.int16))
    assert torch.equal(qs.cpu().view(torch.uint8), want_qs.contiguous().view(torch.uint8))
    if rows % 16 == 0 and cols % 256 == 0:
        # random bit patterns as block scales: the byte permutation is what is tested, not the scale limit of the kernels
        direct = H.gguf_ingest(raw.to(device), gt, E, rows, cols, packed=True, check_scales=False)
        via = planar.prepack()
        for a, b in zip(direct.keep, via.keep):
            assert (a is None) == (b is None)
            if a is not None:
                assert torch.equal(a.view(torch.uint8), b.view(torch.uint8))
        back = direct.unpack()
        for a, b in zip(back.keep, planar.keep):
            if a is not None:
                assert torch.equal(a.view(torch.uint8), b.view(torch.uint8))
    else:
        with pytest.raises(RuntimeError, match="rows % 16 == 0"):
            H.gguf_ingest(raw.to(device), gt, E, rows, cols, packed=True)


@pytest.mark.parametrize("fmt", ["q8_0", "q4_1"])
def test_layer_from_gguf_raw_blocks(device, fmt):
    """A MoeBlock whose expert weights are raw ggml blocks on the device gives the same output, bit for bit, as the
    block built from the planar planes of the same blocks."""
    import moe_cases as MC
    from sharktank_amd import types as ST
    from sharktank_amd.layers import MoeBlock

    case = MC.build(MC.Case(T=24, K=256, N=512, fmt=fmt, dtype=torch.float16, seed=95))
    theta = MC.make_theta(case, device)
    ref_block = MoeBlock(theta, expert_count=case.E, expert_used_count=case.k, rms_epsilon=case.eps)
    tree = dict(theta.flatten())
    for name, key in (("ffn_gate_exps", "gate"), ("ffn_up_exps", "up"), ("ffn_down_exps", "down")):
        p = case.planes[key]
        shape = list(tree[f"{name}.weight"].shape)
        if fmt == "q8_0":
            raw = torch.cat([p["d"].view(torch.uint8).reshape(-1, 2), p["qs"].view(torch.uint8).reshape(-1, 32)], dim=1).reshape(-1)
            tree[f"{name}.weight"] = ST.Q8_0(raw=raw.to(device), shape=shape, name=f"{name}.weight")
        else:
            ggml = O.interleave_linear_i4_block(p["qs"]).reshape(-1, 16)
            raw = torch.cat([p["d"].view(torch.uint8).reshape(-1, 2), p["m"].view(torch.uint8).reshape(-1, 2), ggml], dim=1).reshape(-1)
            tree[f"{name}.weight"] = ST.Q4_1(raw=raw.to(device), shape=shape, name=f"{name}.weight")
    raw_block = MoeBlock(ST.Theta(tree), expert_count=case.E, expert_used_count=case.k, rms_epsilon=case.eps)
    h = case.planes["h"].to(device).reshape(1, case.T, case.K)
    assert torch.equal(raw_block(h), ref_block(h))
    assert raw_block.experts.device_weights()[0].is_packed
    # to_planar() of device-resident raw blocks equals the view-based unpack of the same blocks on the host
    t = tree["ffn_gate_exps.weight"]
    planar = t.to_planar().unpack()
    host = type(t)(raw=t.raw.cpu(), shape=t.shape).unpack()
    assert torch.equal(planar.d.cpu(), host.d)
    if fmt == "q8_0":
        assert torch.equal(planar.qs.cpu(), host.qs)
    else:
        assert torch.equal(planar.m.cpu(), host.m) and torch.equal(planar.qs_bit_packed.cpu(), host.qs_bit_packed)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16, torch.float32])
@pytest.mark.parametrize("n,kind", [(1, "normal"), (1000, "normal"), (70001, "normal"), (4096, "zeros"), (4096, "large"), (3000, "tiny")])
def test_dynamic_quantizer_bit_exact(device, dtype, n, kind):
    """DynamicScaledQuantizer for float8_e4m3fn (sharktank/sharktank/types/quantizers.py:368-389): samples and the
    reciprocal scale equal the oracle's, which follows eager torch step by step, bit for bit."""
    from sharktank_amd import types as ST

    g = torch.Generator().manual_seed(123 + n)
    x = torch.randn(n, generator=g)
    if kind == "zeros":
        x = torch.zeros(n)
    elif kind == "large":
        x = x * 3000.0
    elif kind == "tiny":
        x = x * 1e-3
    x = x.to(dtype)
    want_qs, want_rscale = O.dynamic_quantize(x, torch.float8_e4m3fn)
    qt = ST.DynamicScaledQuantizer(dtype=torch.float8_e4m3fn).quantize(x.to(device).reshape(-1, 1) if n > 1 else x.to(device))
    lay = qt.unpack()
    assert lay.d.dtype == dtype and lay.dtype == dtype
    assert torch.equal(lay.d.cpu().reshape(()), want_rscale.reshape(()))
    assert torch.equal(lay.qs.cpu().reshape(-1).view(torch.uint8), want_qs.reshape(-1).view(torch.uint8))
    # and the layout dequantises as the reference's TensorScaledLayout does
    assert torch.equal(lay.dequant().cpu().reshape(-1), O.dequant_tensor_scaled(want_rscale, want_qs, layout_dtype=dtype).reshape(-1))


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16, torch.float32])
def test_dynamic_quantizer_scale_is_reciprocal_times_number(device, dtype):
    """The reference's `finfo.max / amax.clamp(eps)` divides a Python number by a tensor, which torch evaluates as
    `amax.reciprocal() * 448`: two roundings in the tensor's dtype.  A single division rounds differently for about one
    maximum in four (amax = 4.8867 in fp16: 91.625 against 91.6875), which moves every sample that sits near a rounding
    boundary.  Sixty maxima, among them that one."""
    from sharktank_amd import types as ST

    g = torch.Generator().manual_seed(77)
    q = ST.DynamicScaledQuantizer(dtype=torch.float8_e4m3fn)
    differs = 0
    for i in range(60):
        x = torch.randn(257, generator=g) * (0.05 + 3.0 * float(torch.rand((), generator=g)))
        if i == 0:
            x = x.clamp(-4.0, 4.0)
            x[5] = 4.8867
        x = x.to(dtype)
        want_qs, want_rscale = O.dynamic_quantize(x, torch.float8_e4m3fn)
        lay = q.quantize(x.to(device)).unpack()
        assert torch.equal(lay.d.cpu().reshape(()), want_rscale.reshape(())), (i, float(x.abs().max()))
        assert torch.equal(lay.qs.cpu().view(torch.uint8), want_qs.view(torch.uint8)), (i, float(x.abs().max()))
        amax = x.abs().max().clamp(0.125)
        differs += int((torch.tensor(448.0, dtype=dtype) / amax) != 448.0 / amax)
    if dtype == torch.float16:
        assert differs >= 5, "the sample no longer tells the two formulas apart"


@pytest.mark.gpu
@pytest.mark.parametrize("kind", [0, 1])
def test_matrix_core_probe_runs(device, kind):
    """The ceiling probe (a launch of nothing but MFMA instructions) completes and reports a rate between a tenth of the
    published peak and the peak itself (fp16 2500, fp8 5000 TFLOP/s): a measurement aid, so only its plausibility is checked."""
    from sharktank_amd import _hip

    peak = 2500.0 if kind == 0 else 5000.0
    for random_operands in (True, False):
        rate = _hip.probe_mfma(device, kind, random_operands, iters=2000, launches=2, warm_launches=2)
        assert 0.1 * peak < rate <= 1.02 * peak, f"kind {kind}, random {random_operands}: {rate:.0f} TFLOP/s"


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_fake_quant_every_16_bit_value_against_eager_torch(device, dtype):
    """The fake-quantisation arithmetic the kernels share (the quotient from a correctly rounded reciprocal and one residual
    step, the hardware's e4m3fn rounding) must give eager torch's bits -- `t / reciprocal_scale` in fp32 rounded to the
    tensor's dtype, clamped, cast to float8_e4m3fn, widened and multiplied back (the oracle runs those torch operations on
    the host) -- for every input there is: all 65536 bit patterns of the dtype, each with 150 scales (powers of two,
    scales next to them, scales whose reciprocal is far from representable, very small and very large ones)."""
    bits = torch.arange(65536, dtype=torch.int32).to(torch.int16)
    x = bits.view(dtype)
    g = torch.Generator().manual_seed(91)
    scales = [2.0 ** e for e in range(-12, 5)] + [float(torch.tensor(2.0 ** e).nextafter(torch.tensor(4.0 if i else 0.0))) for e in range(-6, 2) for i in (0, 1)]
    scales += [4.0 * 1.25 / 448.0, 8.0 * 2.0 / 448.0, 1.0 / 3.0, 0.1, 0.7, 1e-6, 300.0]
    scales += (torch.rand(150 - len(scales), generator=g).double() * 0.2 + 1e-3).tolist()
    xd = x.to(device)
    for s in scales:
        rs = torch.tensor(s, dtype=torch.float32)
        want = O.fake_quant_per_tensor(x, rs)
        got = _hip().fake_quant_fp8(xd, rs.to(device)).cpu()
        same = (got.view(torch.int16) == want.view(torch.int16)) | (torch.isnan(got) & torch.isnan(want))
        assert bool(same.all()), f"scale {s!r}: {int((~same).sum())} of 65536 values differ, first at bits {int(bits[~same][0]) & 0xffff:#06x}"
        # the quantizer's samples themselves (the fp8 matrix-core path consumes them as bytes)
        want_qs, _, _ = O.static_quantize_per_tensor(x, rs, torch.float8_e4m3fn)
        got_qs = _hip().quantize_fp8(xd, rs.to(device)).cpu()
        a, b = got_qs.view(torch.uint8), want_qs.view(torch.uint8)
        same = (a == b) | ((a & 0x7f) == 0x7f) & ((b & 0x7f) == 0x7f)  # (any NaN code for NaN)
        assert bool(same.all()), f"scale {s!r}: {int((~same).sum())} quantised samples differ, first at bits {int(bits[~same][0]) & 0xffff:#06x}"
