"""Pins the CPU oracle: the reference's own known-answer vectors, exact-arithmetic checks and brute force.

Vectors are restated as values from the reference's tests (file:line in each test)."""

from fractions import Fraction

import numpy as np
import pytest
import torch
import torch.nn.functional as F

from oracle import moe_oracle as O

import json
import os

with open(os.path.join(os.path.dirname(__file__), "golden", "reference_vectors.json")) as _f:
    GOLDEN = json.load(_f)


# ---- i4 nibble utilities: sharktank/tests/types/layout_utils_test.py:15-65 ---------------------------------
def test_linearize_and_interleave_known_answer():
    v = GOLDEN["i4_interleaved_to_linear"]
    inter = torch.tensor([v["interleaved"]], dtype=torch.uint8)
    linear = O.linearize_interleaved_i4_block(inter)
    assert linear.tolist() == [v["linear"]]
    assert O.interleave_linear_i4_block(linear).tolist() == inter.tolist()


def test_promote_i4_known_answer():
    v = GOLDEN["i4_promote"]
    linear = torch.tensor([v["linear"]], dtype=torch.uint8)
    u = O.promote_linear_i4_block_to_i8(linear)
    assert u.dtype == torch.uint8 and u.tolist() == [v["unsigned"]]
    s = O.promote_linear_i4_block_to_i8(linear, signed=True)
    assert s.dtype == torch.int8 and s.tolist() == [v["signed"]]


def test_linearize_is_a_permutation_of_nibbles():
    g = torch.Generator().manual_seed(0)
    raw = torch.randint(0, 256, (5, 16), generator=g, dtype=torch.uint8)
    lin = O.promote_linear_i4_block_to_i8(O.linearize_interleaved_i4_block(raw))
    # ggml order: byte i holds element i (low) and element i+16 (high)
    want = torch.cat([raw & 0xF, raw >> 4], dim=-1)
    assert torch.equal(lin, want)


# ---- TensorScaledLayout: sharktank/tests/types/layouts_test.py:107-125 ---------------------------------------
def test_tensor_scaled_known_answer():
    v = GOLDEN["tensor_scaled_dequant"]
    got = O.dequant_tensor_scaled(torch.tensor(v["d"]), torch.tensor(v["qs"], dtype=torch.float16), torch.tensor(v["m"]))
    assert got.dtype == torch.float32 and got.tolist() == v["want"]


# ---- block-scaled dequant: exact rational arithmetic with a hand-written round-to-nearest-even -----------------
def _rne_f16(x: Fraction) -> float:
    """Round an exact rational to the nearest fp16 (ties to even), subnormals kept, no overflow expected."""
    if x == 0:
        return 0.0
    sign = -1 if x < 0 else 1
    a = abs(x)
    e = 0
    while a >= 2:
        a /= 2
        e += 1
    while a < 1:
        a *= 2
        e -= 1
    e_eff = max(e, -14)  # subnormal: fixed exponent
    scale = Fraction(2) ** (e_eff - 10)
    q = abs(x) / scale
    fl = q.numerator // q.denominator
    rem = q - fl
    if rem > Fraction(1, 2) or (rem == Fraction(1, 2) and fl % 2 == 1):
        fl += 1
    return float(sign * fl * scale)


def test_q8_0_dequant_exact():
    g = torch.Generator().manual_seed(1)
    d = (torch.rand(6, 1, generator=g) * 1e-3).to(torch.float16)
    d[0] = 6e-8  # smallest subnormal region
    d[1] = 0.0
    qs = torch.randint(-128, 128, (6, 32), generator=g, dtype=torch.int8)
    got = O.dequant_block_scaled(d, qs)
    assert got.dtype == torch.float16
    for b in range(6):
        for i in range(32):
            want = _rne_f16(Fraction(float(d[b, 0])) * int(qs[b, i]))
            assert float(got[b, i]) == want, (b, i)


def test_q4_1_dequant_exact_two_roundings():
    g = torch.Generator().manual_seed(2)
    d = (torch.rand(4, 1, generator=g) * 1e-2).to(torch.float16)
    m = (torch.randn(4, 1, generator=g) * 1e-1).to(torch.float16)
    packed = torch.randint(0, 256, (4, 16), generator=g, dtype=torch.uint8)
    got = O.dequant_block_scaled_i4(d, packed, m)
    for b in range(4):
        for i in range(32):
            byte = int(packed[b, i // 2])
            q = (byte & 0xF) if i % 2 == 0 else (byte >> 4)
            scaled = _rne_f16(Fraction(float(d[b, 0])) * q)
            want = _rne_f16(Fraction(scaled) + Fraction(float(m[b, 0])))
            assert float(got[b, i]) == want, (b, i)


# ---- quantizers: sharktank/tests/types/quantizers_test.py ------------------------------------------------------
def test_static_per_tensor_roundtrip():  # :40-51
    orig = torch.tensor([1.0, 2.0, 3.0, 4.0], dtype=torch.float16)
    qs, d, m = O.static_quantize_per_tensor(orig, torch.tensor(0.5), torch.uint8)
    assert qs.tolist() == [2, 4, 6, 8]
    torch.testing.assert_close(O.dequant_tensor_scaled(d, qs, m, layout_dtype=orig.dtype), orig, atol=1e-3, rtol=1e-3)


def test_static_per_tensor_offset_roundtrip():  # :53-64
    orig = torch.tensor([9.0, 10.0, 11.0, 12.0], dtype=torch.float16)
    off = torch.tensor(8, dtype=torch.int8)
    qs, d, m = O.static_quantize_per_tensor(orig, torch.tensor(0.5), torch.int8, offset=off)
    assert qs.tolist() == [26, 28, 30, 32]
    torch.testing.assert_close(O.dequant_tensor_scaled(d, qs, m, layout_dtype=orig.dtype), orig, atol=1e-3, rtol=1e-3)


def test_static_per_axis_roundtrip():  # :83-101
    orig = torch.tensor([[1.0, -2.0, 3.0], [10.0, -20.0, 60.0]], dtype=torch.float16)
    qs, d, m = O.static_quantize_per_axis(orig, torch.tensor([8.0, 4.0, 2.0]), 1, torch.int8)
    assert qs.tolist() == [[8, -8, 6], [80, -80, 120]]
    torch.testing.assert_close(O.dequant_tensor_scaled(d, qs, m, layout_dtype=orig.dtype), orig, atol=1e-3, rtol=1e-3)


@pytest.mark.parametrize("dtype", [torch.int8, torch.float16, torch.float8_e4m3fn, torch.float8_e4m3fnuz])
def test_dynamic_quantizer_roundtrip(dtype):  # :133-170
    orig = torch.tensor([-5.0, -2.0, 3.0, 4.5], dtype=torch.float32)
    qs, rscale = O.dynamic_quantize(orig, dtype)
    got = O.dequant_tensor_scaled(rscale, qs, layout_dtype=torch.float32)
    torch.testing.assert_close(orig, got, atol=1e-1, rtol=1e-1)


QUARK_FP8 = GOLDEN["quark_fp8"]["int8_bit_patterns"]


def test_quark_fp8_vector():  # :172-244
    scale = torch.tensor(0.0118, dtype=torch.float64)
    orig = torch.tensor(QUARK_FP8, dtype=torch.int8).view(torch.float8_e4m3fn)
    orig = (orig.to(torch.float64) * scale).to(torch.float16)
    qs_fn, d_fn, _ = O.static_quantize_per_tensor(orig, scale, torch.float8_e4m3fn)
    qs_uz, d_uz, _ = O.static_quantize_per_tensor(orig, scale * 2, torch.float8_e4m3fnuz)
    deq_fn = O.dequant_tensor_scaled(d_fn, qs_fn, layout_dtype=orig.dtype)
    deq_uz = O.dequant_tensor_scaled(d_uz, qs_uz, layout_dtype=orig.dtype)
    torch.testing.assert_close(orig, deq_uz, atol=1e-3, rtol=1e-3)
    torch.testing.assert_close(orig, deq_fn, atol=1e-3, rtol=1e-3)
    # the e4m3fn bit patterns survive the round trip exactly
    assert torch.equal(qs_fn.view(torch.int8), torch.tensor(QUARK_FP8, dtype=torch.int8))


def test_fake_quant_is_quantize_then_dequant_and_idempotent():
    """fake_quant_per_tensor on the quark vector gives the vector back (its samples are e4m3fn values times the scale),
    applying it twice changes nothing, and values beyond 448 * scale saturate."""
    scale = torch.tensor(0.0118, dtype=torch.float32)
    orig = torch.tensor(QUARK_FP8[:-2], dtype=torch.int8).view(torch.float8_e4m3fn)  # drop the NaN / -0 patterns
    x = (orig.to(torch.float32) * scale).to(torch.float16)
    fq = O.fake_quant_per_tensor(x, scale)
    torch.testing.assert_close(fq, x, atol=1e-3, rtol=1e-3)
    assert torch.equal(O.fake_quant_per_tensor(fq, scale), fq)
    big = torch.tensor([100.0, -100.0], dtype=torch.float16)
    assert O.fake_quant_per_tensor(big, scale).tolist() == [(torch.tensor(448.0) * scale).to(torch.float16).item()] * 1 + [
        (torch.tensor(-448.0) * scale).to(torch.float16).item()]


# ---- GGUF raw blocks: struct layouts quoted at sharktank/sharktank/types/gguf_interop/layouts.py:33-39,263-270 --
def test_q8_0_unpack_hand_assembled_block():
    d = np.float16(0.25)
    qs = np.arange(-16, 16, dtype=np.int8)
    raw = torch.from_numpy(np.frombuffer(d.tobytes() + qs.tobytes(), dtype=np.uint8).copy())
    dd, qq = O.q8_0_unpack(raw, [1, 32])
    assert dd.shape == (1, 1, 1) and qq.shape == (1, 1, 32)
    assert float(dd[0, 0, 0]) == 0.25 and qq[0, 0].tolist() == list(range(-16, 16))
    assert O.dequant_block_scaled(dd, qq).reshape(32).tolist() == [0.25 * v for v in range(-16, 16)]


def test_q4_1_unpack_hand_assembled_block():
    d, m = np.float16(0.5), np.float16(-1.0)
    elems = [(3 * i + 1) % 16 for i in range(32)]
    packed = bytes((elems[i] | (elems[i + 16] << 4)) for i in range(16))  # ggml: byte i = element i | element i+16 << 4
    raw = torch.from_numpy(np.frombuffer(d.tobytes() + m.tobytes() + packed, dtype=np.uint8).copy())
    dd, mm, qs = O.q4_1_unpack(raw, [1, 32])
    assert O.promote_linear_i4_block_to_i8(qs)[0, 0].tolist() == elems
    got = O.dequant_block_scaled_i4(dd, qs, mm).reshape(32).tolist()
    assert got == [0.5 * e - 1.0 for e in elems]


def test_synthetic_quantizers_reconstruct_within_half_step():
    g = torch.Generator().manual_seed(3)
    w = torch.randn(8, 64, generator=g) * 0.02
    d, qs = O.quantize_q8_0(w)
    err = (O.dequant_block_scaled(d.float(), qs).reshape(8, 64) - w).abs().reshape(8, 2, 32).amax(-1)
    assert bool((err <= 0.6 * d.float().reshape(8, 2) + 1e-8).all())
    d4, m4, q4 = O.quantize_q4_1(w)
    err4 = (O.dequant_block_scaled_i4(d4.float(), q4, m4.float()).reshape(8, 64) - w).abs().reshape(8, 2, 32).amax(-1)
    assert bool((err4 <= 0.6 * d4.float().reshape(8, 2) + 1e-4).all())


# ---- rms_norm: formula of sharktank/tests/ops/ops_test.py:228-232 --------------------------------------------------
def test_rms_norm_formula():
    g = torch.Generator().manual_seed(4)
    x = torch.randn(5, 96, generator=g)
    w = torch.randn(96, generator=g)
    want = (x.double() * w.double()) / torch.sqrt((x.double() ** 2).mean(-1, keepdim=True) + 1e-6)
    torch.testing.assert_close(O.rms_norm(x, w, 1e-6).double(), want, atol=1e-6, rtol=1e-6)
    # dtype round trip: fp16 in -> fp16 out, statistics in fp32
    x16 = x.to(torch.float16)
    got = O.rms_norm(x16, w, 1e-6)
    assert got.dtype == torch.float16
    want16 = (x16.double() * w.double()) / torch.sqrt((x16.double() ** 2).mean(-1, keepdim=True) + 1e-6)
    assert O.rel_l2(got, want16) < 1e-3


def test_rms_norm_ordered_pins():
    g = torch.Generator().manual_seed(44)
    # small integers: every partial sum of squares is exact, so the order cannot matter -> bit-identical to rms_norm
    x = torch.randint(-8, 9, (6, 1536), generator=g).to(torch.float16)
    w = torch.ones(1536) + 0.25 * torch.randint(-2, 3, (1536,), generator=g).float()
    assert torch.equal(O.rms_norm_ordered(x, w, 1e-5), O.rms_norm(x, w, 1e-5))
    # general values: agrees with torch's order up to fp32 rounding, and with a pure-Python restatement of the order
    x = torch.randn(2, 1100, generator=g).to(torch.float16)  # 1100 = 2 full passes of 512 + a ragged third
    w = torch.ones(1100) + 0.1 * torch.randn(1100, generator=g)
    got = O.rms_norm_ordered(x, w, 1e-5)
    assert O.rel_l2(got, O.rms_norm(x, w, 1e-5)) < 1e-3
    f32 = np.float32
    for t in range(2):
        th = [f32(0.0)] * 512
        for i in range(1100):
            v = f32(x[t, i])
            th[i % 512] = f32(th[i % 512] + f32(v * v))
        groups = []
        for gidx in range(8):
            lanes = th[gidx * 64 : (gidx + 1) * 64]
            for off in (32, 16, 8, 4, 2, 1):
                lanes = [f32(lanes[l] + lanes[l ^ off]) for l in range(64)]
            groups.append(lanes[0])
        total = f32(f32(f32(groups[0] + groups[1]) + f32(groups[2] + groups[3])) + f32(f32(groups[4] + groups[5]) + f32(groups[6] + groups[7])))
        rs = f32(f32(1.0) / f32(np.sqrt(f32(f32(total / f32(1100)) + f32(1e-5)))))
        for i in (0, 7, 511, 512, 1099):
            want = np.float16(f32(f32(w[i]) * f32(f32(x[t, i]) * rs)))
            assert float(got[t, i]) == float(want)


# ---- router -----------------------------------------------------------------------------------------------------
def test_topk_tie_rule_brute_force():
    vals = torch.tensor([[0.1, 0.3, 0.3, 0.2, 0.3], [0.5, 0.5, 0.5, 0.5, 0.5], [0.0, 1.0, 0.0, 1.0, 0.5]])
    v, i = O.topk_lower_index_first(vals, 3)
    assert i.tolist() == [[1, 2, 4], [0, 1, 2], [1, 3, 4]]
    for r in range(3):  # pure-Python restatement
        order = sorted(range(5), key=lambda e: (-float(vals[r, e]), e))[:3]
        assert i[r].tolist() == order


def test_route_matches_float64_brute_force():
    g = torch.Generator().manual_seed(5)
    logits = torch.randn(40, 8, generator=g).to(torch.float16)
    idx, gate, probs = O.route(logits, 2)
    p64 = torch.softmax(logits.double(), dim=1)
    for t in range(40):
        order = sorted(range(8), key=lambda e: (-float(p64[t, e]), e))[:2]
        assert idx[t].tolist() == order
        gsum = float(p64[t, order[0]] + p64[t, order[1]])
        for j in range(2):
            assert abs(float(gate[t, j]) - float(p64[t, order[j]]) / gsum) < 1e-3
    assert torch.allclose(probs.sum(-1), torch.ones(40), atol=1e-6)


def test_ordered_logits_exact_cases_and_python_restatement():
    # integers: every partial sum is exact, so any summation order gives the same bits
    g = torch.Generator().manual_seed(6)
    x = torch.randint(-4, 5, (3, 1024), generator=g).to(torch.float16)
    w = torch.randint(-4, 5, (8, 1024), generator=g).to(torch.float16)
    got = O.router_logits_ordered(x, w)
    assert torch.equal(got.float(), (x.double() @ w.double().T).float())
    # general values: pure-Python sequential restatement of the documented order on one tiny row
    x = torch.randn(1, 1032, generator=g).to(torch.float16)  # 1032 = 2 full chunks + a ragged third
    w = torch.randn(2, 1032, generator=g).to(torch.float16)
    got = O.router_logits_ordered(x, w)
    for e in range(2):
        lanes = [np.float32(0.0)] * 64
        for c in range(3):
            for l in range(64):
                for j in range(8):
                    k = (c * 64 + l) * 8 + j
                    if k < 1032:
                        lanes[l] = np.float32(lanes[l] + np.float32(np.float32(x[0, k]) * np.float32(w[e, k])))
        for off in (32, 16, 8, 4, 2, 1):
            lanes = [np.float32(lanes[l] + lanes[l ^ off]) for l in range(64)]
        assert float(got[0, e]) == float(np.float16(lanes[0]))
    # and it agrees with torch's own matmul except on rounding boundaries
    assert O.rel_l2(got, O.router_logits(x, w)) < 1e-3


# ---- dispatch permutation ------------------------------------------------------------------------------------------
def test_dispatch_permutation_brute_force():
    g = torch.Generator().manual_seed(7)
    idx = torch.randint(0, 5, (13, 3), generator=g)
    counts, offsets, perm, inv = O.dispatch_permutation(idx, 6)
    flat = idx.reshape(-1).tolist()
    want = [p for e in range(6) for p in range(len(flat)) if flat[p] == e]
    assert perm.tolist() == want
    assert counts.tolist() == [flat.count(e) for e in range(6)]
    assert offsets.tolist() == [sum(flat.count(e) for e in range(j)) for j in range(7)]
    assert [perm.tolist()[i] for i in inv.tolist()] == list(range(len(flat)))


# ---- FFN formulations ----------------------------------------------------------------------------------------------
def _tiny_layer(dtype, act=F.silu, seed=8):
    g = torch.Generator().manual_seed(seed)
    T, K, N, E, k = 10, 32, 48, 4, 2
    h = torch.randn(T, K, generator=g).to(dtype)
    wg = (torch.randn(E, N, K, generator=g) * 0.2).to(dtype)
    wu = (torch.randn(E, N, K, generator=g) * 0.2).to(dtype)
    wd = (torch.randn(E, K, N, generator=g) * 0.2).to(dtype)
    experts = torch.stack([torch.randperm(E, generator=g)[:k] for _ in range(T)])
    gate = torch.rand(T, k, generator=g).to(dtype)
    return h, experts, gate, wg, wu, wd


@pytest.mark.parametrize("act", [F.silu, F.gelu])
def test_ffn_float64_brute_force(act):
    h, experts, gate, wg, wu, wd = _tiny_layer(torch.float32, act)
    got = O.pre_gather_ffn_moe(h, experts, gate, wg, wu, wd, act)
    for t in range(h.shape[0]):
        acc = torch.zeros(h.shape[1], dtype=torch.float64)
        for j in range(experts.shape[1]):
            e = int(experts[t, j])
            a = act(wg[e].double() @ h[t].double())
            u = wu[e].double() @ h[t].double()
            acc += gate[t, j].double() * (wd[e].double() @ (a * u))
        assert torch.allclose(got[t].double(), acc, atol=1e-5, rtol=1e-5)


@pytest.mark.parametrize("dtype,tol", [(torch.float32, 1e-6), (torch.float16, 1e-3), (torch.bfloat16, 8e-3)])
def test_gather_and_grouped_formulations_agree(dtype, tol):
    h, experts, gate, wg, wu, wd = _tiny_layer(dtype)
    a = O.pre_gather_ffn_moe(h, experts, gate, wg, wu, wd, chunk=3)
    b = O.grouped_ffn_moe(h, experts, gate, wg, wu, wd)
    assert a.dtype == dtype and O.rel_l2(a, b) < tol


def test_toy_config_formulations_agree():
    """BASELINE config 1 (64 tokens, hidden 512, FFN 1024, 8 experts, top-2, fp32, seed 0)."""
    import moe_cases as MC

    case = MC.build(MC.Case(T=64, K=512, N=1024, fmt="dense", dtype=torch.float32, seed=0))
    ya, ia, _ = MC.oracle_block(case, formulation="gather", ordered_logits=False)
    yb, ib, _ = MC.oracle_block(case, formulation="grouped", ordered_logits=True)
    assert torch.equal(ia, ib)
    assert O.rel_l2(ya, yb) < 1e-6
