"""BASELINE.json configurations 2-5 at their full shapes on the GPU.

The reference's own formulation (a gathered weight stack per token) cannot run these shapes on the CPU in reasonable time,
but tokens are independent given their routing, so the oracle is evaluated expert by expert on the rows routed to each
(one dense FFN per expert: seconds per configuration) and EVERY token of every configuration is compared:
  * routing indices of every token against the oracle (bit-exact),
  * the layer output of every token against the oracle.  The MoE contribution y - h is held to the tolerance on its own
    (the residual h ~ N(0, 1) would hide an error of the FFN kernels): 1e-3 for fp16 and for bf16, 2e-2 for fp8 weights
    or activations; the worst single token is held to a multiple of it (a wrong row or a wrong run of features in one row
    cannot hide in the average over thousands of rows),
  * a second kernel family (the 128 x 128 tile kernel) on all rows,
  * size-independent properties on all tokens: token-permutation equivariance (routing bit-exact; outputs equal up to
    the fp32 summation grouping of the few rows whose down-projection tile is split along the reduction) and run-to-run
    bit-identity (no float atomics).
"""

import pytest
import torch
import torch.nn.functional as F

from oracle import moe_oracle as O
import moe_cases as MC

pytestmark = pytest.mark.gpu

# bf16 keeps 8 significant bits, and the gated intermediate, the down projection and the gate-weighted slot values are each
# rounded to it.  Where the kernel and the oracle round the same fp32 value they agree exactly, so what is measured is how
# often a different order of the fp32 sums moves a value across a bf16 rounding boundary: 4e-4 to 8e-4 on the MoE
# contribution at these shapes (long reductions average the flips out; layers with a hidden size of 512 measure 2e-3, see
# tests/test_gpu_layer.py).  The limit is the north-star figure for the layer, held on the MoE contribution alone as well.
BF16_TOL = 1e-3


def build_device_case(device, T, K, N, fmt, dtype, act="silu", seed=0, E=8, k=2, out_norm=False, act_quant=False):
    """Weights N(0, 0.02) generated and quantized on the device (data generation only); returns (theta, pieces)."""
    from sharktank_amd import types as ST

    gg = torch.Generator(device=device).manual_seed(seed)
    gc = torch.Generator().manual_seed(seed)
    tensors, planes = {}, {}
    for name, shape in (("gate", [E, N, K]), ("up", [E, N, K]), ("down", [E, K, N])):
        per = []
        for e in range(E):
            w = torch.randn(shape[1:], generator=gg, device=device) * 0.02
            if fmt == "q8_0":
                per.append(O.quantize_q8_0(w))
            elif fmt == "q4_1":
                per.append(O.quantize_q4_1(w))
            elif fmt == "fp8":
                per.append((w,))
            del w
        if fmt == "fp8":
            w_all = torch.stack([p[0] for p in per])
            d, qs = O.quantize_fp8_per_tensor(w_all)
            p = {"d": d, "qs": qs}
        elif fmt == "q8_0":
            p = {"d": torch.stack([x[0] for x in per]), "qs": torch.stack([x[1] for x in per])}
        else:
            p = {"d": torch.stack([x[0] for x in per]), "m": torch.stack([x[1] for x in per]), "qs": torch.stack([x[2] for x in per])}
        planes[name] = p
        tensors[f"ffn_{name}_exps.weight"] = MC.to_inference_tensor(fmt, p, shape, f"ffn_{name}_exps.weight", device)
    router = torch.randn(E, K, generator=gc) * 0.02
    ffn_norm = torch.ones(K) + 0.1 * torch.randn(K, generator=gc)
    out_norm_w = (torch.ones(K) + 0.1 * torch.randn(K, generator=gc)) if out_norm else None
    h = torch.randn(T, K, generator=gc).to(dtype)
    tensors["ffn_gate_inp.weight"] = ST.DefaultPrimitiveTensor(name="ffn_gate_inp.weight", data=router.to(device))
    tensors["ffn_norm.weight"] = ST.DefaultPrimitiveTensor(name="ffn_norm.weight", data=ffn_norm.to(device))
    if out_norm_w is not None:
        tensors["layer_output_norm.weight"] = ST.DefaultPrimitiveTensor(name="layer_output_norm.weight", data=out_norm_w.to(device))
    act_fn = F.silu if act == "silu" else F.gelu
    x_rscale = z_rscale = None
    if act_quant:
        # static e4m3fn quantizers calibrated on a sample: 8 tokens through expert 0, with head-room
        xn = O.rms_norm(h[:8], ffn_norm, 1e-5)
        dense0 = {}
        for name, shape in (("gate", [N, K]), ("up", [N, K])):
            pe = {kk: (v[0].cpu() if v.dim() > 0 and v.shape[0] == E else v.cpu()) for kk, v in planes[name].items()}
            dense0[name] = MC.dense_from_planes(fmt, pe, shape, dtype)
        z = act_fn(O._mm_rt(xn, dense0["gate"])) * O._mm_rt(xn, dense0["up"])
        x_rscale = (xn.float().abs().amax() * 1.25 / 448.0).to(torch.float32)
        z_rscale = (z.float().abs().amax() * 2.0 / 448.0).to(torch.float32)
        for key, rs in (("ffn_gate_exps.q_input", x_rscale), ("ffn_down_exps.q_input", z_rscale)):
            tensors[key] = ST.StaticScaledQuantizer(name=key, scale=(1.0 / rs).to(device), reciprocal_scale=rs.to(device),
                                                    dtype=torch.float8_e4m3fn)
    return ST.Theta(tensors), dict(planes=planes, router=router, ffn_norm=ffn_norm, out_norm=out_norm_w, h=h, fmt=fmt,
                                   dtype=dtype, act=act_fn, E=E, k=k, K=K, N=N, T=T, x_rscale=x_rscale, z_rscale=z_rscale)


def expert_dense(pc, name, e):
    """Expert e's matrix of plane set `name`, dequantised on the CPU the way the reference does (dequantise, cast)."""
    E, N, K = pc["E"], pc["N"], pc["K"]
    shape = [K, N] if name == "down" else [N, K]
    p = pc["planes"][name]
    pe = {kk: (v[e].cpu() if v.dim() > 0 and v.shape[0] == E else v.cpu()) for kk, v in p.items()}
    return MC.dense_from_planes(pc["fmt"], pe, shape, pc["dtype"])


def oracle_route(pc, eps=1e-5):
    x = O.rms_norm_ordered(pc["h"], pc["ffn_norm"], eps)
    idx, gate, _ = O.route(O.router_logits_ordered(x, pc["router"]), pc["k"])
    return x, idx, gate


def oracle_pair_outputs(pc, x, idx, tokens):
    """down(act(gate x) * up x) of every (token, slot) pair of the given tokens, [len(tokens), k, K]: per expert one dense
    FFN on the rows routed to it (rows are independent, so this is the reference's per-token product row by row)."""
    k, K = pc["k"], pc["K"]
    tok = torch.tensor(tokens, dtype=torch.long)
    out = torch.empty(len(tokens), k, K, dtype=pc["dtype"])
    sel = idx[tok]  # [n, k]
    for e in sorted(set(sel.reshape(-1).tolist())):
        n_i, j_i = (sel == e).nonzero(as_tuple=True)
        xt = x[tok[n_i]]
        if pc.get("x_rscale") is not None:
            xt = O.fake_quant_per_tensor(xt, pc["x_rscale"])
        wg, wu = expert_dense(pc, "gate", e), expert_dense(pc, "up", e)
        z = pc["act"](O._mm_rt(xt, wg)) * O._mm_rt(xt, wu)
        del wg, wu
        if pc.get("z_rscale") is not None:
            z = O.fake_quant_per_tensor(z, pc["z_rscale"])
        out[n_i, j_i] = O._mm_rt(z, expert_dense(pc, "down", e))
    return out


def oracle_rows(pc, rows, eps=1e-5):
    """Oracle layer output for the given token rows (and routing of all tokens)."""
    x, idx, gate = oracle_route(pc, eps)
    tok = torch.tensor(rows, dtype=torch.long)
    pairs = oracle_pair_outputs(pc, x, idx, rows)
    o = torch.sum(gate[tok].unsqueeze(-1) * pairs, dim=1)
    if pc["out_norm"] is not None:
        o = O.rms_norm(o, pc["out_norm"], eps)
    return pc["h"][tok] + o, idx, gate


def token_tiles(idx, E):
    """Number of (expert, token tile of 256 sorted rows) pairs of a routing: the units of a prefill launch per feature tile."""
    counts = torch.bincount(idx.reshape(-1).long(), minlength=E)
    return int(((counts + 255) // 256).sum())


def run_layer(theta, pc, device, variant=0, h=None):
    from sharktank_amd.layers import MoeBlock

    block = MoeBlock(theta, pc["E"], pc["k"], 1e-5, moe_activation=pc["act"])
    block.experts.kernel_variant = variant
    hh = pc["h"] if h is None else h
    y, idx, gate = block(hh.reshape(1, -1, pc["K"]).to(device), return_routing=True)
    return y.reshape(-1, pc["K"]), idx, gate, block


def moe_tolerance(pc):
    if pc["fmt"] == "fp8" or pc.get("x_rscale") is not None:
        return 2e-2
    return BF16_TOL if pc["dtype"] == torch.bfloat16 else 1e-3


# The worst single token against the tolerance of the whole: rows differ in how much of their contribution cancels, so one
# row's relative error scatters around the average; measured maxima are 1.3 to 2.2 times the average at these shapes.
WORST_ROW_FACTOR = 4.0


def row_rel_l2(got, want):
    d = (got.double() - want.double()).norm(dim=-1)
    return d / want.double().norm(dim=-1).clamp_min(1e-30)


def check_against_oracle(y, idx, pc, rows=None, tol=None, want=None, worst_tol=None):
    """Routing of every token bit-exact; on `rows` (default: every token) the layer output within 1e-3 (the north-star
    figure for the layer), the MoE contribution y - h on its own within `tol`, and the MoE contribution of the worst
    single token within `worst_tol` (default WORST_ROW_FACTOR * tol).  `want`: the result of oracle_rows(pc, rows) when
    the caller has it."""
    tol = tol or moe_tolerance(pc)
    worst_tol = worst_tol or WORST_ROW_FACTOR * tol
    rows = list(range(pc["h"].shape[0])) if rows is None else rows
    want, want_idx, _ = want if want is not None else oracle_rows(pc, rows)
    assert torch.equal(idx.cpu().long(), want_idx), "routing indices differ"
    got = y[rows].cpu()
    h = pc["h"][rows].float()
    err = O.rel_l2(got, want)
    moe = O.rel_l2(got.float() - h, want.float() - h)
    per_row = row_rel_l2(got.float() - h, want.float() - h)
    worst = float(per_row.max())
    print(f"  {len(rows)} rows: layer rel-L2 {err:.2e}, MoE contribution rel-L2 {moe:.2e} (limit {tol:.0e}), "
          f"worst token {worst:.2e} (row {rows[int(per_row.argmax())]})")
    assert torch.isfinite(got.float()).all()
    assert err < tol, f"layer output rel-L2 {err:.3e}"
    assert moe < tol, f"MoE contribution rel-L2 {moe:.3e}"
    assert worst < worst_tol, f"MoE contribution of token {rows[int(per_row.argmax())]}: rel-L2 {worst:.3e}"
    return moe


def check_second_kernel_family(theta, pc, device, y, tol):
    """The 128 x 128 tile kernel (an independent implementation: other tiling, no specialised wavefronts, no absorbed
    tails, no split reductions) gives the same layer output on every row."""
    y2, _, _, _ = run_layer(theta, pc, device, variant=2)
    h = pc["h"].float()
    moe = O.rel_l2(y2.cpu().float() - h, y.cpu().float() - h)
    assert moe < tol, f"kernel families differ: MoE contribution rel-L2 {moe:.3e}"


def pre_gather_block(theta, pc):
    from sharktank_amd.layers import PreGatherFFNMOE

    return PreGatherFFNMOE(theta, activation=pc["act"])


def check_pre_gather_ffn_moe(theta, pc, device, x, idx, gate, tokens, tol):
    """PreGatherFFNMOE.forward on its own (no norm, no router, no residual): every slot sum against the oracle's."""
    experts = pre_gather_block(theta, pc)
    got = experts(x.to(device), idx.to(device), gate.to(device)).cpu()
    tok = torch.tensor(tokens, dtype=torch.long)
    want = torch.sum(gate[tok].unsqueeze(-1) * oracle_pair_outputs(pc, x, idx, tokens), dim=1)
    err = O.rel_l2(got[tok], want)
    worst = float(row_rel_l2(got[tok], want).max())
    print(f"  PreGatherFFNMOE.forward, {len(tokens)} rows: rel-L2 {err:.2e} (limit {tol:.0e}), worst token {worst:.2e}")
    assert torch.isfinite(got.float()).all()
    assert err < tol, f"PreGatherFFNMOE output rel-L2 {err:.3e}"
    assert worst < WORST_ROW_FACTOR * tol, f"PreGatherFFNMOE output, worst token: rel-L2 {worst:.3e}"
    return got


def test_config2_mixtral_q8_0_prefill_and_decode(device):
    """Mixtral-8x7B layer, Q8_0, fp16: prefill 2048 tokens and decode 32 tokens."""
    theta, pc = build_device_case(device, 2048, 4096, 14336, "q8_0", torch.float16, seed=0)
    y, idx, gate, block = run_layer(theta, pc, device)
    rows = list(range(2048))  # every token
    counts = torch.bincount(idx.cpu().reshape(-1).long(), minlength=8).tolist()
    print(f"  rows per expert {counts}: {token_tiles(idx.cpu(), 8)} token tiles")
    check_against_oracle(y, idx, pc, rows)
    check_second_kernel_family(theta, pc, device, y, 1e-3)
    # PreGatherFFNMOE on its own, with the router's choices
    x, idx_o, gate_o = oracle_route(pc)
    check_pre_gather_ffn_moe(theta, pc, device, x, idx_o, gate_o, rows, 1e-3)
    # permutation equivariance: every output row depends on its own token only.  Routing is bit-exact; an output row
    # changes in its last bits only if its down-projection tile is one of the last units of the launch in one order and
    # not in the other (those units add four fp32 partial sums instead of one running sum), or if it is computed as a
    # row that rides along with a full token tile in one order and as a row of a token tile in the other
    perm = torch.randperm(2048, generator=torch.Generator().manual_seed(1))
    y2, idx2, _ = block(pc["h"][perm].reshape(1, 2048, 4096).to(device), return_routing=True)
    assert torch.equal(idx2.cpu(), idx.cpu()[perm])
    a, b = y2.reshape(2048, 4096).cpu(), y.cpu()[perm]
    assert O.rel_l2(a, b) < 1e-4
    assert (a != b).float().mean().item() < 0.05
    # run-to-run identity
    y3 = block(pc["h"].reshape(1, 2048, 4096).to(device))
    assert torch.equal(y3.reshape(2048, 4096).view(torch.int16), y.view(torch.int16))
    # decode batch = first 32 tokens through the streaming kernel: same routing, outputs within tolerance of prefill's
    yd, idxd, _ = block(pc["h"][:32].reshape(1, 32, 4096).to(device), return_routing=True)
    assert torch.equal(idxd.cpu(), idx.cpu()[:32])
    assert O.rel_l2(yd.reshape(32, 4096).cpu(), y[:32].cpu()) < 1e-3
    check_against_oracle(yd.reshape(32, 4096), idxd, {**pc, "h": pc["h"][:32]}, list(range(32)))


def test_config2_prefill_with_split_reductions(device):
    """The same layer at 1900 tokens: the units of the two prefill launches no longer fill whole rounds over the compute
    units, so the last ones are cut along the reduction and their chunks added by the workgroup that finishes last."""
    theta, pc = build_device_case(device, 1900, 4096, 14336, "q8_0", torch.float16, seed=7)
    y, idx, gate, block = run_layer(theta, pc, device)
    check_against_oracle(y, idx, pc)  # every token
    check_second_kernel_family(theta, pc, device, y, 1e-3)


@pytest.mark.parametrize("T", [1, 8, 32, 128])
def test_config3_mixtral_q4_1_bf16_decode_sweep(device, T):
    theta, pc = build_device_case(device, T, 4096, 14336, "q4_1", torch.bfloat16, seed=3)
    y, idx, gate, block = run_layer(theta, pc, device)
    rows = list(range(T))  # every token
    check_against_oracle(y, idx, pc, rows)
    # the 128 x 128 tile kernel gives the same answer as the kernel the dispatcher picked
    check_second_kernel_family(theta, pc, device, y, BF16_TOL)
    x, idx_o, gate_o = oracle_route(pc)
    check_pre_gather_ffn_moe(theta, pc, device, x, idx_o, gate_o, rows, BF16_TOL)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_config4_grok_q4_1_gelu_skewed_routing(device, dtype):
    """Grok-1 shape: hidden 6144, FFN 32768, GELU, Q4_1, output norm, 1024 tokens, router logits shifted by a Zipf prior
    (log p_e, p_e ~ 1/(e+1)) so that two experts receive about 60 % of the (token, slot) pairs."""
    E = 8
    theta, pc = build_device_case(device, 1024, 6144, 32768, "q4_1", dtype, act="gelu", seed=4, out_norm=True)
    # the prior enters through a direction u that every token shares: tokens get the offset 40 u, the router rows
    # get (log p_e - mean) u / 40, so every token's logit of expert e moves by log p_e - mean (up to rounding)
    g = torch.Generator().manual_seed(40)
    u = torch.randn(6144, generator=g)
    u = u / u.norm()
    logp = torch.log(1.0 / (torch.arange(E, dtype=torch.float32) + 1.0))
    pc["router"] = pc["router"] + (logp - logp.mean()).reshape(E, 1) * u.reshape(1, -1) / 40.0
    pc["h"] = (pc["h"].float() + 40.0 * u.reshape(1, -1)).to(dtype)
    from sharktank_amd import types as ST

    flat = theta.flatten()
    flat["ffn_gate_inp.weight"] = ST.DefaultPrimitiveTensor(name="ffn_gate_inp.weight", data=pc["router"].to(device))
    theta = ST.Theta(flat)
    y, idx, gate, block = run_layer(theta, pc, device)
    counts = torch.bincount(idx.cpu().reshape(-1).long(), minlength=E)
    top2 = counts.sort(descending=True).values[:2].sum().item() / counts.sum().item()
    print(f"  (token, slot) pairs per expert {counts.tolist()}: the two busiest experts take {top2:.3f}")
    assert 0.55 <= top2 <= 0.65, f"routing skew off the stated 60 %: {counts.tolist()}"
    rows = list(range(1024))  # every token
    check_against_oracle(y, idx, pc, rows)
    check_second_kernel_family(theta, pc, device, y, moe_tolerance(pc))
    x, idx_o, gate_o = oracle_route(pc)
    check_pre_gather_ffn_moe(theta, pc, device, x, idx_o, gate_o, rows, moe_tolerance(pc))


def uniform_routing(T, E=8):
    """The stated routing of configuration 5: token t goes to experts 2t mod E and 2t + 1 mod E."""
    t = torch.arange(T)
    return torch.stack([(2 * t) % E, (2 * t + 1) % E], dim=1)


def test_config5_mixtral_fp8_weights(device):
    """fp8 e4m3 per-tensor-scaled expert weights, fp16 activations; 4096-token prefill and a 1-token decode: once with the
    stated uniform routing (token t to experts 2t mod 8 and 2t + 1 mod 8, through PreGatherFFNMOE.forward, seeded gates)
    and once through the whole block, where the router decides."""
    theta, pc = build_device_case(device, 4096, 4096, 14336, "fp8", torch.float16, seed=5)
    T = 4096
    x = O.rms_norm_ordered(pc["h"], pc["ffn_norm"], 1e-5)
    experts = uniform_routing(T)
    gg = torch.rand(T, 2, generator=torch.Generator().manual_seed(50)) + 0.25
    gates = (gg / gg.sum(dim=1, keepdim=True)).to(torch.float16)
    assert torch.bincount(experts.reshape(-1), minlength=8).tolist() == [1024] * 8
    rows = list(range(T))  # every token
    assert token_tiles(experts, 8) == 32
    check_pre_gather_ffn_moe(theta, pc, device, x, experts, gates, rows, 2e-2)
    got1 = pre_gather_block(theta, pc)(x[:1].to(device), experts[:1].to(device), gates[:1].to(device)).cpu()
    want1 = torch.sum(gates[:1].unsqueeze(-1) * oracle_pair_outputs(pc, x, experts, [0]), dim=1)
    assert O.rel_l2(got1, want1) < 2e-2
    # the whole block
    y, idx, gate, block = run_layer(theta, pc, device)
    check_against_oracle(y, idx, pc, rows)
    check_second_kernel_family(theta, pc, device, y, 2e-2)
    y1, idx1, _ = block(pc["h"][:1].reshape(1, 1, 4096).to(device), return_routing=True)
    assert torch.equal(idx1.cpu(), idx.cpu()[:1])
    assert O.rel_l2(y1.reshape(1, 4096).cpu(), y[:1].cpu()) < 1e-3


def test_config5_mixtral_fp8_weights_and_activations(device):
    """Config 5 with static e4m3fn quantizers on the FFN input and on the gated intermediate.  With fp16 activations the
    prefill runs both operands on the fp8 matrix cores by default (the same kernels as kernel variant 5); decode, and
    every launch under VARIANT_STEP_BY_STEP, quantise, dequantise and multiply in the activation dtype (the reference's
    arithmetic, held to the 16-bit tolerance).  The matrix-core arithmetic is held to the fp8 tolerance of 2e-2 on the MoE
    contribution; the stated uniform routing runs through PreGatherFFNMOE.forward on both paths."""
    from sharktank_amd import _hip

    theta, pc = build_device_case(device, 4096, 4096, 14336, "fp8", torch.float16, seed=5, act_quant=True)
    T = 4096
    x = O.rms_norm_ordered(pc["h"], pc["ffn_norm"], 1e-5)
    experts = uniform_routing(T)
    gates = torch.full((T, 2), 0.5, dtype=torch.float16)
    rows = list(range(T))  # every token
    tok = torch.tensor(rows, dtype=torch.long)
    want = torch.sum(gates[tok].unsqueeze(-1) * oracle_pair_outputs(pc, x, experts, rows), dim=1)
    outs = {}
    for variant, tol in ((_hip.VARIANT_STEP_BY_STEP, 1e-3), (_hip.VARIANT_AUTO, 2e-2), (_hip.VARIANT_FP8_MFMA, 2e-2)):
        ffn = pre_gather_block(theta, pc)
        ffn.kernel_variant = variant
        got = ffn(x.to(device), experts.to(device), gates.to(device)).cpu()
        err = O.rel_l2(got[tok], want)
        print(f"  PreGatherFFNMOE.forward, uniform routing, kernel variant {variant}: rel-L2 {err:.2e} (limit {tol:.0e})")
        assert err < tol
        outs[variant] = got
    # the automatic choice for fp16 activations at this size is the matrix-core arithmetic
    assert torch.equal(outs[_hip.VARIANT_AUTO], outs[_hip.VARIANT_FP8_MFMA])
    y, idx, gate, block = run_layer(theta, pc, device, variant=_hip.VARIANT_STEP_BY_STEP)
    want_all = oracle_rows(pc, rows)
    # the reference's arithmetic step by step: 16-bit tolerance on the whole.  A single token is held to the fp8 tolerance:
    # where the two sides' fp32 sums differ in the last bit, an element of the intermediate can land on the other side of
    # an e4m3 rounding boundary, a step of 1/16 of that element, and a few such elements among a token's largest move
    # that token by several 1e-3 (measured worst token 4.6e-3 at an average of 3.2e-4)
    check_against_oracle(y, idx, pc, rows, 1e-3, want=want_all, worst_tol=2e-2)
    y0, idx0, _, _ = run_layer(theta, pc, device)
    check_against_oracle(y0, idx0, pc, rows, 2e-2, want=want_all)  # the default: fp8 matrix cores
    y1, idx1, _ = block(pc["h"][:1].reshape(1, 1, 4096).to(device), return_routing=True)
    assert torch.equal(idx1.cpu(), idx.cpu()[:1])
    assert O.rel_l2(y1.reshape(1, 4096).cpu(), want_all[0][:1]) < 1e-3  # the decode path follows the reference's arithmetic
    # run-to-run bit identity
    y2, _, _, _ = run_layer(theta, pc, device, variant=_hip.VARIANT_STEP_BY_STEP)
    assert torch.equal(y2, y)
    # fp8 matrix cores
    y8, idx8, _, _ = run_layer(theta, pc, device, variant=_hip.VARIANT_FP8_MFMA)
    check_against_oracle(y8, idx8, pc, rows, 2e-2, want=want_all)
    y8b, _, _, _ = run_layer(theta, pc, device, variant=_hip.VARIANT_FP8_MFMA)
    assert torch.equal(y8b, y8) and torch.equal(y0, y8)
