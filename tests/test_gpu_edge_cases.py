"""Edge cases of the grouped FFN path through the C ABI: empty inputs, experts without rows, one expert, k = E, rows per
expert that need several passes or several token tiles, shapes that fall off the fast kernels, strided inputs."""

import pytest
import torch

from oracle import moe_oracle as O
import moe_cases as MC

pytestmark = pytest.mark.gpu


def _run(device, case, idx, *, prepack=True, variant=0):
    """grouped_ffn + combine with the given routing; returns (got, want)."""
    from sharktank_amd import _hip as hip
    from sharktank_amd.ops import device_weight

    x = case.planes["h"]
    T, k = idx.shape
    g = torch.Generator().manual_seed(case.seed + 7)
    gate = torch.rand(T, k, generator=g)
    gate = (gate / gate.sum(-1, keepdim=True)).to(case.dtype)
    wg, wu, wd = MC.dense_weights(case)
    want = O.grouped_ffn_moe(x, idx, gate, wg, wu, wd, case.activation)
    E, N, K = case.E, case.N, case.K
    dws = [device_weight(MC.to_inference_tensor(case.fmt, case.planes[n], shp, n, device), stacked=True, prepack=prepack)
           for n, shp in (("gate", [E, N, K]), ("up", [E, N, K]), ("down", [E, K, N]))]
    _, offsets, perm, inv = hip.dispatch_build(idx.to(torch.int32).to(device), E)
    act = hip.ACT_SILU if case.act == "silu" else hip.ACT_GELU_ERF
    y = hip.grouped_ffn(x.to(device), dws[0], dws[1], dws[2], act, offsets, perm, k, variant=variant)
    got = hip.combine(y, gate.to(device), inv, T, k).cpu()
    return got, want


def test_empty_batch(device):
    from sharktank_amd.layers import MoeBlock

    case = MC.build(MC.Case(T=4, K=256, N=512, fmt="q8_0", dtype=torch.float16, seed=70))
    block = MoeBlock(MC.make_theta(case, device), case.E, case.k, case.eps)
    y = block(torch.empty(1, 0, case.K, dtype=torch.float16, device=device))
    assert tuple(y.shape) == (1, 0, case.K)


@pytest.mark.parametrize("fmt", ["q8_0", "q4_1", "fp8"])
def test_prefill_with_experts_that_get_no_rows(device, fmt):
    """600 tokens all routed to experts 2 and 5 of 8: two experts with 600 rows (three token tiles, the last one
    partial), six without rows; the launch is small enough that units are split along the reduction."""
    case = MC.build(MC.Case(T=600, K=512, N=768, E=8, k=2, fmt=fmt, dtype=torch.float16, seed=71))
    idx = torch.tensor([[2, 5]]).repeat(600, 1)
    idx[::2] = torch.tensor([5, 2])
    got, want = _run(device, case, idx)
    assert O.rel_l2(got, want) < 1e-3


def test_prefill_single_expert_top1(device):
    case = MC.build(MC.Case(T=700, K=512, N=512, E=1, k=1, fmt="q8_0", dtype=torch.bfloat16, seed=72))
    got, want = _run(device, case, torch.zeros(700, 1, dtype=torch.long))
    assert O.rel_l2(got, want) < 8e-3


def test_every_expert_selected(device):
    """k = E: every token visits every expert (one full and one partial token tile per expert)."""
    case = MC.build(MC.Case(T=300, K=256, N=512, E=4, k=4, fmt="q4_1", dtype=torch.float16, seed=73))
    idx = torch.stack([torch.randperm(4, generator=torch.Generator().manual_seed(t)) for t in range(300)])
    got, want = _run(device, case, idx)
    assert O.rel_l2(got, want) < 1e-3


@pytest.mark.parametrize("fmt", ["q8_0", "q4_1", "fp8"])
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("T,rows", [(73, {0: 3, 1: 16, 2: 17, 3: 40, 4: 70}), (122, {0: 33, 1: 48, 2: 64, 3: 65, 4: 32, 5: 2})])
def test_streaming_kernel_packed_rows_per_expert(device, fmt, dtype, T, rows):
    """The packed streaming kernels (token rows shared through LDS) with 2 ... 70 rows on the experts: passes of one, two
    and four 16-row token tiles against one set of weight registers (up to 16, 32 and 64 rows), both sides of each limit,
    and experts that need a second pass over their weights (65 = 64 + 1, 70 = 64 + 6)."""
    E, k = 8, 2
    case = MC.build(MC.Case(T=T, K=512, N=1024, E=E, k=k, fmt=fmt, dtype=dtype, seed=74))
    pairs = [e for e, n in rows.items() for _ in range(n)]  # 146 = T * k pairs
    assert len(pairs) == T * k
    # deal the pairs so that a token never gets the same expert twice
    idx = torch.empty(T, k, dtype=torch.long)
    order = sorted(range(len(pairs)), key=lambda i: (i % T, i // T))
    by_token = [[] for _ in range(T)]
    for i, e in enumerate(sorted(pairs, key=lambda e: -rows[e])):
        by_token[i % T].append(e)
    for t in range(T):
        assert len(set(by_token[t])) == k
        idx[t] = torch.tensor(by_token[t])
    got, want = _run(device, case, idx, variant=3)
    assert O.rel_l2(got, want) < (1e-3 if dtype == torch.float16 else 8e-3)


@pytest.mark.parametrize("N,K", [(96, 512), (992, 256), (512, 528)])
def test_shapes_off_the_fast_paths(device, N, K):
    """Feature counts that are not whole tiles or groups of four tiles, and a reduction length that is not a multiple
    of 256: the launchers fall back to kernels that take them (planar order when the packed one does not apply)."""
    for T in (5, 300):
        case = MC.build(MC.Case(T=T, K=K, N=N, E=4, k=2, fmt="q8_0" if K % 32 == 0 else "dense", dtype=torch.float16, seed=75))
        g = torch.Generator().manual_seed(76)
        idx = torch.stack([torch.randperm(4, generator=g)[:2] for _ in range(T)])
        from sharktank_amd.ops import device_weight

        can = N % 16 == 0 and K % 256 == 0
        got, want = _run(device, case, idx, prepack=can)
        assert O.rel_l2(got, want) < 1e-3, (N, K, T)


def test_strided_input_view(device):
    """h given as a non-contiguous view (every other row of a larger buffer)."""
    from sharktank_amd.layers import MoeBlock

    case = MC.build(MC.Case(T=40, K=256, N=512, fmt="q8_0", dtype=torch.float16, seed=77))
    block = MoeBlock(MC.make_theta(case, device), case.E, case.k, case.eps)
    big = torch.zeros(80, case.K, dtype=torch.float16, device=device)
    big[::2] = case.planes["h"].to(device)
    y = block(big[::2].reshape(1, 40, case.K))
    want, _, _ = MC.oracle_block(case)
    assert O.rel_l2(y.reshape(40, case.K).cpu(), want) < 1e-3


def test_three_experts_top3_router(device):
    from sharktank_amd.layers import MoeBlock

    case = MC.build(MC.Case(T=33, K=256, N=256, E=3, k=3, fmt="q8_0", dtype=torch.float16, seed=78))
    block = MoeBlock(MC.make_theta(case, device), case.E, case.k, case.eps)
    y, idx, gate = block(case.planes["h"].reshape(1, 33, case.K).to(device), return_routing=True)
    want, want_idx, want_gate = MC.oracle_block(case)
    assert torch.equal(idx.cpu().long(), want_idx)
    assert O.rel_l2(y.reshape(33, case.K).cpu(), want) < 1e-3


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("E,k,T,K,N,routing", [
    (8, 2, 400, 256, 128, "random"),      # smallest tile counts the 256 x 256 fp8 kernel takes; every token tile partial
    (3, 1, 900, 1024, 384, "random"),     # three experts, one slot, full and partial token tiles
    (8, 2, 600, 512, 768, "two"),         # six experts without rows
    (1, 1, 513, 256, 256, "random"),      # one expert: two full tiles and a one-row tile
])
def test_fp8_matrix_core_kernels_agree(device, dtype, E, k, T, K, N, routing):
    """fp8 activations x fp8 weights: the 256 x 256 kernel with direct global -> LDS loads (variant 5) against the
    128 x 128 kernel (variant 7) -- the same arithmetic, up to the order of the fp32 sums -- and both against the
    oracle's quantise-dequantise arithmetic at the fp8 tolerance."""
    from sharktank_amd import _hip as hip
    from sharktank_amd.ops import device_weight

    case = MC.build(MC.Case(T=T, K=K, N=N, E=E, k=k, fmt="fp8", dtype=dtype, act_quant=True, seed=90 + E + T))
    g = torch.Generator().manual_seed(case.seed)
    if routing == "two":
        idx = torch.tensor([[1, 6]]).repeat(T, 1)
    else:
        idx = torch.stack([torch.randperm(E, generator=g)[:k] for _ in range(T)])
    x = case.planes["h"]
    gate = torch.rand(T, k, generator=g)
    gate = (gate / gate.sum(-1, keepdim=True)).to(dtype)
    wg, wu, wd = MC.dense_weights(case)
    xs, zs = case.planes["x_rscale"], case.planes["z_rscale"]
    want = O.grouped_ffn_moe(x, idx, gate, wg, wu, wd, case.activation, x_rscale=xs, z_rscale=zs)
    dws = [device_weight(MC.to_inference_tensor("fp8", case.planes[n], shp, n, device), stacked=True, prepack=True)
           for n, shp in (("gate", [E, N, K]), ("up", [E, N, K]), ("down", [E, K, N]))]
    _, offsets, perm, inv = hip.dispatch_build(idx.to(torch.int32).to(device), E)
    outs = {}
    for variant in (hip.VARIANT_FP8_MFMA, hip.VARIANT_FP8_TILE):
        y = hip.grouped_ffn(x.to(device), dws[0], dws[1], dws[2], hip.ACT_SILU, offsets, perm, k, variant=variant,
                            x_scale=xs.to(device), z_scale=zs.to(device))
        outs[variant] = hip.combine(y, gate.to(device), inv, T, k).cpu()
    a, b = outs[hip.VARIANT_FP8_MFMA], outs[hip.VARIANT_FP8_TILE]
    assert O.rel_l2(a, b) < (2e-3 if dtype == torch.float16 else 1.5e-2), "the two fp8 kernels disagree"
    assert O.rel_l2(a, want) < 6e-2 and O.rel_l2(b, want) < 6e-2


@pytest.mark.parametrize("fmt", ["q8_0", "q4_1", "fp8"])
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_streaming_kernel_two_row_tiles_in_one_pass(device, fmt, dtype):
    """33 tokens over 16 experts with one expert taking 30 rows: the streaming kernel multiplies two 16-row tiles of
    that expert with one weight fragment.  (The first tile once read fp8 fragments whose fp16 halves had been written by
    half-register instructions one cycle earlier, without the wait state that such a read needs.)"""
    case = MC.build(MC.Case(T=33, K=1024, N=1024, E=16, k=2, fmt=fmt, dtype=dtype, seed=1006))
    idx = torch.zeros(33, 2, dtype=torch.long)
    idx[:, 1] = 1 + torch.arange(33) % 15
    idx[30:, 0] = torch.tensor([2, 3, 4])
    idx[30:, 1] = torch.tensor([5, 6, 7])
    got, want = _run(device, case, idx)
    assert O.rel_l2(got, want) < (1e-3 if dtype == torch.float16 else 8e-3)


def _routing_with_rows(rows, T, k, seed):
    """idx [T,k] (no expert twice in a token) that gives expert e exactly rows[e] pairs; sum(rows) == T*k."""
    assert sum(rows) == T * k and max(rows) <= T
    g = torch.Generator().manual_seed(seed)
    left = list(rows)
    idx = torch.empty(T, k, dtype=torch.long)
    for t in range(T):
        # the k experts with the most pairs left (ties in random order): greedy, always feasible while max(left) <= tokens left
        order = sorted(range(len(left)), key=lambda e: (-left[e], torch.rand(1, generator=g).item()))
        pick = order[:k]
        assert all(left[e] > 0 for e in pick)
        for j, e in enumerate(pick):
            left[e] -= 1
        idx[t] = torch.tensor([pick[i] for i in torch.randperm(k, generator=g).tolist()])
    assert not any(left)
    return idx[torch.randperm(T, generator=g)]


@pytest.mark.parametrize("fmt,dtype", [("q8_0", torch.float16), ("q4_1", torch.bfloat16), ("fp8", torch.float16)])
@pytest.mark.parametrize("rows", [
    [261, 517, 512 + 32, 512 + 33, 256 + 16, 256 + 17, 300, 122],  # absorbed: 5, 5, 32 (two tiles x 16), 16; not: 33, 17
    [768 + 48, 768 + 1, 256, 255, 1, 0, 270, 257],                  # three full tiles x 16; one-row tails; an expert without rows
    [128, 129, 127, 1, 18, 64, 256 + 128, 256 + 129],               # token tiles of at most 128 rows (8 loaders, 4 consumers) and both sides of that limit
    [470, 511, 385, 384, 256 + 128 + 1, 512 + 200, 491, 130],       # a full tile and more than half of another: equal tiles (235 + 235, 256 + 255, 193 + 192; Q8_0 also 712 = 3 x 237+); not: 384
    [900, 1100, 650, 1290, 770, 1024 + 200, 768 + 129, 301],        # several full tiles and a large remainder (Q8_0: 4 x 225, 5 x 220, 3 x 217, ...; other formats keep full + partial tiles)
])
def test_prefill_tails_that_ride_along_with_full_token_tiles(device, fmt, dtype, rows):
    """Row counts a few rows above a multiple of 256: the prefill kernel lets every full token tile of such an expert take up
    to 16 of the extra rows along (computed by its loader wavefronts) instead of running a partial token tile for them.
    Token tiles of at most 128 rows run with eight loader and four consumer wavefronts instead of four and eight.
    An expert with one full token tile and more than half of a second one gets two tiles of equal size instead.
    Every output row is checked against the oracle, every expert's rows and the tail rows also on their own, and the whole
    result against the vector-ALU kernel."""
    from sharktank_amd import _hip as hip
    from sharktank_amd.ops import device_weight

    E, k = len(rows), 2
    T = sum(rows) // k
    assert sum(rows) == T * k
    case = MC.build(MC.Case(T=T, K=512, N=768, E=E, k=k, fmt=fmt, dtype=dtype, seed=4100 + rows[0]))
    idx = _routing_with_rows(rows, T, k, seed=rows[1])
    assert torch.bincount(idx.reshape(-1), minlength=E).tolist() == rows
    x = case.planes["h"]
    wg, wu, wd = MC.dense_weights(case)
    ones = torch.ones(T, k, dtype=dtype)
    N, K = case.N, case.K
    dws = [device_weight(MC.to_inference_tensor(fmt, case.planes[n], shp, n, device), stacked=True, prepack=True)
           for n, shp in (("gate", [E, N, K]), ("up", [E, N, K]), ("down", [E, K, N]))]
    _, offsets, perm, inv = hip.dispatch_build(idx.to(torch.int32).to(device), E)
    tol = 1e-3 if dtype == torch.float16 else 8e-3
    y = {}
    for variant in (hip.VARIANT_MFMA_WS, hip.VARIANT_GENERIC):
        y[variant] = hip.grouped_ffn(x.to(device), dws[0], dws[1], dws[2], hip.ACT_SILU, offsets, perm, k, variant=variant).cpu()
    got = y[hip.VARIANT_MFMA_WS]
    assert O.rel_l2(got.float(), y[hip.VARIANT_GENERIC].float()) < (2e-3 if dtype == torch.float16 else 1.2e-2)
    # oracle per sorted row: row i belongs to pair perm[i] = t*k + j of expert idx[t, j]
    perm_c, off_c = perm.cpu().long(), offsets.cpu().long()
    pair_rows = O.grouped_ffn_pairs(x, idx, wg, wu, wd, case.activation)  # [T, k, K]
    want = pair_rows.reshape(T * k, K)[perm_c]
    assert O.rel_l2(got, want) < tol
    for e in range(E):
        r = rows[e]
        if r > 0:
            a, b = int(off_c[e]), int(off_c[e + 1])
            err = O.rel_l2(got[a:b], want[a:b])
            assert err < 2 * tol, f"expert {e} ({r} rows): rel-L2 {err:.3e}"
        c, t = r // 256, r % 256
        if c >= 1 and 0 < t <= 16 * c:  # an absorbed tail: its rows on their own
            a, b = int(off_c[e]) + c * 256, int(off_c[e + 1])
            err = O.rel_l2(got[a:b], want[a:b])
            assert err < 2 * tol, f"expert {e}: tail rows {a}..{b}: rel-L2 {err:.3e}"
            assert torch.isfinite(got[a:b].float()).all()


@pytest.mark.parametrize("E", [2, 4, 6])
@pytest.mark.parametrize("T", [50, 96, 127])
@pytest.mark.parametrize("routing", ["uniform", "two experts take everything"])
def test_few_experts_between_100_and_255_rows(device, E, T, routing):
    """Launches of 100-254 sorted rows with 2-6 experts sit between the streaming kernel (up to 128 rows in all, or 16-28
    rows per expert on average) and the prefill kernel, whichever the automatic choice picks from the row total; with all tokens on two
    experts each of those holds T rows, several passes of the streaming kernel or one partial token tile.  Checked
    against the oracle pair by pair."""
    from sharktank_amd import _hip as hip
    from sharktank_amd.ops import device_weight

    k = 2
    case = MC.build(MC.Case(T=T, K=512, N=768, E=E, k=k, fmt="q8_0", dtype=torch.float16, seed=900 + E + T))
    g = torch.Generator().manual_seed(E * 1000 + T)
    if routing == "uniform":
        idx = torch.stack([torch.randperm(E, generator=g)[:k] for _ in range(T)])
    else:
        idx = torch.tensor([[0, 1], [1, 0]])[torch.randint(0, 2, (T,), generator=g)]
    x = case.planes["h"]
    wg, wu, wd = MC.dense_weights(case)
    N, K = case.N, case.K
    dws = [device_weight(MC.to_inference_tensor("q8_0", case.planes[n], shp, n, device), stacked=True, prepack=True)
           for n, shp in (("gate", [E, N, K]), ("up", [E, N, K]), ("down", [E, K, N]))]
    _, offsets, perm, inv = hip.dispatch_build(idx.to(torch.int32).to(device), E)
    got = hip.grouped_ffn(x.to(device), dws[0], dws[1], dws[2], hip.ACT_SILU, offsets, perm, k).cpu()
    want = O.grouped_ffn_pairs(x, idx, wg, wu, wd, case.activation).reshape(T * k, K)[perm.cpu().long()]
    assert torch.isfinite(got.float()).all()
    assert O.rel_l2(got, want) < 1e-3


def test_q4_1_block_scale_beyond_the_packed_limit_stays_planar(device):
    """The kernels on packed Q4_1 weights need |d| < 64 (they would give NaN beyond, without an error).  A tensor with one
    block scale of 100 must keep the planar order when asked to prepack, and the product through ops.matmul must match the
    oracle; the same tensor with ordinary scales is packed."""
    from sharktank_amd import _hip as hip
    from sharktank_amd.ops import device_weight

    g = torch.Generator().manual_seed(77)
    N, K = 64, 512
    d, m, qs = O.quantize_q4_1(torch.randn(N, K, generator=g) * 0.02)
    shape = [N, K]
    ok = device_weight(MC.to_inference_tensor("q4_1", {"d": d, "m": m, "qs": qs}, shape, "w", device), stacked=False, prepack=True)
    assert ok.is_packed
    d_big = d.clone()
    d_big[3, 5] = 100.0
    planes = {"d": d_big, "m": m, "qs": qs}
    dw = device_weight(MC.to_inference_tensor("q4_1", planes, shape, "w", device), stacked=False, prepack=True)
    assert not dw.is_packed, "a block scale of 100 must keep the tensor off the packed kernels"
    x = (torch.randn(40, K, generator=g) * 0.1).to(torch.float16)
    got = hip.mmt(x.to(device), dw).cpu()
    want = O.mmt(x, MC.dense_from_planes("q4_1", planes, shape, torch.float16))
    assert torch.isfinite(got.float()).all()
    assert O.rel_l2(got, want) < 1e-3
    # raw ggml blocks take the same decision
    raw = torch.cat([d_big.reshape(-1, 1).view(torch.uint8), m.reshape(-1, 1).view(torch.uint8), qs.reshape(-1, 16)], dim=1).contiguous()
    ing = hip.gguf_ingest(raw.reshape(-1).to(device), hip.GGUF_Q4_1, 1, N, K, packed=True)
    assert not ing.is_packed


def test_expert_ids_out_of_range_raise_with_checks_on(device):
    """The dispatch kernel clamps ids into range; with the debug checks on, PreGatherFFNMOE.forward raises IndexError as
    the reference's weights[experts] would."""
    from sharktank_amd.layers import PreGatherFFNMOE
    from sharktank_amd.utils import debugging

    case = MC.build(MC.Case(T=8, K=256, N=256, E=4, k=2, fmt="q8_0", dtype=torch.float16, seed=5))
    ffn = PreGatherFFNMOE(MC.make_theta(case, device))
    x = case.planes["h"].to(device)
    experts = torch.tensor([[0, 1]] * 7 + [[2, 4]], dtype=torch.int32, device=device)
    gate = torch.full((8, 2), 0.5, dtype=torch.float16, device=device)
    old = debugging.flags.enable_nan_checks
    try:
        debugging.flags.enable_nan_checks = True
        with pytest.raises(IndexError):
            ffn(x, experts, gate)
        debugging.flags.enable_nan_checks = False
        y = ffn(x, experts, gate)  # clamped: finite output, no fault
        assert torch.isfinite(y.float()).all()
    finally:
        debugging.flags.enable_nan_checks = old


def test_random_shapes_automatic_choice_against_vector_alu_kernel(device):
    """Seeded random shapes, formats, routings and activations: the automatically chosen kernels against the vector-ALU
    kernel (an independent implementation of the same arithmetic)."""
    import random
    from sharktank_amd import _hip as hip
    from sharktank_amd.ops import device_weight

    rng = random.Random(2024)
    for it in range(40):
        fmt = rng.choice(["q8_0", "q4_1", "fp8", "dense"])
        dtype = rng.choice([torch.float16, torch.bfloat16])
        E = rng.choice([1, 2, 3, 5, 8, 16])
        k = rng.randint(1, min(E, 3))
        K = rng.choice([256, 512, 768, 1024])
        N = rng.choice([128, 256, 384, 512, 1024])
        T = rng.choice([1, 3, 17, 33, 64, 100, 200, 330, 600, 1100])
        mode = rng.choice(["uniform", "skew", "few"])
        case = MC.build(MC.Case(T=T, K=K, N=N, E=E, k=k, fmt=fmt, dtype=dtype, seed=3000 + it))
        g = torch.Generator().manual_seed(it)
        if mode == "uniform":
            idx = torch.stack([torch.randperm(E, generator=g)[:k] for _ in range(T)])
        elif mode == "skew":
            w = torch.tensor([1.0 / (e + 1) ** 2 for e in range(E)])
            idx = torch.stack([torch.multinomial(w, k, replacement=False, generator=g) for _ in range(T)])
        else:
            idx = torch.randperm(E, generator=g)[:k].repeat(T, 1)
        what = f"case {it}: {fmt} {dtype} E={E} k={k} K={K} N={N} T={T} {mode}"
        print(what, flush=True)
        dws = [device_weight(MC.to_inference_tensor(fmt, case.planes[n], shp, n, device), stacked=True, prepack=True)
               for n, shp in (("gate", [E, N, K]), ("up", [E, N, K]), ("down", [E, K, N]))]
        _, offsets, perm, _ = hip.dispatch_build(idx.to(torch.int32).to(device), E)
        x = case.planes["h"].to(device)
        act = rng.choice([hip.ACT_SILU, hip.ACT_GELU_ERF])
        auto = hip.grouped_ffn(x, *dws, act, offsets, perm, k, variant=hip.VARIANT_AUTO)
        alu = hip.grouped_ffn(x, *dws, act, offsets, perm, k, variant=hip.VARIANT_GENERIC)
        err = O.rel_l2(auto.float().cpu(), alu.float().cpu())
        assert torch.isfinite(auto.float()).all() and err < (2e-3 if dtype == torch.float16 else 1.2e-2), f"{what}: rel-L2 {err:.3e}"
