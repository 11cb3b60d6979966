"""The MoE side of the model loops: MoeBlocks stacked from the `blk.<n>.*` sub-trees of one theta, prefill and decode
block after block, the decode step replayed as a HIP graph, and the golden dumps of the loop's trace points reproduced by
the CPU oracle block by block (sharktank/sharktank/models/mixtral/mixtral.py:111-233 without attention, KV cache and
embeddings)."""

import pytest
import torch

from oracle import moe_oracle as O
import moe_cases as MC

pytestmark = pytest.mark.gpu

L, E, KTOP, K, N = 3, 8, 2, 512, 768


def build_stack(device, dtype=torch.float16, fmt="q8_0", token_mixer=None):
    from sharktank_amd import types as ST
    from sharktank_amd.models import MoeStack

    cases, tensors = [], {}
    for n in range(L):
        case = MC.build(MC.Case(T=1, K=K, N=N, E=E, k=KTOP, fmt=fmt, dtype=dtype, seed=700 + n))
        cases.append(case)
        for name, t in MC.make_theta(case, device).flatten().items():
            tensors[f"blk.{n}.{name}"] = t
    stack = MoeStack(ST.Theta(tensors), block_count=L, expert_count=E, expert_used_count=KTOP, rms_epsilon=1e-5,
                     token_mixer=token_mixer)
    return stack, cases


def oracle_block(case, h):
    wg, wu, wd = MC.dense_weights(case)
    y, idx, _ = O.moe_block(h, case.planes["ffn_norm"], case.planes["router"], wg, wu, wd, KTOP, 1e-5, case.activation)
    return y, idx


def mixer(block_idx, h):
    """Stands in for the attention block: mixes neighbouring tokens (a roll along the sequence) and rescales."""
    return (0.5 * h + 0.5 * torch.roll(h, 1, dims=1)).to(h.dtype)


def test_prefill_golden_dumps_reproduced_by_the_oracle(device, tmp_path):
    from safetensors.torch import load_file
    from sharktank_amd.utils import debugging

    stack, cases = build_stack(device, token_mixer=mixer)
    h = torch.randn(2, 48, K, generator=torch.Generator().manual_seed(1)).to(torch.float16)
    old = (debugging.flags.save_goldens_path, debugging.flags.golden_sequence_value)
    try:
        debugging.flags.save_goldens_path = tmp_path
        debugging.flags.golden_sequence_value = 0
        out = stack.prefill(h.to(device)).cpu()
    finally:
        debugging.flags.save_goldens_path, debugging.flags.golden_sequence_value = old
    files = sorted(p.name for p in tmp_path.iterdir())
    # per block: the input that enters the MoE block (the reference's attn_block output), the block's own record
    # (routing and output), and the loop's trace point after the block
    assert len(files) == 3 * L, files
    for n in range(L):
        x_in = load_file(str(tmp_path / [f for f in files if f.endswith(f"mixtral.attn_block.{n}.output.safetensors")][0]))["default"]
        rec = load_file(str(tmp_path / [f for f in files if f.endswith("_moe_block.safetensors")][n]))
        y_out = load_file(str(tmp_path / [f for f in files if f.endswith(f"mixtral.moe_block.{n}.output.safetensors")][0]))["default"]
        assert torch.equal(rec["output"], y_out)
        want, want_idx = oracle_block(cases[n], x_in.reshape(-1, K))
        assert torch.equal(rec["top_k_experts"].long(), want_idx), f"block {n}: routing differs from the oracle"
        hin = x_in.reshape(-1, K).float()
        err = O.rel_l2(y_out.reshape(-1, K).float() - hin, want.float() - hin)
        assert err < 1e-3, f"block {n}: MoE contribution rel-L2 {err:.3e}"
    assert torch.equal(out, y_out)
    # the loop as a whole against the oracle's own loop (errors may add up over the blocks; routing is compared per block above)
    hh = h
    for n in range(L):
        hh = mixer(n, hh)
        hh = oracle_block(cases[n], hh.reshape(-1, K))[0].reshape(h.shape)
    assert O.rel_l2(out, hh) < 2e-3


@pytest.mark.parametrize("dtype,fmt", [(torch.float16, "q8_0"), (torch.bfloat16, "q4_1")])
def test_decode_graph_replays_equal_eager_steps(device, dtype, fmt):
    """A decode loop of 6 steps, each step's output fed back (normalised) as the next input: every replay of the captured
    step is compared bit for bit with the same step run eagerly, with eager work and synchronisations between replays."""
    stack, cases = build_stack(device, dtype=dtype, fmt=fmt)
    bs = 4
    h0 = torch.randn(bs, 1, K, generator=torch.Generator().manual_seed(2)).to(dtype).to(device)
    eager = []
    h = h0
    for step in range(6):
        y = stack.decode(h)  # no graph yet: eager
        eager.append(y.clone())
        h = (y / y.float().pow(2).mean(dim=-1, keepdim=True).sqrt().to(dtype)).to(dtype)
    torch.cuda.synchronize()
    stack.capture_decode(bs, dtype, device)
    assert stack._graph is not None
    h = h0
    for step in range(6):
        y = stack.decode(h)  # replays the graph
        torch.cuda.synchronize()
        assert torch.equal(y.view(torch.int16), eager[step].view(torch.int16)), f"step {step}: replay differs from the eager step"
        # eager work between replays: the same blocks at another batch size, and a reduction of torch's own
        stack.moe_blocks[0](torch.randn(1, 7, K, device=device).to(dtype))
        assert torch.isfinite(y.float().sum()).item()
        h = (y / y.float().pow(2).mean(dim=-1, keepdim=True).sqrt().to(dtype)).to(dtype)
    # the first step against the oracle
    want = h0.cpu().reshape(bs, K)
    for n in range(L):
        want = oracle_block(cases[n], want)[0]
    assert O.rel_l2(eager[0].cpu().reshape(bs, K), want) < (2e-3 if dtype == torch.float16 else 1e-2)
    # another batch size falls back to the eager loop
    y2 = stack.decode(h0[:2])
    assert y2.shape == (2, 1, K)
    stack.release_decode_graph()
