"""The forward that allocates nothing (stmoe_moe_forward_static) against stmoe_moe_forward with a caller-owned
workspace: the same kernels on the same inputs, so outputs, routing indices and gates must be identical bit for bit.
Two calls in a row share the library's built-in workspace; the second one is smaller, so whatever the first call left
behind in the array must not leak into it."""

import ctypes

import pytest
import torch

import moe_cases as MC
from sharktank_amd import _hip
from sharktank_amd.layers import MoeBlock
from sharktank_amd.types import unbox_tensor

pytestmark = pytest.mark.gpu


def _both(block, case, T, dev):
    """(static-workspace result, caller-workspace result) for the first T tokens of the case."""
    h = case.planes["h"][:T].to(dev).contiguous()
    wg, wu, wd = block.experts.device_weights()
    norm_w = unbox_tensor(block.ffn_norm.weight)
    out_norm_w = unbox_tensor(block.layer_output_norm.weight) if case.out_norm else None
    router_w = block._router_weight(h.dtype)
    xs, zs = (_hip._scale1(s) for s in block.experts.activation_scales())
    out = torch.full_like(h, float("nan"))
    idx = torch.full((T, case.k), -1, dtype=torch.int32, device=dev)
    gate = torch.full((T, case.k), float("nan"), dtype=h.dtype, device=dev)
    _hip.moe_forward_static(h, norm_w, out_norm_w, case.eps, router_w, wg, wu, wd, block.experts._act, case.k, out,
                            idx=idx, gate=gate, x_scale=xs, z_scale=zs)
    want, want_idx, want_gate = _hip.moe_forward(h, norm_w, out_norm_w, case.eps, router_w, wg, wu, wd, block.experts._act,
                                                 case.k, want_routing=True, x_scale=xs, z_scale=zs)
    torch.cuda.synchronize()
    return (out, idx, gate), (want, want_idx, want_gate)


@pytest.mark.parametrize("fmt,dtype,act,out_norm", [
    ("q8_0", torch.float16, "silu", False),
    ("q4_1", torch.bfloat16, "gelu", True),
    ("fp8", torch.float16, "silu", False),
])
def test_static_workspace_forward_equals_caller_workspace_forward(device, fmt, dtype, act, out_norm):
    case = MC.build(MC.Case(T=64, K=512, N=1024, fmt=fmt, dtype=dtype, act=act, out_norm=out_norm, seed=11))
    block = MoeBlock(MC.make_theta(case, device), case.E, case.k, case.eps, moe_activation=case.activation)
    for T in (64, 24, 1):  # in a row on one GPU: each call finds the previous call's contents in the array
        got, want = _both(block, case, T, device)
        assert torch.equal(got[1], want[1]), f"T={T}: routing indices differ"
        assert torch.equal(got[2].view(torch.int16), want[2].view(torch.int16)), f"T={T}: gates differ"
        assert torch.equal(got[0].view(torch.int16), want[0].view(torch.int16)), f"T={T}: outputs differ"
        assert not torch.isnan(got[0].float()).any()


def test_static_workspace_refuses_shapes_beyond_its_size(device):
    """A prefill-sized batch of a Mixtral layer needs 260 MB of workspace: refused before any launch, with a message that
    names both sizes."""
    lib = _hip.load_library()
    w = _hip.StmoeWeight(format=_hip.W_Q8_0, dtype=0, experts=8, rows=14336, cols=4096, qs=256, d=256, m=None, d_count=1)
    rc = lib.stmoe_moe_forward_static(256, _hip.F16, 2048, 4096, 14336, 8, 2, 256, None, _hip.F32, 1e-5, 256, ctypes.byref(w),
                                      ctypes.byref(w), ctypes.byref(w), 0, None, None, 256, None, None, 0, None)
    assert rc == 6
    msg = lib.stmoe_last_error().decode()
    assert str(_hip.STATIC_SCRATCH_BYTES) in msg and "workspace" in msg
    need = _hip.moe_forward_workspace_bytes(32, 2, 8, 4096, 14336, torch.float16)
    assert need <= _hip.STATIC_SCRATCH_BYTES, "a 32-token Mixtral decode step must fit the built-in workspace"
