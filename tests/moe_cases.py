"""Seeded synthetic MoE layers shared by the parity tests: CPU planes for the oracle and the same planes wrapped
in the product's tensor types for the device.  Weights and the router matrix are N(0, 0.02), activations N(0, 1),
generated on the CPU with torch.manual_seed(seed)."""

from __future__ import annotations

from dataclasses import dataclass, field
from typing import Optional

import torch
import torch.nn.functional as F

from oracle import moe_oracle as O


@dataclass
class Case:
    T: int
    K: int
    N: int
    E: int = 8
    k: int = 2
    fmt: str = "q8_0"  # dense | q8_0 | q4_1 | fp8
    dtype: torch.dtype = torch.float16
    act: str = "silu"
    seed: int = 0
    eps: float = 1e-5
    out_norm: bool = False
    act_quant: bool = False  # static per-tensor e4m3fn quantizers on the FFN input and on the gated intermediate
    router_bias: Optional[torch.Tensor] = None  # added to the router rows' effect via a skewed input direction
    planes: dict = field(default_factory=dict)

    @property
    def activation(self):
        return F.silu if self.act == "silu" else F.gelu


def _quantize(fmt: str, w: torch.Tensor):
    if fmt == "q8_0":
        d, qs = O.quantize_q8_0(w)
        return {"d": d, "qs": qs}
    if fmt == "q4_1":
        d, m, qs = O.quantize_q4_1(w)
        return {"d": d, "m": m, "qs": qs}
    if fmt == "fp8":
        d, qs = O.quantize_fp8_per_tensor(w)
        return {"d": d, "qs": qs}
    raise ValueError(fmt)


def dense_from_planes(fmt: str, p: dict, shape, dtype: torch.dtype) -> torch.Tensor:
    """The reference's dequantize-then-cast view of a weight (unbox_tensor -> .to(lhs.dtype))."""
    if fmt == "dense":
        return p["w"].to(dtype)
    if fmt == "q8_0":
        return O.dequant_block_scaled(p["d"], p["qs"]).reshape(shape).to(dtype)
    if fmt == "q4_1":
        return O.dequant_block_scaled_i4(p["d"], p["qs"], p["m"]).reshape(shape).to(dtype)
    if fmt == "fp8":
        return O.dequant_tensor_scaled(p["d"], p["qs"]).to(dtype)
    raise ValueError(fmt)


def build(case: Case, dense_dtype: Optional[torch.dtype] = None) -> Case:
    g = torch.Generator().manual_seed(case.seed)
    E, N, K = case.E, case.N, case.K
    raw = {
        "gate": torch.randn(E, N, K, generator=g) * 0.02,
        "up": torch.randn(E, N, K, generator=g) * 0.02,
        "down": torch.randn(E, K, N, generator=g) * 0.02,
    }
    case.planes = {}
    for name, w in raw.items():
        if case.fmt == "dense":
            case.planes[name] = {"w": w.to(dense_dtype or case.dtype)}
        else:
            case.planes[name] = _quantize(case.fmt, w)
    case.planes["router"] = torch.randn(E, K, generator=g) * 0.02
    case.planes["ffn_norm"] = torch.ones(K) + 0.1 * torch.randn(K, generator=g)
    case.planes["out_norm"] = (torch.ones(K) + 0.1 * torch.randn(K, generator=g)) if case.out_norm else None
    case.planes["h"] = torch.randn(case.T, K, generator=g).to(case.dtype)
    case.planes["x_rscale"] = case.planes["z_rscale"] = None
    if case.act_quant:
        # calibrate as a static quantizer would be: amax over a sample of the unquantised activations, 448 = e4m3fn max
        xn = O.rms_norm(case.planes["h"][:16], case.planes["ffn_norm"], case.eps)
        wg, wu, _ = dense_weights(case)
        z = case.activation(O._mm_rt(xn, wg[0])) * O._mm_rt(xn, wu[0])
        case.planes["x_rscale"] = (xn.float().abs().amax() * 1.25 / 448.0).to(torch.float32)
        case.planes["z_rscale"] = (z.float().abs().amax() * 2.0 / 448.0).to(torch.float32)
    return case


def dense_weights(case: Case):
    E, N, K = case.E, case.N, case.K
    return (
        dense_from_planes(case.fmt, case.planes["gate"], [E, N, K], case.dtype),
        dense_from_planes(case.fmt, case.planes["up"], [E, N, K], case.dtype),
        dense_from_planes(case.fmt, case.planes["down"], [E, K, N], case.dtype),
    )


def to_inference_tensor(fmt: str, p: dict, shape, name: str, device):
    from sharktank_amd import types as ST

    if fmt == "dense":
        return ST.DefaultPrimitiveTensor(name=name, data=p["w"].to(device))
    if fmt == "q8_0":
        layout = ST.BlockScaledLayout(shape, p["d"].to(device), p["qs"].to(device))
    elif fmt == "q4_1":
        layout = ST.BlockScaledI4Layout(shape, p["d"].to(device), p["qs"].to(device), m=p["m"].to(device), signed=False)
    elif fmt == "fp8":
        layout = ST.TensorScaledLayout(shape=shape, d=p["d"].to(device), qs=p["qs"].to(device))
    else:
        raise ValueError(fmt)
    return ST.PlanarQuantizedTensor(name=name, shape=shape, layout=layout)


def make_theta(case: Case, device):
    from sharktank_amd import types as ST

    E, N, K = case.E, case.N, case.K
    tensors = {
        "ffn_gate_inp.weight": ST.DefaultPrimitiveTensor(name="ffn_gate_inp.weight", data=case.planes["router"].to(device)),
        "ffn_norm.weight": ST.DefaultPrimitiveTensor(name="ffn_norm.weight", data=case.planes["ffn_norm"].to(device)),
        "ffn_gate_exps.weight": to_inference_tensor(case.fmt, case.planes["gate"], [E, N, K], "ffn_gate_exps.weight", device),
        "ffn_up_exps.weight": to_inference_tensor(case.fmt, case.planes["up"], [E, N, K], "ffn_up_exps.weight", device),
        "ffn_down_exps.weight": to_inference_tensor(case.fmt, case.planes["down"], [E, K, N], "ffn_down_exps.weight", device),
    }
    if case.act_quant:
        for key, rs in (("ffn_gate_exps.q_input", case.planes["x_rscale"]), ("ffn_down_exps.q_input", case.planes["z_rscale"])):
            tensors[key] = ST.StaticScaledQuantizer(name=key, scale=(1.0 / rs).to(device), reciprocal_scale=rs.to(device),
                                                    dtype=torch.float8_e4m3fn)
    if case.planes["out_norm"] is not None:
        tensors["layer_output_norm.weight"] = ST.DefaultPrimitiveTensor(
            name="layer_output_norm.weight", data=case.planes["out_norm"].to(device))
    return ST.Theta(tensors)


def oracle_block(case: Case, formulation: str = "grouped", ordered_logits: bool = True):
    wg, wu, wd = dense_weights(case)
    return O.moe_block(
        case.planes["h"], case.planes["ffn_norm"], case.planes["router"], wg, wu, wd, case.k, case.eps,
        case.activation, out_norm_w=case.planes["out_norm"], formulation=formulation, ordered_logits=ordered_logits,
        x_rscale=case.planes["x_rscale"], z_rscale=case.planes["z_rscale"],
    )
