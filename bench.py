#!/usr/bin/env python3
"""Benchmark of the MoE layer hot path on one MI355X.

Workload (BASELINE.json configs[1]): one Mixtral-8x7B MoE layer, Q8_0 block-scaled expert weights, hidden 4096,
FFN 14336, 8 experts, top-2, SiLU, fp16 activations; prefill with 2048 tokens (the headline metric) and decode
with 32 tokens (reported beside it).  A step is one forward of the layer over the batch, inputs resident in HBM, issued
as the single C-ABI call that MoeBlock.forward makes (stmoe_moe_forward, with the workspace allocated once);
`e2e_ms_per_step` is the same step through MoeBlock.forward itself (Python layer included).

Prints ONE JSON line.  `value` = prefill tokens/s.  `roofline` prices the dominant prefill kernel (the fused
gate/up projection) against the dense fp16 MFMA peak; `decode.roofline` prices the same kernel at T=32 against
HBM bandwidth on its expert-weight bytes.  Kernel durations are measured live with HIP events recorded on the
launch stream around the kernel, in a pass of the same K steps right before the timed one (an event between two
launches costs stream time, so the step time itself is taken without events).  `cpu_baseline` times the CPU oracle (a restatement of
the reference's eager per-token-gather algorithm) on the host cores for a bounded token sample.
`configs` holds one short leg for each of the other BASELINE configurations (3: Q4_1 / bf16 decode sweep, 4: Grok shape
with skewed routing, 5: fp8 weights and activations) and for the dense quantized linear next to the path; the headline
line is not affected by them (`--no-configs` skips them).
"""

import argparse
import ctypes
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.join(ROOT, "shark-platform_amd"))
sys.path.insert(0, ROOT)

K_HID, N_FFN, E, TOPK = 4096, 14336, 8, 2
HBM_PEAK_GBPS = 8000.0
MFMA_F16_PEAK_TFLOPS = 2500.0
STAGES = ["ffn_norm", "router", "dispatch", "gate_up", "down", "combine"]


def quantize_q8_0(w):
    """ggml Q8_0 convention: per 32-block d = amax/127 (fp16), q = round(w/d) (int8).  Synthetic-data helper."""
    import torch

    wb = w.reshape(*w.shape[:-1], -1, 32)
    d = wb.abs().amax(dim=-1, keepdim=True) / 127.0
    inv = torch.where(d > 0, 1.0 / d, torch.zeros_like(d))
    qs = torch.round(wb * inv).clamp_(-127, 127).to(torch.int8)
    return d.to(torch.float16), qs


def quantize_q4_1(w):
    """ggml Q4_1 convention: per 32-block d = (max - min) / 15, m = min (fp16), q = round((w - m) / d) in 0..15, two per
    byte in linear order (element 2i in the low nibble).  Synthetic-data helper."""
    import torch

    wb = w.reshape(*w.shape[:-1], -1, 32)
    mn = wb.amin(dim=-1, keepdim=True)
    d = (wb.amax(dim=-1, keepdim=True) - mn) / 15.0
    inv = torch.where(d > 0, 1.0 / d, torch.zeros_like(d))
    q = torch.floor((wb - mn) * inv + 0.5).clamp_(0, 15).to(torch.uint8)
    return d.to(torch.float16), mn.to(torch.float16), q[..., 0::2] | (q[..., 1::2] << 4)


def build_layer(dev, seed=0, fmt="q8_0", K=K_HID, N=N_FFN, act=None, out_norm=False, router=None, act_quant=None):
    """One MoE layer with synthetic weights N(0, 0.02) quantised on the device.  `router`: optional [E, K] matrix;
    `act_quant`: optional (x reciprocal scale, z reciprocal scale) of static e4m3fn activation quantizers."""
    import torch
    import torch.nn.functional as F
    from sharktank_amd import types as ST
    from sharktank_amd.layers import MoeBlock

    g = torch.Generator(device="cpu").manual_seed(seed)
    gg = torch.Generator(device=dev).manual_seed(seed)
    tensors = {}
    for name, shape in (("ffn_gate_exps", [E, N, K]), ("ffn_up_exps", [E, N, K]), ("ffn_down_exps", [E, K, N])):
        per = []
        for e in range(E):  # per expert to bound the fp32 staging memory
            w = torch.randn(shape[1:], generator=gg, device=dev, dtype=torch.float32) * 0.02
            per.append(quantize_q8_0(w) if fmt == "q8_0" else quantize_q4_1(w) if fmt == "q4_1" else (w.to(torch.float16),))
            del w
        if fmt == "q8_0":
            layout = ST.BlockScaledLayout(shape, torch.stack([p[0] for p in per]), torch.stack([p[1] for p in per]))
        elif fmt == "q4_1":
            layout = ST.BlockScaledI4Layout(shape, torch.stack([p[0] for p in per]), torch.stack([p[2] for p in per]),
                                            m=torch.stack([p[1] for p in per]), signed=False)
        else:  # fp8 e4m3fn, one fp32 scale per tensor (amax / 448)
            w_all = torch.stack([p[0] for p in per]).float()
            d = (w_all.abs().amax() / 448.0).to(torch.float32)
            layout = ST.TensorScaledLayout(shape=shape, d=d, qs=(w_all / d).to(torch.float8_e4m3fn))
            del w_all
        del per
        tensors[f"{name}.weight"] = ST.PlanarQuantizedTensor(name=f"{name}.weight", shape=shape, layout=layout)
    if router is None:
        router = torch.randn(E, K, generator=g) * 0.02
    tensors["ffn_gate_inp.weight"] = ST.DefaultPrimitiveTensor(name="ffn_gate_inp.weight", data=router.to(dev))
    tensors["ffn_norm.weight"] = ST.DefaultPrimitiveTensor(name="ffn_norm.weight", data=torch.ones(K, device=dev))
    if out_norm:
        tensors["layer_output_norm.weight"] = ST.DefaultPrimitiveTensor(name="layer_output_norm.weight", data=torch.ones(K, device=dev))
    if act_quant is not None:
        for key, rs in (("ffn_gate_exps.q_input", act_quant[0]), ("ffn_down_exps.q_input", act_quant[1])):
            rs = torch.tensor(float(rs), dtype=torch.float32, device=dev)
            tensors[key] = ST.StaticScaledQuantizer(name=key, scale=1.0 / rs, reciprocal_scale=rs, dtype=torch.float8_e4m3fn)
    theta = ST.Theta(tensors)
    return MoeBlock(theta, E, TOPK, 1e-5, moe_activation=act or F.silu), theta


class HipEvents:
    """hipEvent_t handles created through the HIP runtime that torch already loaded."""

    def __init__(self, n):
        self.hip = ctypes.CDLL("libamdhip64.so")
        self.hip.hipEventCreate.argtypes = [ctypes.POINTER(ctypes.c_void_p)]
        self.hip.hipEventElapsedTime.argtypes = [ctypes.POINTER(ctypes.c_float), ctypes.c_void_p, ctypes.c_void_p]
        self.hip.hipEventDestroy.argtypes = [ctypes.c_void_p]
        self.arr = (ctypes.c_void_p * n)()
        for i in range(n):
            ev = ctypes.c_void_p()
            rc = self.hip.hipEventCreate(ctypes.byref(ev))
            assert rc == 0, f"hipEventCreate -> {rc}"
            self.arr[i] = ev

    def elapsed_ms(self, a, b):
        out = ctypes.c_float()
        rc = self.hip.hipEventElapsedTime(ctypes.byref(out), self.arr[a], self.arr[b])
        assert rc == 0, f"hipEventElapsedTime -> {rc}"
        return out.value

    def destroy(self):
        for ev in self.arr:
            self.hip.hipEventDestroy(ev)


def run_leg(block, h, steps, warmup, e2e=False):
    """Times `steps` forwards.  In the timed loop only the dominant kernel (the gate/up projection) is bracketed by
    HIP events on the launch stream; a second, untimed pass of the same length brackets every stage for the
    breakdown.  Returns (ms_per_step, gate_up_ms, {stage: avg ms}, out, idx[, ms per MoeBlock.forward]); the stage
    dictionary also carries "step_with_dominant_bracket", the step time of the pass that brackets the dominant kernel."""
    import torch
    from sharktank_amd import _hip
    from sharktank_amd.layers import RMSNormLayer
    from sharktank_amd.types import unbox_tensor

    T, K = h.shape[1], h.shape[2]
    x = h.reshape(T, K)
    wg, wu, wd = block.experts.device_weights()
    need = _hip.moe_forward_workspace_bytes(T, TOPK, E, K, wg.rows, h.dtype)
    ws = torch.empty(need, dtype=torch.uint8, device=h.device)
    out = torch.empty_like(x)
    norm_w = unbox_tensor(block.ffn_norm.weight)
    out_norm_w = unbox_tensor(block.layer_output_norm.weight) if isinstance(block.layer_output_norm, RMSNormLayer) else None
    router_w = block._router_weight(h.dtype)
    xs, zs = block.experts.activation_scales()
    evsets = [HipEvents(12) for _ in range(steps)]
    dominant = []
    for ev in evsets:  # the same handles, all but the gate/up bracket masked out
        arr = (ctypes.c_void_p * 12)()
        arr[6], arr[7] = ev.arr[6], ev.arr[7]
        dominant.append(arr)

    def fwd(events=None, want_routing=False):
        return _hip.moe_forward(x, norm_w, out_norm_w, block.rms_epsilon, router_w, wg, wu, wd, block.experts._act, TOPK,
                                variant=block.experts.kernel_variant, workspace=ws, out=out, events=events,
                                want_routing=want_routing, x_scale=xs, z_scale=zs)

    # Order: first the two instrumented passes (every stage bracketed by HIP events on the launch stream, then only the
    # dominant kernel), which also bring the clocks up; then W warm-up steps and the K timed steps without any event
    # (recording an event between two launches costs stream time: several per cent of a 32-token step).
    for _ in range(warmup):
        fwd()
    for s in range(steps):
        fwd(evsets[s].arr)
    torch.cuda.synchronize()
    stage_ms = {name: sum(ev.elapsed_ms(2 * i, 2 * i + 1) for ev in evsets) / steps for i, name in enumerate(STAGES)}
    t0 = time.perf_counter()
    for s in range(steps):
        fwd(dominant[s])
    torch.cuda.synchronize()
    stage_ms["step_with_dominant_bracket"] = (time.perf_counter() - t0) * 1e3 / steps
    gate_up_ms = sum(ev.elapsed_ms(6, 7) for ev in evsets) / steps

    for _ in range(warmup):
        fwd()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for s in range(steps):
        fwd()
    torch.cuda.synchronize()
    ms = (time.perf_counter() - t0) * 1e3 / steps
    for ev in evsets:
        ev.destroy()
    _, idx, _ = fwd(want_routing=True)
    if not e2e:
        return ms, gate_up_ms, stage_ms, out, idx
    for _ in range(warmup):
        block(h)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for s in range(steps):
        block(h)
    torch.cuda.synchronize()
    return ms, gate_up_ms, stage_ms, out, idx, (time.perf_counter() - t0) * 1e3 / steps


def cpu_model():
    try:
        with open("/proc/cpuinfo") as f:
            for line in f:
                if line.startswith("model name"):
                    return line.split(":", 1)[1].strip()
    except OSError:
        pass
    return "unknown"


def config_legs(dev, steps, warmup):
    """Short legs for BASELINE configurations 3, 4, 5 and the dense quantized linear: {name: figures}."""
    import torch
    import torch.nn.functional as F
    from sharktank_amd import _hip
    from sharktank_amd.layers import PreGatherFFNMOE
    from sharktank_amd.ops import device_weight

    legs = {}
    g = torch.Generator().manual_seed(11)

    # configuration 3: Mixtral shape, Q4_1, bf16, decode sweep; HBM-bound on the weights of the experts that are hit
    block, theta = build_layer(dev, seed=3, fmt="q4_1")
    sweep = {}
    for T in (1, 8, 32, 128):
        h = torch.randn(1, T, K_HID, generator=g).to(torch.bfloat16).to(dev)
        ms, gu_ms, st, _, idx = run_leg(block, h, max(steps, 30), warmup)
        hit = int(torch.unique(idx).numel())
        wbytes = hit * N_FFN * K_HID * 20.0 / 32.0  # Q4_1 bytes of one matrix, experts that are hit only
        sweep[str(T)] = {"ms_per_step": round(ms, 4), "tokens_per_s": round(T / (ms * 1e-3), 1), "experts_hit": hit,
                         "layer_frac_hbm": round(3 * wbytes / (ms * 1e-3) / 1e9 / HBM_PEAK_GBPS, 4),
                         "gate_up_ms": round(gu_ms, 4),
                         "gate_up_frac_hbm": round(2 * wbytes / (gu_ms * 1e-3) / 1e9 / HBM_PEAK_GBPS, 4)}
    legs["c3_mixtral_q4_1_bf16_decode"] = {"bound": "hbm", "peak_GBps": HBM_PEAK_GBPS, "tokens": sweep}
    del block, theta
    torch.cuda.empty_cache()

    # configuration 4: Grok-1 shape, Q4_1, fp16, GELU, output norm, 1024 tokens, Zipf prior (p_e ~ 1/(e+1)) on the router
    K4, N4, T4 = 6144, 32768, 1024
    u = torch.randn(K4, generator=g)
    u = u / u.norm()
    router0 = torch.randn(E, K4, generator=g) * 0.02
    h = (torch.randn(1, T4, K4, generator=g) + 40.0 * u.reshape(1, 1, -1)).to(torch.float16)
    # Zipf exponent: the one (of a small grid) whose routing, estimated with plain fp32 arithmetic on the host, puts the
    # share of the two busiest experts closest to the stated 60 %; the realised histogram is read back from the GPU run
    xn = h[0].float()
    xn = xn * torch.rsqrt(xn.pow(2).mean(dim=1, keepdim=True) + 1e-5)
    best = None
    for zipf in [0.4 + 0.1 * i for i in range(13)]:
        logp = torch.log(1.0 / (torch.arange(E, dtype=torch.float32) + 1.0) ** zipf)
        cand = router0 + (logp - logp.mean()).reshape(E, 1) * u.reshape(1, -1) / 40.0
        top = torch.topk(xn @ cand.t(), TOPK, dim=1).indices
        c = torch.bincount(top.reshape(-1), minlength=E).sort(descending=True).values
        share = float(c[:2].sum()) / float(c.sum())
        if best is None or abs(share - 0.60) < abs(best[0] - 0.60):
            best = (share, zipf, cand)
    _, zipf, router = best
    block, theta = build_layer(dev, seed=4, fmt="q4_1", K=K4, N=N4, act=F.gelu, out_norm=True, router=router)
    h = h.to(dev)
    ms, gu_ms, st, _, idx = run_leg(block, h, steps, warmup)
    counts = torch.bincount(idx.reshape(-1).long().cpu(), minlength=E).tolist()
    fl = 2.0 * T4 * TOPK * 2 * N4 * K4
    legs["c4_grok_q4_1_f16_prefill"] = {
        "tokens": T4, "ms_per_step": round(ms, 4), "tokens_per_s": round(T4 / (ms * 1e-3), 1),
        "zipf_exponent": round(zipf, 2), "pairs_per_expert": counts, "top2_share": round(sum(sorted(counts)[-2:]) / sum(counts), 3),
        "gate_up_ms": round(gu_ms, 4), "bound": "mfma", "peak_TFLOPs": MFMA_F16_PEAK_TFLOPS,
        "gate_up_frac": round(fl / (gu_ms * 1e-3) / 1e12 / MFMA_F16_PEAK_TFLOPS, 4),
        "layer_tflops": round(1.5 * fl / (ms * 1e-3) / 1e12, 1), "stage_ms": {k: round(v, 4) for k, v in st.items()}}
    del block, theta, h
    torch.cuda.empty_cache()

    # configuration 5: Mixtral shape, fp8 e4m3 weights and static fp8 activation quantizers; 4096 tokens with the stated
    # uniform routing (token t -> experts 2t, 2t+1 mod 8) through PreGatherFFNMOE.forward, and a one-token forward
    T5 = 4096
    block, theta = build_layer(dev, seed=5, fmt="fp8", act_quant=(4.0 * 1.25 / 448.0, 8.0 * 2.0 / 448.0))
    x = torch.randn(T5, K_HID, generator=g).to(torch.float16).to(dev)
    t = torch.arange(T5)
    experts = torch.stack([(2 * t) % E, (2 * t + 1) % E], dim=1).to(torch.int32).to(dev)
    gates = torch.full((T5, TOPK), 0.5, dtype=torch.float16, device=dev)
    fl5 = 2.0 * T5 * TOPK * 3 * N_FFN * K_HID
    c5 = {"tokens": T5, "routing": "token t -> experts 2t mod 8, 2t+1 mod 8"}
    # the default for fp16 activations is the fp8 matrix-core arithmetic; VARIANT_STEP_BY_STEP is the reference's
    # quantise, dequantise, multiply in fp16
    for label, variant, peak in (("dequantise_then_f16_mfma", _hip.VARIANT_STEP_BY_STEP, MFMA_F16_PEAK_TFLOPS),
                                 ("fp8_mfma", _hip.VARIANT_AUTO, 5000.0)):
        ffn = PreGatherFFNMOE(theta)
        ffn._dw = block.experts.device_weights()
        ffn.kernel_variant = variant
        for _ in range(warmup):
            ffn(x, experts, gates)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(steps):
            ffn(x, experts, gates)
        torch.cuda.synchronize()
        ms = (time.perf_counter() - t0) * 1e3 / steps
        c5[label] = {"ms_per_step": round(ms, 4), "tokens_per_s": round(T5 / (ms * 1e-3), 1), "bound": "mfma", "peak_TFLOPs": peak,
                     "ffn_tflops": round(fl5 / (ms * 1e-3) / 1e12, 1), "ffn_frac": round(fl5 / (ms * 1e-3) / 1e12 / peak, 4)}
    h1 = torch.randn(1, 1, K_HID, generator=g).to(torch.float16).to(dev)
    ms, gu_ms, st, _, idx = run_leg(block, h1, max(steps, 50), warmup)
    wb = 2 * N_FFN * K_HID * 1.0  # two experts, one byte per weight
    c5["decode_1_token"] = {"latency_us": round(ms * 1e3, 1), "layer_frac_hbm": round(3 * wb / (ms * 1e-3) / 1e9 / HBM_PEAK_GBPS, 4)}
    legs["c5_mixtral_fp8"] = c5
    del block, theta
    torch.cuda.empty_cache()

    # the dense quantized linear next to the path: ops.matmul(x, Q8_0 weight) on one [14336, 4096] matrix
    gg = torch.Generator(device=dev).manual_seed(9)
    from sharktank_amd import types as ST

    d, qs = quantize_q8_0(torch.randn(N_FFN, K_HID, generator=gg, device=dev) * 0.02)
    w = ST.PlanarQuantizedTensor(name="w", shape=[N_FFN, K_HID], layout=ST.BlockScaledLayout([N_FFN, K_HID], d, qs))
    dw = device_weight(w, stacked=False, prepack=True)
    lin = {}
    for M in (1, 32, 256, 2048):
        a = torch.randn(M, K_HID, generator=g).to(torch.float16).to(dev)
        for _ in range(warmup):
            _hip.mmt(a, dw)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(max(steps, 50)):
            _hip.mmt(a, dw)
        torch.cuda.synchronize()
        ms = (time.perf_counter() - t0) * 1e3 / max(steps, 50)
        lin[str(M)] = {"us": round(ms * 1e3, 1), "tflops": round(2.0 * M * N_FFN * K_HID / (ms * 1e-3) / 1e12, 1),
                       "weight_GBps": round(N_FFN * K_HID * 34.0 / 32.0 / (ms * 1e-3) / 1e9, 1)}
    legs["dense_linear_q8_0_14336x4096"] = {"rows": lin}
    return legs


def cpu_baseline(theta, h_cpu, sample_tokens):
    """The oracle's per-token-gather formulation (the reference's eager algorithm) on the host cores."""
    import torch
    from oracle import moe_oracle as O

    torch.set_num_threads(os.cpu_count() if (os.cpu_count() or 1) <= 16 else 16)
    cores = torch.get_num_threads()
    dense = []
    for name in ("ffn_gate_exps", "ffn_up_exps", "ffn_down_exps"):
        lay = theta.tensor(name, "weight").unpack()
        d, qs = lay.d.cpu(), lay.qs.cpu()
        dense.append(O.dequant_block_scaled(d, qs).reshape(lay.shape))
    router = theta.tensor("ffn_gate_inp", "weight").as_torch().cpu()
    norm_w = theta.tensor("ffn_norm", "weight").as_torch().cpu()
    hs = h_cpu[:sample_tokens]
    t0 = time.perf_counter()
    y_gather, _, _ = O.moe_block(hs, norm_w, router, dense[0], dense[1], dense[2], TOPK, 1e-5, formulation="gather")
    t_gather = time.perf_counter() - t0
    t0 = time.perf_counter()
    y_grouped, _, _ = O.moe_block(hs, norm_w, router, dense[0], dense[1], dense[2], TOPK, 1e-5, formulation="grouped")
    t_grouped = time.perf_counter() - t0
    return {
        "value": round(sample_tokens / t_gather, 3),
        "unit": "tokens/s",
        "cores": cores,
        "cpu_model": cpu_model(),
        "kind": "port",
        "sample": f"first {sample_tokens} of the 2048 prefill tokens, reference per-token-gather formulation in chunks of 8 "
                  f"({t_gather:.1f} s); per-expert grouped formulation of the same tokens: {sample_tokens / t_grouped:.2f} tokens/s",
    }, y_gather


def measured_traffic(key):
    """HBM bytes per launch from the committed rocprofv3 counter runs (profiles/traffic.json), or None."""
    try:
        with open(os.path.join(ROOT, "profiles", "traffic.json")) as f:
            t = json.load(f)[key]
        return t["read_bytes"] + t["write_bytes"]
    except (OSError, KeyError, ValueError):
        return None


def traffic_measured_at():
    """Which sources the counter runs behind profiles/traffic.json were made with (the file's own stamp), or None."""
    try:
        with open(os.path.join(ROOT, "profiles", "traffic.json")) as f:
            return json.load(f).get("measured_at")
    except (OSError, ValueError):
        return None


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--prefill-tokens", type=int, default=2048)
    ap.add_argument("--decode-tokens", type=int, default=32)
    ap.add_argument("--cpu-sample", type=int, default=16, help="tokens timed on the CPU baseline (0 to skip)")
    ap.add_argument("--no-configs", action="store_true", help="skip the legs of the other BASELINE configurations")
    ap.add_argument("--no-probe", action="store_true", help="skip the matrix-core ceiling probe")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="also run a plain 1 GiB device copy (5 times) so that rocprofv3 FETCH_SIZE/WRITE_SIZE readings "
                         "of the kernels can be scaled by what the same counters read for a copy of known size")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py measures one GPU: every box of this run has a single MI355X, so --gpus must be 1", file=sys.stderr)
        sys.exit(2)

    import torch

    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    block, theta = build_layer(dev)
    g = torch.Generator().manual_seed(1)
    h_pre = torch.randn(1, args.prefill_tokens, K_HID, generator=g).to(torch.float16)
    h_dec = torch.randn(1, args.decode_tokens, K_HID, generator=g).to(torch.float16)

    ms, gu_ms, st, out_pre, _, e2e_ms = run_leg(block, h_pre.to(dev), args.steps, args.warmup, e2e=True)
    T = args.prefill_tokens
    gateup_flops = 2.0 * T * TOPK * 2 * N_FFN * K_HID
    layer_flops = 2.0 * T * TOPK * 3 * N_FFN * K_HID + 2.0 * T * E * K_HID
    achieved = gateup_flops / (gu_ms * 1e-3) / 1e12
    roofline = {
        "kernel": "grouped gate/up projection (prefill)", "bound": "mfma", "achieved": round(achieved, 2),
        "peak": MFMA_F16_PEAK_TFLOPS, "unit": "TFLOP/s", "frac": round(achieved / MFMA_F16_PEAK_TFLOPS, 4),
        "traffic": measured_traffic("prefill_gate_up") if T == 2048 else None, "traffic_measured_at": traffic_measured_at(),
        "avg_kernel_ms": round(gu_ms, 4), "algorithmic": gateup_flops, "algorithmic_unit": "flop per launch",
    }

    dms, dgu_ms, dst, _, _, de2e_ms = run_leg(block, h_dec.to(dev), max(args.steps, 50), args.warmup, e2e=True)
    wbytes_one = E * N_FFN * K_HID * 34.0 / 32.0  # Q8_0 bytes of one stacked matrix (all 8 experts are hit at T=32)
    d_achieved = 2 * wbytes_one / (dgu_ms * 1e-3) / 1e9
    decode = {
        "tokens": args.decode_tokens, "steps": max(args.steps, 50), "ms_per_step": round(dms, 4),
        "e2e_ms_per_step": round(de2e_ms, 4),
        "tokens_per_s": round(args.decode_tokens / (dms * 1e-3), 1),
        "layer_weight_GBps": round(3 * wbytes_one / (dms * 1e-3) / 1e9, 1),
        "layer_frac_hbm": round(3 * wbytes_one / (dms * 1e-3) / 1e9 / HBM_PEAK_GBPS, 4),
        "stage_ms": {k: round(v, 4) for k, v in dst.items()},
        "roofline": {"kernel": "grouped gate/up projection (decode)", "bound": "hbm", "achieved": round(d_achieved, 1),
                     "peak": HBM_PEAK_GBPS, "unit": "GB/s", "frac": round(d_achieved / HBM_PEAK_GBPS, 4),
                     "traffic": measured_traffic("decode_gate_up") if args.decode_tokens == 32 else None,
                     "avg_kernel_ms": round(dgu_ms, 4), "algorithmic": 2 * wbytes_one,
                     "algorithmic_unit": "expert-weight bytes per launch"},
    }

    # What the matrix cores of this very machine sustain on nothing but MFMA instructions (the chip lowers its clock with
    # their activity and with the switching of the operand bits): the practical ceiling beside the data-sheet one.
    probe = None
    if not args.no_probe:
        from sharktank_amd import _hip

        probe = {
            "f16_random_operands_TFLOPs": round(_hip.probe_mfma(dev, 0, True), 1),
            "f16_constant_operands_TFLOPs": round(_hip.probe_mfma(dev, 0, False), 1),
            "fp8_random_operands_TFLOPs": round(_hip.probe_mfma(dev, 1, True), 1),
            "fp8_constant_operands_TFLOPs": round(_hip.probe_mfma(dev, 1, False), 1),
            "what": "256 workgroups x 8 wavefronts of independent v_mfma_f32_16x16x32_f16 / v_mfma_scale_f32_32x32x64_f8f6f4 "
                    "on register operands; 8 timed launches of 20000 loop passes after 12 untimed ones",
        }
        roofline["frac_of_mfma_only_probe"] = round(achieved / probe["f16_random_operands_TFLOPs"], 4)

    if args.copy_calibration:
        src = torch.empty(1 << 30, dtype=torch.uint8, device=dev).fill_(1)
        dst = torch.empty_like(src)
        for _ in range(5):
            dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst

    cpu = None
    if args.cpu_sample > 0:
        cpu, y_cpu = cpu_baseline(theta, h_pre[0], args.cpu_sample)
        from oracle import moe_oracle as O

        cpu["gpu_vs_cpu_rel_l2"] = float(f"{O.rel_l2(out_pre[: args.cpu_sample].cpu(), y_cpu):.3e}")

    configs = None
    if not args.no_configs:
        del block, theta
        torch.cuda.empty_cache()
        configs = config_legs(dev, min(args.steps, 10), args.warmup)

    line = {
        "metric": "MoE-layer tokens/s (Mixtral Q8_0 prefill)", "value": round(T / (ms * 1e-3), 1), "unit": "tokens/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(ms, 4), "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": "f16", "data": "synthetic",
        "config": {"workload": f"Mixtral-8x7B MoE layer, prefill {T} tokens, Q8_0 weights, fp16, 8 experts top-2, 4096 x 14336, SiLU",
                   "parallelism": "1 GPU"},
        "layer_tflops": round(layer_flops / (ms * 1e-3) / 1e12, 2),
        "e2e_ms_per_step": round(e2e_ms, 4),
        "stage_ms": {k: round(v, 4) for k, v in st.items()},
        "roofline": roofline, "mfma_only_probe": probe, "decode": decode, "cpu_baseline": cpu, "configs": configs,
    }
    print(json.dumps(line))


if __name__ == "__main__":
    main()
