#!/usr/bin/env python3
"""Benchmark of the MoE layer hot path on one MI355X.

Workload (BASELINE.json configs[1]): one Mixtral-8x7B MoE layer, Q8_0 block-scaled expert weights, hidden 4096,
FFN 14336, 8 experts, top-2, SiLU, fp16 activations; prefill with 2048 tokens (the headline metric) and decode
with 32 tokens (reported beside it).  A step is one MoeBlock.forward over the batch, inputs resident in HBM.

Prints ONE JSON line.  `value` = prefill tokens/s.  `roofline` prices the dominant prefill kernel (the fused
gate/up projection) against the dense fp16 MFMA peak; `decode.roofline` prices the same kernel at T=32 against
HBM bandwidth on its expert-weight bytes.  Kernel durations are measured live with HIP events recorded on the
launch stream around each kernel inside the timed loop.  `cpu_baseline` times the CPU oracle (a restatement of
the reference's eager per-token-gather algorithm) on the host cores for a bounded token sample.
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


def build_layer(dev, seed=0):
    import torch
    from sharktank_amd import types as ST
    from sharktank_amd.layers import MoeBlock

    g = torch.Generator(device="cpu").manual_seed(seed)
    gg = torch.Generator(device=dev).manual_seed(seed)
    tensors = {}
    for name, shape in (("ffn_gate_exps", [E, N_FFN, K_HID]), ("ffn_up_exps", [E, N_FFN, K_HID]), ("ffn_down_exps", [E, K_HID, N_FFN])):
        planes_d, planes_q = [], []
        for e in range(E):  # per expert to bound the fp32 staging memory
            w = torch.randn(shape[1:], generator=gg, device=dev, dtype=torch.float32) * 0.02
            d, qs = quantize_q8_0(w)
            planes_d.append(d)
            planes_q.append(qs)
            del w
        layout = ST.BlockScaledLayout(shape, torch.stack(planes_d), torch.stack(planes_q))
        tensors[f"{name}.weight"] = ST.PlanarQuantizedTensor(name=f"{name}.weight", shape=shape, layout=layout)
    tensors["ffn_gate_inp.weight"] = ST.DefaultPrimitiveTensor(
        name="ffn_gate_inp.weight", data=(torch.randn(E, K_HID, generator=g) * 0.02).to(dev))
    tensors["ffn_norm.weight"] = ST.DefaultPrimitiveTensor(name="ffn_norm.weight", data=torch.ones(K_HID, device=dev))
    theta = ST.Theta(tensors)
    return MoeBlock(theta, E, TOPK, 1e-5), theta


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


def run_leg(block, h, steps, warmup):
    """Times `steps` forwards.  In the timed loop only the dominant kernel (the gate/up projection) is bracketed by
    HIP events on the launch stream; a second, untimed pass of the same length brackets every stage for the
    breakdown.  Returns (ms_per_step, gate_up_ms, {stage: avg ms}, out)."""
    import torch
    from sharktank_amd import _hip
    from sharktank_amd.types import unbox_tensor

    T = h.shape[1]
    x = h.reshape(T, K_HID)
    wg, wu, wd = block.experts.device_weights()
    need = _hip.moe_forward_workspace_bytes(T, TOPK, E, K_HID, N_FFN, h.dtype)
    ws = torch.empty(need, dtype=torch.uint8, device=h.device)
    out = torch.empty_like(x)
    norm_w = unbox_tensor(block.ffn_norm.weight)
    router_w = block._router_weight(h.dtype)
    evsets = [HipEvents(12) for _ in range(steps)]
    dominant = []
    for ev in evsets:  # the same handles, all but the gate/up bracket masked out
        arr = (ctypes.c_void_p * 12)()
        arr[6], arr[7] = ev.arr[6], ev.arr[7]
        dominant.append(arr)

    def fwd(events=None):
        _hip.moe_forward(x, norm_w, None, block.rms_epsilon, router_w, wg, wu, wd, block.experts._act, TOPK,
                         workspace=ws, out=out, events=events)

    for _ in range(warmup):
        fwd()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for s in range(steps):
        fwd(dominant[s])
    torch.cuda.synchronize()
    ms = (time.perf_counter() - t0) * 1e3 / steps
    gate_up_ms = sum(ev.elapsed_ms(6, 7) for ev in evsets) / steps

    for s in range(steps):
        fwd(evsets[s].arr)
    torch.cuda.synchronize()
    stage_ms = {name: sum(ev.elapsed_ms(2 * i, 2 * i + 1) for ev in evsets) / steps for i, name in enumerate(STAGES)}
    for ev in evsets:
        ev.destroy()
    return ms, gate_up_ms, stage_ms, out


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


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--prefill-tokens", type=int, default=2048)
    ap.add_argument("--decode-tokens", type=int, default=32)
    ap.add_argument("--cpu-sample", type=int, default=16, help="tokens timed on the CPU baseline (0 to skip)")
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

    ms, gu_ms, st, out_pre = run_leg(block, h_pre.to(dev), args.steps, args.warmup)
    T = args.prefill_tokens
    gateup_flops = 2.0 * T * TOPK * 2 * N_FFN * K_HID
    layer_flops = 2.0 * T * TOPK * 3 * N_FFN * K_HID + 2.0 * T * E * K_HID
    achieved = gateup_flops / (gu_ms * 1e-3) / 1e12
    roofline = {
        "kernel": "grouped gate/up projection (prefill)", "bound": "mfma", "achieved": round(achieved, 2),
        "peak": MFMA_F16_PEAK_TFLOPS, "unit": "TFLOP/s", "frac": round(achieved / MFMA_F16_PEAK_TFLOPS, 4),
        "traffic": measured_traffic("prefill_gate_up") if T == 2048 else None, "avg_kernel_ms": round(gu_ms, 4),
        "algorithmic": gateup_flops, "algorithmic_unit": "flop per launch",
    }

    dms, dgu_ms, dst, _ = run_leg(block, h_dec.to(dev), max(args.steps, 50), args.warmup)
    wbytes_one = E * N_FFN * K_HID * 34.0 / 32.0  # Q8_0 bytes of one stacked matrix (all 8 experts are hit at T=32)
    d_achieved = 2 * wbytes_one / (dgu_ms * 1e-3) / 1e9
    decode = {
        "tokens": args.decode_tokens, "steps": max(args.steps, 50), "ms_per_step": round(dms, 4),
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

    line = {
        "metric": "MoE-layer tokens/s (Mixtral Q8_0 prefill)", "value": round(T / (ms * 1e-3), 1), "unit": "tokens/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(ms, 4), "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": "f16", "data": "synthetic",
        "config": {"workload": "Mixtral-8x7B MoE layer, Q8_0 expert weights, fp16 activations, hidden 4096, FFN 14336, "
                               f"8 experts, top-2, SiLU; prefill {T} tokens", "parallelism": "1 GPU"},
        "layer_tflops": round(layer_flops / (ms * 1e-3) / 1e12, 2),
        "stage_ms": {k: round(v, 4) for k, v in st.items()},
        "roofline": roofline, "decode": decode, "cpu_baseline": cpu,
    }
    print(json.dumps(line))


if __name__ == "__main__":
    main()
