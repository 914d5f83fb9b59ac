"""Benchmark of the FP8 lm_head + fused softcapped cross-entropy, forward + backward, on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

Workload: Benchmark configuration 3 -- x bf16 [49152, 768] ~ N(0,1), W bf16 [50304, 768] ~ N(0, 1/768),
lm_head scales x_s = 100/448, w_s = 1.6/448, grad_s = 0.75/448, int64 targets uniform in [0, 50257),
outputs per-token losses, dx bf16, dW fp32.  One "step" = one forward + one backward of the path
with all inputs already resident in HBM.  Algorithmic work per step: 6*M*K*V FLOP (three GEMMs;
the logits recomputed in the backward are not counted).

Prints one JSON line.  Besides the whole-step throughput it carries
  roofline      for the kernel that takes the most time, timed with HIP events on its stream,
  cpu_baseline  the CPU oracle (PyTorch eager restatement) on a bounded row sample of the same workload.
"""
from __future__ import annotations

import argparse
import ctypes
import json
import os
import sys
import time

import torch

PEAK_FP8_TFLOPS = 5033.0      # MI355X dense FP8 MFMA (published)
M, K, V = 49152, 768, 50304
SLOT_NAMES = ["lm_head_ce_fwd", "dlogits_recompute", "dx_gemm", "dw_gemm", "other_gemm"]
# HBM bytes (read + write) per launch at this workload, from rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE runs of
# this script scaled by a 1 GiB copy in the same run (FETCH_SIZE x 2 KiB, WRITE_SIZE x 1 KiB); the runs and
# their commands are in profiles/lmhead_ce_cfg3_hbm_traffic.txt.  Counters cannot be read from inside the
# process, so these are recorded values, not live ones.
MEASURED_HBM_BYTES = {
    "lm_head_ce_fwd": 975.0e6 + 3.8e6,
    "dlogits_recompute": 2475.7e6 + 2495.6e6,
    "dx_gemm": 3332.3e6 + 134.3e6 + 16.8e6 + 25.2e6,
    "dw_gemm": 3360.8e6 + 195.2e6 + 20.3e6,
}


def profile_read(lib):
    out = {}
    for slot, name in enumerate(SLOT_NAMES):
        ms, n = ctypes.c_double(0), ctypes.c_int(0)
        lib.ngpt_profile_read(slot, ctypes.byref(ms), ctypes.byref(n))
        out[name] = (ms.value, n.value)
    return out


def make_cfg1(seed: int = 0, M: int = 1024, N: int = 3072, K: int = 768):
    """Configuration 1: x ~ N(0,1) bf16 [M,K]; W ~ N(0,1/K) bf16 [N,K]; x_s = 1, w_s = 1/32 (drawn on the CPU, fp32 then cast)."""
    import math
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(M, K, generator=g).bfloat16()
    w = (torch.randn(N, K, generator=g) / math.sqrt(K)).bfloat16()
    return x, w, 1.0, 1.0 / 32


def make_cfg3(seed: int = 0, M: int = 49152, K: int = 768, V: int = 50304, n_tok: int = 50257):
    """Configuration 3: x ~ N(0,1), W ~ N(0,1/K) (out,in), the reference's lm_head scales (train_gpt.py:1225), uniform targets."""
    import math
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(M, K, generator=g).bfloat16()
    w = (torch.randn(V, K, generator=g) / math.sqrt(K)).bfloat16()
    t = torch.randint(0, n_tok, (M,), generator=g, dtype=torch.int64)
    return x, w, t, dict(x_s=100 / 448, w_s=1.6 / 448, grad_s=0.75 / 448, grad_scale=1.0, A=23.0, B=5.0, C=7.5)


def cpu_baseline(x, w, t, sc, budget_s=20.0):
    # the only place where this script touches the CPU oracle: as the baseline that is timed beside the GPU path
    from oracle import nanogpt_fp8_oracle as oracle
    """Oracle forward+backward on the first rows of the same inputs; ~budget_s seconds of CPU work."""
    threads = torch.get_num_threads()
    rows_per_chunk = 1024
    oracle.lm_head_ce_chunked(x, t, w, **sc, rows_per_chunk=rows_per_chunk, max_rows=rows_per_chunk)   # warm-up
    t0 = time.perf_counter()
    oracle.lm_head_ce_chunked(x, t, w, **sc, rows_per_chunk=rows_per_chunk, max_rows=rows_per_chunk)
    per_chunk = time.perf_counter() - t0
    n_chunks = max(1, min(M // rows_per_chunk, int(budget_s / max(per_chunk, 1e-3))))
    rows = n_chunks * rows_per_chunk
    t0 = time.perf_counter()
    _, _, _, done = oracle.lm_head_ce_chunked(x, t, w, **sc, rows_per_chunk=rows_per_chunk, max_rows=rows)
    dt = time.perf_counter() - t0
    return {
        "value": done / dt, "unit": "tokens/s", "cores": threads, "kind": "port",
        "sample": f"first {done} of {M} rows, K={K}, V={V}, forward+backward in {rows_per_chunk}-row chunks, "
                  f"{dt:.1f} s of PyTorch-eager fp32 on the host CPU",
        "tflops": 6.0 * done * K * V / dt / 1e12,
    }


def calibrate_copy(dev) -> None:
    """One 1 GiB device-to-device copy: the kernel of known size that scales the profiler's FETCH_SIZE / WRITE_SIZE."""
    src = torch.empty(1 << 30, dtype=torch.uint8, device=dev).fill_(3)
    dst = torch.empty_like(src)
    dst.copy_(src)
    torch.cuda.synchronize()
    del src, dst


def secondary(args, amd) -> int:
    """Other workloads of the path, same JSON shape; timed with events on the current stream."""
    import math
    dev = torch.device("cuda:0")
    g = torch.Generator().manual_seed(0)
    wl = args.workload
    if wl == "mm_cfg1":
        x, w, x_s, w_s = make_cfg1(seed=0)
        xd, wd = x.to(dev), w.to(dev)
        step = lambda: torch.ops.nanogpt.mm(xd, wd, x_s, w_s, 1.0)
        flops, desc, tokens = 2.0 * x.shape[0] * w.shape[0] * x.shape[1], "config 1: nanogpt::mm forward, M=1024 N=3072 K=768", x.shape[0]
    elif wl == "mm_lmhead":
        Mm, Nn, Kk = 16384, 50304, 768
        xd = torch.randn(Mm, Kk, generator=g).bfloat16().to(dev)
        wd = (torch.randn(Nn, Kk, generator=g) / math.sqrt(Kk)).bfloat16().to(dev)
        gd = (torch.randn(Mm, Nn, generator=g) * 1e-3).bfloat16().to(dev)
        x_s, w_s, grad_s = 100 / 448, 1.6 / 448, 0.75 / 448 * 1e-2

        def step():
            out, x_f8, w_f8 = torch.ops.nanogpt.mm(xd, wd, x_s, w_s, grad_s)
            return torch.ops.nanogpt.mm_backward(gd, x_f8, w_f8, x_s, w_s, grad_s)
        flops, desc, tokens = 6.0 * Mm * Nn * Kk, "nanogpt::mm forward + mm_backward at the lm_head shape, M=16384 N=50304 K=768", Mm
    elif wl in ("mlp_fwd", "mlp_fwd_bwd"):
        Mm, D, H = 49152, 768, 3072
        xr = (torch.randn(Mm, D, generator=g) * 2).bfloat16().to(dev)
        w_fc = (torch.randn(H, D, generator=g) / math.sqrt(D)).bfloat16().to(dev)
        w_pt = (torch.randn(D, H, generator=g) / math.sqrt(H)).bfloat16().T.contiguous().to(dev)
        dy = (torch.randn(1, Mm, D, generator=g) * 1e-3).bfloat16().to(dev)
        w_f8, scales = torch.ops.nanogpt.quant_up_weights(w_fc[None])
        bwd = wl == "mlp_fwd_bwd"
        if bwd:
            xr.requires_grad_(True); w_fc.requires_grad_(True); w_pt.requires_grad_(True)

        def step():
            normed, x_f8, dequant = torch.ops.nanogpt.mlp_input_quant(xr, scales[0:1])
            out = amd.ReLUSqrdMLP(normed[None], w_fc, w_pt, w_f8[0], dequant, x_f8[None])
            if bwd:
                xr.grad = w_fc.grad = w_pt.grad = None
                out.backward(dy)
            return out
        flops = (12.0 if bwd else 4.0) * Mm * D * H
        desc = ("config 4 (one layer): " if bwd else "config 2: ") + "norm + quantise + FP8 c_fc with ReLU^2 + bf16 c_proj" + \
               (", forward+backward" if bwd else ", forward") + ", M=49152 D=768 H=3072"
        tokens = Mm
    elif wl == "mlp_cfg4":
        # configuration 4 as worded: twelve layers with their own weights, forward+backward, back to back on one stream
        Mm, D, H, L = 49152, 768, 3072, 12
        xr = (torch.randn(Mm, D, generator=g) * 2).bfloat16().to(dev).requires_grad_(True)
        w_fc = [(torch.randn(H, D, generator=g) / math.sqrt(D)).bfloat16().to(dev).requires_grad_(True) for _ in range(L)]
        w_pt = [(torch.randn(D, H, generator=g) / math.sqrt(H)).bfloat16().T.contiguous().to(dev).requires_grad_(True) for _ in range(L)]
        dy = (torch.randn(1, Mm, D, generator=g) * 1e-3).bfloat16().to(dev)
        w_f8, scales = torch.ops.nanogpt.quant_up_weights(torch.stack([w.detach() for w in w_fc]))

        def step():
            xr.grad = None
            for l in range(L):
                w_fc[l].grad = w_pt[l].grad = None
                normed, x_f8, dequant = torch.ops.nanogpt.mlp_input_quant(xr, scales[l:l + 1])
                out = amd.ReLUSqrdMLP(normed[None], w_fc[l], w_pt[l], w_f8[l], dequant, x_f8[None])
                out.backward(dy)
            return out
        flops = 12.0 * Mm * D * H * L
        desc = "config 4: 12 layers (own weights) of norm + quantise + FP8 c_fc with ReLU^2 + bf16 c_proj, forward+backward, M=49152 D=768 H=3072"
        tokens = Mm
    elif wl == "cfg5":
        # medium-track shapes: FP8 lm_head + softcapped CE forward+backward and one FP8 MLP layer forward+backward per step
        Mm, D, H, Vv = 65536, 1024, 4096, 50304
        xh = torch.randn(Mm, D, generator=g).bfloat16().to(dev).requires_grad_(True)
        wh = (torch.randn(Vv, D, generator=g) / math.sqrt(D)).bfloat16().to(dev).requires_grad_(True)
        tg = torch.randint(0, 50257, (Mm,), generator=g).to(dev)
        xr = (torch.randn(Mm, D, generator=g) * 2).bfloat16().to(dev).requires_grad_(True)
        w_fc = (torch.randn(H, D, generator=g) / math.sqrt(D)).bfloat16().to(dev).requires_grad_(True)
        w_pt = (torch.randn(D, H, generator=g) / math.sqrt(H)).bfloat16().T.contiguous().to(dev).requires_grad_(True)
        dy = (torch.randn(1, Mm, D, generator=g) * 1e-3).bfloat16().to(dev)
        w_f8, scales = torch.ops.nanogpt.quant_up_weights(w_fc.detach()[None])

        def step():
            xh.grad = wh.grad = xr.grad = w_fc.grad = w_pt.grad = None
            losses = amd.FusedSoftcappedCrossEntropy.apply(xh, tg, None, None, None, wh, 100 / 448, 1.6 / 448, 0.75 / 448, 1.0,
                                                           23.0, 5.0, 7.5, "out_in")
            losses.sum().backward()
            normed, x_f8, dequant = torch.ops.nanogpt.mlp_input_quant(xr, scales[0:1])
            out = amd.ReLUSqrdMLP(normed[None], w_fc, w_pt, w_f8[0], dequant, x_f8[None])
            out.backward(dy)
            return out
        flops = 6.0 * Mm * D * Vv + 12.0 * Mm * D * H
        desc, tokens = "config 5: lm_head + softcapped CE forward+backward and one FP8 MLP layer forward+backward, M=65536 D=1024 H=4096 V=50304", Mm
    elif wl == "ce_logits":
        # the logits-in-HBM compatibility op: one pass over bf16 logits in, e5m2 gradient out (HBM-bound)
        Mm, Vv = 49152, 50304
        logits = torch.empty(Mm, Vv, dtype=torch.bfloat16, device=dev)
        for r in range(0, Mm, 8192):   # N(0, 4) in slices, to keep the fp32 temporaries small
            logits[r:r + 8192] = (torch.randn(8192, Vv, device=dev) * 2).bfloat16()
        targets = torch.randint(0, 50257, (Mm,), generator=g).to(dev)
        mtp = torch.ones(1, device=dev)
        ptg = torch.full((Mm,), -1, dtype=torch.int64, device=dev)
        pw = torch.zeros(1, device=dev)
        losses = torch.empty(Mm, dtype=torch.float32, device=dev)
        grad = torch.empty(Mm, Vv, dtype=torch.float8_e5m2, device=dev)
        step = lambda: torch.ops.nanogpt.ce_fwd_bwd(logits, targets, mtp, ptg, pw, losses, grad, Mm, 1, 23.0, 5.0, 7.5,
                                                    0.75 / 448, 1.0)
        hbm_bytes = Mm * Vv * 3 + Mm * 12
        flops, desc, tokens = 0.0, "nanogpt::ce_fwd_bwd on materialised logits, M=49152 V=50304 (bf16 in, e5m2 gradient out)", Mm
    else:
        print(f"bench.py: unknown workload {wl}", file=sys.stderr)
        return 2
    if args.calibrate_copy:
        calibrate_copy(dev)
    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    e0.record()
    for _ in range(args.steps):
        step()
    e1.record()
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    ms = dt / args.steps * 1e3
    tflops = flops / (ms * 1e-3) / 1e12
    peak = PEAK_FP8_TFLOPS
    if wl == "ce_logits":
        gbs = hbm_bytes / (ms * 1e-3) / 1e9
        print(json.dumps({
            "metric": "tokens/s (secondary workload of the FP8 path)", "value": tokens / (ms * 1e-3), "unit": "tokens/s",
            "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": ms, "higher_is_better": True,
            "scaling": "weak", "vs_baseline": None, "dtype": "bf16 in, fp32 arithmetic, e5m2 out", "data": "synthetic",
            "config": {"workload": desc}, "event_ms_per_step": e0.elapsed_time(e1) / args.steps,
            "roofline": {"bound": "hbm", "achieved": gbs, "peak": 8000.0, "unit": "GB/s", "frac": gbs / 8000.0,
                         "traffic": 4991.2e6 + 2479.8e6,
                         "note": "algorithmic bytes M*V*(2+1) + M*12 per pass / its duration; traffic = recorded rocprofv3 "
                                 "FETCH_SIZE + WRITE_SIZE measurement in bytes per launch (profiles/ce_logits_hbm_traffic.txt)"},
        }))
        return 0
    print(json.dumps({
        "metric": "tokens/s (secondary workload of the FP8 path)", "value": tokens / (ms * 1e-3), "unit": "tokens/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": ms, "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": "fp8", "data": "synthetic", "config": {"workload": desc},
        "tflops": tflops, "event_ms_per_step": e0.elapsed_time(e1) / args.steps,
        "roofline": {"bound": "mfma", "achieved": tflops, "peak": peak, "unit": "TFLOP/s", "frac": tflops / peak, "traffic": None,
                     "note": "whole step against the dense FP8 peak; bf16 GEMMs inside count at the same peak"},
    }))
    return 0


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--workload", default="lmhead_ce",
                    help="lmhead_ce (default, the headline configuration 3) | mm_cfg1 | mm_lmhead | mlp_fwd | mlp_fwd_bwd | mlp_cfg4 | ce_logits | cfg5")
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=10)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="also run one 1 GiB device-to-device copy, the known-size kernel that scales "
                         "the FETCH_SIZE / WRITE_SIZE counters of a rocprofv3 --pmc run")
    args = ap.parse_args()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print("bench.py: this path is built and measured on ONE GPU (the kernel on one GPU's share of the "
              "batch, M=49152); runs with more than one GPU are not part of this build.", file=sys.stderr)
        return 2

    sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))
    import modded_nanogpt_amd as amd
    lib = amd._lib.load()
    assert torch.cuda.is_available(), "bench.py needs a GPU"
    if args.workload != "lmhead_ce":
        return secondary(args, amd)
    dev = torch.device("cuda:0")
    x, w, t, sc = make_cfg3(seed=0)
    xd, wd, td = x.to(dev), w.to(dev), t.to(dev)
    mtp = torch.tensor([1.0], device=dev)
    pt = torch.full((M,), -1, dtype=torch.int64, device=dev)
    pw = torch.zeros(1, device=dev)

    def step():
        losses, lse, sig, x_f8, w_f8 = torch.ops.nanogpt.lmhead_ce_fwd(
            xd, wd, td, mtp, pt, pw, sc["x_s"], sc["w_s"], sc["A"], sc["B"], sc["C"], False)
        dx, dw = torch.ops.nanogpt.lmhead_ce_bwd(
            x_f8, w_f8, td, mtp, pt, pw, lse, sig, sc["x_s"], sc["w_s"], sc["grad_s"], sc["grad_scale"],
            sc["A"], sc["B"], sc["C"], False)
        return losses, dx, dw

    if args.calibrate_copy:
        calibrate_copy(dev)
    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    lib.ngpt_profile_enable(1)
    profile_read(lib)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        out = step()
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    prof = profile_read(lib)
    lib.ngpt_profile_enable(0)

    ms_per_step = dt / args.steps * 1e3
    flops_step = 6.0 * M * K * V
    tflops = flops_step / (ms_per_step * 1e-3) / 1e12
    mean_loss = float(out[0].mean())

    # roofline of the kernel with the largest share of the step
    flops_per_launch = {   # algorithmic FLOP of one launch of each kernel at this workload
        "lm_head_ce_fwd": 2.0 * M * K * V,
        "dlogits_recompute": None,      # recompute: executed 2*Mc*K*V per launch, algorithmic share 0
        "dx_gemm": None, "dw_gemm": None, "other_gemm": None,
    }
    kernels = {}
    for name, (ms, n) in prof.items():
        if n:
            kernels[name] = {"launches_per_step": n / args.steps, "avg_ms": ms / n, "ms_per_step": ms / args.steps}
    for name in ("dlogits_recompute", "dx_gemm", "dw_gemm"):
        if name in kernels:
            flops_per_launch[name] = 2.0 * M * K * V / kernels[name]["launches_per_step"]
    dominant = max(kernels, key=lambda k: kernels[k]["ms_per_step"])
    dom = kernels[dominant]
    achieved = flops_per_launch[dominant] / (dom["avg_ms"] * 1e-3) / 1e12
    roofline = {
        "bound": "mfma", "kernel": dominant, "achieved": achieved, "peak": PEAK_FP8_TFLOPS, "unit": "TFLOP/s",
        "frac": achieved / PEAK_FP8_TFLOPS, "traffic": MEASURED_HBM_BYTES.get(dominant),
        "traffic_unit": "bytes per launch (recorded rocprofv3 FETCH_SIZE + WRITE_SIZE measurement, see profiles/)",
        "avg_launch_ms": dom["avg_ms"], "flop_per_launch": flops_per_launch[dominant],
        "note": "executed 2*rows*K*V FLOP per launch of each GEMM-shaped kernel / its HIP-event duration",
    }

    result = {
        "metric": "lm_head+CE fwd+bwd tokens/s at M=49152 (FP8 TFLOP/s and fraction of dense FP8 peak alongside)",
        "value": M / (ms_per_step * 1e-3), "unit": "tokens/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": ms_per_step,
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "fp8", "data": "synthetic",
        "config": {"workload": "config 3: FP8 lm_head + fused softcapped cross-entropy, forward+backward, "
                               "M=49152 K=768 V=50304, (out,in) weight, n_predict=1"},
        "tflops": tflops, "frac_fp8_peak": tflops / PEAK_FP8_TFLOPS, "peak_fp8_tflops": PEAK_FP8_TFLOPS,
        "flop_per_step": flops_step, "mean_loss": mean_loss,
        "kernels": kernels, "roofline": roofline,
    }
    if not args.no_cpu_baseline:
        result["cpu_baseline"] = cpu_baseline(x, w, t, sc)
    print(json.dumps(result))
    return 0


if __name__ == "__main__":
    sys.exit(main())
