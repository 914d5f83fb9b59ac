"""Benchmark of the FP8 contraction path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload NAME]

Default workload (`lmhead_ce`): benchmark configuration 3 -- x bf16 [49152, 768] ~ N(0,1), W bf16 [50304, 768]
~ N(0, 1/768), lm_head scales x_s = 100/448, w_s = 1.6/448, grad_s = 0.75/448, int64 targets uniform in [0, 50257),
outputs per-token losses, dx bf16, dW fp32.  One "step" = one forward + one backward of the path with all inputs
already resident in HBM.  Algorithmic work per step: 6*M*K*V FLOP (three GEMMs; the logits recomputed in the
backward are not counted).

Every workload prints one JSON line with the whole-step throughput (mean over the timed steps, the median of the
per-step HIP-event times beside it) and
  kernels       HIP-event time per kernel group on the launch stream (the library's profile slots),
  roofline      for the kernel group that takes the most time: algorithmic FLOP (or bytes) per launch / its
                average launch duration, against the published peak; `traffic` = HBM bytes per launch from the
                rocprofv3 counter runs recorded in profiles/hbm_traffic.json (counters cannot be read in-process),
  cpu_baseline  the CPU oracle (PyTorch eager restatement) on a bounded sample of the same workload.
The default line also carries `tail47_ms` (the same step with 47 vocabulary columns below the sigma-code window, as the
padding ids of a trained model are) and `secondary`: configurations 1, 2 (bf16 and FP8 down projection), 4 and 5 timed briefly.
Other workloads: mm_cfg1 (configuration 1), mlp_fwd (2), mlp_fwd_fp8down, mlp_fwd_bwd (one layer of 4), mlp_cfg4 (4: twelve layers),
cfg5 (5), mm_lmhead, ce_logits, and `ceiling`: what an fp8 GEMM reaches on this machine (matrix pipe alone and the
k-step skeleton on zero / random operands, the shipped tile kernel without its epilogue, the vendor library; needs the
measurement build of the library, `python -m modded_nanogpt_amd.build`).
"""
from __future__ import annotations

import argparse
import ctypes
import glob
import json
import math
import os
import statistics
import sys
import time

import torch

ROOT = os.path.dirname(os.path.abspath(__file__))
PEAK_FP8_TFLOPS = 5000.0      # MI355X dense FP8 MFMA, the published figure every fp8 fraction below is taken against
PEAK_BF16_TFLOPS = 2500.0     # dense BF16 (published)
PEAK_HBM_GBS = 8000.0
M, K, V = 49152, 768, 50304
SLOT_NAMES = ["lm_head_ce_fwd", "dlogits_recompute", "dx_gemm", "dw_gemm", "fp8_gemm", "fc_relu2", "dpre", "bf16_gemm",
              "mlp_input_producers"]


def profile_read(lib):
    out = {}
    for slot, name in enumerate(SLOT_NAMES):
        ms, n = ctypes.c_double(0), ctypes.c_int(0)
        lib.ngpt_profile_read(slot, ctypes.byref(ms), ctypes.byref(n))
        out[name] = (ms.value, n.value)
    return out


def recorded_traffic(workload: str):
    """HBM bytes per launch of each kernel group, from the rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE runs summarised
    in profiles/hbm_traffic.json (which names the profile file and the commit each figure came from)."""
    try:
        with open(os.path.join(ROOT, "profiles", "hbm_traffic.json")) as f:
            rec = json.load(f)
        entry = rec.get(workload)
        if entry:
            return entry["bytes_per_launch"], {"file": entry["source"], "commit": entry.get("commit")}
    except (OSError, ValueError, KeyError):
        pass
    return {}, None


def device_info(lib):
    """Compute units the persistent grids are sized to and the number of XCDs (each with its own L2), as queried."""
    info = {"compute_units": int(lib.ngpt_num_cus()), "xcds": None, "name": torch.cuda.get_device_name(0)}
    for path in glob.glob("/sys/class/kfd/kfd/topology/nodes/*/properties"):
        try:
            props = dict(line.split() for line in open(path) if len(line.split()) == 2)
            if int(props.get("simd_count", "0")) > 0 and "num_xcc" in props:
                info["xcds"] = int(props["num_xcc"])
                break
        except (OSError, ValueError):
            continue
    return info


# ---------------------------------------------------------------------------------------------- inputs
def make_cfg1(seed: int = 0, M: int = 1024, N: int = 3072, K: int = 768):
    """Configuration 1: x ~ N(0,1) bf16 [M,K]; W ~ N(0,1/K) bf16 [N,K]; x_s = 1, w_s = 1/32 (drawn on the CPU, fp32 then cast)."""
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(M, K, generator=g).bfloat16()
    w = (torch.randn(N, K, generator=g) / math.sqrt(K)).bfloat16()
    return x, w, 1.0, 1.0 / 32


def make_cfg3(seed: int = 0, M: int = 49152, K: int = 768, V: int = 50304, n_tok: int = 50257):
    """Configuration 3: x ~ N(0,1), W ~ N(0,1/K) (out,in), the reference's lm_head scales (train_gpt.py:1225), uniform targets."""
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(M, K, generator=g).bfloat16()
    w = (torch.randn(V, K, generator=g) / math.sqrt(K)).bfloat16()
    t = torch.randint(0, n_tok, (M,), generator=g, dtype=torch.int64)
    return x, w, t, dict(x_s=100 / 448, w_s=1.6 / 448, grad_s=0.75 / 448, grad_scale=1.0, A=23.0, B=5.0, C=7.5)


def make_mlp(seed: int, M: int, D: int, H: int, layers: int = 1):
    """Configurations 2 / 4 / 5 (MLP part): x ~ 2 N(0,1) before the norm, W_fc ~ N(0,1/D), W_proj ~ N(0,1/H) stored [H, D], dY ~ 1e-3 N(0,1)."""
    g = torch.Generator().manual_seed(seed)
    x = (torch.randn(M, D, generator=g) * 2).bfloat16()
    w_fc = [(torch.randn(H, D, generator=g) / math.sqrt(D)).bfloat16() for _ in range(layers)]
    w_pt = [(torch.randn(D, H, generator=g) / math.sqrt(H)).bfloat16().T.contiguous() for _ in range(layers)]
    dy = (torch.randn(1, M, D, generator=g) * 1e-3).bfloat16()
    return x, w_fc, w_pt, dy


# ---------------------------------------------------------------------------------------------- CPU baselines
# The only places where this script touches the CPU oracle: as the baseline that is timed beside the GPU path.
def cpu_baseline(x, w, t, sc, budget_s=20.0):
    """Oracle forward+backward of the lm_head + CE on the first rows of the same inputs; ~budget_s seconds of CPU work."""
    from oracle import nanogpt_fp8_oracle as oracle
    threads = torch.get_num_threads()
    rows_total, Kd = x.shape
    Vd = w.shape[0]
    rows_per_chunk = 1024
    oracle.lm_head_ce_chunked(x, t, w, **sc, rows_per_chunk=rows_per_chunk, max_rows=rows_per_chunk)   # warm-up
    t0 = time.perf_counter()
    oracle.lm_head_ce_chunked(x, t, w, **sc, rows_per_chunk=rows_per_chunk, max_rows=rows_per_chunk)
    per_chunk = time.perf_counter() - t0
    n_chunks = max(1, min(rows_total // rows_per_chunk, int(budget_s / max(per_chunk, 1e-3))))
    rows = n_chunks * rows_per_chunk
    t0 = time.perf_counter()
    _, _, _, done = oracle.lm_head_ce_chunked(x, t, w, **sc, rows_per_chunk=rows_per_chunk, max_rows=rows)
    dt = time.perf_counter() - t0
    return {
        "value": done / dt, "unit": "tokens/s", "cores": threads, "kind": "port",
        "sample": f"first {done} of {rows_total} rows, K={Kd}, V={Vd}, forward+backward in {rows_per_chunk}-row chunks, "
                  f"{dt:.1f} s of PyTorch-eager fp32 on the host CPU",
        "tflops": 6.0 * done * Kd * Vd / dt / 1e12,
    }


def cpu_baseline_mm(x, w, x_s, w_s):
    """Oracle nanogpt::mm forward, whole (configuration 1 is CPU-sized)."""
    from oracle import nanogpt_fp8_oracle as oracle
    oracle.mm_fwd(x, w, x_s, w_s)
    reps, t0 = 0, time.perf_counter()
    while reps < 3 or time.perf_counter() - t0 < 2.0:
        oracle.mm_fwd(x, w, x_s, w_s)
        reps += 1
    dt = (time.perf_counter() - t0) / reps
    Mm, Kk = x.shape
    return {"value": Mm / dt, "unit": "tokens/s", "cores": torch.get_num_threads(), "kind": "port",
            "sample": f"the whole problem ({Mm} x {w.shape[0]} x {Kk}), mean of {reps} runs of PyTorch-eager fp32 on the host CPU",
            "tflops": 2.0 * Mm * w.shape[0] * Kk / dt / 1e12}


def cpu_baseline_mlp(x, w_fc, w_pt, dy, backward: bool, budget_s=10.0):
    """Oracle FP8 MLP forward (+ bf16 backward) of one layer in row chunks (the quantisation scale is taken from the
    whole input first, as it is a global amax); weight gradients accumulate over the chunks."""
    from oracle import nanogpt_fp8_oracle as oracle
    threads = torch.get_num_threads()
    Mm, D = x.shape
    H = w_fc.shape[0]
    w_f8, scales = oracle.quantize_up_weights(w_fc[None])
    normed = oracle.rms_norm(x)
    x_f8, dequant = oracle.mlp_input_quant(normed, scales[0:1])
    chunk = 1024

    def run(rows):
        dw1 = dw2 = None
        for r0 in range(0, rows, chunk):
            r = slice(r0, r0 + chunk)
            out, post = oracle.mlp_fwd(normed[None, r], w_fc, w_pt, w_f8[0], dequant, x_f8[None, r])
            if backward:
                _, a, b = oracle.mlp_bwd(dy[:, r], normed[None, r], w_fc, w_pt, post)
                dw1 = a.float() if dw1 is None else dw1 + a.float()
                dw2 = b.float() if dw2 is None else dw2 + b.float()
    run(chunk)
    t0 = time.perf_counter()
    run(chunk)
    per_chunk = time.perf_counter() - t0
    rows = max(1, min(Mm // chunk, int(budget_s / max(per_chunk, 1e-3)))) * chunk
    t0 = time.perf_counter()
    run(rows)
    dt = time.perf_counter() - t0
    return {"value": rows / dt, "unit": "tokens/s", "cores": threads, "kind": "port",
            "sample": f"first {rows} of {Mm} rows of one layer, D={D}, H={H}, forward{'+backward' if backward else ''} in {chunk}-row chunks "
                      f"(input norm and quantisation scale from the whole tensor, outside the timed part), {dt:.1f} s of PyTorch-eager fp32 on the host CPU",
            "tflops": (12.0 if backward else 4.0) * rows * D * H / dt / 1e12}


# ---------------------------------------------------------------------------------------------- timing
def calibrate_copy(dev) -> None:
    """One 1 GiB device-to-device copy: the kernel of known size that scales the profiler's FETCH_SIZE / WRITE_SIZE."""
    src = torch.empty(1 << 30, dtype=torch.uint8, device=dev).fill_(3)
    dst = torch.empty_like(src)
    dst.copy_(src)
    torch.cuda.synchronize()
    del src, dst


def run_timed(lib, step, steps: int, warmup: int):
    """`warmup` untimed steps, then exactly `steps` steps between two synchronisations (wall clock -> mean), each step
    also bracketed by HIP events on the current stream (-> median), the library's per-kernel events switched on."""
    for _ in range(warmup):
        step()
    torch.cuda.synchronize()
    lib.ngpt_profile_enable(1)
    profile_read(lib)
    ev = [torch.cuda.Event(enable_timing=True) for _ in range(steps + 1)]
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    ev[0].record()
    out = None
    for i in range(steps):
        out = step()
        ev[i + 1].record()
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    prof = profile_read(lib)
    lib.ngpt_profile_enable(0)
    per_step = [ev[i].elapsed_time(ev[i + 1]) for i in range(steps)]
    kernels = {}
    for name, (ms, n) in prof.items():
        if n:
            kernels[name] = {"launches_per_step": n / steps, "avg_ms": ms / n, "ms_per_step": ms / steps}
    return out, dt / steps * 1e3, statistics.median(per_step), kernels


def roofline_of(kernels, work, traffic, traffic_src):
    """Roofline entry for the kernel group with the largest share of the step.  work[name] = (amount per step, bound):
    FLOP for "mfma-fp8" / "mfma-bf16", bytes for "hbm"."""
    timed = {k: v for k, v in kernels.items() if k in work}
    if not timed:
        return None
    dominant = max(timed, key=lambda k: timed[k]["ms_per_step"])
    per_step, bound = work[dominant]
    dom = timed[dominant]
    per_launch = per_step / dom["launches_per_step"]
    if bound == "hbm":
        achieved, peak, unit = per_launch / (dom["avg_ms"] * 1e-3) / 1e9, PEAK_HBM_GBS, "GB/s"
    else:
        achieved, unit = per_launch / (dom["avg_ms"] * 1e-3) / 1e12, "TFLOP/s"
        peak = PEAK_FP8_TFLOPS if bound == "mfma-fp8" else PEAK_BF16_TFLOPS
    return {"bound": "hbm" if bound == "hbm" else "mfma", "kernel": dominant, "achieved": achieved, "peak": peak, "unit": unit,
            "frac": achieved / peak, "traffic": traffic.get(dominant),
            "traffic_unit": "HBM bytes per launch, rocprofv3 FETCH_SIZE + WRITE_SIZE (recorded; null = not recorded for this kernel)",
            "traffic_source": traffic_src, "avg_launch_ms": dom["avg_ms"], "per_launch": per_launch,
            "per_launch_unit": "bytes" if bound == "hbm" else "FLOP (2 * rows * cols * contraction of the launch)",
            "arithmetic": {"mfma-fp8": "fp8 MFMA", "mfma-bf16": "bf16 MFMA", "hbm": "memory"}[bound]}


def emit(args, lib, desc, tokens, flops, ms, median_ms, kernels, work, traffic_key, dtype="fp8", extra=None, cpu=None,
         metric="tokens/s (secondary workload of the FP8 path)"):
    traffic, src = recorded_traffic(traffic_key)
    result = {
        "metric": metric, "value": tokens / (ms * 1e-3), "unit": "tokens/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": ms, "median_ms_per_step": median_ms,
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": dtype, "data": "synthetic",
        "config": {"workload": desc}, "device": device_info(lib),
    }
    if flops:
        tf = flops / (ms * 1e-3) / 1e12
        result.update({"tflops": tf, "frac_fp8_peak": tf / PEAK_FP8_TFLOPS, "peak_fp8_tflops": PEAK_FP8_TFLOPS, "flop_per_step": flops})
    if extra:
        result.update(extra)
    result["kernels"] = kernels
    result["roofline"] = roofline_of(kernels, work, traffic, src)
    if cpu is not None:
        result["cpu_baseline"] = cpu
    return result


# ---------------------------------------------------------------------------------------------- workloads
def workload_lmhead_ce(args, amd, lib, dev):
    x, w, t, sc = make_cfg3(seed=0)
    if args.tail_columns:
        # What a trained model looks like to the sigma-code backward: the last vocabulary entries (ids that never occur
        # as targets, such as the padding ids 50257..50303) have logits near -20 for every token, below the code window,
        # and the rows' factors are above the limit under which such gradients are exact zeros (here by a larger
        # grad_scale; in a trained model by a smaller lse).  The tiles that hold those columns are then recomputed.
        x[:, 0] = 13.5
        w[w.shape[0] - args.tail_columns:, 0] = -1.5      # inside the e4m3 range of w / w_s
        sc["grad_scale"] = 64.0
    xd, wd, td = x.to(dev), w.to(dev), t.to(dev)
    mtp = torch.tensor([1.0], device=dev)
    pt = torch.full((M,), -1, dtype=torch.int64, device=dev)
    pw = torch.zeros(1, device=dev)

    fwd_args = (xd, wd, td, mtp, pt, pw, sc["x_s"], sc["w_s"], sc["A"], sc["B"], sc["C"], False)
    bwd_tail = (sc["x_s"], sc["w_s"], sc["grad_s"], sc["grad_scale"], sc["A"], sc["B"], sc["C"], False)

    def step_recompute():      # nothing of size [tokens, vocabulary] kept: the backward runs the logits GEMM again
        losses, lse, sig, x_f8, w_f8 = torch.ops.nanogpt.lmhead_ce_fwd(*fwd_args)
        dx, dw = torch.ops.nanogpt.lmhead_ce_bwd(x_f8, w_f8, td, mtp, pt, pw, lse, sig, *bwd_tail)
        return losses, dx, dw

    def step_codes():          # the forward keeps one code byte of bf16(sigma) per logit, the backward rebuilds dl from it
        losses, lse, sig, x_f8, w_f8, codes = torch.ops.nanogpt.lmhead_ce_fwd_codes(*fwd_args)
        dx, dw = torch.ops.nanogpt.lmhead_ce_bwd_codes(x_f8, w_f8, td, mtp, pt, pw, lse, sig, codes, *bwd_tail)
        return losses, dx, dw

    codes_mode = args.ce_backward == "codes"
    step, other = (step_codes, step_recompute) if codes_mode else (step_recompute, step_codes)
    if args.calibrate_copy:
        calibrate_copy(dev)
    out, ms, median_ms, kernels = run_timed(lib, step, args.steps, args.warmup)
    gemm = 2.0 * M * K * V      # executed FLOP of each GEMM-shaped kernel per step
    work = {n: (gemm, "mfma-fp8") for n in ("lm_head_ce_fwd", "dlogits_recompute", "dx_gemm", "dw_gemm")}
    mode_desc = "the backward recomputes the logits (four GEMM passes)"
    if codes_mode:              # the second slot then is the code -> e5m2 conversion, a memory-bound pass over 2 x M x V bytes
        kernels["dlogits_from_codes"] = kernels.pop("dlogits_recompute", {"launches_per_step": 0.0, "avg_ms": 0.0, "ms_per_step": 0.0})
        del work["dlogits_recompute"]
        work["dlogits_from_codes"] = (2.0 * M * V, "hbm")
        mode_desc = "the forward keeps one sigma code byte per logit for the backward (three GEMM passes)"
    extra = {"mean_loss": float(out[0].mean()), "ce_backward": args.ce_backward}
    # device memory of size ~ M x V that each mode of the backward needs: the code panel lives from the forward to the
    # backward (the reference keeps an e5m2 gradient of that size there), the dlogits panel is backward workspace
    bwd_ws = int(lib.ngpt_lmhead_ce_bwd_workspace_bytes(M, K, V, 0))
    extra["memory_bytes"] = {"codes": {"saved_for_backward": int(lib.ngpt_lmhead_ce_codes_bytes(M, V)), "backward_workspace": bwd_ws},
                             "recompute": {"saved_for_backward": 0, "backward_workspace": bwd_ws},
                             "forward_workspace": int(lib.ngpt_lmhead_ce_fwd_workspace_bytes(M, K, V, 0))}
    if args.tail_columns:
        extra["tail_columns"] = args.tail_columns
    if not args.no_other_mode:  # the other mode of the backward, timed the same way on a few steps, for the record
        _, o_ms, o_med, _ = run_timed(lib, other, max(5, args.steps // 5), 3)
        extra["other_mode"] = {"ce_backward": "recompute" if codes_mode else "codes", "ms_per_step": o_ms,
                               "median_ms_per_step": o_med, "tokens_per_s": M / (o_ms * 1e-3)}
    if not args.tail_columns and not args.no_tail:
        # the same step on logits as a trained model has them in the padding ids: 47 vocabulary columns below the code window
        tail = argparse.Namespace(**{**vars(args), "tail_columns": 47, "no_other_mode": True, "no_cpu_baseline": True, "no_tail": True,
                                     "steps": max(5, args.steps // 5), "warmup": 3})
        extra["tail47_ms"] = workload_lmhead_ce(tail, amd, lib, dev)["ms_per_step"]
    cpu = None if args.no_cpu_baseline else cpu_baseline(x, w, t, sc)
    return emit(args, lib, "config 3: FP8 lm_head + fused softcapped cross-entropy, forward+backward, M=49152 K=768 V=50304, "
                    "(out,in) weight, n_predict=1; " + mode_desc, M, 6.0 * M * K * V, ms, median_ms, kernels, work,
         "lmhead_ce" if codes_mode else "lmhead_ce_recompute", extra=extra, cpu=cpu,
         metric="lm_head+CE fwd+bwd tokens/s at M=49152 (FP8 TFLOP/s and fraction of dense FP8 peak alongside)")


def mlp_work(Mm, D, H, backward, layers=1):
    g = 2.0 * Mm * D * H * layers
    work = {"fc_relu2": (g, "mfma-fp8"), "bf16_gemm": (g * (4 if backward else 1), "mfma-bf16"),
            "mlp_input_producers": (Mm * D * (2 + 2 + 2 + 1) * layers + (Mm * D * 6 * layers if backward else 0), "hbm")}
    if backward:
        work["dpre"] = (g, "mfma-bf16")
    return work


def secondary(args, amd, lib, dev):
    """Other workloads of the path, same JSON shape (None for an unknown name)."""
    g = torch.Generator().manual_seed(0)
    wl = args.workload
    cpu, work, traffic_key, dtype, extra = None, {}, wl, "fp8", None
    if wl == "mm_cfg1":
        x, w, x_s, w_s = make_cfg1(seed=0)
        xd, wd = x.to(dev), w.to(dev)
        step = lambda: torch.ops.nanogpt.mm(xd, wd, x_s, w_s, 1.0)
        flops, desc, tokens = 2.0 * x.shape[0] * w.shape[0] * x.shape[1], "config 1: nanogpt::mm forward, M=1024 N=3072 K=768", x.shape[0]
        work = {"fp8_gemm": (flops, "mfma-fp8")}
        if not args.no_cpu_baseline:
            cpu = cpu_baseline_mm(x, w, x_s, w_s)
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
        work = {"fp8_gemm": (flops, "mfma-fp8")}
    elif wl in ("mlp_fwd", "mlp_fwd_fp8down", "mlp_fwd_bwd", "mlp_cfg4"):
        Mm, D, H = 49152, 768, 3072
        L = 12 if wl == "mlp_cfg4" else 1
        bwd = wl in ("mlp_fwd_bwd", "mlp_cfg4")
        fp8down = wl == "mlp_fwd_fp8down"
        x, w_fc_c, w_pt_c, dy_c = make_mlp(0, Mm, D, H, L)
        xr = x.to(dev).requires_grad_(bwd)
        w_fc = [w.to(dev).requires_grad_(bwd) for w in w_fc_c]
        w_pt = [w.to(dev).requires_grad_(bwd) for w in w_pt_c]
        dy = dy_c.to(dev)
        w_f8, scales = torch.ops.nanogpt.quant_up_weights(torch.stack([w.detach() for w in w_fc]))
        down = None
        if fp8down:
            # the delayed-scaling state of the FP8 down projection (reference train_gpt.py:1423-1434, 1670-1675): e4m3 copy of
            # W_proj stored [D, H] with its scale, the activation scale from a first pass's amax with the reference's headroom
            w2_scale = (w_pt[0].detach().float().abs().max() / 448).reshape(1)
            w2_dh = torch.empty((1, D, H), dtype=torch.float8_e4m3fn, device=dev)
            nxt, part = torch.empty(1, device=dev), torch.zeros((1, (H // 64) * (D // 64)), device=dev)
            amd.fused.quantize_transpose_mlp_down_weights(w_pt[0].detach()[None], w2_dh, nxt, w2_scale, part)
            normed, x_f8, dequant = torch.ops.nanogpt.mlp_input_quant(xr, scales[0:1])
            act_scale = (torch.ops.nanogpt.fc_relu2_fwd(x_f8, w_f8[0], dequant).float().max() * 1.25 / 448).reshape(1)
            down = (w2_dh[0].T, w2_scale, act_scale, torch.zeros(1024, device=dev))

        def step():
            xr.grad = None
            for l in range(L):     # the layers run back to back on one stream, nothing synchronises in between
                w_fc[l].grad = w_pt[l].grad = None
                normed, x_f8, dequant = torch.ops.nanogpt.mlp_input_quant(xr, scales[l:l + 1])
                if down is not None:
                    out = amd.ReLUSqrdMLP(normed[None], w_fc[l], w_pt[l], w_f8[l], dequant, x_f8[None], *down)
                else:
                    out = amd.ReLUSqrdMLP(normed[None], w_fc[l], w_pt[l], w_f8[l], dequant, x_f8[None])
                if bwd:
                    out.backward(dy)
            return out
        flops = (12.0 if bwd else 4.0) * Mm * D * H * L
        desc = {"mlp_fwd": "config 2: norm + quantise + FP8 c_fc with ReLU^2 + bf16 c_proj, forward",
                "mlp_fwd_fp8down": "config 2 with the FP8 down projection: norm + quantise + FP8 c_fc with ReLU^2 and e4m3 copy + FP8 c_proj, forward",
                "mlp_fwd_bwd": "config 4 (one layer): norm + quantise + FP8 c_fc with ReLU^2 + bf16 c_proj, forward+backward",
                "mlp_cfg4": "config 4: 12 layers (own weights) of norm + quantise + FP8 c_fc with ReLU^2 + bf16 c_proj, forward+backward"}[wl] \
            + ", M=49152 D=768 H=3072"
        tokens = Mm
        work = mlp_work(Mm, D, H, bwd, L)
        if fp8down:
            work["fp8_gemm"] = work.pop("bf16_gemm")[0], "mfma-fp8"
        if not args.no_cpu_baseline:
            cpu = cpu_baseline_mlp(x, w_fc_c[0], w_pt_c[0], dy_c, bwd)
            if L > 1:
                cpu["value"] /= L
                cpu["sample"] += f"; tokens/s divided by the {L} layers of a step"
    elif wl == "cfg5":
        # medium-track shapes: FP8 lm_head + softcapped CE forward+backward and one FP8 MLP layer forward+backward per step
        Mm, D, H, Vv = 65536, 1024, 4096, 50304
        xh_c, wh_c, tg_c, sc = make_cfg3(seed=5, M=Mm, K=D, V=Vv)
        xh, wh, tg = xh_c.to(dev).requires_grad_(True), wh_c.to(dev).requires_grad_(True), tg_c.to(dev)
        x, w_fc_c, w_pt_c, dy_c = make_mlp(5, Mm, D, H)
        xr, w_fc, w_pt, dy = x.to(dev).requires_grad_(True), w_fc_c[0].to(dev).requires_grad_(True), w_pt_c[0].to(dev).requires_grad_(True), dy_c.to(dev)
        w_f8, scales = torch.ops.nanogpt.quant_up_weights(w_fc.detach()[None])

        def step():
            xh.grad = wh.grad = xr.grad = w_fc.grad = w_pt.grad = None
            losses = amd.FusedSoftcappedCrossEntropy.apply(xh, tg, None, None, None, wh, sc["x_s"], sc["w_s"], sc["grad_s"], 1.0,
                                                           23.0, 5.0, 7.5, "out_in")
            losses.sum().backward()
            normed, x_f8, dequant = torch.ops.nanogpt.mlp_input_quant(xr, scales[0:1])
            out = amd.ReLUSqrdMLP(normed[None], w_fc, w_pt, w_f8[0], dequant, x_f8[None])
            out.backward(dy)
            return out
        flops = 6.0 * Mm * D * Vv + 12.0 * Mm * D * H
        desc, tokens = "config 5: lm_head + softcapped CE forward+backward and one FP8 MLP layer forward+backward, M=65536 D=1024 H=4096 V=50304", Mm
        work = mlp_work(Mm, D, H, True)
        work.update({n: (2.0 * Mm * D * Vv, "mfma-fp8") for n in ("lm_head_ce_fwd", "dx_gemm", "dw_gemm")})
        # the slot named dlogits_recompute holds the code -> e5m2 pass (2 x M x V bytes) unless the backward recomputes the logits
        work["dlogits_recompute"] = (2.0 * Mm * Vv, "hbm") if amd.fused.CE_BACKWARD == "codes" else (2.0 * Mm * D * Vv, "mfma-fp8")
        if not args.no_cpu_baseline:
            a = cpu_baseline(xh_c, wh_c, tg_c, sc, budget_s=10.0)
            b = cpu_baseline_mlp(x, w_fc_c[0], w_pt_c[0], dy_c, True, budget_s=8.0)
            cpu = {"value": 1.0 / (1.0 / a["value"] + 1.0 / b["value"]), "unit": "tokens/s", "cores": a["cores"], "kind": "port",
                   "sample": "the two halves timed separately and combined as time per token: [" + a["sample"] + "] and [" + b["sample"] + "]"}
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
        flops, desc, tokens = 0.0, "nanogpt::ce_fwd_bwd on materialised logits, M=49152 V=50304 (bf16 in, e5m2 gradient out)", Mm
        dtype = "bf16 in, fp32 arithmetic, e5m2 out"
    else:
        return None
    if args.calibrate_copy:
        calibrate_copy(dev)
    out, ms, median_ms, kernels = run_timed(lib, step, args.steps, args.warmup)
    if wl == "ce_logits":
        # a single kernel with no profile slot: the step is the launch
        hbm_bytes = tokens * 50304 * 3 + tokens * 12
        kernels = {"ce_rows": {"launches_per_step": 1.0, "avg_ms": median_ms, "ms_per_step": median_ms}}
        work = {"ce_rows": (hbm_bytes, "hbm")}
    return emit(args, lib, desc, tokens, flops, ms, median_ms, kernels, work, traffic_key, dtype=dtype, extra=extra, cpu=cpu)


SECONDARY_IN_DEFAULT_LINE = (("cfg1", "mm_cfg1"), ("cfg2", "mlp_fwd"), ("cfg2_fp8_down", "mlp_fwd_fp8down"), ("cfg4", "mlp_cfg4"), ("cfg5", "cfg5"))


def secondary_summary(args, amd, lib, dev):
    """The other benchmark configurations, timed briefly (no CPU baseline), for the default line's "secondary" entry."""
    out = {}
    for key, wl in SECONDARY_IN_DEFAULT_LINE:
        sub = argparse.Namespace(**{**vars(args), "workload": wl, "no_cpu_baseline": True, "calibrate_copy": False,
                                    "steps": 20 if wl != "mlp_cfg4" else 10, "warmup": 3})
        r = secondary(sub, amd, lib, dev)
        roof = r.get("roofline") or {}
        out[key] = {"workload": r["config"]["workload"], "ms": r["ms_per_step"], "tflops": r.get("tflops"),
                    "tokens_per_s": r["value"], "kernel": roof.get("kernel"), "roofline_frac": roof.get("frac"),
                    "roofline_peak": roof.get("peak"), "roofline_unit": roof.get("unit")}
        torch.cuda.empty_cache()
    return out


def workload_ceiling(args, amd, dev) -> int:
    """What bounds an fp8 GEMM on this machine: the matrix pipe alone and the k-step skeleton (LDS fragment reads,
    barrier, direct-to-LDS loads) on zero and on random operands with the shader clock they run at, the shipped kernel
    without its epilogue, and the vendor library's fp8 GEMM on the shapes of this path."""
    lib = amd._lib.load_bench()
    st = torch.cuda.current_stream().cuda_stream
    cus = lib.ngpt_num_cus()
    E4 = torch.float8_e4m3fn
    res = {"workload": "ceiling", "device": torch.cuda.get_device_name(0), "compute_units": cus, "peak_fp8_tflops": PEAK_FP8_TFLOPS, "rows": []}
    stride = 16384
    nbytes = (512 << 10) + cus * stride + (64 << 10)
    sink = torch.zeros(512, device=dev)
    ticks = torch.zeros(cus, 2, dtype=torch.int64, device=dev)
    iters = 4000
    for data in ("zeros", "random fp8"):
        src = torch.zeros(nbytes, dtype=torch.uint8, device=dev) if data == "zeros" else \
            torch.randint(0, 120, (nbytes,), dtype=torch.uint8, device=dev)          # finite e4m3 codes
        for mode, what in ((0, "matrix pipe alone"), (1, "+ LDS fragment reads"), (3, "+ barrier per k-step"), (7, "+ direct-to-LDS operand loads")):
            for _ in range(2):
                rc = lib.ngpt_bench_kstep_rate(src.data_ptr(), stride, mode, iters, cus, sink.data_ptr(), ticks.data_ptr(), st)
                assert rc == 0, lib.ngpt_last_error()
            torch.cuda.synchronize()
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            lib.ngpt_bench_kstep_rate(src.data_ptr(), stride, mode, iters, cus, sink.data_ptr(), ticks.data_ptr(), st)
            e1.record()
            torch.cuda.synchronize()
            ms = e0.elapsed_time(e1)
            tk = ticks.double().mean(0)
            res["rows"].append({"what": f"k-step skeleton, {what}", "operands": data, "ms": ms,
                                "tflops": 2.0 * 256 * 256 * 128 * iters * cus / ms / 1e9,
                                "cycles_per_kstep": float(tk[0]) / iters, "shader_clock_mhz": float(tk[0] / tk[1] * 100.0)})
    # the shipped GEMM kernel, result discarded (contraction loop alone), at the logits shape
    R, C, Kk = 49152, 50304, 768
    for data in ("zeros", "random fp8"):
        mk = (lambda n: torch.zeros(n, Kk, dtype=torch.uint8, device=dev)) if data == "zeros" else \
            (lambda n: torch.randint(0, 120, (n, Kk), dtype=torch.uint8, device=dev))
        a, b = mk(R).view(E4), mk(C).view(E4)
        out = torch.zeros(16, device=dev)
        call = lambda: lib.ngpt_gemm_fp8_tn(a.data_ptr(), 0, Kk, b.data_ptr(), 0, Kk, R, C, Kk, 1.0, out.data_ptr(), C, 3, st)
        for _ in range(3):
            assert call() == 0, lib.ngpt_last_error()
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(5):
            call()
        e1.record()
        torch.cuda.synchronize()
        ms = e0.elapsed_time(e1) / 5
        tiles = ((R + 255) // 256) * ((C + 255) // 256)
        ksteps = -(-tiles // cus) * (Kk // 128)
        clk, wall = float(out[2]), float(out[3])
        res["rows"].append({"what": f"shipped gemm_tn_kernel, epilogue discarded, {R} x {C} x {Kk}", "operands": data, "ms": ms,
                            "tflops": 2.0 * R * C * Kk / ms / 1e9, "cycles_per_kstep": clk / ksteps,
                            "shader_clock_mhz": clk / max(wall, 1.0) * 100.0})
        del a, b
    # the vendor library (hipBLASLt behind torch._scaled_mm), e4m3 x e4m3 -> bf16, random operands
    one = torch.ones((), device=dev)
    for (Mm, Nn, Kk) in ((8192, 8192, 8192), (16384, 16384, 8192), (16384, 50304, 768), (49152, 768, 50304), (49152, 3072, 768)):
        a = (torch.randn(Mm, Kk, device=dev) * 4).to(E4)
        b = (torch.randn(Nn, Kk, device=dev) * 4).to(E4)
        f = lambda: torch._scaled_mm(a, b.T, scale_a=one, scale_b=one, out_dtype=torch.bfloat16, use_fast_accum=True)
        try:
            for _ in range(3):
                f()
            torch.cuda.synchronize()
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            for _ in range(10):
                f()
            e1.record()
            torch.cuda.synchronize()
            ms = e0.elapsed_time(e1) / 10
            res["rows"].append({"what": f"vendor library torch._scaled_mm {Mm} x {Nn} x {Kk} -> bf16", "operands": "random fp8", "ms": ms,
                                "tflops": 2.0 * Mm * Nn * Kk / ms / 1e9})
        except Exception as e:    # a shape the library refuses is reported, not fatal
            res["rows"].append({"what": f"vendor library torch._scaled_mm {Mm} x {Nn} x {Kk}", "error": str(e)[:200]})
        del a, b
    print(json.dumps(res))
    return 0


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--workload", default="lmhead_ce",
                    help="lmhead_ce (default, the headline configuration 3) | mm_cfg1 | mm_lmhead | mlp_fwd | mlp_fwd_bwd | mlp_cfg4 | "
                         "ce_logits | cfg5 | ceiling")
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--ce-backward", choices=("codes", "recompute"), default="codes",
                    help="headline workload: where the backward takes the e5m2 gradient of the logits from")
    ap.add_argument("--tail-columns", type=int, default=0,
                    help="headline workload: this many of the last vocabulary entries get logits far below the sigma-code window "
                         "in every row (and grad_scale = 64, so that they matter): measures the fallback of the codes backward")
    ap.add_argument("--no-other-mode", action="store_true", help="headline workload: do not also time the other --ce-backward mode")
    ap.add_argument("--no-tail", action="store_true", help="headline workload: do not also time the step with 47 vocabulary columns below the code window")
    ap.add_argument("--no-secondary", action="store_true", help="headline workload: leave out the brief runs of configurations 1, 2, 4 and 5")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="also run one 1 GiB device-to-device copy, the known-size kernel that scales "
                         "the FETCH_SIZE / WRITE_SIZE counters of a rocprofv3 --pmc run")
    args = ap.parse_args()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print("bench.py: this path is built and measured on ONE GPU (the kernel on one GPU's share of the "
              "batch, M=49152); runs with more than one GPU are not part of this build.", file=sys.stderr)
        return 2

    sys.path.insert(0, ROOT)
    import modded_nanogpt_amd as amd
    lib = amd._lib.load()
    assert torch.cuda.is_available(), "bench.py needs a GPU"
    dev = torch.device("cuda:0")
    if args.workload == "ceiling":
        return workload_ceiling(args, amd, dev)
    if args.workload != "lmhead_ce":
        result = secondary(args, amd, lib, dev)
        if result is None:
            print(f"bench.py: unknown workload {args.workload}", file=sys.stderr)
            return 2
    else:
        result = workload_lmhead_ce(args, amd, lib, dev)
        if not args.no_secondary and not args.tail_columns:
            result["secondary"] = secondary_summary(args, amd, lib, dev)
    print(json.dumps(result))
    return 0


if __name__ == "__main__":
    sys.exit(main())
