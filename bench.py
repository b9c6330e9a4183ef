#!/usr/bin/env python3
"""Headline benchmark: effective attention TOPS of the SageAttention forward path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload c2] [--no-cpu-baseline]

A step is one full pass of the hot path over the workload, inputs already resident in HBM:
K mean -> INT8 quantise K and Q -> FP8/FP16 V panels -> fused attention (one `sageattn` call).
`value` is effective TOPS of that whole step; `roofline` is the fused attention kernel alone, timed
with HIP events on the stream it is launched on; `cpu_baseline` is the oracle's PyTorch
quantise + SDPA pipeline timed on this machine's host cores on a bounded sample of the same workload.
Prints one JSON line.
"""
from __future__ import annotations

import argparse
import json
import os
import statistics
import sys
import time

import torch

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

METRIC = "effective attention TOPS at B2 H32 S16k d128 causal; % of MFMA peak"
PEAK_INT8_FP8 = 5033.2   # MI355X dense INT8 / FP8 MFMA peak, TOP/s (256 CUs x 2.4 GHz x 8192 ops/clk)
PEAK_FP16 = 2516.6       # dense FP16 MFMA peak, TFLOP/s


# HBM-side bytes per launch of the attention kernel, from the committed rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE
# runs on this same command (profiles/attn_kernel_c2_pmc.md): (1 245 800 + 262 140) counter units x 2.0 (the factor the
# same counters read for a 512 MiB device copy) x 1 KiB.  Measured for config 2 only.
TRAFFIC_BYTES = {"c2": (1245800 + 262140) * 2.0 * 1024}


def blended_peak(pv: str) -> float:
    """FP8 P.V: both GEMMs run at the INT8/FP8 rate.  FP16 P.V: half of the ops run at the FP16 rate."""
    if pv == "fp8":
        return PEAK_INT8_FP8
    return 1.0 / (0.5 / PEAK_INT8_FP8 + 0.5 / PEAK_FP16)


def time_attention_kernel(sa, S, w, iters: int):
    """Average duration of the fused attention kernel alone, HIP events on the launch stream: the variant
    the one-call pipeline runs (K and V pre-quantised, Q quantised in the kernel's prologue).  Returns
    milliseconds per launch."""
    import ctypes
    from baselinebenchmark_amd._cabi import check, lib
    kw = w.kwargs
    layout = w.layout
    if w.cu_seqlens is not None:
        return None
    q, k, v = w.q, w.k, w.v
    km = sa.k_mean(k, layout)
    qi, qs, ki, ks = sa.per_block_int8(q, k, km=km, BLKQ=kw["BLKQ"], BLKK=kw["BLKK"], tensor_layout=layout)
    panels, vs = sa.prepare_v(v, layout, kw["pv_mode"])
    out = torch.empty_like(q)
    B, Hq, Sq, D, qsb, qsh, qsn = S._layout(qi, layout)
    _, Hkv, Skv, _, ksb, ksh, ksn = S._layout(ki, layout)
    _, _, _, _, osb, osh, osn = S._layout(out, layout)
    pv = S._pv(kw["pv_mode"])
    stream = torch.cuda.current_stream()

    def launch():
        check(lib().sage_attn_fwd_qfused(S._ptr(q), S._dt(q.dtype), float(D ** -0.5), S._ptr(ki), S._ptr(panels), S._ptr(ks),
                                         S._ptr(vs), S._ptr(out), None,
                                         B, Hq, Hkv, Sq, Skv, D, qsb, qsh, qsn, ksb, ksh, ksn, osb, osh, osn,
                                         kw["BLKQ"], kw["BLKK"], int(w.causal), pv, S._dt(q.dtype), None, None, None, 0, 0, 0,
                                         ctypes.c_void_p(stream.cuda_stream)))
    for _ in range(3):
        launch()
    stream.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record(stream)
    for _ in range(iters):
        launch()
    e1.record(stream)
    e1.synchronize()
    return e0.elapsed_time(e1) / iters


def cpu_baseline(name: str, budget_s: float = 20.0):
    """oracle.attention.cpu_quantize_sdpa on a sample of the workload (fewer batch x head pairs), sized so
    that it runs for roughly `budget_s` seconds.  Effective TOPS of the sample / its wall time."""
    from baselinebenchmark_amd import workloads
    from oracle import attention as oa
    threads = torch.get_num_threads()
    heads = 8
    w = workloads.make(name, device="cpu", heads=heads, batch=1)
    kw = w.kwargs
    t0 = time.perf_counter()
    oa.cpu_quantize_sdpa(w.q, w.k, w.v, w.layout, w.causal, None, kw["BLKQ"], kw["BLKK"], True)
    t1 = time.perf_counter() - t0
    reps = max(1, min(64, int(budget_s / max(t1, 1e-3)) - 1))
    t0 = time.perf_counter()
    for _ in range(reps):
        oa.cpu_quantize_sdpa(w.q, w.k, w.v, w.layout, w.causal, None, kw["BLKQ"], kw["BLKK"], True)
    dt = (time.perf_counter() - t0) / reps if reps else t1
    return {
        "value": w.ops / dt / 1e12, "unit": "TOPS", "cores": threads, "kind": "port",
        "sample": f"{name} restricted to batch 1 x {heads} head(s) ({w.ops:.3e} effective ops per pass), "
                  f"{reps} timed pass(es) after 1 warm-up, {dt:.2f} s per pass, torch threads={threads}, "
                  f"os.cpu_count()={os.cpu_count()}",
    }


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=30,
                    help="untimed steps before the timed ones; the first dozen steps after idle run up to 30 %% slower "
                         "while the GPU clocks ramp, so the default covers that transient")
    ap.add_argument("--workload", default="c2", choices=["c0", "c1", "c2", "c3", "c4"])
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--cpu-seconds", type=float, default=20.0)
    ap.add_argument("--copy-calibration", action="store_true",
                    help="also run three 512 MiB device-to-device copies (a kernel of known traffic, used to scale "
                         "the FETCH_SIZE / WRITE_SIZE counters of a rocprofv3 --pmc run)")
    args = ap.parse_args()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print("bench.py measures one GPU: this path is built and measured on a single MI355X "
              "(--gpus must be 1); it shards over (batch, kv-head) with no exchange.", file=sys.stderr)
        sys.exit(2)

    import baselinebenchmark_amd as sa
    from baselinebenchmark_amd import sageattention as S
    from baselinebenchmark_amd import workloads

    torch.cuda.set_device(0)
    w = workloads.make(args.workload, device="cuda")

    if w.cu_seqlens is None:
        def step():
            return sa.sageattn(w.q, w.k, w.v, **w.kwargs)
    else:
        def step():
            return sa.sageattn_varlen(w.q, w.k, w.v, w.cu_seqlens, w.cu_seqlens, w.max_seqlen, w.max_seqlen, **w.kwargs)

    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
    torch.cuda.synchronize()
    ms = (time.perf_counter() - t0) * 1e3 / args.steps
    value = w.ops / (ms * 1e-3) / 1e12

    pv = w.kwargs["pv_mode"]
    peak = blended_peak(pv)
    kms = time_attention_kernel(sa, S, w, max(args.steps, 10))
    roofline = None
    if kms is not None:
        achieved = w.ops / (kms * 1e-3) / 1e12
        roofline = {"bound": "mfma", "achieved": round(achieved, 1), "peak": round(peak, 1), "unit": "TFLOP/s",
                    "frac": round(achieved / peak, 4), "traffic": TRAFFIC_BYTES.get(args.workload),
                    "kernel": "sage::attn_kernel", "kernel_ms": round(kms, 4),
                    "note": "algorithmic ops = 4*B*Hq*Sq*Skv*D*(1/2 causal) per launch / HIP-event average launch time"}
    out = {
        "metric": METRIC, "value": round(value, 1), "unit": "TOPS", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms, 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "int8 QK / " + ("fp8-e4m3 PV" if pv == "fp8" else "fp16 PV") + " / fp32 softmax+accumulate",
        "data": "synthetic",
        "config": {"workload": w.desc, "step": "K mean + INT8 quantise Q,K + V panels + fused attention (sageattn)",
                   "effective_ops": w.ops, "frac_of_mfma_peak_end_to_end": round(value / peak, 4)},
        "roofline": roofline,
    }
    if args.copy_calibration:
        x = torch.empty(128 * 1024 * 1024, device="cuda", dtype=torch.int32)
        y = torch.empty_like(x)
        for _ in range(3):
            y.copy_(x)
        torch.cuda.synchronize()
    if not args.no_cpu_baseline:
        out["cpu_baseline"] = cpu_baseline(args.workload if args.workload != "c4" else "c2", args.cpu_seconds)
    print(json.dumps(out))


if __name__ == "__main__":
    main()
