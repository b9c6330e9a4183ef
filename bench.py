#!/usr/bin/env python3
"""Headline benchmark: effective attention TOPS of the SageAttention forward path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload c0|c1|c2|c3|c4|all] [--no-cpu-baseline]

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
import sys
import time

import torch

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

METRIC = "effective attention TOPS at B2 H32 S16k d128 causal; % of MFMA peak"
PEAK_INT8_FP8 = 5033.2   # MI355X dense INT8 / FP8 MFMA peak, TOP/s (256 CUs x 2.4 GHz x 8192 ops/clk)
PEAK_FP16 = 2516.6       # dense FP16 MFMA peak, TFLOP/s


TRAFFIC_FILE = os.path.join(ROOT, "profiles", "attn_kernel_traffic.json")
KERNEL_SOURCES = ["sage_attn_kernel.h", "sage_attn.hip", "sage_attn_qfuse.hip", "sage_attn_mask.hip", "sage_attn_kinterleave.hip",
                  "sage_common.h", "sage_launch.h"]


def kernel_source_digest() -> str:
    """sha256 over the sources that define the attention kernel: what a committed counter profile is valid for."""
    import hashlib
    h = hashlib.sha256()
    for name in KERNEL_SOURCES:
        with open(os.path.join(ROOT, "baselinebenchmark_amd", "csrc", name), "rb") as f:
            h.update(f.read())
    return h.hexdigest()


def measured_traffic(workload: str):
    """HBM-side bytes per launch of the attention kernel from the committed rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE
    summary (profiles/attn_kernel_traffic.json, written by `python -m baselinebenchmark_amd.benchmarks.traffic_profile`
    from the counter runs), valid only for the kernel sources it was measured on.  Returns (bytes or None, note)."""
    try:
        with open(TRAFFIC_FILE) as f:
            doc = json.load(f)
    except (OSError, ValueError) as exc:
        return None, f"no committed counter profile ({exc.__class__.__name__})"
    if doc.get("kernel_source_sha256") != kernel_source_digest():
        return None, "the committed counter profile was measured on other kernel sources (sha256 differs): re-run the --pmc passes"
    row = doc.get("workloads", {}).get(workload)
    if row is None:
        return None, f"no counter profile for workload {workload}"
    return row["bytes"], (f"FETCH_SIZE {row['fetch_kib']:.0f} KiB x {row['fetch_factor']:.2f} + WRITE_SIZE {row['write_kib']:.0f} KiB x "
                          f"{row['write_factor']:.2f} per launch (factors from a 512 MiB device copy in the same runs)")


def blended_peak(pv: str) -> float:
    """FP8 P.V: both GEMMs run at the INT8/FP8 rate.  FP16 P.V: half of the ops run at the FP16 rate."""
    if pv == "fp8":
        return PEAK_INT8_FP8
    return 1.0 / (0.5 / PEAK_INT8_FP8 + 0.5 / PEAK_FP16)


def time_attention_kernel(sa, S, w, iters: int):
    """Average duration of the fused attention kernel alone, HIP events on the launch stream: the variant
    the one-call pipeline runs (K and V pre-quantised, Q quantised in the kernel's prologue), for fixed-length
    and packed workloads alike.  Returns milliseconds per launch."""
    import ctypes
    from baselinebenchmark_amd._cabi import check, lib
    kw = w.kwargs
    layout = w.layout
    q, k, v = w.q, w.k, w.v
    pv = S._pv(kw["pv_mode"])
    out = torch.empty_like(q)
    stream = torch.cuda.current_stream()
    st = ctypes.c_void_p(stream.cuda_stream)
    if w.cu_seqlens is None:
        km = sa.k_mean(k, layout)
        _, _, ki, ks = sa.per_block_int8(q, k, km=km, BLKQ=kw["BLKQ"], BLKK=kw["BLKK"], tensor_layout=layout)
        panels, vs = sa.prepare_v(v, layout, kw["pv_mode"])
        B, Hq, Sq, D, qsb, qsh, qsn = S._layout(q, layout)
        _, Hkv, Skv, _, ksb, ksh, ksn = S._layout(ki, layout)
        _, _, _, _, osb, osh, osn = S._layout(out, layout)
        args = (B, Hq, Hkv, Sq, Skv, D, qsb, qsh, qsn, ksb, ksh, ksn, osb, osh, osn, kw["BLKQ"], kw["BLKK"], int(w.causal), pv,
                S._dt(q.dtype), None, None, None, 0, 0, 0, st)
    else:
        # packed batch: the same pieces through the C ABI -- plan, K mean per sequence, INT8 K, V panels
        cu, nseq, L = w.cu_seqlens, w.cu_seqlens.numel() - 1, w.max_seqlen
        Tq, Hq, D = q.shape
        Tk, Hkv, _ = k.shape
        km = torch.empty((nseq, Hkv, D), device=q.device, dtype=k.dtype)
        nb = lib().sage_k_mean_workspace_bytes(nseq, Hkv, L, D)
        ws = torch.empty(max(nb, 8), device=q.device, dtype=torch.uint8)
        check(lib().sage_k_mean(S._ptr(k), S._ptr(km), S._ptr(ws), nb, nseq, Hkv, L, D, 0, k.stride(1), k.stride(0), S._dt(k.dtype),
                                S._ptr(cu), st))
        _, _, ki, ks, plan, offs = sa.per_block_int8_varlen(q, k, cu, cu, L, L, km=km, BLKQ=kw["BLKQ"], BLKK=kw["BLKK"])
        plan, offs = sa.varlen_plan(cu, cu, Tq, kw["BLKQ"], kw["BLKK"], is_causal=w.causal)   # (tile order for this mask)
        panel_sh = Tk // 128 + nseq
        panels = torch.zeros(Hkv * panel_sh * 128 * D * (1 if pv else 2), device=q.device, dtype=torch.uint8)
        vs = torch.empty((nseq, Hkv, D), device=q.device, dtype=torch.float32) if pv else None
        nb = lib().sage_prep_v_workspace_bytes(nseq, Hkv, L, D, pv)
        ws = torch.empty(max(nb, 8), device=q.device, dtype=torch.uint8)
        check(lib().sage_prep_v(S._ptr(v), S._ptr(panels), S._ptr(vs), S._ptr(ws), nb, nseq, Hkv, L, D, 0, v.stride(1), v.stride(0),
                                S._dt(v.dtype), pv, S._ptr(cu), ctypes.c_void_p(plan.data_ptr() + 4 * offs[2]), panel_sh, st))
        args = (nseq, Hq, Hkv, L, L, D, 0, q.stride(1), q.stride(0), 0, ki.stride(1), ki.stride(0), 0, out.stride(1), out.stride(0),
                kw["BLKQ"], kw["BLKK"], int(w.causal), pv, S._dt(q.dtype), S._ptr(cu), S._ptr(cu), S._ptr(plan), Tq,
                ks.shape[1], panel_sh, st)

    def launch():
        check(lib().sage_attn_fwd_qfused(S._ptr(q), S._dt(q.dtype), float(D ** -0.5), S._ptr(ki), S._ptr(panels), S._ptr(ks),
                                         S._ptr(vs), S._ptr(out), None, *args))
    # (not part of the timed steps: untimed launches until the clocks have settled after idle -- 50 ms of them, at least 20)
    t_warm, n_warm = time.perf_counter(), 0
    while n_warm < 20 or time.perf_counter() - t_warm < 0.05:
        for _ in range(5):
            launch()
        stream.synchronize()
        n_warm += 5
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record(stream)
    for _ in range(iters):
        launch()
    e1.record(stream)
    e1.synchronize()
    return e0.elapsed_time(e1) / iters, out


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


def run_workload(name: str, args, sa, S, workloads) -> dict:
    w = workloads.make(name, device="cuda")
    if args.constant_inputs:
        # diagnostic: the same instruction streams on operands that toggle no bits (every element 1.0) -- the part holds a
        # higher clock on them, which separates what the schedule costs from what the data cost
        for t in (w.q, w.k, w.v):
            t.fill_(1.0)
    if w.cu_seqlens is None:
        def step():
            return sa.sageattn(w.q, w.k, w.v, **w.kwargs)
    else:
        def step():
            return sa.sageattn(w.q, w.k, w.v, cu_seqlens_q=w.cu_seqlens, cu_seqlens_k=w.cu_seqlens, max_seqlen_q=w.max_seqlen,
                               max_seqlen_k=w.max_seqlen, **w.kwargs)

    # The attention kernel alone first (the roofline figure; its own untimed launches come first), so that the timed steps
    # below find the clocks settled whatever --warmup says.
    pv = w.kwargs["pv_mode"]
    peak = blended_peak(pv)
    kms, kout = time_attention_kernel(sa, S, w, max(args.steps, 10))
    ref = None
    for _ in range(args.warmup):
        ref = step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        last = step()
    torch.cuda.synchronize()
    ms = (time.perf_counter() - t0) * 1e3 / args.steps
    value = w.ops / (ms * 1e-3) / 1e12
    if not torch.equal(kout, ref if ref is not None else last):
        raise RuntimeError("the separately launched attention kernel does not reproduce the one-call result")
    achieved = w.ops / (kms * 1e-3) / 1e12
    traffic, traffic_note = measured_traffic(name)
    roofline = {"bound": "mfma", "achieved": round(achieved, 1), "peak": round(peak, 1), "unit": "TFLOP/s",
                "frac": round(achieved / peak, 4), "traffic": traffic, "traffic_note": traffic_note,
                "kernel": "sage::attn_kernel", "kernel_ms": round(kms, 4),
                "note": "algorithmic ops = 4*B*Hq*Sq*Skv*D*(1/2 causal) per launch / HIP-event average launch time"}
    out = {
        "metric": METRIC, "value": round(value, 1), "unit": "TOPS", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms, 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "int8 QK / " + ("fp8-e4m3 PV" if pv == "fp8" else "fp16 PV") + " / fp32 softmax+accumulate",
        "data": "synthetic" if not args.constant_inputs else "constant 1.0 everywhere (diagnostic run: not the benchmark's data)",
        "config": {"workload": w.desc, "step": "K mean + INT8 quantise Q,K + V panels + fused attention (sageattn)",
                   "effective_ops": w.ops, "frac_of_mfma_peak_end_to_end": round(value / peak, 4)},
        "roofline": roofline,
    }
    if not args.no_cpu_baseline:
        out["cpu_baseline"] = cpu_baseline(name if name != "c4" else "c2", args.cpu_seconds)
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=30,
                    help="untimed steps before the timed ones; the first dozen steps after idle run up to 30 %% slower "
                         "while the GPU clocks ramp, so the default covers that transient")
    ap.add_argument("--workload", default="c2", choices=["c0", "c1", "c2", "c3", "c4", "all"],
                    help="BASELINE configuration; 'all' prints one JSON line per configuration (the CPU baseline only on c2)")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--cpu-seconds", type=float, default=20.0)
    ap.add_argument("--constant-inputs", action="store_true",
                    help="diagnostic: fill q, k and v with 1.0 (same kernels and launch geometry; shows how much of the time "
                         "is the clock the part holds on random operands)")
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
    names = ["c0", "c1", "c2", "c3", "c4"] if args.workload == "all" else [args.workload]
    for name in names:
        if args.workload == "all" and name != "c2":
            saved, args.no_cpu_baseline = args.no_cpu_baseline, True
            out = run_workload(name, args, sa, S, workloads)
            args.no_cpu_baseline = saved
        else:
            out = run_workload(name, args, sa, S, workloads)
        print(json.dumps(out), flush=True)
        torch.cuda.empty_cache()
    if args.copy_calibration:
        x = torch.empty(128 * 1024 * 1024, device="cuda", dtype=torch.int32)
        y = torch.empty_like(x)
        for _ in range(3):
            y.copy_(x)
        torch.cuda.synchronize()


if __name__ == "__main__":
    main()
