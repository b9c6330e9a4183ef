"""SageAttention forward benchmark for the MI355X backend.

Counterpart of backends/_enflame/benchmarks/sage_attention_native_benchmark.py (the 20-shape table of
:70-78, synthetic quantised operands :253-273, correctness gate before timing :294-354 and :408-425,
TSV columns :392-395, ops = 4*B*HQ*T*T*D :447-455, --isolate-shapes :200-250) and of the core / end-to-end
split of backends/_mthreads/benchmarks/sage_attention_benchmark_compare.py:505-559:

  core : forward() on INT8 operands and scales that already exist (what the reference table times)
  e2e  : sageattn() on fp16/bf16 tensors, i.e. K mean + both quantisers + V preparation + attention

Per docs/benchmark_conventions.md:24-51 every row reports mean / median / p99 over per-iteration HIP-event
samples, and one machine-readable result file per run is written under ``results/`` (untracked).

    python -m baselinebenchmark_amd.benchmarks.sage_attention_benchmark                  # the 20-shape table
    python -m baselinebenchmark_amd.benchmarks.sage_attention_benchmark --path e2e --causal --pv fp8
    python -m baselinebenchmark_amd.benchmarks.sage_attention_benchmark --custom-shapes --batch-size 2 \\
        --num-heads 32 --head-dim 128 --seq-lens 16384 --dtype bfloat16 --causal --pv fp8 --blkq 64 --blkk 128
"""
from __future__ import annotations

import argparse
import json
import math
import subprocess
import sys
import time
from pathlib import Path

TABLE_BATCH_SEQ = ((1, 1024), (4, 1024), (1, 4096), (1, 8192), (1, 16384))
TABLE_HEAD_DIMS = (64, 128)
TABLE_DTYPES = ("float16", "bfloat16")
TABLE_HEADS = 32
GATE_Q_LEN, GATE_KV_LEN = 129, 70
COLUMNS = ("provider", "backend", "path", "B", "T", "HQ", "HKV", "D", "dtype", "causal", "pv", "latency_ms", "median_ms",
           "p99_ms", "tflops", "status", "gate_max_abs")


def build_parser() -> argparse.ArgumentParser:
    p = argparse.ArgumentParser(description="Benchmark the MI355X SageAttention forward")
    p.add_argument("--path", choices=("core", "e2e", "both"), default="core",
                   help="core = forward() on quantised operands; e2e = sageattn() including the quantisers")
    p.add_argument("--custom-shapes", action="store_true",
                   help="use --batch-size/--num-heads/--num-kv-heads/--head-dim/--seq-lens/--dtype instead of the 20-shape table")
    p.add_argument("--isolate-shapes", action="store_true", help="run every shape in a fresh Python process")
    p.add_argument("--batch-size", type=int, default=1)
    p.add_argument("--num-heads", type=int, default=32)
    p.add_argument("--num-kv-heads", type=int, help="defaults to --num-heads; smaller for GQA/MQA")
    p.add_argument("--head-dim", type=int, choices=(64, 128), default=128)
    p.add_argument("--seq-lens", type=int, nargs="+", default=(1024, 4096, 8192, 16384))
    p.add_argument("--dtype", choices=TABLE_DTYPES, default="float16")
    p.add_argument("--causal", action="store_true", help="causal mask (effective ops are halved)")
    p.add_argument("--pv", choices=("fp16", "fp8"), default="fp16", help="precision of the P.V product")
    p.add_argument("--blkq", type=int, choices=(16, 32, 64, 128), default=128)
    p.add_argument("--blkk", type=int, choices=(16, 32, 64, 128), default=64)
    p.add_argument("--q-interleave", type=int, choices=(1, 8), default=1,
                   help="8: eight interleaved scales per Q block (rows r, r+8, ... share one: upstream's per-thread Q granularity)")
    p.add_argument("--k-interleave", type=int, choices=(1, 4), default=1,
                   help="4: four interleaved scales per K block (keys n with equal (n %% 8) // 2 share one; K blocks of 32+ keys)")
    p.add_argument("--warmup", type=int, default=5)
    p.add_argument("--rep", type=int, default=20)
    g = p.add_mutually_exclusive_group()
    g.add_argument("--check-reference", dest="check_reference", action="store_true",
                   help="run a small CPU-reference gate before timing (default)")
    g.add_argument("--no-check-reference", dest="check_reference", action="store_false")
    p.set_defaults(check_reference=True)
    p.add_argument("--atol", type=float, default=3e-2)
    p.add_argument("--rtol", type=float, default=3e-2)
    p.add_argument("--seed", type=int, default=2026)
    p.add_argument("--results-dir", default="results", help="where the per-run result file goes ('' disables it)")
    return p


def configs(args):
    """(B, T, HQ, HKV, D, dtype) tuples: the custom list or the default table, dtype-major like the reference."""
    if args.custom_shapes:
        hkv = args.num_kv_heads or args.num_heads
        return [(args.batch_size, t, args.num_heads, hkv, args.head_dim, args.dtype) for t in args.seq_lens]
    return [(b, t, TABLE_HEADS, TABLE_HEADS, d, dt) for dt in TABLE_DTYPES for d in TABLE_HEAD_DIMS for b, t in TABLE_BATCH_SEQ]


def validate(args) -> None:
    sizes = [args.batch_size, args.num_heads, args.head_dim, args.warmup, args.rep, *args.seq_lens]
    if args.num_kv_heads is not None:
        sizes.append(args.num_kv_heads)
    if any(v <= 0 for v in sizes):
        raise ValueError("all sizes, warmup, and rep must be positive")
    if args.num_heads % (args.num_kv_heads or args.num_heads):
        raise ValueError("num-kv-heads must divide num-heads")
    if args.atol < 0 or args.rtol < 0:
        raise ValueError("atol and rtol must be non-negative")
    if args.k_interleave == 4 and args.blkk == 16:
        raise ValueError("four interleaved K scales need K blocks of 32, 64 or 128 keys")


def effective_ops(batch, heads, seq, dim, causal) -> float:
    return 4.0 * batch * heads * seq * seq * dim * (0.5 if causal else 1.0)


def summarise(samples_ms):
    s = sorted(samples_ms)
    n = len(s)
    p99 = s[min(n - 1, math.ceil(0.99 * n) - 1)]
    median = s[n // 2] if n % 2 else 0.5 * (s[n // 2 - 1] + s[n // 2])
    return {"samples": n, "mean_ms": sum(s) / n, "median_ms": median, "p99_ms": p99, "min_ms": s[0]}


def _paths(args):
    return ("core", "e2e") if args.path == "both" else (args.path,)


def run_isolated(args) -> None:
    """One child process per shape; this parent never touches the GPU."""
    shapes = configs(args)
    for index, (b, t, hq, hkv, d, dt) in enumerate(shapes, start=1):
        print(f"# isolated shape {index}/{len(shapes)}: B={b}, T={t}, HQ={hq}, HKV={hkv}, D={d}, dtype={dt}", flush=True)
        cmd = [sys.executable, "-m", "baselinebenchmark_amd.benchmarks.sage_attention_benchmark", "--custom-shapes",
               "--path", args.path, "--batch-size", str(b), "--num-heads", str(hq), "--num-kv-heads", str(hkv),
               "--head-dim", str(d), "--seq-lens", str(t), "--dtype", dt, "--pv", args.pv, "--blkq", str(args.blkq),
               "--blkk", str(args.blkk), "--q-interleave", str(args.q_interleave), "--k-interleave", str(args.k_interleave),
               "--warmup", str(args.warmup), "--rep", str(args.rep), "--atol", str(args.atol),
               "--rtol", str(args.rtol), "--seed", str(args.seed), "--results-dir", args.results_dir,
               "--check-reference" if args.check_reference else "--no-check-reference"]
        if args.causal:
            cmd.append("--causal")
        subprocess.run(cmd, check=True)


# ------------------------------------------------------------------------------------------------
# everything below touches torch / the GPU
# ------------------------------------------------------------------------------------------------
def _quantised_inputs(torch, b, hq, hkv, t, d, blkq, blkk, dev, qg=1, kg=1):
    """Synthetic operands of the reference table: small INT8 values, random scales, N(0,1) V."""
    q = torch.randint(-16, 16, (b, hq, t, d), device=dev, dtype=torch.int8)
    k = torch.randint(-16, 16, (b, hkv, t, d), device=dev, dtype=torch.int8)
    v = torch.randn((b, hkv, t, d), device=dev, dtype=torch.float16)
    qs = 0.005 + 0.015 * torch.rand((b, hq, -(-t // blkq) * qg), device=dev, dtype=torch.float32)
    ks = 0.005 + 0.015 * torch.rand((b, hkv, -(-t // blkk) * kg), device=dev, dtype=torch.float32)
    return q, k, v, qs, ks


def _expand(torch, scale, blk, groups, length):
    """Per-row scales from per-block ones; with interleaved scales row n takes scale (n // blk) * groups + its group."""
    if groups == 1:
        return scale.cpu().repeat_interleave(blk, dim=-1)[..., :length, None]
    n = torch.arange(length)
    g = n % 8 if groups == 8 else (n % 8) // 2
    return scale.cpu()[..., (n // blk) * groups + g, None]


def _formula_on_cpu(torch, q, k, v, qs, ks, blkq, blkk, causal, qg=1, kg=1):
    """softmax(ln2 * (q*qs)(k*ks)^T) v in fp32 on the host: the gate's yardstick."""
    q, k, v = q.cpu().float(), k.cpu().float(), v.cpu().float()
    q = q * _expand(torch, qs, blkq, qg, q.shape[-2])
    k = k * _expand(torch, ks, blkk, kg, k.shape[-2])
    g = q.shape[1] // k.shape[1]
    k, v = k.repeat_interleave(g, dim=1), v.repeat_interleave(g, dim=1)
    logits = torch.matmul(q, k.transpose(-1, -2)) * math.log(2.0)
    if causal:
        i = torch.arange(q.shape[-2])[:, None]
        j = torch.arange(k.shape[-2])[None, :]
        logits = logits.masked_fill(j > i, -float("inf"))
    return torch.matmul(torch.softmax(logits, dim=-1), v)


def reference_gate(torch, sa, hq, hkv, d, out_dtype, args):
    """129 x 70 case (tail blocks, GQA) against the fp32 formula, as the reference does before timing."""
    groups = hq // hkv
    gkv = min(hkv, 2)
    ghq = gkv * groups
    dev = "cuda"
    q = torch.randint(-8, 8, (1, ghq, GATE_Q_LEN, d), device=dev, dtype=torch.int8)
    k = torch.randint(-8, 8, (1, gkv, GATE_KV_LEN, d), device=dev, dtype=torch.int8)
    v = torch.randn((1, gkv, GATE_KV_LEN, d), device=dev, dtype=torch.float16)
    qg, kg = args.q_interleave, args.k_interleave
    qs = 0.005 + 0.015 * torch.rand((1, ghq, -(-GATE_Q_LEN // args.blkq) * qg), device=dev, dtype=torch.float32)
    ks = 0.005 + 0.015 * torch.rand((1, gkv, -(-GATE_KV_LEN // args.blkk) * kg), device=dev, dtype=torch.float32)
    out, _ = sa.forward(q, k, v, qs, ks, output_dtype=out_dtype, BLKQ=args.blkq, BLKK=args.blkk, is_causal=args.causal,
                        pv_mode=args.pv, q_interleave=qg, k_interleave=kg)
    expected = _formula_on_cpu(torch, q, k, v, qs, ks, args.blkq, args.blkk, args.causal, qg, kg)
    actual = out.cpu().float()
    max_abs = (actual - expected).abs().max().item()
    if args.pv == "fp8":
        # FP8 V and P carry 3 mantissa bits: element-wise closeness at 3e-2 is not the right yardstick (a causal
        # row that sees one key returns that key's fp8-rounded V).  Gate on direction and energy of the error instead.
        cosine = torch.nn.functional.cosine_similarity(actual.flatten(), expected.flatten(), dim=0).item()
        rel_rmse = ((actual - expected).square().mean().sqrt() / (expected.square().mean().sqrt() + 1e-12)).item()
        return cosine >= 0.999 and rel_rmse < 5e-2, max_abs
    loose = out_dtype == torch.bfloat16                           # bf16 output rounds more coarsely
    atol = max(args.atol, 4e-2) if loose else args.atol
    rtol = max(args.rtol, 4e-2) if loose else args.rtol
    return bool(torch.allclose(actual, expected, atol=atol, rtol=rtol)), max_abs


def _time(torch, fn, warmup, rep):
    out = fn()
    out = out[0] if isinstance(out, tuple) else out
    if not bool(torch.isfinite(out).all().item()):
        raise RuntimeError("forward produced non-finite output")
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    samples = []
    for _ in range(rep):
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        fn()
        e1.record()
        e1.synchronize()
        samples.append(e0.elapsed_time(e1))
    return summarise(samples)


def _metadata(torch, sa):
    commit = "unknown"
    try:
        root = Path(__file__).resolve().parents[2]
        commit = subprocess.run(["git", "-C", str(root), "rev-parse", "--short", "HEAD"], capture_output=True, text=True,
                                timeout=10).stdout.strip() or "unknown"
    except Exception:
        pass
    return {"backend": "_amd", "implementation": sa.backend_name(), "device": torch.cuda.get_device_name(0),
            "operator": "sage_attention_forward", "framework_version": torch.__version__,
            "driver_version": str(getattr(torch.version, "hip", "unknown")), "commit": commit}


def benchmark(args) -> list:
    validate(args)
    if args.isolate_shapes:
        run_isolated(args)
        return []
    import torch

    import baselinebenchmark_amd as sa

    torch.manual_seed(args.seed)
    print(f"# backend: {sa.backend_name()}; device: {torch.cuda.get_device_name(0)}")
    print("# core = forward() on INT8 operands; e2e = sageattn() incl. K mean, quantisers and V preparation")
    print("# timed region: the call only (HIP events on the current stream, one sample per iteration); inputs resident;"
          " outputs and workspaces are allocated inside the call by torch's caching allocator")
    print("\t".join(COLUMNS))
    rows, gate_cache = [], {}
    for b, t, hq, hkv, d, dtype_name in configs(args):
        dtype = getattr(torch, dtype_name)
        gate_key = (hq // hkv, d, dtype_name)
        if args.check_reference and gate_key not in gate_cache:
            gate_cache[gate_key] = reference_gate(torch, sa, hq, hkv, d, dtype, args)
        correct, max_abs = gate_cache.get(gate_key, (True, None))
        for path in _paths(args):
            base = {"provider": "mi355x", "backend": "hip", "path": path, "B": b, "T": t, "HQ": hq, "HKV": hkv, "D": d,
                    "dtype": dtype_name, "causal": int(args.causal), "pv": args.pv,
                    "gate_max_abs": "" if max_abs is None else f"{max_abs:.6f}"}
            if not correct:
                rows.append({**base, "latency_ms": "", "median_ms": "", "p99_ms": "", "tflops": "", "status": "INCORRECT"})
                print("\t".join(str(rows[-1][c]) for c in COLUMNS), flush=True)
                continue
            if path == "core":
                q, k, v, qs, ks = _quantised_inputs(torch, b, hq, hkv, t, d, args.blkq, args.blkk, "cuda", args.q_interleave,
                                                    args.k_interleave)
                fn = lambda: sa.forward(q, k, v, qs, ks, output_dtype=dtype, BLKQ=args.blkq, BLKK=args.blkk,  # noqa: E731
                                        is_causal=args.causal, pv_mode=args.pv, q_interleave=args.q_interleave,
                                        k_interleave=args.k_interleave)
            else:
                q = torch.randn((b, hq, t, d), device="cuda", dtype=dtype)
                k = torch.randn((b, hkv, t, d), device="cuda", dtype=dtype)
                v = torch.randn((b, hkv, t, d), device="cuda", dtype=dtype)
                fn = lambda: sa.sageattn(q, k, v, is_causal=args.causal, pv_mode=args.pv, BLKQ=args.blkq,  # noqa: E731
                                         BLKK=args.blkk, q_interleave=args.q_interleave, k_interleave=args.k_interleave)
            stats = _time(torch, fn, args.warmup, args.rep)
            tflops = effective_ops(b, hq, t, d, args.causal) / stats["mean_ms"] * 1e-9
            rows.append({**base, "latency_ms": f"{stats['mean_ms']:.4f}", "median_ms": f"{stats['median_ms']:.4f}",
                         "p99_ms": f"{stats['p99_ms']:.4f}", "tflops": f"{tflops:.2f}", "status": "PASS",
                         "samples": stats["samples"], "warmup": args.warmup, "latency_us": stats["mean_ms"] * 1e3,
                         "blkq": args.blkq, "blkk": args.blkk, "shape": [b, hq, t, d]})
            print("\t".join(str(rows[-1][c]) for c in COLUMNS), flush=True)
            del q, k, v
    if args.results_dir:
        out_dir = Path(args.results_dir)
        out_dir.mkdir(parents=True, exist_ok=True)
        name = out_dir / f"sage_attention_mi355x_{time.strftime('%Y%m%d_%H%M%S')}_{abs(hash(tuple(sys.argv))) % 10000:04d}.json"
        name.write_text(json.dumps({**_metadata(torch, sa), "tolerance": {"atol": args.atol, "rtol": args.rtol,
                                    "method": "129x70 case against the fp32 formula before timing: allclose (fp16 P.V) or cosine >= 0.999 and relative RMSE < 5e-2 (fp8 P.V)"},
                                    "cases": rows}, indent=1))
        print(f"# result file: {name}")
    return rows


if __name__ == "__main__":
    benchmark(build_parser().parse_args())
