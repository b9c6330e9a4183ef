"""Where a q-tile's time goes inside the fused attention kernel: the timing build of the library stamps eight
points of every workgroup on the GPU's constant-rate counter (entry, tile decoded, raw Q arrived, Q operand ready,
first barrier of the main loop, main loop done, stores issued, stores acknowledged) and sums the intervals; the kernel's
wall time says what a workgroup costs beyond them.

    python -m baselinebenchmark_amd.build --timing
    SAGE_MI355X_LIB=baselinebenchmark_amd/csrc/libsage_mi355x_timing.so python -m baselinebenchmark_amd.benchmarks.tile_timing

Prints, per shape, the average per workgroup in nanoseconds for the first, the last and the other wavefronts.  The
timing build is slower than the shipped one (the stamps and their atomics); the intervals are what it is for.  No
counterpart in the reference: a measurement aid.
"""
from __future__ import annotations

import argparse
import ctypes

import torch

import baselinebenchmark_amd as sa
from baselinebenchmark_amd._cabi import LIB_PATH, lib

INTERVALS = ["decode + first requests", "raw Q arrives", "Q maximum + quantise", "first loop barrier", "main loop",
             "epilogue to last store", "store acknowledge"]
TICK_NS = 10.0   # s_memrealtime runs at 100 MHz


def _read():
    fn = getattr(lib(), "sage_tile_timing", None)
    if fn is None:
        raise SystemExit(f"{LIB_PATH} is not a timing build: run `python -m baselinebenchmark_amd.build --timing` and set "
                         "SAGE_MI355X_LIB to csrc/libsage_mi355x_timing.so")
    buf = (ctypes.c_ulonglong * 48)()
    if fn(buf) != 0:
        raise RuntimeError("sage_tile_timing failed")
    return list(buf)


def measure(B, H, S, D, causal, dtype=torch.bfloat16, pv_mode="fp8", blkq=64, blkk=128, launches=5):
    g = torch.Generator(device="cuda").manual_seed(0)
    q, k, v = (torch.randn((B, H, S, D), dtype=dtype, device="cuda", generator=g) for _ in range(3))
    _, _, ki, ks = sa.per_block_int8(q, k, BLKQ=blkq, BLKK=blkk)
    call = lambda: sa.forward_fused_q(q, ki, v, ks, is_causal=causal, pv_mode=pv_mode, BLKQ=blkq, BLKK=blkk)
    prep = lambda: sa.prepare_v(v, "HND", pv_mode)
    for _ in range(10):
        call()
    # wall time of the attention kernel alone: the call minus its V preparation pass, HIP events on the current stream
    def wall(fn):
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(launches):
            fn()
        e1.record()
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) * 1e6 / launches
    prep()
    t_prep = wall(prep)
    _read()
    t_call = wall(call)
    d = _read()
    rows = {}
    for cls, name in enumerate(("first wavefront", "last wavefront", "other wavefronts")):
        n = max(d[cls * 8 + 7], 1)
        rows[name] = [d[cls * 8 + i] * TICK_NS / n for i in range(7)]
    tiles = d[24] / max(d[7], 1)
    # main loop of the FP8 kernels, per period and group: first phase, wait at the odd barrier, second phase, wait at the
    # even barrier (group 0: matrix phase first; group 1: vector phase first)
    for g in (0, 1):
        n = max(d[40 + g], 1)
        rows[f"group {g} phases"] = [d[32 + 4 * g + k] * TICK_NS / n for k in range(4)]
    rows["request issue"] = [d[42] * TICK_NS / max(d[43], 1)]
    rows["raw Q wait"] = [d[44] * TICK_NS / max(d[45], 1)]
    # what a workgroup's slot on a compute unit costs beyond the time its wavefronts measure themselves: the kernel's
    # wall time divided by the workgroups a compute unit runs one after the other, minus a workgroup's own total
    cus = torch.cuda.get_device_properties(q.device).multi_processor_count
    per_cu = B * H * ((S + 255) // 256) / cus
    own = sum(rows["other wavefronts"])
    rows["between workgroups"] = [t_call - t_prep, per_cu, (t_call - t_prep) / per_cu - own]
    return rows, tiles


def timeline(B, H, S, D, causal, dtype=torch.bfloat16, pv_mode="fp8", blkq=64, blkk=128, dump=None):
    """One launch seen from the compute units: the timing build records, per workgroup, its first and last stamp on the
    chip-wide 100 MHz counter and the compute unit it ran on.  Returns, in nanoseconds: the span of the launch (first
    stamp of any workgroup to last stamp of any), and per compute unit (averaged, with the maximum) the time before its
    first workgroup, the gaps between consecutive workgroups, the time inside workgroups and the idle time after its
    last workgroup until the launch ends; also each XCD's finish time relative to the end of the launch."""
    fn = getattr(lib(), "sage_wg_timeline", None)
    if fn is None:
        raise SystemExit(f"{LIB_PATH} is not a timing build")
    if B == 0:      # the packed benchmark configuration (16 sequences of 512..32768 rows, 32 q-heads on 8 KV heads)
        from baselinebenchmark_amd import workloads
        wl = workloads.make("c4")
        for _ in range(4):
            sa.sageattn_varlen(wl.q, wl.k, wl.v, wl.cu_seqlens, wl.cu_seqlens, wl.max_seqlen, wl.max_seqlen, **wl.kwargs)
        n = sum((L + 255) // 256 for L in wl.extra["lens"]) * wl.q.shape[1]
    else:
        g = torch.Generator(device="cuda").manual_seed(0)
        q, k, v = (torch.randn((B, H, S, D), dtype=dtype, device="cuda", generator=g) for _ in range(3))
        _, _, ki, ks = sa.per_block_int8(q, k, BLKQ=blkq, BLKK=blkk)
        for _ in range(6):
            sa.forward_fused_q(q, ki, v, ks, is_causal=causal, pv_mode=pv_mode, BLKQ=blkq, BLKK=blkk)
        n = B * H * ((S + 255) // 256)
    buf = (ctypes.c_ulonglong * (4 * n))()
    got = fn(buf, n)
    if got <= 0:
        raise RuntimeError("sage_wg_timeline failed")
    if dump:     # raw records, one row per workgroup index: first stamp, last stamp, XCC_ID << 32 | HW_ID, K tiles
        import numpy as np
        np.save(dump, np.frombuffer(buf, dtype=np.uint64).reshape(-1, 4)[:got].copy())
    per_cu: dict = {}
    for i in range(got):
        t0, t1, where, tiles = buf[4 * i], buf[4 * i + 1], buf[4 * i + 2], buf[4 * i + 3]
        hw = where & 0xFFFFFFFF
        key = ((where >> 32) & 0xF, (hw >> 13) & 0x7, (hw >> 12) & 0x1, (hw >> 8) & 0xF)   # XCD, shader engine, array, CU
        per_cu.setdefault(key, []).append((t0, t1, tiles))
    first = min(w[0] for ws in per_cu.values() for w in ws)
    last = max(w[1] for ws in per_cu.values() for w in ws)
    lead, gaps, inside, tail, counts, tiles_cu = [], [], [], [], [], []
    xcd_end: dict = {}
    for key, ws in per_cu.items():
        ws.sort()
        lead.append((ws[0][0] - first) * TICK_NS)
        gaps.append(sum(max(b[0] - a[1], 0) for a, b in zip(ws, ws[1:])) * TICK_NS)
        inside.append(sum(w[1] - w[0] for w in ws) * TICK_NS)
        tail.append((last - ws[-1][1]) * TICK_NS)
        counts.append(len(ws))
        tiles_cu.append(sum(w[2] for w in ws))
        xcd_end[key[0]] = max(xcd_end.get(key[0], 0), ws[-1][1])
    stat = lambda xs: (sum(xs) / len(xs), min(xs), max(xs))
    return {"workgroups": got, "compute_units": len(per_cu), "span_ns": (last - first) * TICK_NS,
            "workgroups_per_cu": stat(counts), "k_tiles_per_cu": stat(tiles_cu),
            "before_first_ns": stat(lead), "gaps_ns": stat(gaps), "inside_ns": stat(inside), "after_last_ns": stat(tail),
            "gap_per_handover_ns": sum(gaps) / max(sum(c - 1 for c in counts), 1),
            "xcd_finish_before_end_ns": {x: (last - t) * TICK_NS for x, t in sorted(xcd_end.items())}}


def main():
    ap = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("--shapes", default="2x32x16384x128:1,2x32x16384x128:0,16x32x4096x128:1,64x32x1024x128:1",
                    help="comma-separated BxHxSxD:causal (with --timeline also c4: the packed benchmark configuration)")
    ap.add_argument("--dump", default=None, help="with --timeline: folder that receives the raw per-workgroup records (.npy per shape)")
    ap.add_argument("--timeline", action="store_true",
                    help="per compute unit: time before the first workgroup, between workgroups, inside them, and idle at the end")
    args = ap.parse_args()
    for spec in args.shapes.split(","):
        if spec == "c4":     # (--timeline only) the packed benchmark configuration
            dims, causal, B, H, S, D = "c4", "1", 0, 32, 0, 128
        else:
            dims, causal = spec.split(":")
            B, H, S, D = (int(x) for x in dims.split("x"))
        if args.timeline:
            dump = None
            if args.dump:
                import os
                os.makedirs(args.dump, exist_ok=True)
                dump = os.path.join(args.dump, f"timeline_{dims}_{causal}.npy")
            t = timeline(B, H, S, D, bool(int(causal)), dump=dump)
            f = lambda s3: f"{s3[0]:9.0f} (min {s3[1]:.0f}, max {s3[2]:.0f})"
            print(f"B{B} H{H} S{S} D{D} causal={bool(int(causal))}: {t['workgroups']} workgroups on {t['compute_units']} compute units, "
                  f"launch span {t['span_ns'] / 1e3:.1f} us", flush=True)
            print(f"  workgroups per compute unit {f(t['workgroups_per_cu'])}; K tiles per compute unit {f(t['k_tiles_per_cu'])}")
            print(f"  per compute unit, ns: before its first workgroup {f(t['before_first_ns'])}")
            print(f"                        inside workgroups          {f(t['inside_ns'])}")
            print(f"                        between workgroups         {f(t['gaps_ns'])} = {t['gap_per_handover_ns']:.0f} per hand-over")
            print(f"                        idle after its last one    {f(t['after_last_ns'])}")
            print("  XCD finishes before the end of the launch, ns: " +
                  ", ".join(f"{x}: {v:.0f}" for x, v in t["xcd_finish_before_end_ns"].items()), flush=True)
            continue
        rows, tiles = measure(B, H, S, D, bool(int(causal)))
        print(f"B{B} H{H} S{S} D{D} causal={bool(int(causal))}: {tiles:.1f} K tiles per workgroup", flush=True)
        for name, vals in rows.items():
            if name == "raw Q wait":
                print(f"  {name:17s} {vals[0]:.0f} ns from a wavefront's last prologue request to the arrival of its raw Q rows", flush=True)
                continue
            if len(vals) == 1:
                print(f"  {name:17s} {vals[0]:.0f} ns per period for the wavefront that issues the tile requests", flush=True)
                continue
            if name == "between workgroups":
                print(f"  {name:17s} kernel {vals[0] / 1e3:.0f} us for {vals[1]:.1f} workgroups per compute unit: "
                      f"{vals[2]:.0f} ns per workgroup beyond its own stamps (dispatch, wavefront start-up, imbalance)", flush=True)
                continue
            if len(vals) == 4:
                print(f"  {name:17s} per period {sum(vals):6.0f} ns | first phase {vals[0]:.0f}, odd barrier {vals[1]:.0f}, "
                      f"second phase {vals[2]:.0f}, even barrier {vals[3]:.0f}", flush=True)
                continue
            parts = ", ".join(f"{lbl} {v:.0f}" for lbl, v in zip(INTERVALS, vals))
            print(f"  {name:17s} total {sum(vals):8.0f} ns | {parts} | main loop per tile {vals[4] / max(tiles, 1e-9):.0f}", flush=True)


if __name__ == "__main__":
    main()
