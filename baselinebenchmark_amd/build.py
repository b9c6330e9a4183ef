"""Builds libsage_mi355x.so (the gfx950 HIP kernels and their C ABI) in-tree with hipcc.

Run as ``python -m baselinebenchmark_amd.build``.  The library lands next to the sources in
``baselinebenchmark_amd/csrc/`` where ``_cabi.py`` loads it from; nothing is built lazily at
import time, so a missing library is a loud error.
"""
from __future__ import annotations

import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor
from pathlib import Path

CSRC = Path(__file__).resolve().parent / "csrc"
LIB = CSRC / "libsage_mi355x.so"
SOURCES = ["sage_quant.hip", "sage_attn.hip", "sage_attn_mask.hip", "sage_attn_qfuse.hip", "sage_attn_kinterleave.hip", "sage_api.hip",
           "sage_static.hip"]
FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC",
    # correctly rounded fp32 divide (the INT8 quantiser's contract) and no packed-fp32 selection
    "-fhip-fp32-correctly-rounded-divide-sqrt",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
]


# The instantiation units of the shipped attention kernels are scheduled for instruction-level parallelism rather than
# for occupancy (which is fixed at two wavefronts per SIMD anyway): +0.9 % on config 2 and on FP16 P.V at 16k keys, equal
# elsewhere, no scratch.  The explicit-mask variants (sage_attn_mask.hip), which spill under either strategy, keep the default.
# -fno-honor-nans: these kernels produce -inf (masked scores) but never a NaN, and without the flag every fmaxf on a
# loaded or exchanged value is preceded by an instruction that only quiets signalling NaNs (four per tile: 0.6 % on
# config 2, bit-identical outputs).
EXTRA_FLAGS = {src: ["-mllvm", "-amdgpu-sched-strategy=max-ilp", "-fno-honor-nans"]
               for src in ("sage_attn.hip", "sage_attn_qfuse.hip", "sage_attn_kinterleave.hip")}


def _hipcc() -> str:
    return os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")


TIMING_LIB = CSRC / "libsage_mi355x_timing.so"   # same library with in-kernel interval timers (a measurement aid)


def _compile(src: str, timing: bool = False) -> Path:
    obj = CSRC / (src.replace(".hip", ".timing.o" if timing else ".o"))
    cmd = [_hipcc(), *FLAGS, *EXTRA_FLAGS.get(src, []), *(["-DSAGE_TIMING=1"] if timing else []), "-c", str(CSRC / src), "-o", str(obj)]
    res = subprocess.run(cmd, capture_output=True, text=True)
    noise = "is not a recognized feature for this target"
    err = "\n".join(l for l in res.stderr.splitlines() if noise not in l)
    if res.returncode != 0:
        raise RuntimeError(f"hipcc failed for {src}:\n{err}")
    if err.strip():
        print(err, file=sys.stderr)
    return obj


def _link(objs, lib: Path, verbose: bool) -> Path:
    cmd = [_hipcc(), "--offload-arch=gfx950", "-shared", "-fPIC", *map(str, objs), "-o", str(lib)]
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError(f"link failed:\n{res.stderr}")
    if verbose:
        print(f"built {lib} ({lib.stat().st_size} bytes)")
    return lib


def build(verbose: bool = True, timing: bool = False) -> Path:
    """Builds the library; ``timing=True`` builds the instrumented twin (``-DSAGE_TIMING=1``) next to it instead,
    for ``python -m baselinebenchmark_amd.benchmarks.tile_timing``."""
    with ThreadPoolExecutor(max_workers=len(SOURCES)) as ex:
        objs = list(ex.map(lambda src: _compile(src, timing), SOURCES))
    return _link(objs, TIMING_LIB if timing else LIB, verbose)


BENCH = Path(__file__).resolve().parent / "benchmarks"
HWRATES_LIB = BENCH / "libsage_hwrates.so"      # hardware-rate micro-benchmarks (benchmarks/hw_rates.py)
CABI_BENCH = BENCH / "sage_bench"               # C++ benchmark driver that calls the C ABI directly


def build_tools(verbose: bool = True) -> list[Path]:
    """Builds what the benchmark tools need and the drop-in library does not contain: the instrumented twin of the
    library (tile_timing), the hardware-rate micro-benchmarks (hw_rates) and the C++ benchmark driver."""
    out = [build(verbose, timing=True)]
    objs = []
    # (the attention kernels' scheduling flags: the micro-benchmarks reproduce their instruction streams; the replica of
    # the 64-rows-per-wavefront design keeps its scores in vector registers, see hw_rates_rows64.hip)
    for name, extra in (("hw_rates", []), ("hw_rates_rows64", ["-mllvm", "-amdgpu-mfma-vgpr-form"])):
        obj = BENCH / f"{name}.o"
        res = subprocess.run([_hipcc(), *FLAGS, *EXTRA_FLAGS["sage_attn.hip"], *extra, "-c", str(BENCH / f"{name}.hip"), "-o", str(obj)],
                             capture_output=True, text=True)
        if res.returncode != 0:
            raise RuntimeError(f"hipcc failed for {name}.hip:\n{res.stderr}")
        objs.append(obj)
    out.append(_link(objs, HWRATES_LIB, verbose))
    src = BENCH / "sage_bench.cpp"
    if src.exists():
        cmd = [_hipcc(), "-O2", "-std=c++17", "-x", "hip", "--offload-arch=gfx950", str(src), "-I", str(CSRC.parent.parent / "include"),
               "-L", str(CSRC), "-lsage_mi355x", f"-Wl,-rpath,{CSRC}", "-o", str(CABI_BENCH)]
        res = subprocess.run(cmd, capture_output=True, text=True)
        if res.returncode != 0:
            raise RuntimeError(f"hipcc failed for sage_bench.cpp:\n{res.stderr}")
        if verbose:
            print(f"built {CABI_BENCH}")
        out.append(CABI_BENCH)
    return out


if __name__ == "__main__":
    if "--tools" in sys.argv[1:]:
        build_tools()
    else:
        build(timing="--timing" in sys.argv[1:])
