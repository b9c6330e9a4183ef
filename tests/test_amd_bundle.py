"""The ``backends/_amd`` bundle (ops / benchmarks / test / doc, the layout of backends/README.md:5-9 and of
backends/_hygon/): its interface file re-exports the package's entry points unchanged, its benchmark file reaches the
benchmark's parser, and its correctness script passes on the GPU."""
import importlib.util
import sys
from pathlib import Path

import pytest

import baselinebenchmark_amd as pkg

BUNDLE = Path(__file__).resolve().parents[1] / "backends" / "_amd"


def _load(path, name):
    spec = importlib.util.spec_from_file_location(name, path, submodule_search_locations=[str(path.parent)] if path.name == "__init__.py" else None)
    mod = importlib.util.module_from_spec(spec)
    sys.modules[name] = mod
    spec.loader.exec_module(mod)
    return mod


def test_layout_is_the_vendor_bundle_layout():
    for sub in ("ops/sage_attention/__init__.py", "ops/sage_attention/sageattention_hip.py",
                "benchmarks/benchmark_sageattention_amd.py", "test/sage_attention/test_sageattention_hip.py",
                "doc/SAGEATTENTION_AMD.md"):
        assert (BUNDLE / sub).is_file(), sub


def test_interface_file_re_exports_the_package():
    ops = _load(BUNDLE / "ops" / "sage_attention" / "__init__.py", "amd_bundle_sage_attention")
    for name in ("per_block_int8", "forward", "sageattn", "sageattn_varlen", "backend_name"):   # sageattention_hip.py:37-80
        assert getattr(ops, name) is getattr(pkg, name)
    assert sorted(ops.__all__) == sorted(pkg.__all__)
    assert ops.backend_name().startswith("mi355x_hip")


def test_benchmark_file_reaches_the_parser():
    src = (BUNDLE / "benchmarks" / "benchmark_sageattention_amd.py").read_text()
    compile(src, "benchmark_sageattention_amd.py", "exec")
    from baselinebenchmark_amd.benchmarks.sage_attention_benchmark import build_parser
    args = build_parser().parse_args(["--path", "e2e", "--causal", "--pv", "fp8"])
    assert args.path == "e2e" and args.causal and args.pv == "fp8"


@pytest.mark.gpu
def test_correctness_script_passes():
    script = _load(BUNDLE / "test" / "sage_attention" / "test_sageattention_hip.py", "amd_bundle_correctness_script")
    script.test_forward_cases()
    script.test_one_call_cases()
