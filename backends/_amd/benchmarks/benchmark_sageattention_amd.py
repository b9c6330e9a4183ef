"""Benchmark entry point of the ``backends/_amd`` bundle (compare
backends/_hygon/benchmarks/benchmark_sageattention_hygon.py and
backends/_enflame/benchmarks/sage_attention_native_benchmark.py).

    python backends/_amd/benchmarks/benchmark_sageattention_amd.py                       # the 20-shape table
    python backends/_amd/benchmarks/benchmark_sageattention_amd.py --path e2e --causal --pv fp8

All options are those of ``python -m baselinebenchmark_amd.benchmarks.sage_attention_benchmark``, which does the work.
"""
from baselinebenchmark_amd.benchmarks.sage_attention_benchmark import benchmark, build_parser

if __name__ == "__main__":
    benchmark(build_parser().parse_args())
