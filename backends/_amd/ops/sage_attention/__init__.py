"""SageAttention for AMD Instinct MI355X (gfx950): the operator files of the ``backends/_amd`` bundle.

The bundle follows the layout the other vendors use (backends/README.md:5-9; compare
backends/_hygon/ops/sageattention/): ``ops/`` holds the operator's public interface, ``benchmarks/`` its benchmark
entry point, ``test/`` a correctness script, ``doc/`` a usage note.  Everything here is a thin file: the kernels and
the C ABI live in the ``baselinebenchmark_amd`` package, which must be importable (on ``PYTHONPATH`` or installed)
and built (``python -m baselinebenchmark_amd.build``).
"""
from .sageattention_hip import *          # noqa: F401,F403
from .sageattention_hip import __all__    # noqa: F401
