"""Public SageAttention interface for AMD Instinct MI355X.

The names, arguments and error behaviour are those of the other vendors' interface files
(backends/_hygon/ops/sageattention/sageattention_hip.py:37-80 for ``per_block_int8`` / ``forward`` /
``backend_name``; backends/_metax/ops/sage_attention/official_wheel.py:18-24 for ``sageattn``, whose packed counterpart
here is ``sageattn_varlen``).  The work is
done by the HIP library behind the ``baselinebenchmark_amd`` package; this file adds nothing to it.  There is no
fallback: importing this file without the built library raises.
"""
from __future__ import annotations

from baselinebenchmark_amd import _cabi
from baselinebenchmark_amd import (backend_name, forward, forward_fused_q, k_mean, per_block_int8, per_block_int8_varlen, prepare_v,
                                   sageattn, sageattn_varlen, varlen_plan)

_cabi.lib()   # fail at import, not at the first call, when libsage_mi355x.so has not been built

__all__ = ["backend_name", "forward", "forward_fused_q", "k_mean", "per_block_int8", "per_block_int8_varlen", "prepare_v", "sageattn",
           "sageattn_varlen", "varlen_plan"]
