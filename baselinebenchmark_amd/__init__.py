"""MI355X (gfx950) SageAttention forward: per-block INT8 Q/K quantiser with K mean-smoothing, fused
INT8-QK / FP16-or-FP8-PV attention and a varlen/GQA tile scheduler, behind the reference's
``per_block_int8`` / ``forward`` / ``sageattn`` entry points.  Hand-written HIP kernels behind a C ABI
(include/sage_mi355x.h); no fallback implementation exists."""
from .sageattention import (backend_name, forward, forward_fused_q, k_mean, per_block_int8, per_block_int8_varlen, prepare_v, sageattn,
                            sageattn_varlen, varlen_plan)

__all__ = ["backend_name", "forward", "forward_fused_q", "k_mean", "per_block_int8", "per_block_int8_varlen", "prepare_v", "sageattn",
           "sageattn_varlen", "varlen_plan"]
