"""Host-side description of the V panel byte order (mirrors panel_index_fp8 / panel_index_fp16 in
csrc/sage_common.h).  Used to inspect panels; the kernels never need it."""
from __future__ import annotations

import numpy as np
import torch

PANEL_ROWS = 128


def _index_fp8(D: int) -> np.ndarray:
    n = np.arange(PANEL_ROWS)[:, None]
    d = np.arange(D)[None, :]
    ks, nn = n >> 6, n & 63
    half, r = nn >> 5, nn & 31
    a, h, b = r >> 3, (r >> 2) & 1, r & 3
    lane, dt = 32 * h + (d & 31), d >> 5
    return (((ks * (D // 32) + dt) * 2 + half) * 64 + lane) * 16 + 4 * a + b


def _index_fp16(D: int) -> np.ndarray:
    n = np.arange(PANEL_ROWS)[:, None]
    d = np.arange(D)[None, :]
    ks, r = n >> 4, n & 15
    a, h, b = r >> 3, (r >> 2) & 1, r & 3
    lane, dt = 32 * h + (d & 31), d >> 5
    return ((ks * (D // 32) + dt) * 64 + lane) * 8 + 4 * a + b


def unpack_panels(panels: torch.Tensor, B: int, H: int, L: int, D: int, pv_mode: str) -> torch.Tensor:
    """CPU uint8 panel buffer -> [B, H, ceil(L/128)*128, D] tensor (uint8 fp8 bit patterns, or float16)."""
    npan = (L + PANEL_ROWS - 1) // PANEL_ROWS
    if pv_mode == "fp8":
        idx = torch.from_numpy(_index_fp8(D).reshape(-1).astype(np.int64))
        flat = panels[: B * H * npan * PANEL_ROWS * D].reshape(B * H * npan, PANEL_ROWS * D)
        return flat[:, idx].reshape(B, H, npan * PANEL_ROWS, D)
    idx = torch.from_numpy(_index_fp16(D).reshape(-1).astype(np.int64))
    flat = panels[: B * H * npan * PANEL_ROWS * D * 2].view(torch.float16).reshape(B * H * npan, PANEL_ROWS * D)
    return flat[:, idx].reshape(B, H, npan * PANEL_ROWS, D)
