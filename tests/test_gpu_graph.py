"""The one-call pipeline under HIP graph capture: every kernel goes to the caller's stream, nothing is
allocated, synchronised or cleared with a memset node by the library, so a captured `sageattn` must replay
bit-identically to the eager call -- on every replay, with fresh inputs copied into the captured tensors and
eager work of the program in between."""
import pytest
import torch

import baselinebenchmark_amd as sa
from tests.helpers import randn

pytestmark = [pytest.mark.gpu, pytest.mark.sage_attention]
DEV = "cuda"


def _inputs(seed, layout, B, Hq, Hkv, S, D, dtype):
    g = torch.Generator().manual_seed(seed)
    return (randn(layout, B, Hq, S, D, dtype, g), randn(layout, B, Hkv, S, D, dtype, g), randn(layout, B, Hkv, S, D, dtype, g))


@pytest.mark.parametrize("cfg", [
    dict(layout="HND", B=2, Hq=4, Hkv=2, S=700, D=128, dtype=torch.bfloat16, causal=True, pv="fp8", blk=(64, 128)),
    dict(layout="NHD", B=1, Hq=2, Hkv=2, S=333, D=64, dtype=torch.float16, causal=False, pv="fp16", blk=(128, 64)),
])
def test_captured_sageattn_replays_like_eager(cfg):
    kw = dict(tensor_layout=cfg["layout"], is_causal=cfg["causal"], pv_mode=cfg["pv"], BLKQ=cfg["blk"][0], BLKK=cfg["blk"][1])
    shape = (cfg["layout"], cfg["B"], cfg["Hq"], cfg["Hkv"], cfg["S"], cfg["D"], cfg["dtype"])
    q, k, v = (t.to(DEV) for t in _inputs(1, *shape))
    # warm-up on a side stream (the usual capture recipe), then capture one call
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        sa.sageattn(q, k, v, **kw)
    torch.cuda.current_stream().wait_stream(side)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        out = sa.sageattn(q, k, v, **kw)
    for seed in (2, 3, 4):
        nq, nk, nv = (t.to(DEV) for t in _inputs(seed, *shape))
        eager = sa.sageattn(nq, nk, nv, **kw)     # the program's own eager work between replays
        torch.cuda.synchronize()
        q.copy_(nq); k.copy_(nk); v.copy_(nv)
        graph.replay()
        torch.cuda.synchronize()
        assert torch.isfinite(out.float()).all()
        assert torch.equal(out, eager), f"replay with seed {seed} differs from the eager call"
