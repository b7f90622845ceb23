"""Chunk-local prefix sums of log-gates.

Restates ``chunk_local_cumsum`` (``fla/ops/utils/cumsum.py:389-407``; scalar
kernel ``:24-57``, vector kernel ``:72-110``): an inclusive prefix sum along
time that restarts at every chunk boundary, chunk boundaries counted from the
start of each sequence; ``reverse=True`` gives inclusive suffix sums; output is
always fp32.  Seq-first layout ``[B, T, H]`` or ``[B, T, H, S]``.

Test infrastructure only.
"""
from typing import Optional, Sequence

import torch


def chunk_local_cumsum(g: torch.Tensor, chunk_size: int, reverse: bool = False,
                       offsets: Optional[Sequence[int]] = None) -> torch.Tensor:
    g32 = g.detach().to(torch.float32).cpu()
    out = torch.empty_like(g32)
    B, T = g32.shape[:2]
    if offsets is None:
        spans = [(b, 0, T) for b in range(B)]
    else:
        assert B == 1
        offs = [int(x) for x in offsets]
        spans = [(0, offs[i], offs[i + 1]) for i in range(len(offs) - 1)]
    for b, bos, eos in spans:
        for s in range(bos, eos, chunk_size):
            e = min(s + chunk_size, eos)
            blk = g32[b, s:e]
            if reverse:
                out[b, s:e] = torch.flip(torch.cumsum(torch.flip(blk, [0]), 0), [0])
            else:
                out[b, s:e] = torch.cumsum(blk, 0)
    return out
