"""``chunk_local_cumsum`` with the reference's signature
(``fla/ops/utils/cumsum.py:389-407``), served by ``fla_chunk_local_cumsum``."""
from typing import Optional

import torch

from ... import _backend as be
from ...utils import VarlenPlan


def chunk_local_cumsum(
    g: torch.Tensor,
    chunk_size: int,
    reverse: bool = False,
    offsets: Optional[torch.Tensor] = None,
    indices: Optional[torch.Tensor] = None,
    head_first: bool = True,
) -> torch.Tensor:
    if offsets is not None:
        assert g.shape[0] == 1, "Only batch size 1 is supported when offsets are provided"
    if g.dim() not in (3, 4):
        raise ValueError(f"Unsupported input shape {g.shape}. "
                         f"which should be (B, H, T, dim) if `head_first=True` "
                         f"or (batch_size, num_heads, seq_len) otherwise")
    assert chunk_size == 2 ** (chunk_size.bit_length() - 1), "chunk_size must be a power of 2"
    be.require_gpu(g)
    if head_first:
        # the kernels are seq-first; head-first is served by a transpose
        out = chunk_local_cumsum(g.transpose(1, 2), chunk_size, reverse, offsets, indices, head_first=False)
        return out.transpose(1, 2).contiguous()
    g = g.contiguous()
    B, T, H = g.shape[:3]
    S = g.shape[3] if g.dim() == 4 else 1
    out = torch.empty_like(g, dtype=torch.float32)
    NT = 0
    if offsets is not None:
        if indices is None:
            plan = VarlenPlan(offsets, chunk_size)
            offsets, indices = plan.offsets, plan.indices
        offsets = offsets.to(torch.int64).contiguous()
        indices = indices.to(torch.int64).contiguous()
        NT = indices.shape[0]
    be.check(be.lib().fla_chunk_local_cumsum(
        be.ptr(g), be.ptr(out), be.dt(g), B, T, H, S, chunk_size, int(bool(reverse)),
        be.ptr(offsets), be.ptr(indices), NT, be.stream_of(g)), "fla_chunk_local_cumsum")
    return out
