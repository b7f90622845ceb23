"""``chunk_local_cumsum`` and ``chunk_global_cumsum`` with the reference's signatures
(``fla/ops/utils/cumsum.py:389-407`` and ``:366-386``), served by ``fla_chunk_local_cumsum`` and
``fla_chunk_global_cumsum``."""
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


def chunk_local_cumsum_inverse(
    g_cumsum: torch.Tensor,
    chunk_size: int,
    reverse: bool = False,
    offsets: Optional[torch.Tensor] = None,
    indices: Optional[torch.Tensor] = None,
    head_first: bool = True,
) -> torch.Tensor:
    """The raw values whose ``chunk_local_cumsum`` is ``g_cumsum`` (fp32): differences of consecutive rows
    inside every chunk (``fla_chunk_local_cumsum_inverse``).  No counterpart in the reference, whose internal
    entry points take the cumulative gates as they are; the kernels here start from the raw gates."""
    be.require_gpu(g_cumsum)
    if head_first:
        out = chunk_local_cumsum_inverse(g_cumsum.transpose(1, 2), chunk_size, reverse, offsets, indices, head_first=False)
        return out.transpose(1, 2).contiguous()
    g = g_cumsum.float().contiguous()
    B, T, H = g.shape[:3]
    S = g.shape[3] if g.dim() == 4 else 1
    out = torch.empty_like(g)
    NT = 0
    if offsets is not None:
        if indices is None:
            plan = VarlenPlan(offsets, chunk_size)
            offsets, indices = plan.offsets, plan.indices
        offsets = offsets.to(torch.int64).contiguous()
        indices = indices.to(torch.int64).contiguous()
        NT = indices.shape[0]
    be.check(be.lib().fla_chunk_local_cumsum_inverse(
        be.ptr(g), be.ptr(out), B, T, H, S, chunk_size, int(bool(reverse)), be.ptr(offsets), be.ptr(indices), NT,
        be.stream_of(g)), "fla_chunk_local_cumsum_inverse")
    return out


def chunk_global_cumsum(
    s: torch.Tensor,
    dtype: Optional[torch.dtype] = None,
    reverse: bool = False,
    offsets: Optional[torch.Tensor] = None,
    head_first: bool = True,
) -> torch.Tensor:
    """Cumulative sum along time over each whole sequence; ``s`` is ``[B,H,T]`` / ``[B,H,T,D]``
    (``[B,T,H]`` / ``[B,T,H,D]`` if not ``head_first``), the result has dtype ``dtype or s.dtype``."""
    if offsets is not None:
        assert s.shape[0] == 1, "Only batch size 1 is supported when offsets are provided"
    if s.dim() not in (3, 4):
        raise ValueError(f"Unsupported input shape {s.shape}. "
                         f"which should be [B, H, T]/[B, H, T, D] if `head_first=True` "
                         f"or [B, T, H]/[B, T, H, D] otherwise")
    be.require_gpu(s)
    if head_first:
        out = chunk_global_cumsum(s.transpose(1, 2), dtype, reverse, offsets, head_first=False)
        return out.transpose(1, 2).contiguous()
    s = s.contiguous()
    B, T, H = s.shape[:3]
    S = s.shape[3] if s.dim() == 4 else 1
    out = torch.empty_like(s, dtype=dtype or s.dtype)
    if s.numel() == 0:
        return out
    # parallel grain: at most about 64 chunks per sequence, so the carry pass stays short
    longest = T
    chunk_size = 64
    while chunk_size * 64 < longest:
        chunk_size *= 2
    indices, NT = None, 0
    if offsets is not None:
        plan = VarlenPlan(offsets, chunk_size)
        offsets, indices = plan.offsets.to(torch.int64).contiguous(), plan.indices.to(torch.int64).contiguous()
        NT = indices.shape[0]
    ws = torch.empty_like(s, dtype=torch.float32)
    be.check(be.lib().fla_chunk_global_cumsum(
        be.ptr(s), be.ptr(ws), be.ptr(out), be.dt(s), be.dt(out), B, T, H, S, chunk_size, int(bool(reverse)),
        be.ptr(offsets), be.ptr(indices), NT, be.stream_of(s)), "fla_chunk_global_cumsum")
    return out
