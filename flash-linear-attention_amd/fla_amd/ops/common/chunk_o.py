"""``chunk_fwd_o`` for scalar-gated models (``fla/ops/common/chunk_o.py:444-495``),
served by ``fla_chunk_fwd_o``."""
from typing import Optional

import torch

from ... import _backend as be

BT = 64


def chunk_fwd_o(
    q: torch.Tensor,
    k: torch.Tensor,
    v: torch.Tensor,
    h: torch.Tensor,
    g: Optional[torch.Tensor] = None,
    scale: Optional[float] = None,
    offsets: Optional[torch.Tensor] = None,
    indices: Optional[torch.Tensor] = None,
    head_first: bool = True,
    chunk_size: int = 64,
) -> torch.Tensor:
    """``o = scale * (exp(g) * (q h) + tril(q k^T * exp(g_i - g_j)) v)`` per chunk.
    ``h`` must be the MFMA-fragment-order states written by the scan kernels;
    ``g`` is the fp32 chunk-local cumsum ``[B,T,H]`` or ``None``."""
    if head_first or chunk_size != BT:
        raise NotImplementedError("fla_amd chunk_fwd_o: seq-first, chunk size 64 only")
    be.require_gpu(q, k, v, h)
    B, T, H, K = q.shape
    V = v.shape[-1]
    if scale is None:
        scale = K ** -0.5
    NT = 0
    if offsets is not None:
        NT = indices.shape[0]
        offsets = offsets.to(torch.int64).contiguous()
    if g is not None and g.dtype != torch.float32:
        g = g.float()
    o = torch.empty_like(v)
    be.check(be.lib().fla_chunk_fwd_o(
        be.ptr(q), be.ptr(k), be.ptr(v), be.ptr(g), be.ptr(h), be.ptr(o), be.ptr(offsets), be.ptr(indices), NT,
        be.dt(q), B, T, H, K, V, float(scale), be.stream_of(q)), "fla_chunk_fwd_o")
    return o
