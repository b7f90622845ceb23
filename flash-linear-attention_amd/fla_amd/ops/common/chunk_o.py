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
    *,
    fragment_layout: bool = False,
) -> torch.Tensor:
    """``o = scale * (exp(g) * (q h) + tril(q k^T * exp(g_i - g_j)) v)`` per chunk
    (``fla/ops/common/chunk_o.py:444-496``).  ``h`` ``[B,NT,H,K,V]`` is row-major as in the reference
    (fp32 or 16-bit; re-ordered for the kernel by one extra pass over the states), or, with
    ``fragment_layout=True``, the MFMA-fragment-order states the scan kernels of this library write;
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
    if not fragment_layout:
        h = states_to_fragments(h, q.dtype)
    o = torch.empty_like(v)
    be.check(be.lib().fla_chunk_fwd_o(
        be.ptr(q), be.ptr(k), be.ptr(v), be.ptr(g), be.ptr(h), be.ptr(o), be.ptr(offsets), be.ptr(indices), NT,
        be.dt(q), B, T, H, K, V, float(scale), be.stream_of(q)), "fla_chunk_fwd_o")
    return o


def states_to_fragments(h: torch.Tensor, dtype: torch.dtype, transposed: bool = False) -> torch.Tensor:
    """Row-major states ``[..., K, V]`` (fp32 or ``dtype``) in the MFMA-fragment order the output-stage and
    backward kernels read (``transposed``: every 32x32 tile transposed, the backward kernels' order)."""
    K, V = h.shape[-2:]
    if K % 32 or V % 32:
        raise NotImplementedError("fla_amd states_to_fragments: K and V must be multiples of 32")
    h = h.contiguous()
    out = torch.empty(h.shape, dtype=dtype, device=h.device)
    be.check(be.lib().fla_states_to_fragments(
        be.ptr(h), be.ptr(out), be.dt(h), be._DTYPES[dtype], int(transposed), h.numel() // (K * V), K, V,
        be.stream_of(h)), "fla_states_to_fragments")
    return out
