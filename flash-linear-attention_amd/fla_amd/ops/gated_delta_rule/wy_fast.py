"""WY representation of the gated delta rule
(``fla/ops/gated_delta_rule/wy_fast.py:320-426``), served by ``fla_gdr_fwd_wy``."""
from typing import Optional, Tuple

import torch

from ... import _backend as be

BT = 64


def fwd_prepare_wy_repr(
    k: torch.Tensor,
    v: torch.Tensor,
    beta: torch.Tensor,
    g: Optional[torch.Tensor],
    offsets: Optional[torch.Tensor] = None,
    indices: Optional[torch.Tensor] = None,
    head_first: bool = True,
    chunk_size: int = 64,
    *,
    store_A: bool = True,
    store_Au: bool = True,
    q: Optional[torch.Tensor] = None,
    scale: float = 1.0,
):
    """Returns ``(w, u, Aw, Au)`` with ``Aw = (I + strict_lower(diag(beta) K K^T))^-1``,
    ``Au = Aw * exp(g_i - g_j)``, ``w = Aw (beta K)``, ``u = Au (beta V)``; ``g`` is the
    fp32 chunk-local cumsum of the log-gate (or ``None``).

    With ``q`` the same launch also produces the gated causal scores of the output stage,
    ``Aqk[i, j] = scale (q_i . k_j) exp(g_i - g_j)`` for ``j <= i`` (else 0), ``[B, T, H, 64]``,
    and the return value is ``(w, u, Aw, Au, Aqk)``."""
    if head_first or chunk_size != BT:
        raise NotImplementedError("fla_amd fwd_prepare_wy_repr: seq-first, chunk size 64 only")
    be.require_gpu(k, v, beta)
    B, T, H, K = k.shape
    V = v.shape[-1]
    NT = 0
    if offsets is not None:
        NT = indices.shape[0]
        offsets = offsets.to(torch.int64).contiguous()
    beta = beta.float().contiguous()
    if g is not None:
        g = g.float().contiguous()
    w, u = torch.empty_like(k), torch.empty_like(v)
    Aw = k.new_empty(B, T, H, BT) if store_A else None
    Au = k.new_empty(B, T, H, BT) if (store_A and store_Au) else None
    Aqk = k.new_empty(B, T, H, BT) if q is not None else None
    be.check(be.lib().fla_gdr_fwd_wy(
        be.ptr(k), be.ptr(v), be.ptr(beta), be.ptr(g), be.ptr(w), be.ptr(u), be.ptr(Aw), be.ptr(Au),
        be.ptr(q), be.ptr(Aqk), float(scale),
        be.ptr(offsets), be.ptr(indices), NT, be.dt(k), B, T, H, K, V, be.stream_of(k)), "fla_gdr_fwd_wy")
    if q is not None:
        return w, u, Aw, Au, Aqk
    return w, u, Aw, Au
