"""``fused_recurrent_gla`` with the reference's signature
(``fla/ops/gla/fused_recurrent.py:11-116``)."""
from typing import Optional, Tuple

import torch

from ...utils import check_varlen_args, resolve_offsets
from ..common.fused_recurrent import fused_recurrent


def fused_recurrent_gla(
    q: torch.Tensor,
    k: torch.Tensor,
    v: torch.Tensor,
    gk: Optional[torch.Tensor] = None,
    gv: Optional[torch.Tensor] = None,
    scale: Optional[int] = None,
    initial_state: Optional[torch.Tensor] = None,
    output_final_state: bool = False,
    reverse: bool = False,
    offsets: Optional[torch.LongTensor] = None,
    head_first: bool = True,
    cu_seqlens: Optional[torch.LongTensor] = None,
    inplace_state: bool = False,
) -> Tuple[torch.Tensor, Optional[torch.Tensor]]:
    r"""
    Args mirror the reference: q, k ``[B,H,T,K]`` (``[B,T,H,K]`` if not
    ``head_first``), v ``[.., V]``, log-gates ``gk`` / ``gv``, ``scale``
    (default ``K ** -0.5``), ``initial_state`` ``[N,H,K,V]``,
    ``output_final_state``, ``reverse``, ``offsets`` (int64 ``[N+1]``, batch 1).

    Extensions: ``cu_seqlens`` is a synonym of ``offsets``; ``inplace_state=True``
    writes the final state over ``initial_state`` (fp32, contiguous) instead of
    allocating a new tensor - the decode loop's read-modify-write.

    Returns ``(o, final_state)`` with ``final_state`` fp32 ``[N,H,K,V]`` or ``None``.
    """
    offsets = resolve_offsets(offsets, cu_seqlens)
    check_varlen_args(q, offsets, head_first, initial_state)
    if scale is None:
        scale = k.shape[-1] ** -0.5
    return fused_recurrent(q=q, k=k, v=v, g=None, gk=gk, gv=gv, scale=scale, initial_state=initial_state,
                           output_final_state=output_final_state, reverse=reverse, offsets=offsets,
                           head_first=head_first, inplace_state=inplace_state)
