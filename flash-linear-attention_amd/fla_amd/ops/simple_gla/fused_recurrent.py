"""``fused_recurrent_simple_gla`` (``fla/ops/simple_gla/fused_recurrent.py:11-120``): the common
token-by-token recurrence with a head-wise gate, served by ``fla_fused_recurrent_fwd``."""
from typing import Optional, Tuple

import torch

from ...utils import check_varlen_args, resolve_offsets
from ..common.fused_recurrent import fused_recurrent


def fused_recurrent_simple_gla(
    q: torch.Tensor,
    k: torch.Tensor,
    v: torch.Tensor,
    g: torch.Tensor,
    scale: Optional[float] = None,
    initial_state: Optional[torch.Tensor] = None,
    output_final_state: bool = False,
    reverse: bool = False,
    offsets: Optional[torch.LongTensor] = None,
    head_first: bool = True,
    cu_seqlens: Optional[torch.LongTensor] = None,
    inplace_state: bool = False,
) -> Tuple[torch.Tensor, torch.Tensor]:
    """Same arguments as the reference; ``g`` is the head-wise log decay ``[B, H, T]`` /
    ``[B, T, H]``.  Returns ``(o, final_state)``."""
    offsets = resolve_offsets(offsets, cu_seqlens)
    check_varlen_args(q, offsets, head_first, initial_state)
    if scale is None:
        scale = k.shape[-1] ** -0.5
    return fused_recurrent(q=q, k=k, v=v, g=g, scale=scale, initial_state=initial_state,
                           output_final_state=output_final_state, reverse=reverse, offsets=offsets,
                           head_first=head_first, inplace_state=inplace_state)
