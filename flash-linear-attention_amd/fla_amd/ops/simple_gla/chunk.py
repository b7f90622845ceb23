"""``chunk_simple_gla`` with the reference's signature (``fla/ops/simple_gla/chunk.py:213-320``).

Head-wise (scalar) log-decay: ``h_t = e^{g_t} h_{t-1} + k_t v_t^T``, ``o_t = s q_t^T h_t``.  That is
GLA with the same gate on every key channel, so the operator is served by the GLA kernels
(forward and backward) on the gate broadcast over K; autograd reduces the gate gradient
over the key channels.  A forward that will not be differentiated skips the ``[B,T,H,K]`` gate
tensor: ``fla_chunk_simple_gla_fwd_fused`` reads the per-head gates as they are."""
from typing import Optional, Tuple

import torch

from ...utils import check_varlen_args, resolve_offsets
from ..gla.chunk import chunk_gla, chunk_gla_fwd_fused


def chunk_simple_gla(
    q: torch.Tensor,
    k: torch.Tensor,
    v: torch.Tensor,
    g: torch.Tensor,
    scale: Optional[float] = None,
    initial_state: Optional[torch.Tensor] = None,
    output_final_state: bool = False,
    offsets: Optional[torch.LongTensor] = None,
    head_first: bool = True,
    cu_seqlens: Optional[torch.LongTensor] = None,
) -> Tuple[torch.Tensor, torch.Tensor]:
    r"""
    Args:
        q, k: ``[B, H, T, K]`` if ``head_first`` else ``[B, T, H, K]``.
        v: ``[B, H, T, V]`` / ``[B, T, H, V]``.
        g: head-wise log decay ``[B, H, T]`` / ``[B, T, H]`` (or ``None`` for no decay).
        scale: default ``K ** -0.5``.
        initial_state: ``[N, H, K, V]`` or ``None``; output_final_state: return the fp32 final state.
        offsets (synonym ``cu_seqlens``): int64 ``[N+1]`` boundaries of a packed batch (batch 1, seq-first).

    Returns ``(o, final_state)``.
    """
    offsets = resolve_offsets(offsets, cu_seqlens)
    check_varlen_args(q, offsets, head_first, initial_state)
    if scale is None:
        scale = k.shape[-1] ** -0.5
    K = k.shape[-1]
    V = v.shape[-1]
    needs_grad = torch.is_grad_enabled() and any(
        t is not None and t.requires_grad for t in (q, k, v, g, initial_state))
    if (g is not None and not needs_grad and not head_first and K in (64, 128) and V in (64, 128)
            and q.dtype in (torch.bfloat16, torch.float16) and k.dtype == q.dtype and v.dtype == q.dtype):
        return chunk_gla_fwd_fused(q.contiguous(), k.contiguous(), v.contiguous(), g.float().contiguous(), scale,
                                   initial_state, output_final_state, offsets=offsets, head_gates=True)
    if g is None:
        gk = q.new_zeros(q.shape, dtype=torch.float32)
    else:
        gk = g.float().unsqueeze(-1).expand(*g.shape, K)
    return chunk_gla(q, k, v, gk, scale=scale, initial_state=initial_state, output_final_state=output_final_state,
                     offsets=offsets, head_first=head_first)
