"""``chunk_delta_rule`` with the reference's signature (``fla/ops/delta_rule/chunk.py:243-345``).

The un-gated delta rule is the gated one without the decay: the reference's
``chunk_delta_rule_fwd`` / ``_bwd`` (``fla/ops/delta_rule/chunk.py:18-163``) launch the same
WY, state-scan and output kernels with ``g=None``, and so does this wrapper (forward and
backward of ``chunk_gated_delta_rule`` with a NULL gate pointer)."""
from typing import Optional, Tuple

import torch

from ...utils import check_varlen_args, resolve_offsets
from ..gated_delta_rule.chunk import apply_in_value_slabs


def chunk_delta_rule(
    q: torch.Tensor,
    k: torch.Tensor,
    v: torch.Tensor,
    beta: torch.Tensor,
    scale: float = None,
    initial_state: torch.Tensor = None,
    output_final_state: bool = False,
    offsets: Optional[torch.LongTensor] = None,
    head_first: bool = True,
    cu_seqlens: Optional[torch.LongTensor] = None,
) -> Tuple[torch.Tensor, torch.Tensor]:
    r"""
    Args:
        q, k: ``[B, H, T, K]`` if ``head_first`` else ``[B, T, H, K]`` (bf16 / fp16; keys are expected L2-normalised).
        v: ``[B, H, T, V]`` / ``[B, T, H, V]``.
        beta: ``[B, H, T]`` / ``[B, T, H]``.
        scale: default ``K ** -0.5``.
        initial_state: ``[N, H, K, V]`` or ``None``; output_final_state: return the fp32 final state.
        offsets (synonym ``cu_seqlens``): int64 ``[N+1]`` boundaries of a packed batch (batch 1, seq-first).

    Returns ``(o, final_state)``.
    """
    assert q.dtype == k.dtype == v.dtype
    assert q.dtype != torch.float32, "ChunkDeltaRuleFunction does not support float32. Please use bfloat16."
    assert len(beta.shape) == 3, "beta must be of shape (batch size, num of head, seq len)."
    offsets = resolve_offsets(offsets, cu_seqlens)
    check_varlen_args(q, offsets, head_first, initial_state)
    scale = k.shape[-1] ** -0.5 if scale is None else scale
    return apply_in_value_slabs(q, k, v, None, beta, scale, initial_state, output_final_state, offsets, head_first)
