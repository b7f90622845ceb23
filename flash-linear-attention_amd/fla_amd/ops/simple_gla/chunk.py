"""``chunk_simple_gla`` with the reference's signature (``fla/ops/simple_gla/chunk.py:213-320``).

Head-wise (scalar) log-decay: ``h_t = e^{g_t} h_{t-1} + k_t v_t^T``, ``o_t = s q_t^T h_t``.  That is
GLA with the same gate on every key channel, so the operator is served by the GLA kernels
(forward and backward) on the gate broadcast over K; autograd reduces the gate gradient
over the key channels.  For 16-bit seq-first inputs with K, V in {64, 128} the forward skips the
``[B,T,H,K]`` gate tensor: ``fla_chunk_simple_gla_fwd_fused`` reads the per-head gates as they are
(``ChunkSimpleGLAFunction`` when gradients are needed: only its backward forms the gate tensor)."""
from typing import Optional, Tuple

import torch

import os

from ... import _backend as be
from ...utils import VarlenPlan, check_varlen_args, contiguous, resolve_offsets
from ..gla import chunk as gla_chunk
from ..gla.chunk import chunk_gla, chunk_gla_bwd_device, chunk_gla_fwd_fused


# A forward without gradients runs on the delta-rule scan kernel with the delta rule taken out
# (``fla_chunk_simple_gla_fwd_scan``): raw q and k tiles, gates on the score blocks and on rows, no range guard.
# ``FLA_AMD_SIMPLE_GLA_FUSED=1`` sends it through the GLA kernel's per-head-gate instantiation instead.
SCAN_FORWARD = os.environ.get("FLA_AMD_SIMPLE_GLA_FUSED", "0") != "1"


def chunk_simple_gla_fwd_scan(q, k, v, g, scale, initial_state, output_final_state, offsets=None):
    """``fla_chunk_simple_gla_fwd_scan``: seq-first 16-bit ``q, k, v``, raw per-head log-gates ``g`` ``[B,T,H]`` (any
    float dtype; ``None`` for no decay), K in {64, 128}, V a multiple of 64.  Returns ``(o, final_state)``."""
    be.require_gpu(q, k, v)
    B, T, H, K = k.shape
    V = v.shape[-1]
    N, co, order = B, None, None
    if offsets is not None:
        plan = VarlenPlan(offsets, 64)
        N, offsets, co, order = plan.N, plan.offsets, plan.chunk_offsets, plan.seq_order
    o = torch.empty_like(v)
    ht = k.new_empty(N, H, K, V, dtype=torch.float32) if output_final_state else None
    h0 = None
    if initial_state is not None:
        h0 = (initial_state if initial_state.dtype == torch.float32 else initial_state.float()).contiguous()
    gf = None if g is None else (g if g.dtype == torch.float32 else g.float()).contiguous()
    be.check(be.lib().fla_chunk_simple_gla_fwd_scan(
        be.ptr(q), be.ptr(k), be.ptr(v), be.ptr(gf), be.ptr(h0), be.ptr(o), be.ptr(ht), be.ptr(offsets), be.ptr(co),
        be.ptr(order), be.dt(k), B, T, H, K, V, N, float(scale), be.stream_of(k)), "fla_chunk_simple_gla_fwd_scan")
    return o, ht


class ChunkSimpleGLAFunction(torch.autograd.Function):
    """Seq-first, K and V in {64, 128}, 16-bit q/k/v: the forward reads the per-head gates as they are
    (``fla_chunk_simple_gla_fwd_fused``, which also keeps the per-chunk states for the backward pass unless
    recomputation is asked for, and the gated queries and chunk decays its reverse state scan streams); the backward
    pass runs on the GLA kernels' per-head-gate instantiations (``fla_chunk_simple_gla_bwd``) - only when it
    recomputes the states does it form the ``[B,T,H,K]`` gate tensor and reduce the gate gradient over the key
    channels afterwards
    (the reference: ``fla/ops/simple_gla/chunk.py:134-210``)."""

    @staticmethod
    @contiguous
    def forward(ctx, q, k, v, g, scale, initial_state, output_final_state, offsets):
        be.require_gpu(q, k, v, g)
        gf = g.float().contiguous()
        h0 = initial_state
        flags_states = [] if gla_chunk.KEEP_STATES_FOR_BACKWARD and any(ctx.needs_input_grad) else None
        o, ht, wide = chunk_gla_fwd_fused(q, k, v, gf, scale, h0, output_final_state, offsets=offsets,
                                          return_flags=True, states_out=flags_states, head_gates=True)
        ctx.save_for_backward(q, k, v, gf, h0, offsets, wide, *(flags_states or ()))
        ctx.scale, ctx.g_dtype = scale, g.dtype
        ctx.h0_dtype = None if initial_state is None else initial_state.dtype
        return o, ht

    @staticmethod
    @contiguous
    def backward(ctx, do, dht):
        q, k, v, gf, h0, offsets, wide, *kept = ctx.saved_tensors
        hT = kept[0] if kept else None
        qg, decay = (kept[1], kept[2]) if len(kept) > 2 else (None, None)
        kh, scores = (kept[3], kept[4]) if len(kept) > 4 else (None, None)
        h0f = None if h0 is None else h0.float().contiguous()
        dq, dk, dv, dg, dh0 = chunk_gla_bwd_device(q, k, v, gf, ctx.scale, h0f, do.to(q.dtype).contiguous(), dht,
                                                   offsets, wide, hT=hT, qg=qg, decay=decay, head_gates=True, kh=kh,
                                                   scores=scores)
        if dh0 is not None:
            dh0 = dh0.to(ctx.h0_dtype)
        return dq, dk, dv, dg.to(ctx.g_dtype), None, dh0, None, None


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
    if (g is not None and not head_first and K in (64, 128) and V in (64, 128)
            and q.dtype in (torch.bfloat16, torch.float16) and k.dtype == q.dtype and v.dtype == q.dtype):
        if needs_grad:
            return ChunkSimpleGLAFunction.apply(q, k, v, g, scale, initial_state, output_final_state, offsets)
        if SCAN_FORWARD:
            return chunk_simple_gla_fwd_scan(q.contiguous(), k.contiguous(), v.contiguous(), g, scale, initial_state,
                                             output_final_state, offsets=offsets)
        return chunk_gla_fwd_fused(q.contiguous(), k.contiguous(), v.contiguous(), g.float().contiguous(), scale,
                                   initial_state, output_final_state, offsets=offsets, head_gates=True)
    if g is None:
        gk = q.new_zeros(q.shape, dtype=torch.float32)
    else:
        gk = g.float().unsqueeze(-1).expand(*g.shape, K)
    return chunk_gla(q, k, v, gk, scale=scale, initial_state=initial_state, output_final_state=output_final_state,
                     offsets=offsets, head_first=head_first)
