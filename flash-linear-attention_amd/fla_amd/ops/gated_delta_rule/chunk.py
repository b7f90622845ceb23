"""``chunk_gated_delta_rule`` with the reference's signature
(``fla/ops/gated_delta_rule/chunk.py:258-363``).

Forward on the device (chunk size 64), two launches: ``fla_gdr_fwd_prep`` (chunk-parallel, reads k: prefix sum of
the gate, KK^T, block inverse; leaves one packed triangular 64x64 tile per chunk and head) ->
``fla_chunk_gated_delta_rule_fwd_scan`` (gated causal q k^T scores, state scan and output in one pass over q, k,
v; w, u, v_new and the per-chunk states are never formed).
A forward pass that will be differentiated runs the same two launches with more outputs and keeps w, Aw, v_new
and the per-chunk states for the backward; with ``KEEP_STATES_FOR_BACKWARD = False`` the backward recomputes
them with ``fla_chunk_gated_delta_rule_fwd_h`` like the reference.
"""
import os
import warnings
from typing import Optional, Tuple

import torch
import torch.nn.functional as F

from ... import _backend as be
from ...utils import (VarlenPlan, autocast_custom_bwd, autocast_custom_fwd, check_varlen_args, contiguous,
                      empty_batch_result, resolve_offsets)
from ..common.chunk_delta_h import (chunk_gated_delta_rule_fwd_h, chunk_gated_delta_rule_fwd_h_both,
                                    chunk_gated_delta_rule_fwd_onepass, chunk_gated_delta_rule_fwd_scan)
from ..common.chunk_o import chunk_fwd_o
from ..utils.cumsum import chunk_local_cumsum
from .wy_fast import fwd_prepare_scan_operands, fwd_prepare_wy_repr

BT = 64
_SUPPORTED_KV = {(64, 64), (128, 128), (64, 128), (128, 64), (256, 64), (256, 128)}
_FUSED_MAX_K = 128  # the one-pass forward kernel holds at most 128 key channels of the state

# A forward pass that will be differentiated keeps w, Aw, v_new and the per-chunk states for its
# backward pass (about 2.3 bytes per q/k/v byte) instead of recomputing them there as the reference
# does (fla/ops/gated_delta_rule/chunk.py:95-116): with 288 GB of HBM the second WY launch and the
# second state scan cost more than the memory.  FLA_AMD_RECOMPUTE_STATES=1 (or setting this flag to
# False) restores the reference's behaviour.
KEEP_STATES_FOR_BACKWARD = os.environ.get("FLA_AMD_RECOMPUTE_STATES", "0") in ("", "0")
# FLA_AMD_GDR_ONEPASS=1: a forward that is not differentiated runs as ONE launch (the WY blocks of a chunk are formed
# inside the scan's workgroups, fla_chunk_gated_delta_rule_fwd_onepass) once 64-column slabs give every CU a
# workgroup.  Off by default: the launch moves only the operator's own bytes, but the extra work lands on the
# scan's matrix waves, which are on the critical path of a chunk period, and measured slower than the two launches
# (212 against 190 us at B=8, T=4096, H=16, K=V=128).
ONEPASS_FORWARD = os.environ.get("FLA_AMD_GDR_ONEPASS", "0") not in ("", "0")
_ONEPASS_MIN_WORKGROUPS = 129


def _round64(d: int) -> int:
    return -(-d // 64) * 64


def _round_k(d: int) -> int:
    """Key head dims run on tiles of 64, 128 or 256 channels (zero padding is exact)."""
    return 64 if d <= 64 else 128 if d <= 128 else 256 if d <= 256 else _round64(d)


def chunk_gated_delta_rule_fwd(q, k, v, g, beta, scale, initial_state, output_final_state,
                               offsets=None, indices=None, head_first=True, chunk_size=64,
                               *, plan: Optional[VarlenPlan] = None, store_A: bool = True, fused: bool = True,
                               l2norm_eps: Optional[float] = None, want_g_cumsum: bool = True):
    """Reference-shaped forward (``fla/ops/gated_delta_rule/chunk.py:20-73``): returns
    ``(g_cumsum, o, Aw, Au, final_state)``.  ``fused=False`` runs the reference's steps one by one
    (cumsum, WY representation, state scan, output stage); the default two-launch form does not form
    ``Aw`` / ``Au`` and returns ``None`` for them.  ``l2norm_eps`` (two-launch form only): ``q`` and ``k`` are
    un-normalised and both launches l2-normalise the rows as they stage them.  ``want_g_cumsum=False``: the caller
    does not read the cumulative gates, which lets a large enough batch run as one launch (``g_cumsum`` is then
    returned as ``None``)."""
    if head_first or chunk_size != BT:
        raise NotImplementedError("fla_amd chunk_gated_delta_rule_fwd: seq-first, chunk size 64 only")
    if offsets is not None and plan is None:
        plan = VarlenPlan(offsets, BT)
    offs = None if plan is None else plan.offsets
    idx = None if plan is None else plan.indices
    co = None if plan is None else plan.chunk_offsets
    if fused and ONEPASS_FORWARD and want_g_cumsum is False:
        N = q.shape[0] if plan is None else plan.N
        if N * q.shape[2] * (v.shape[-1] // 64) >= _ONEPASS_MIN_WORKGROUPS:
            o, final_state = chunk_gated_delta_rule_fwd_onepass(
                q, k, v, g, beta, scale, initial_state, output_final_state, offsets=offs,
                seq_order=None if plan is None else plan.seq_order, l2norm_eps=l2norm_eps)
            return None, o, None, None, final_state
    if fused:
        # two launches; Aw / Au are not formed on this path
        AT, g, *rstd = fwd_prepare_scan_operands(k, beta, g, offsets=offs, indices=idx, l2norm_eps=l2norm_eps)
        o, final_state = chunk_gated_delta_rule_fwd_scan(q, k, v, AT, g, scale, initial_state, output_final_state,
                                                         offsets=offs, chunk_offsets=co,
                                                         seq_order=None if plan is None else plan.seq_order,
                                                         l2norm_eps=l2norm_eps, k_rstd=rstd[0] if rstd else None)
        return g, o, None, None, final_state
    if l2norm_eps is not None:
        raise ValueError("l2norm_eps needs the two-launch form")
    g = None if g is None else chunk_local_cumsum(g, BT, offsets=offs, indices=idx, head_first=False)
    w, u, Aw, Au = fwd_prepare_wy_repr(k, v, beta, g, offsets=offs, indices=idx, head_first=False, chunk_size=BT,
                                       store_A=store_A)
    h, v_new, final_state = chunk_gated_delta_rule_fwd_h(
        k=k, w=w, u=u, g=g, initial_state=initial_state, output_final_state=output_final_state,
        offsets=offs, indices=idx, head_first=False, chunk_size=BT, fragment_layout=True, chunk_offsets=co)
    o = chunk_fwd_o(q=q, k=k, v=v_new, h=h, g=g, scale=scale, offsets=offs, indices=idx, head_first=False, fragment_layout=True,
                    chunk_size=BT)
    return g, o, Aw, Au, final_state


def chunk_gated_delta_rule_fwd_keep(q, k, v, g, beta, scale, initial_state, output_final_state, offsets=None):
    """Forward of a pass that will be differentiated.  Returns ``(g_cumsum, o, final_state, kept)``
    with ``kept = (w, Aw, v_new, hT[, Aqk])`` for :func:`chunk_gated_delta_rule_bwd`.  Key dims up to 128: the
    two-launch forward, whose first launch also writes ``w`` and ``Aw`` and whose scan also writes ``v_new`` and
    the state entering every chunk.  K = 256: the reference's decomposition (WY launch, state scan, output stage)."""
    plan = VarlenPlan(offsets, BT) if offsets is not None else None
    offs = None if plan is None else plan.offsets
    idx = None if plan is None else plan.indices
    co = None if plan is None else plan.chunk_offsets
    beta = beta.float().contiguous()
    if q.shape[-1] <= _FUSED_MAX_K:
        AT, g, w, Aw = fwd_prepare_scan_operands(k, beta, g, offsets=offs, indices=idx, keep_w=True)
        o, final_state, v_new, hT, Aqk = chunk_gated_delta_rule_fwd_scan(
            q, k, v, AT, g, scale, initial_state, output_final_state, offsets=offs, chunk_offsets=co,
            seq_order=None if plan is None else plan.seq_order, keep=True)
        return g, o, final_state, (w, Aw, v_new, hT, Aqk)
    g = None if g is None else chunk_local_cumsum(g, BT, offsets=offs, indices=idx, head_first=False)
    w, u, Aw, _ = fwd_prepare_wy_repr(k, v, beta, g, offsets=offs, indices=idx, head_first=False, chunk_size=BT,
                                      store_A=True, store_Au=False)
    h, hT, v_new, final_state = chunk_gated_delta_rule_fwd_h_both(
        k, w, u, g, initial_state, output_final_state, offsets=offs, indices=idx, chunk_offsets=co)
    o = chunk_fwd_o(q=q, k=k, v=v_new, h=h, g=g, scale=scale, offsets=offs, indices=idx, head_first=False, fragment_layout=True,
                    chunk_size=BT)
    return g, o, final_state, (w, Aw, v_new, hT)


def chunk_gated_delta_rule_bwd(q, k, v, g_cumsum, beta, scale, initial_state, do, dht, offsets=None, kept=None):
    """Backward on prepared tensors (seq-first, 16-bit, 64-aligned head dims; ``g_cumsum``
    the fp32 chunk-local cumsum saved by the forward).  Without ``kept`` it recomputes w, u, Aw, the
    per-chunk states and v_new like the reference (``fla/ops/gated_delta_rule/chunk.py:95-116``).
    Returns ``(dq, dk, dv, dbeta, dg, dh0)``."""
    plan = VarlenPlan(offsets, BT) if offsets is not None else None
    offs = None if plan is None else plan.offsets
    idx = None if plan is None else plan.indices
    co = None if plan is None else plan.chunk_offsets
    B, T, H, K = q.shape
    V = v.shape[-1]
    N = B if plan is None else plan.N
    NT = 0 if plan is None else plan.NT
    beta = beta.float().contiguous()
    Aqk = None
    if kept is not None:
        w, Aw, v_new, hT = kept[:4]
        Aqk = kept[4] if len(kept) > 4 else None   # the score tiles of the two-launch forward (K <= 128)
    else:
        w, u, Aw, _ = fwd_prepare_wy_repr(k, v, beta, g_cumsum, offsets=offs, indices=idx, head_first=False,
                                          chunk_size=BT, store_A=True, store_Au=False)
        hT, v_new, _ = chunk_gated_delta_rule_fwd_h(
            k=k, w=w, u=u, g=g_cumsum, initial_state=initial_state, output_final_state=False, offsets=offs,
            indices=idx, head_first=False, chunk_size=BT, fragment_layout=True, transposed_fragments=True,
            chunk_offsets=co)
    ws_dvl, ws_dv2 = (torch.empty_like(v) if Aqk is None else None), torch.empty_like(v)
    ws_dh = torch.empty_like(hT)
    ws_dw, ws_dkp = torch.empty_like(k), torch.empty_like(k)
    ws_dgam = q.new_empty(K // 64, B * T, H, dtype=torch.float32)
    dq, dk, dv = torch.empty_like(q), torch.empty_like(k), torch.empty_like(v)
    dbeta = q.new_empty(B, T, H, dtype=torch.float32)
    dg = q.new_empty(B, T, H, dtype=torch.float32)   # the last launch sums the partials and takes the reverse cumsum
    dh0 = q.new_empty(N, H, K, V, dtype=torch.float32) if initial_state is not None else None
    if dht is not None:
        dht = (dht if dht.dtype == torch.float32 else dht.float()).contiguous()
    be.check(be.lib().fla_chunk_gated_delta_rule_bwd(
        be.ptr(q), be.ptr(k), be.ptr(v), be.ptr(w), be.ptr(v_new), be.ptr(beta), be.ptr(g_cumsum), be.ptr(Aw),
        be.ptr(do), be.ptr(dht), be.ptr(hT), be.ptr(Aqk), be.ptr(ws_dvl), be.ptr(ws_dv2), be.ptr(ws_dh), be.ptr(ws_dw),
        be.ptr(ws_dkp), be.ptr(ws_dgam), be.ptr(dq), be.ptr(dk), be.ptr(dv), be.ptr(dbeta), be.ptr(dg),
        be.ptr(dh0), be.ptr(offs), be.ptr(idx), be.ptr(co), NT, be.dt(q), B, T, H, K, V, N, float(scale),
        be.stream_of(q)), "fla_chunk_gated_delta_rule_bwd")
    return dq, dk, dv, dbeta, (dg if g_cumsum is not None else None), dh0


class ChunkGatedDeltaRuleFunction(torch.autograd.Function):

    @staticmethod
    @contiguous
    @autocast_custom_fwd
    def forward(ctx, q, k, v, g, beta, scale, initial_state, output_final_state, offsets=None, head_first=True):
        be.require_gpu(q, k, v, beta)
        in_dtypes = (q.dtype, k.dtype, v.dtype, None if g is None else g.dtype, beta.dtype)
        if head_first:
            q, k, v = (x.transpose(1, 2).contiguous() for x in (q, k, v))
            beta = beta.transpose(1, 2).contiguous()
            g = None if g is None else g.transpose(1, 2).contiguous()
        K, V = q.shape[-1], v.shape[-1]
        KP, VP = _round_k(K), _round64(V)
        if (KP, VP) not in _SUPPORTED_KV:
            raise NotImplementedError(f"fla_amd chunk_gated_delta_rule: head dims K={K}, V={V} are outside the built "
                                      f"tiles {sorted(_SUPPORTED_KV)} (after rounding up to multiples of 64)")
        h0 = initial_state
        if (KP, VP) != (K, V):
            q, k = F.pad(q, (0, KP - K)), F.pad(k, (0, KP - K))
            v = F.pad(v, (0, VP - V))
            if h0 is not None:
                h0 = F.pad(h0, (0, VP - V, 0, KP - K))
        kept = ()
        if KEEP_STATES_FOR_BACKWARD and any(ctx.needs_input_grad):
            gc, o, ht, kept = chunk_gated_delta_rule_fwd_keep(q, k, v, g, beta, scale, h0, output_final_state,
                                                              offsets=offsets)
        else:
            _, o, _, _, ht = chunk_gated_delta_rule_fwd(q, k, v, g, beta, scale, h0, output_final_state,
                                                        offsets=offsets, head_first=False, chunk_size=BT,
                                                        store_A=False, fused=KP <= _FUSED_MAX_K, want_g_cumsum=False)
            # a backward that recomputes starts from the raw gate, like the reference's
            gc = None if g is None else g.float().contiguous()
        ctx.save_for_backward(q, k, v, gc, beta, h0, offsets, *kept)
        ctx.scale, ctx.head_first, ctx.dims, ctx.in_dtypes = scale, head_first, (K, V, KP, VP), in_dtypes
        ctx.h0_dtype = None if initial_state is None else initial_state.dtype
        if (KP, VP) != (K, V):
            o = o[..., :V]
            if ht is not None:
                ht = ht[..., :K, :V].contiguous()
        if head_first:
            o = o.transpose(1, 2).contiguous()
        return o.to(in_dtypes[0]), ht

    @staticmethod
    @contiguous
    @autocast_custom_bwd
    def backward(ctx, do, dht):
        q, k, v, gc, beta, h0, offsets, *kept = ctx.saved_tensors
        K, V, KP, VP = ctx.dims
        if ctx.head_first:
            do = do.transpose(1, 2)
        do = do.to(q.dtype)
        if VP != V:
            do = F.pad(do, (0, VP - V))
        do = do.contiguous()
        if dht is not None and (KP, VP) != (K, V):
            dht = F.pad(dht, (0, VP - V, 0, KP - K))
        if not kept and gc is not None:   # the raw gate was saved: its prefix sums as the kept-states forward forms them
            plan = VarlenPlan(offsets, BT) if offsets is not None else None
            gc = chunk_local_cumsum(gc, BT, offsets=None if plan is None else plan.offsets,
                                    indices=None if plan is None else plan.indices, head_first=False)
        dq, dk, dv, db, dg, dh0 = chunk_gated_delta_rule_bwd(q, k, v, gc, beta, ctx.scale, h0, do, dht, offsets,
                                                             kept=tuple(kept) if kept else None)
        if (KP, VP) != (K, V):
            dq, dk, dv = dq[..., :K], dk[..., :K], dv[..., :V]
            if dh0 is not None:
                dh0 = dh0[..., :K, :V]
        if ctx.head_first:
            dq, dk, dv, db = (x.transpose(1, 2) for x in (dq, dk, dv, db))
            dg = None if dg is None else dg.transpose(1, 2)
        qd, kd, vd, gd, bd = ctx.in_dtypes
        if dh0 is not None:
            dh0 = dh0.to(ctx.h0_dtype)
        return (dq.to(qd), dk.to(kd), dv.to(vd), None if dg is None else dg.to(gd), db.to(bd), None, dh0,
                None, None, None)


def _direct_launch_ok(q, k, v, g, beta, initial_state, head_first) -> bool:
    """True when a call can go straight to the two forward launches: no operand takes part in autograd and every
    operand already has the layout, dtype and head dims the kernels read.  Anything else takes the autograd
    function, which converts and pads."""
    if head_first or q.dtype not in (torch.bfloat16, torch.float16):
        return False
    K, V = q.shape[-1], v.shape[-1]
    if K > _FUSED_MAX_K or (K, V) not in _SUPPORTED_KV:
        return False
    if torch.is_autocast_enabled():
        return False
    ts = (q, k, v, beta) if g is None else (q, k, v, beta, g)
    if torch.is_grad_enabled() and (any(t.requires_grad for t in ts) or
                                    (initial_state is not None and initial_state.requires_grad)):
        return False
    if not all(t.is_cuda and t.is_contiguous() for t in ts):
        return False
    return initial_state is None or (initial_state.dtype == torch.float32 and initial_state.is_contiguous())


def apply_in_value_slabs(q, k, v, g, beta, scale, initial_state, output_final_state, offsets, head_first):
    """The autograd function on heads of any supported width (``g`` may be None: un-gated rule)."""
    K, V = k.shape[-1], v.shape[-1]
    if K > 256:
        raise NotImplementedError(f"fla_amd chunk_gated_delta_rule: key head dims up to 256 are covered (got {K}), "
                                  f"as in the reference (fla/ops/common/chunk_delta_h.py:272)")
    if V > 128:
        # the delta rule is independent per value column: wider heads run as slabs of 128 columns
        # (autograd sums the slabs' gradients of q, k, g and beta)
        outs, states = [], []
        for v0 in range(0, V, 128):
            h0 = None if initial_state is None else initial_state[..., v0:v0 + 128]
            o, ht = ChunkGatedDeltaRuleFunction.apply(q, k, v[..., v0:v0 + 128], g, beta, scale, h0, output_final_state,
                                                      offsets, head_first)
            outs.append(o)
            states.append(ht)
        return torch.cat(outs, dim=-1), (torch.cat(states, dim=-1) if output_final_state else None)
    return ChunkGatedDeltaRuleFunction.apply(q, k, v, g, beta, scale, initial_state, output_final_state, offsets,
                                             head_first)


def chunk_gated_delta_rule(
    q: torch.Tensor,
    k: torch.Tensor,
    v: torch.Tensor,
    g: torch.Tensor,
    beta: torch.Tensor,
    scale: float = None,
    initial_state: torch.Tensor = None,
    output_final_state: bool = False,
    offsets: Optional[torch.LongTensor] = None,
    head_first: bool = True,
    cu_seqlens: Optional[torch.LongTensor] = None,
    use_qk_l2norm_in_kernel: bool = False,
) -> Tuple[torch.Tensor, torch.Tensor]:
    r"""
    Args:
        q, k: ``[B, H, T, K]`` if ``head_first`` else ``[B, T, H, K]`` (bf16 / fp16).
        v: ``[B, H, T, V]`` / ``[B, T, H, V]``.
        g: per-head log decay ``[B, H, T]`` / ``[B, T, H]``.
        beta: ``[B, H, T]`` / ``[B, T, H]``.
        scale: default ``K ** -0.5``; must be positive.
        initial_state: ``[N, H, K, V]`` or ``None``; output_final_state: return the fp32 final state.
        offsets (synonym ``cu_seqlens``): int64 ``[N+1]`` boundaries of a packed batch (batch 1, seq-first).
        use_qk_l2norm_in_kernel (extension, default off): ``q`` and ``k`` are un-normalised and the operator
            applies ``l2_norm`` (eps 1e-6, ``fla/modules/l2norm.py``) to both, as the layer does in front of it
            (``fla/layers/gated_deltanet.py:234-235``).  A forward that is not differentiated normalises the rows
            inside its two launches; otherwise the stand-alone ``l2_norm`` runs first, with its backward.

    Returns ``(o, final_state)``.
    """
    assert q.dtype == k.dtype == v.dtype
    assert q.dtype != torch.float32, "ChunkDeltaRuleFunction does not support float32. Please use bfloat16."
    assert len(beta.shape) == 3, "beta must be of shape [B, H, T] if head_first=True, or [B, T, H] if head_first=False."
    offsets = resolve_offsets(offsets, cu_seqlens)
    check_varlen_args(q, offsets, head_first, initial_state)
    if scale is None:
        scale = k.shape[-1] ** -0.5
    else:
        assert scale > 0, "Scale must be positive."
    if q.numel() == 0:
        return empty_batch_result(q.transpose(1, 2) if head_first else q, v, offsets, initial_state, output_final_state)
    direct = _direct_launch_ok(q, k, v, g, beta, initial_state, head_first)
    if use_qk_l2norm_in_kernel and not direct:
        from ...modules.l2norm import l2_norm
        q, k = l2_norm(q), l2_norm(k)
    if direct:
        # nothing to differentiate and nothing to convert: no autograd node, no copies
        _, o, _, _, ht = chunk_gated_delta_rule_fwd(q, k, v, g, beta, scale, initial_state, output_final_state,
                                                    offsets=offsets, head_first=False, chunk_size=BT, store_A=False,
                                                    l2norm_eps=1e-6 if use_qk_l2norm_in_kernel else None,
                                                    want_g_cumsum=False)
        return o, ht
    return apply_in_value_slabs(q, k, v, g, beta, scale, initial_state, output_final_state, offsets, head_first)
