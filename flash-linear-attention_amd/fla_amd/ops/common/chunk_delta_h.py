"""``chunk_gated_delta_rule_fwd_h`` (``fla/ops/common/chunk_delta_h.py:248-320``),
served by ``fla_chunk_gated_delta_rule_fwd_h``, and ``chunk_gated_delta_rule_bwd_dhu`` (``:323-391``),
served by ``fla_chunk_gated_delta_rule_bwd_dhu``."""
from typing import Optional, Tuple

import torch

from ... import _backend as be
from ...utils import prepare_chunk_offsets

BT = 64


def chunk_gated_delta_rule_fwd_h(
    k: torch.Tensor,
    w: torch.Tensor,
    u: torch.Tensor,
    g: Optional[torch.Tensor],
    initial_state: Optional[torch.Tensor],
    output_final_state: bool,
    offsets: Optional[torch.Tensor] = None,
    indices: Optional[torch.Tensor] = None,
    head_first: bool = True,
    chunk_size: int = 64,
    *,
    states_in_fp32: bool = False,
    fragment_layout: bool = False,
    transposed_fragments: bool = False,
    chunk_offsets: Optional[torch.Tensor] = None,
    store_v_new: bool = True,
) -> Tuple[torch.Tensor, Optional[torch.Tensor], Optional[torch.Tensor]]:
    """Returns ``(h, v_new, final_state)``; ``g`` is the fp32 chunk-local cumsum of
    the log-gate ``[B,T,H]`` (or ``None``).  ``h`` is ``[B,NT,H,K,V]`` holding the
    state entering each chunk (row-major, or MFMA-fragment order for
    ``fla_chunk_fwd_o`` when ``fragment_layout``)."""
    if chunk_size != BT:
        raise NotImplementedError("fla_amd chunk_gated_delta_rule_fwd_h: chunk size 64 only")
    if head_first:
        # head-first operands ([B,H,T,*]) are transposed on the way in, h ([B,H,NT,K,V]) and v_new on the way out
        if fragment_layout:
            raise NotImplementedError("fla_amd chunk_gated_delta_rule_fwd_h: fragment-order states are seq-first")
        tr = lambda x: None if x is None else x.transpose(1, 2).contiguous()
        h, v_new, ht = chunk_gated_delta_rule_fwd_h(
            tr(k), tr(w), tr(u), tr(g), initial_state, output_final_state, offsets, indices, False, chunk_size,
            states_in_fp32=states_in_fp32, chunk_offsets=chunk_offsets, store_v_new=store_v_new)
        return h.transpose(1, 2), (None if v_new is None else v_new.transpose(1, 2)), ht
    be.require_gpu(k, w, u)
    B, T, H, K = k.shape
    V = u.shape[-1]
    if offsets is None:
        N, NT = B, -(-T // BT)
    else:
        if chunk_offsets is None:
            chunk_offsets = prepare_chunk_offsets(offsets, BT, device=k.device)
        N = len(offsets) - 1
        NT = int(indices.shape[0]) if indices is not None else int(prepare_chunk_offsets(offsets, BT)[-1])
        offsets = offsets.to(torch.int64).contiguous()
    h_dtype = torch.float32 if states_in_fp32 else k.dtype
    h = k.new_empty(B, NT, H, K, V, dtype=h_dtype)
    v_new = torch.empty_like(u) if store_v_new else None
    ht = k.new_empty(N, H, K, V, dtype=torch.float32) if output_final_state else None
    h0 = None
    if initial_state is not None:
        h0 = (initial_state if initial_state.dtype == torch.float32 else initial_state.float()).contiguous()
    if g is not None and g.dtype != torch.float32:
        g = g.float()
    be.check(be.lib().fla_chunk_gated_delta_rule_fwd_h(
        be.ptr(k), be.ptr(w), be.ptr(u), be.ptr(g), be.ptr(h0), be.ptr(h), be.ptr(v_new), be.ptr(ht),
        be.ptr(offsets), be.ptr(chunk_offsets), be.dt(k), be._DTYPES[h_dtype],
        (be.FLA_H_FRAGMENT_T if transposed_fragments else be.FLA_H_FRAGMENT) if fragment_layout
        else be.FLA_H_ROW_MAJOR,
        B, T, H, K, V, N, be.stream_of(k)), "fla_chunk_gated_delta_rule_fwd_h")
    return h, v_new, ht


def chunk_gated_delta_rule_fwd_h_both(
    k: torch.Tensor,
    w: torch.Tensor,
    u: torch.Tensor,
    g: Optional[torch.Tensor],
    initial_state: Optional[torch.Tensor],
    output_final_state: bool,
    offsets: Optional[torch.Tensor] = None,
    indices: Optional[torch.Tensor] = None,
    chunk_offsets: Optional[torch.Tensor] = None,
) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor, Optional[torch.Tensor]]:
    """The state scan for a forward pass whose states are kept for the backward pass: returns
    ``(h, hT, v_new, final_state)`` with the per-chunk states in MFMA-fragment order (for
    ``chunk_fwd_o``) and in transposed fragment order (for ``fla_chunk_gated_delta_rule_bwd``).
    Seq-first, chunk size 64; served by ``fla_chunk_gated_delta_rule_fwd_h_both``."""
    be.require_gpu(k, w, u)
    B, T, H, K = k.shape
    V = u.shape[-1]
    if offsets is None:
        N, NT = B, -(-T // BT)
    else:
        if chunk_offsets is None:
            chunk_offsets = prepare_chunk_offsets(offsets, BT, device=k.device)
        N = len(offsets) - 1
        NT = int(indices.shape[0]) if indices is not None else int(prepare_chunk_offsets(offsets, BT)[-1])
        offsets = offsets.to(torch.int64).contiguous()
    h = k.new_empty(B, NT, H, K, V)
    hT = k.new_empty(B, NT, H, K, V)
    v_new = torch.empty_like(u)
    ht = k.new_empty(N, H, K, V, dtype=torch.float32) if output_final_state else None
    h0 = None
    if initial_state is not None:
        h0 = (initial_state if initial_state.dtype == torch.float32 else initial_state.float()).contiguous()
    if g is not None and g.dtype != torch.float32:
        g = g.float()
    be.check(be.lib().fla_chunk_gated_delta_rule_fwd_h_both(
        be.ptr(k), be.ptr(w), be.ptr(u), be.ptr(g), be.ptr(h0), be.ptr(h), be.ptr(hT), be.ptr(v_new), be.ptr(ht),
        be.ptr(offsets), be.ptr(chunk_offsets), be.dt(k), B, T, H, K, V, N, be.stream_of(k)),
        "fla_chunk_gated_delta_rule_fwd_h_both")
    return h, hT, v_new, ht


def chunk_gated_delta_rule_fwd_scan(
    q: torch.Tensor,
    k: torch.Tensor,
    v: torch.Tensor,
    AT: torch.Tensor,
    g: Optional[torch.Tensor],
    scale: float,
    initial_state: Optional[torch.Tensor],
    output_final_state: bool,
    offsets: Optional[torch.Tensor] = None,
    chunk_offsets: Optional[torch.Tensor] = None,
    seq_order: Optional[torch.Tensor] = None,
    *,
    keep: bool = False,
    l2norm_eps: Optional[float] = None,
    k_rstd: Optional[torch.Tensor] = None,
):
    """Serial half of the one-pass forward (``fla_chunk_gated_delta_rule_fwd_scan``): the work of
    ``chunk_gated_delta_rule_fwd_h`` followed by ``chunk_fwd_o`` (``fla/ops/gated_delta_rule/chunk.py:47-72``)
    on ``q, k, v`` and the packed triangular tiles ``AT`` of ``fwd_prepare_scan_operands``; neither w, u,
    v_new nor the per-chunk states are materialised.  ``g`` is the fp32 chunk-local cumsum.  Seq-first.
    Returns ``(o, final_state)``; with ``keep`` also ``v_new``, the state entering every chunk in
    transposed-fragment order (``[B, NT, H, K, V]``) and the packed score tiles ``Aqk``
    (``[chunks, H, 10, 16, 16]``), what the backward reads: ``(o, final_state, v_new, hT, Aqk)``.
    ``l2norm_eps``: ``q`` and ``k`` are un-normalised and the launch works with their l2-normalised rows
    (``fla_chunk_gated_delta_rule_fwd_scan_l2norm``; ``k_rstd`` are the factors of ``k`` that
    ``fwd_prepare_scan_operands(..., l2norm_eps=...)`` returned; not with ``keep``)."""
    be.require_gpu(q, k, v, AT)
    B, T, H, K = k.shape
    V = v.shape[-1]
    N = B
    if offsets is not None:
        N = len(offsets) - 1
        offsets = offsets.to(torch.int64).contiguous()
    o = torch.empty_like(v)
    ht = k.new_empty(N, H, K, V, dtype=torch.float32) if output_final_state else None
    h0 = None
    if initial_state is not None:
        h0 = (initial_state if initial_state.dtype == torch.float32 else initial_state.float()).contiguous()
    if g is not None and g.dtype != torch.float32:
        g = g.float()
    v_new = hT = Aqk = None
    if keep:
        v_new = torch.empty_like(v)
        hT = k.new_empty(B, AT.shape[0] // B if offsets is None else AT.shape[0], H, K, V)
        Aqk = torch.empty_like(AT)
    if l2norm_eps is not None:
        if keep:
            raise ValueError("l2norm_eps: forward without kept intermediates only")
        if k_rstd is None:
            raise ValueError("l2norm_eps: the scan needs k_rstd from fwd_prepare_scan_operands")
        be.check(be.lib().fla_chunk_gated_delta_rule_fwd_scan_l2norm(
            be.ptr(q), be.ptr(k), be.ptr(v), be.ptr(AT), be.ptr(g), be.ptr(k_rstd), be.ptr(h0), be.ptr(o), be.ptr(ht),
            be.ptr(offsets), be.ptr(chunk_offsets), be.ptr(seq_order), be.dt(k), B, T, H, K, V, N, float(scale),
            float(l2norm_eps), be.stream_of(k)), "fla_chunk_gated_delta_rule_fwd_scan_l2norm")
        return o, ht
    be.check(be.lib().fla_chunk_gated_delta_rule_fwd_scan(
        be.ptr(q), be.ptr(k), be.ptr(v), be.ptr(AT), be.ptr(g), be.ptr(h0), be.ptr(o), be.ptr(ht), be.ptr(v_new),
        be.ptr(hT), be.ptr(Aqk), be.ptr(offsets), be.ptr(chunk_offsets), be.ptr(seq_order), be.dt(k), B, T, H, K, V, N,
        float(scale), be.stream_of(k)), "fla_chunk_gated_delta_rule_fwd_scan")
    if keep:
        return o, ht, v_new, hT, Aqk
    return o, ht


def chunk_gated_delta_rule_fwd_onepass(
    q: torch.Tensor,
    k: torch.Tensor,
    v: torch.Tensor,
    g: Optional[torch.Tensor],
    beta: torch.Tensor,
    scale: float,
    initial_state: Optional[torch.Tensor],
    output_final_state: bool,
    offsets: Optional[torch.Tensor] = None,
    seq_order: Optional[torch.Tensor] = None,
    *,
    l2norm_eps: Optional[float] = None,
):
    """The whole forward (``fla/ops/gated_delta_rule/chunk.py:20-73``) in one launch,
    ``fla_chunk_gated_delta_rule_fwd_onepass``: ``g`` is the raw per-head log-gate ``[B,T,H]`` (or ``None``), ``beta``
    ``[B,T,H]``; the prefix sum of the gate, the WY blocks, the state scan and the output stage all happen inside the
    scan's workgroups.  Seq-first, K in {64, 128}, V a multiple of 64.  Returns ``(o, final_state)``.
    ``l2norm_eps``: ``q`` and ``k`` are un-normalised and are l2-normalised row by row as they are staged."""
    be.require_gpu(q, k, v, beta)
    B, T, H, K = k.shape
    V = v.shape[-1]
    N = B
    if offsets is not None:
        N = len(offsets) - 1
        offsets = offsets.to(torch.int64).contiguous()
    o = torch.empty_like(v)
    ht = k.new_empty(N, H, K, V, dtype=torch.float32) if output_final_state else None
    h0 = None
    if initial_state is not None:
        h0 = (initial_state if initial_state.dtype == torch.float32 else initial_state.float()).contiguous()
    if g is not None:
        g = g.float().contiguous()
    beta = beta.float().contiguous()
    be.check(be.lib().fla_chunk_gated_delta_rule_fwd_onepass(
        be.ptr(q), be.ptr(k), be.ptr(v), be.ptr(g), be.ptr(beta), be.ptr(h0), be.ptr(o), be.ptr(ht), be.ptr(offsets),
        None, be.ptr(seq_order), be.dt(k), B, T, H, K, V, N, float(scale), int(l2norm_eps is not None),
        float(l2norm_eps or 0.0), be.stream_of(k)), "fla_chunk_gated_delta_rule_fwd_onepass")
    return o, ht


def chunk_gated_delta_rule_bwd_dhu(
    q: torch.Tensor,
    k: torch.Tensor,
    w: torch.Tensor,
    g: Optional[torch.Tensor],
    h0: Optional[torch.Tensor],
    dht: Optional[torch.Tensor],
    do: torch.Tensor,
    dv: torch.Tensor,
    scale: float,
    offsets: Optional[torch.Tensor] = None,
    head_first: bool = True,
    chunk_size: int = 64,
    *,
    fragment_layout: bool = False,
) -> Tuple[torch.Tensor, Optional[torch.Tensor], torch.Tensor]:
    """Reverse state scan of the delta rule's backward (``fla/ops/common/chunk_delta_h.py:323-391``):
    returns ``(dh, dh0, dv2)`` with ``dh`` ``[B, NT, H, K, V]`` (``[B, H, NT, K, V]`` if ``head_first``) in the
    q/k dtype, the gradient w.r.t. the state leaving every chunk; ``g`` is the chunk-local cumsum ``[B,T,H]``.
    ``fragment_layout=True`` leaves ``dh`` in the transposed-fragment order the next stage reads."""
    if chunk_size != BT:
        raise NotImplementedError("fla_amd chunk_gated_delta_rule_bwd_dhu: chunk size is fixed to 64")
    if head_first:
        q, k, w, do, dv = (x.transpose(1, 2) for x in (q, k, w, do, dv))
        g = None if g is None else g.transpose(1, 2)
    be.require_gpu(q, k, w, do, dv)
    q, k, w, do, dv = (x.contiguous() for x in (q, k, w, do, dv))
    B, T, H, K = q.shape
    V = do.shape[-1]
    if K not in (64, 128, 256) or V % 32:
        raise NotImplementedError("fla_amd chunk_gated_delta_rule_bwd_dhu: K in {64,128,256}, V a multiple of 32")
    if any(x.dtype != q.dtype for x in (k, w, do, dv)) or q.dtype not in (torch.bfloat16, torch.float16):
        raise NotImplementedError("fla_amd chunk_gated_delta_rule_bwd_dhu: q, k, w, do, dv all bf16 or all fp16")
    g = None if g is None else g.float().contiguous()
    co, N, NT = None, B, -(-T // BT)
    if offsets is not None:
        offsets = offsets.to(torch.int64).contiguous()
        co = prepare_chunk_offsets(offsets, BT).to(torch.int64).contiguous()
        N = offsets.numel() - 1
        NT = int(co[-1])
    dh = q.new_empty(B, NT, H, K, V)
    dh0 = q.new_empty(N, H, K, V, dtype=torch.float32) if h0 is not None else None
    dv2 = torch.empty_like(dv)
    dht = None if dht is None else dht.float().contiguous()
    be.check(be.lib().fla_chunk_gated_delta_rule_bwd_dhu(
        be.ptr(q), be.ptr(k), be.ptr(w), be.ptr(g), be.ptr(dht), be.ptr(do), be.ptr(dv), be.ptr(dh), be.ptr(dv2),
        be.ptr(dh0), be.ptr(offsets), be.ptr(co), be.dt(q), B, T, H, K, V, N, float(scale), be.stream_of(q)),
        "fla_chunk_gated_delta_rule_bwd_dhu")
    if not fragment_layout:
        from .chunk_o import fragments_to_states
        dh = fragments_to_states(dh, q.dtype, transposed=True)
        if head_first:
            dh = dh.transpose(1, 2).contiguous()
    if head_first:
        dv2 = dv2.transpose(1, 2).contiguous()
    return dh, dh0, dv2
