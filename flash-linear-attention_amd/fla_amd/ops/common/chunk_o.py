"""``chunk_fwd_o`` for scalar-gated models (``fla/ops/common/chunk_o.py:444-495``), served by
``fla_chunk_fwd_o``, and the backward stages of the same file: ``chunk_bwd_dv_local`` (``:551-599``),
``chunk_bwd_dv`` (``:499-548``), ``chunk_bwd_dqkwg`` (``:602-670``)."""
from typing import Optional, Tuple

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
    ``g`` is the fp32 chunk-local cumsum ``[B,T,H]`` or ``None``.  Head-first operands (``[B,H,T,*]``, states
    ``[B,H,NT,K,V]``) are transposed on the way in and ``o`` on the way out."""
    if chunk_size != BT:
        raise NotImplementedError("fla_amd chunk_fwd_o: chunk size 64 only")
    if head_first:
        if fragment_layout:
            raise NotImplementedError("fla_amd chunk_fwd_o: fragment-order states are seq-first")
        tr = lambda x: None if x is None else x.transpose(1, 2).contiguous()
        return chunk_fwd_o(tr(q), tr(k), tr(v), tr(h), tr(g), scale, offsets, indices, False, chunk_size).transpose(1, 2)
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


def chunk_bwd_dv_local(
    q: torch.Tensor,
    k: torch.Tensor,
    g: Optional[torch.Tensor],
    do: torch.Tensor,
    dh: Optional[torch.Tensor],
    scale: float,
    offsets: Optional[torch.Tensor] = None,
    indices: Optional[torch.Tensor] = None,
    head_first: bool = True,
    chunk_size: int = 64,
) -> torch.Tensor:
    """``dv_j = sum_{i>=j} scale (k_j . q_i) exp(g_i - g_j) do_i`` within each chunk
    (``fla/ops/common/chunk_o.py:551-599``; ``dh`` is unused there as well).  ``g`` is the chunk-local
    cumsum ``[B,T,H]`` or ``None``.  Key dims up to 256 (zero-padded to 64 / 128 / 256), value dims in
    slabs of 128."""
    if chunk_size != BT:
        raise NotImplementedError("fla_amd chunk_bwd_dv_local: chunk size is fixed to 64")
    if q.dtype not in (torch.bfloat16, torch.float16) or k.dtype != q.dtype or do.dtype != q.dtype:
        raise NotImplementedError("fla_amd chunk_bwd_dv_local: q, k and do must all be bf16 or all fp16")
    if head_first:
        q, k, do = (x.transpose(1, 2) for x in (q, k, do))
        g = None if g is None else g.transpose(1, 2)
    be.require_gpu(q, k, do)
    B, T, H, K = k.shape
    V = do.shape[-1]
    if K > 256:
        raise NotImplementedError("fla_amd chunk_bwd_dv_local: K <= 256")
    Kp = 64 if K <= 64 else 128 if K <= 128 else 256
    pad = torch.nn.functional.pad
    qp = (q if Kp == K else pad(q, (0, Kp - K))).contiguous()
    kp = (k if Kp == K else pad(k, (0, Kp - K))).contiguous()
    gp = None if g is None else g.float().contiguous()
    NT = 0
    if offsets is not None:
        if indices is None:
            from ...utils import VarlenPlan
            indices = VarlenPlan(offsets, BT).indices
        NT = indices.shape[0]
        offsets = offsets.to(torch.int64).contiguous()
    outs = []
    for v0 in range(0, V, 128):
        d = do[..., v0:v0 + 128]
        w = d.shape[-1]
        wp = 64 if w <= 64 else 128
        d = (d if wp == w else pad(d, (0, wp - w))).contiguous()
        dv = torch.empty_like(d)
        be.check(be.lib().fla_chunk_bwd_dv_local(
            be.ptr(qp), be.ptr(kp), be.ptr(gp), be.ptr(d), be.ptr(dv), be.ptr(offsets), be.ptr(indices), NT,
            be.dt(qp), B, T, H, Kp, wp, float(scale), be.stream_of(q)), "fla_chunk_bwd_dv_local")
        outs.append(dv[..., :w])
    dv = outs[0] if len(outs) == 1 else torch.cat(outs, -1)
    return dv.transpose(1, 2) if head_first else dv


def fragments_to_states(hf: torch.Tensor, dtype: torch.dtype, transposed: bool = False) -> torch.Tensor:
    """The inverse of :func:`states_to_fragments`: 16-bit states in fragment order back to row-major
    ``[..., K, V]`` in ``dtype`` (fp32 or the fragments' own)."""
    K, V = hf.shape[-2:]
    if K % 32 or V % 32:
        raise NotImplementedError("fla_amd fragments_to_states: K and V must be multiples of 32")
    hf = hf.contiguous()
    out = torch.empty(hf.shape, dtype=dtype, device=hf.device)
    be.check(be.lib().fla_fragments_to_states(
        be.ptr(hf), be.ptr(out), be.dt(hf), be._DTYPES[dtype], int(transposed), hf.numel() // (K * V), K, V,
        be.stream_of(hf)), "fla_fragments_to_states")
    return out


def _states_seq_first(m: torch.Tensor, head_first: bool) -> torch.Tensor:
    return m.transpose(1, 2) if head_first else m


def chunk_bwd_dv(
    q: torch.Tensor,
    k: torch.Tensor,
    g: Optional[torch.Tensor],
    do: torch.Tensor,
    dh: torch.Tensor,
    scale: float,
    offsets: Optional[torch.Tensor] = None,
    indices: Optional[torch.Tensor] = None,
    head_first: bool = True,
    chunk_size: int = 64,
) -> torch.Tensor:
    """``dv_j = sum_{i>=j} scale (k_j . q_i) e^{g_i-g_j} do_i + (k_j e^{g_last-g_j})^T dh_c``
    (``fla/ops/common/chunk_o.py:499-548``, kernel ``:294-375``); ``dh`` row-major ``[B, NT, H, K, V]``.
    Two launches: the intra-chunk part (:func:`chunk_bwd_dv_local`) and the state part on the per-key-gate dv
    stage (``fla_chunk_gla_bwd_dv`` with an all-zero score tile and the gate repeated over the key channels);
    the sibling operators that call this are outside the hot path, so no kernel of its own."""
    from ..gla.chunk import chunk_gla_bwd_dv
    if offsets is not None and indices is None:
        from ...utils import VarlenPlan
        indices = VarlenPlan(offsets, BT).indices
    dv = chunk_bwd_dv_local(q, k, g, do, None, scale, offsets=offsets, indices=indices, head_first=head_first,
                            chunk_size=chunk_size)
    shape = k.shape[:-1]
    gk = k.new_zeros(*k.shape, dtype=torch.float32) if g is None else g.float().unsqueeze(-1).expand(*k.shape).contiguous()
    A = k.new_zeros(*shape, BT, dtype=torch.float32)
    dv_state = chunk_gla_bwd_dv(k, gk, A, do, dh, offsets=offsets, indices=indices, head_first=head_first,
                                chunk_size=chunk_size)
    return dv + dv_state.to(dv.dtype)


def chunk_bwd_dqkwg(
    q: torch.Tensor,
    k: torch.Tensor,
    v: torch.Tensor,
    g: Optional[torch.Tensor],
    do: torch.Tensor,
    h: torch.Tensor,
    dh: torch.Tensor,
    dv: Optional[torch.Tensor] = None,
    w: Optional[torch.Tensor] = None,
    offsets: Optional[torch.Tensor] = None,
    indices: Optional[torch.Tensor] = None,
    chunk_size: int = 64,
    scale: float = 1.0,
    head_first: bool = True,
    *,
    fragment_layout: bool = False,
) -> Tuple[torch.Tensor, torch.Tensor, Optional[torch.Tensor], Optional[torch.Tensor]]:
    """``(dq, dk, dw, dg)`` of the scalar-gated chunk step (``fla/ops/common/chunk_o.py:602-670``): ``v`` is the
    value the output stage saw (``v_new`` for the delta rule), ``h`` / ``dh`` the row-major per-chunk states and
    their gradients ``[B, NT, H, K, V]`` (``fragment_layout=True``: both already in transposed-fragment order),
    ``dv`` / ``w`` the delta rule's extra operands (``dw`` is ``None`` without ``w``).  ``dg`` is fp32 ``[B,T,H]``
    before the reverse cumulative sum, as the reference returns it."""
    if chunk_size != BT:
        raise NotImplementedError("fla_amd chunk_bwd_dqkwg: chunk size is fixed to 64")
    if head_first:
        q, k, v, do = (x.transpose(1, 2) for x in (q, k, v, do))
        g, dv, w = (None if x is None else x.transpose(1, 2) for x in (g, dv, w))
        if not fragment_layout:
            h, dh = h.transpose(1, 2), dh.transpose(1, 2)
    be.require_gpu(q, k, v, do, h, dh)
    B, T, H, K = k.shape
    V = v.shape[-1]
    if K % 64 or V not in (64, 128):
        raise NotImplementedError("fla_amd chunk_bwd_dqkwg: K a multiple of 64, V in {64, 128}")
    if any(x.dtype != q.dtype for x in (k, v, do)) or q.dtype not in (torch.bfloat16, torch.float16):
        raise NotImplementedError("fla_amd chunk_bwd_dqkwg: q, k, v, do all bf16 or all fp16")
    q, k, v, do = (x.contiguous() for x in (q, k, v, do))
    has_w = w is not None
    w = torch.zeros_like(k) if w is None else w.to(q.dtype).contiguous()
    dv = torch.zeros_like(v) if dv is None else dv.to(q.dtype).contiguous()
    gg = None if g is None else g.float().contiguous()
    if not fragment_layout:
        h = states_to_fragments(h, q.dtype, transposed=True)
        dh = states_to_fragments(dh, q.dtype, transposed=True)
    NT = 0
    if offsets is not None:
        if indices is None:
            from ...utils import VarlenPlan
            indices = VarlenPlan(offsets, BT).indices
        indices = indices.to(torch.int64).contiguous()
        NT = indices.shape[0]
        offsets = offsets.to(torch.int64).contiguous()
    dq, dk, dw = torch.empty_like(q), torch.empty_like(k), torch.empty_like(k)
    dg = q.new_empty(K // 64, B, T, H, dtype=torch.float32)
    be.check(be.lib().fla_chunk_bwd_dqkwg(
        be.ptr(q), be.ptr(k), be.ptr(v), be.ptr(w), be.ptr(gg), be.ptr(h), be.ptr(dh), be.ptr(do), be.ptr(dv),
        be.ptr(dq), be.ptr(dk), be.ptr(dw), be.ptr(dg), be.ptr(offsets), be.ptr(indices), NT, be.dt(q), B, T, H, K, V,
        float(scale), be.stream_of(q)), "fla_chunk_bwd_dqkwg")
    dg = None if g is None else dg.sum(0)
    dw = dw if has_w else None
    if head_first:
        dq, dk = dq.transpose(1, 2).contiguous(), dk.transpose(1, 2).contiguous()
        dw = None if dw is None else dw.transpose(1, 2).contiguous()
        dg = None if dg is None else dg.transpose(1, 2).contiguous()
    return dq, dk, dw, dg
