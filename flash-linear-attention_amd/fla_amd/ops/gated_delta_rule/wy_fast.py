"""WY representation of the gated delta rule (``fla/ops/gated_delta_rule/wy_fast.py:320-426``), served by
``fla_gdr_fwd_wy``; ``fwd_recompute_w_u`` (``:320-371``) and ``bwd_prepare_wy_repr`` (``:565-625``) on the
reference's operands, served by ``fla_fwd_recompute_w_u`` and ``fla_bwd_prepare_wy_repr``."""
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
    store_u: bool = True,
):
    """Returns ``(w, u, Aw, Au)`` with ``Aw = (I + strict_lower(diag(beta) K K^T))^-1``,
    ``Au = Aw * exp(g_i - g_j)``, ``w = Aw (beta K)``, ``u = Au (beta V)``; ``g`` is the
    fp32 chunk-local cumsum of the log-gate (or ``None``).  ``store_u=False`` skips ``u`` (returned as ``None``)
    for a forward that forms ``v_new`` from the triangular tiles instead."""
    if chunk_size != BT:
        raise NotImplementedError("fla_amd fwd_prepare_wy_repr: chunk size 64 only")
    if head_first:
        # head-first operands ([B,H,T,*]) are transposed on the way in and every result on the way out
        tr = lambda x: None if x is None else x.transpose(1, 2).contiguous()
        outs = fwd_prepare_wy_repr(tr(k), tr(v), tr(beta), tr(g), offsets, indices, False, chunk_size,
                                   store_A=store_A, store_Au=store_Au, store_u=store_u)
        return tuple(None if x is None else x.transpose(1, 2) for x in outs)
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
    w, u = torch.empty_like(k), (torch.empty_like(v) if store_u else None)
    Aw = k.new_empty(B, T, H, BT) if store_A else None
    Au = k.new_empty(B, T, H, BT) if (store_A and store_Au) else None
    be.check(be.lib().fla_gdr_fwd_wy(
        be.ptr(k), be.ptr(v), be.ptr(beta), be.ptr(g), be.ptr(w), be.ptr(u), be.ptr(Aw), be.ptr(Au),
        be.ptr(offsets), be.ptr(indices), NT, be.dt(k), B, T, H, K, V, be.stream_of(k)), "fla_gdr_fwd_wy")
    return w, u, Aw, Au


TRI_BLOCKS = 10   # 16x16 blocks on and below the diagonal of a 64x64 tile


def fwd_prepare_scan_operands(
    k: torch.Tensor,
    beta: torch.Tensor,
    g: Optional[torch.Tensor],
    offsets: Optional[torch.Tensor] = None,
    indices: Optional[torch.Tensor] = None,
    g_is_cumsum: bool = False,
    keep_w: bool = False,
    l2norm_eps: Optional[float] = None,
):
    """Chunk-parallel half of the one-pass forward (``fla_gdr_fwd_prep``): the work of ``chunk_local_cumsum``
    and ``fwd_prepare_wy_repr`` (``fla/ops/gated_delta_rule/wy_fast.py:320-376``), leaving per (chunk, head) the
    lower-triangular ``Tu = (Aw * Gamma) diag(beta)`` as packed 16x16 blocks: ``AT`` is
    ``[chunks, H, 10, 16, 16]`` in the k dtype (the scan forms the gated scores ``q k^T`` itself).  ``g`` is the raw per-head log-gate
    ``[B, T, H]`` (or its chunk-local cumsum with ``g_is_cumsum``; ``None`` for the un-gated rule).
    Seq-first, K in {64, 128}.  Returns ``(AT, g_cumsum)``; with ``keep_w`` the launch also writes
    ``w = Aw (beta k)`` and ``Aw`` (what ``fwd_prepare_wy_repr`` leaves for the backward) and the return value
    is ``(AT, g_cumsum, w, Aw)``.  ``l2norm_eps``: ``k`` is un-normalised and the launch works with its
    l2-normalised rows (``fla_gdr_fwd_prep_l2norm``; not with ``keep_w``); the return value is then
    ``(AT, g_cumsum, k_rstd)`` with the per-row factors ``1 / sqrt(sum k^2 + eps)`` (fp32 ``[B,T,H]``) the scan reads."""
    be.require_gpu(k, beta)
    B, T, H, K = k.shape
    NT = 0
    chunks = B * (-(-T // BT))
    if offsets is not None:
        NT = chunks = indices.shape[0]
        offsets = offsets.to(torch.int64).contiguous()
    beta = beta.float().contiguous()
    gc = None
    if g is not None:
        g = g.float().contiguous()
        gc = g if g_is_cumsum else torch.empty_like(g)
    AT = k.new_empty(chunks, H, TRI_BLOCKS, 16, 16)
    w = torch.empty_like(k) if keep_w else None
    Aw = k.new_empty(B, T, H, BT) if keep_w else None
    if l2norm_eps is not None:
        if keep_w:
            raise ValueError("l2norm_eps: forward without kept intermediates only")
        k_rstd = k.new_empty(B, T, H, dtype=torch.float32)
        be.check(be.lib().fla_gdr_fwd_prep_l2norm(
            be.ptr(k), be.ptr(beta), be.ptr(g), int(g_is_cumsum), be.ptr(None if g_is_cumsum else gc), be.ptr(AT),
            be.ptr(k_rstd), be.ptr(offsets), be.ptr(indices), NT, be.dt(k), B, T, H, K, float(l2norm_eps),
            be.stream_of(k)), "fla_gdr_fwd_prep_l2norm")
        return AT, gc, k_rstd
    be.check(be.lib().fla_gdr_fwd_prep(
        be.ptr(k), be.ptr(beta), be.ptr(g), int(g_is_cumsum), be.ptr(None if g_is_cumsum else gc),
        be.ptr(AT), be.ptr(w), be.ptr(Aw), be.ptr(offsets), be.ptr(indices), NT, be.dt(k), B, T, H, K,
        be.stream_of(k)), "fla_gdr_fwd_prep")
    return (AT, gc, w, Aw) if keep_w else (AT, gc)


def unpack_triangular_tiles(AT: torch.Tensor) -> torch.Tensor:
    """``[chunks, H, 10, 16, 16]`` packed blocks -> dense ``[chunks, H, 64, 64]`` (zeros above the diagonal
    blocks); for tests and debugging."""
    chunks, H = AT.shape[:2]
    out = AT.new_zeros(chunks, H, 64, 64)
    for i in range(4):
        for j in range(i + 1):
            out[..., 16 * i:16 * i + 16, 16 * j:16 * j + 16] = AT[..., i * (i + 1) // 2 + j, :, :]
    return out


def _chunk_tables(offsets, indices):
    if offsets is None:
        return None, None, 0
    if indices is None:
        from ...utils import VarlenPlan
        indices = VarlenPlan(offsets, BT).indices
    indices = indices.to(torch.int64).contiguous()
    return offsets.to(torch.int64).contiguous(), indices, indices.shape[0]


def fwd_recompute_w_u(
    k: torch.Tensor,
    v: torch.Tensor,
    beta: torch.Tensor,
    Aw: torch.Tensor,
    Au: torch.Tensor,
    offsets: Optional[torch.Tensor] = None,
    indices: Optional[torch.Tensor] = None,
    head_first: bool = True,
    chunk_size: int = 64,
) -> Tuple[torch.Tensor, torch.Tensor]:
    """``w = Aw (beta k)``, ``u = Au (beta v)`` per chunk on matrices the caller kept
    (``fla/ops/gated_delta_rule/wy_fast.py:320-371``); ``Aw`` / ``Au`` ``[B,T,H,64]`` lower triangular."""
    if chunk_size != BT:
        raise NotImplementedError("fla_amd fwd_recompute_w_u: chunk size is fixed to 64")
    if head_first:
        k, v, beta, Aw, Au = (x.transpose(1, 2) for x in (k, v, beta, Aw, Au))
    be.require_gpu(k, v, beta, Aw, Au)
    B, T, H, K = k.shape
    V = v.shape[-1]
    if K not in (64, 128, 256) or V not in (64, 128):
        raise NotImplementedError("fla_amd fwd_recompute_w_u: K in {64,128,256}, V in {64,128}")
    if k.dtype not in (torch.bfloat16, torch.float16) or v.dtype != k.dtype:
        raise NotImplementedError("fla_amd fwd_recompute_w_u: k and v both bf16 or both fp16")
    k, v = k.contiguous(), v.contiguous()
    Aw, Au = Aw.to(k.dtype).contiguous(), Au.to(k.dtype).contiguous()
    beta = beta.float().contiguous()
    offsets, indices, NT = _chunk_tables(offsets, indices)
    w, u = torch.empty_like(k), torch.empty_like(v)
    be.check(be.lib().fla_fwd_recompute_w_u(
        be.ptr(k), be.ptr(v), be.ptr(beta), be.ptr(Aw), be.ptr(Au), be.ptr(w), be.ptr(u), be.ptr(offsets),
        be.ptr(indices), NT, be.dt(k), B, T, H, K, V, be.stream_of(k)), "fla_fwd_recompute_w_u")
    if head_first:
        w, u = w.transpose(1, 2).contiguous(), u.transpose(1, 2).contiguous()
    return w, u


def bwd_prepare_wy_repr(
    k: torch.Tensor,
    v: torch.Tensor,
    g: Optional[torch.Tensor],
    beta: torch.Tensor,
    Aw: torch.Tensor,
    Au: Optional[torch.Tensor],
    dw: torch.Tensor,
    du: torch.Tensor,
    offsets: Optional[torch.Tensor] = None,
    indices: Optional[torch.Tensor] = None,
    head_first: bool = True,
    chunk_size: int = 64,
) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor]:
    """``(dk, dv, dbeta, dg)`` through ``w = Aw (beta k)``, ``u = Au (beta v)``
    (``fla/ops/gated_delta_rule/wy_fast.py:565-625``); ``g`` the chunk-local cumsum, ``dbeta`` / ``dg`` fp32.
    ``Au`` is not read: it equals ``Aw * exp(g_i - g_j)`` and is rebuilt from ``Aw`` and ``g``."""
    if chunk_size != BT:
        raise NotImplementedError("fla_amd bwd_prepare_wy_repr: chunk size is fixed to 64")
    if head_first:
        k, v, beta, Aw, dw, du = (x.transpose(1, 2) for x in (k, v, beta, Aw, dw, du))
        g = None if g is None else g.transpose(1, 2)
    be.require_gpu(k, v, beta, Aw, dw, du)
    B, T, H, K = k.shape
    V = v.shape[-1]
    if K not in (64, 128, 256) or V not in (64, 128):
        raise NotImplementedError("fla_amd bwd_prepare_wy_repr: K in {64,128,256}, V in {64,128}")
    if k.dtype not in (torch.bfloat16, torch.float16) or v.dtype != k.dtype:
        raise NotImplementedError("fla_amd bwd_prepare_wy_repr: k and v both bf16 or both fp16")
    k, v = k.contiguous(), v.contiguous()
    Aw, dw, du = Aw.to(k.dtype).contiguous(), dw.to(k.dtype).contiguous(), du.to(k.dtype).contiguous()
    beta = beta.float().contiguous()
    g = None if g is None else g.float().contiguous()
    offsets, indices, NT = _chunk_tables(offsets, indices)
    dk, dv = torch.empty_like(k), torch.empty_like(v)
    dbeta = k.new_empty(B, T, H, dtype=torch.float32)
    dg = k.new_empty(B, T, H, dtype=torch.float32)
    be.check(be.lib().fla_bwd_prepare_wy_repr(
        be.ptr(k), be.ptr(v), be.ptr(beta), be.ptr(g), be.ptr(Aw), be.ptr(dw), be.ptr(du), None, be.ptr(dk),
        be.ptr(dv), be.ptr(dbeta), be.ptr(dg), be.ptr(offsets), be.ptr(indices), NT, be.dt(k), B, T, H, K, V,
        be.stream_of(k)), "fla_bwd_prepare_wy_repr")
    if head_first:
        dk, dv = dk.transpose(1, 2).contiguous(), dv.transpose(1, 2).contiguous()
        dbeta, dg = dbeta.transpose(1, 2).contiguous(), dg.transpose(1, 2).contiguous()
    return dk, dv, dbeta, dg
