"""``chunk_fwd_h`` for per-key log-gates (``fla/ops/common/chunk_h.py:282-335``),
served by ``fla_chunk_gla_fwd_h``."""
from typing import Optional, Tuple

import torch

from ... import _backend as be
from ...utils import prepare_chunk_offsets

BT = 64


def chunk_fwd_h(
    k: torch.Tensor,
    v: torch.Tensor,
    g: Optional[torch.Tensor],
    gk: Optional[torch.Tensor],
    gv: Optional[torch.Tensor],
    h0: Optional[torch.Tensor],
    output_final_state: bool,
    offsets: Optional[torch.Tensor] = None,
    indices: Optional[torch.Tensor] = None,
    head_first: bool = True,
    chunk_size: int = 64,
    states_in_fp32: bool = False,
    *,
    gates_are_cumsum: bool = True,
    fragment_layout: bool = False,
    transposed_fragments: bool = False,
    chunk_offsets: Optional[torch.Tensor] = None,
    store_states: bool = True,
) -> Tuple[Optional[torch.Tensor], Optional[torch.Tensor]]:
    """Per-chunk states ``h`` ``[B,NT,H,K,V]`` (the state entering each chunk)
    and the final state.  ``gk`` is the chunk-local cumsum of the log-gates, as
    in the reference, unless ``gates_are_cumsum=False`` (raw gates; the prefix
    sum is formed in the kernel).  ``fragment_layout=True`` stores ``h`` in the
    MFMA-fragment order only ``fla_chunk_gla_fwd_o`` understands."""
    if gv is not None:
        raise NotImplementedError("fla_amd chunk_fwd_h: value gates (gv) are not covered")
    if g is not None:
        # per-head gates run on the per-key kernel: the same log-gate on every key channel
        # (what chunk_simple_gla does at the operator level), added to gk when both are given
        gb = g.float().unsqueeze(-1).expand(*g.shape, k.shape[-1])
        gk = gb.contiguous() if gk is None else gk.float() + gb
    if gk is None:
        raise NotImplementedError("fla_amd chunk_fwd_h: g or gk is required")
    if head_first:
        raise NotImplementedError("fla_amd chunk_fwd_h: seq-first layout only (transpose at the operator boundary)")
    if chunk_size != BT:
        raise NotImplementedError("fla_amd chunk_fwd_h: chunk size is fixed to 64")
    be.require_gpu(k, v, gk)
    B, T, H, K = k.shape
    V = v.shape[-1]
    if offsets is None:
        N, NT = B, -(-T // BT)
    else:
        if chunk_offsets is None:
            chunk_offsets = prepare_chunk_offsets(offsets, BT, device=k.device)
        N = len(offsets) - 1
        NT = int(indices.shape[0]) if indices is not None else int(prepare_chunk_offsets(offsets, BT)[-1])
        offsets = offsets.to(torch.int64).contiguous()
    h_dtype = torch.float32 if states_in_fp32 else k.dtype
    if fragment_layout and states_in_fp32:
        raise ValueError("fragment-layout states are 16-bit")
    h = k.new_empty(B, NT, H, K, V, dtype=h_dtype) if store_states else None
    ht = k.new_empty(N, H, K, V, dtype=torch.float32) if output_final_state else None
    if h0 is not None:
        h0 = (h0 if h0.dtype == torch.float32 else h0.float()).contiguous()
    if gates_are_cumsum and gk.dtype != torch.float32:
        gk = gk.float()
    be.check(be.lib().fla_chunk_gla_fwd_h(
        be.ptr(k), be.ptr(v), be.ptr(gk), int(gates_are_cumsum), be.ptr(h0), be.ptr(h), be.ptr(ht),
        be.ptr(offsets), be.ptr(chunk_offsets), be.dt(k), be.dt(gk), be._DTYPES[h_dtype],
        (be.FLA_H_FRAGMENT_T if transposed_fragments else be.FLA_H_FRAGMENT) if fragment_layout
        else be.FLA_H_ROW_MAJOR,
        B, T, H, K, V, N, be.stream_of(k)), "fla_chunk_gla_fwd_h")
    return h, ht


def chunk_bwd_dh(
    q: torch.Tensor,
    k: torch.Tensor,
    v: torch.Tensor,
    g: Optional[torch.Tensor],
    gk: Optional[torch.Tensor],
    gv: Optional[torch.Tensor],
    do: torch.Tensor,
    h0: Optional[torch.Tensor],
    dht: Optional[torch.Tensor],
    scale: float,
    offsets: Optional[torch.Tensor] = None,
    indices: Optional[torch.Tensor] = None,
    head_first: bool = True,
    chunk_size: int = 64,
    states_in_fp32: bool = False,
) -> Tuple[torch.Tensor, Optional[torch.Tensor]]:
    """Reverse state scan with the reference's arguments (``fla/ops/common/chunk_h.py:338-410``):
    ``dh`` ``[B,NT,H,K,V]`` row-major, the gradient w.r.t. the state leaving every chunk, and ``dh0``
    (returned when ``h0`` is given, as in the reference).  ``g`` ``[B,T,H]`` and ``gk`` ``[B,T,H,K]`` are
    chunk-cumulative log-gates; value gates (``gv``) and grouped query heads are not covered.
    ``chunk_gla``'s own backward does not come through here (its scan keeps ``dh`` in fragment order)."""
    if gv is not None:
        raise NotImplementedError("fla_amd chunk_bwd_dh: value gates (gv) are not covered")
    if chunk_size != BT:
        raise NotImplementedError("fla_amd chunk_bwd_dh: chunk size is fixed to 64")
    if head_first:
        q, k, v, do = (x.transpose(1, 2).contiguous() for x in (q, k, v, do))
        g = None if g is None else g.transpose(1, 2).contiguous()
        gk = None if gk is None else gk.transpose(1, 2).contiguous()
    if q.shape[2] != k.shape[2]:
        raise NotImplementedError("fla_amd chunk_bwd_dh: q must have as many heads as k")
    if q.dtype not in (torch.bfloat16, torch.float16) or do.dtype != q.dtype:
        raise NotImplementedError("fla_amd chunk_bwd_dh: q and do must both be bf16 or fp16")
    be.require_gpu(q, do)
    B, T, H, K = k.shape
    V = v.shape[-1]
    Kp, Vp = -(-K // 64) * 64, -(-V // 64) * 64
    pad = torch.nn.functional.pad
    qp = (q if Kp == K else pad(q, (0, Kp - K))).contiguous()
    dop = (do if Vp == V else pad(do, (0, Vp - V))).contiguous()
    gp = None if g is None else g.float().contiguous()
    gkp = None if gk is None else (gk.float() if Kp == K else pad(gk.float(), (0, Kp - K))).contiguous()
    chunk_offsets = None
    if offsets is None:
        N, NT = B, -(-T // BT)
    else:
        offsets = offsets.to(torch.int64).contiguous()
        chunk_offsets = prepare_chunk_offsets(offsets, BT, device=k.device)
        N = len(offsets) - 1
        NT = int(indices.shape[0]) if indices is not None else int(prepare_chunk_offsets(offsets, BT)[-1])
    dhtp = None
    if dht is not None:
        dhtp = dht.float()
        if (Kp, Vp) != (K, V):
            dhtp = pad(dhtp, (0, Vp - V, 0, Kp - K))
        dhtp = dhtp.contiguous()
    dh_dtype = torch.float32 if states_in_fp32 else k.dtype
    dh = k.new_empty(B, NT, H, Kp, Vp, dtype=dh_dtype)
    dh0 = k.new_empty(N, H, Kp, Vp, dtype=torch.float32) if h0 is not None else None
    be.check(be.lib().fla_chunk_bwd_dh(
        be.ptr(qp), be.ptr(gp), be.ptr(gkp), be.ptr(dop), be.ptr(dhtp), be.ptr(dh), be.ptr(dh0),
        be.ptr(offsets), be.ptr(chunk_offsets), be.dt(qp), be._DTYPES[dh_dtype], B, T, H, Kp, Vp, N, float(scale),
        be.stream_of(q)), "fla_chunk_bwd_dh")
    if (Kp, Vp) != (K, V):
        dh = dh[..., :K, :V]
        dh0 = None if dh0 is None else dh0[..., :K, :V]
    if head_first:
        dh = dh.transpose(1, 2)
    return dh, dh0
