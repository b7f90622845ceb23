"""``chunk_fwd_h`` / ``chunk_bwd_dh`` with the reference's arguments
(``fla/ops/common/chunk_h.py:282-335``, ``:338-410``), served by ``fla_chunk_gla_fwd_h`` and
``fla_chunk_bwd_dh``.

The kernels carry the decay on the key axis.  Decay on the value axis (``gv``, what GSA passes,
``fla/ops/gsa/chunk.py:664-675, 794-820``) is the transposed problem: with ``h' = h^T`` the update
``h <- h diag(e^{gv_last}) + k^T (v e^{gv_last - gv})`` reads ``h' <- diag(e^{gv_last}) h' + (v e^{gv_last - gv})^T k``,
i.e. the same launch with k and v (q and do for the reverse scan) exchanged, whose states are transposed
back afterwards.
"""
from typing import Optional, Tuple

import torch
import torch.nn.functional as F

from ... import _backend as be
from ...utils import prepare_chunk_offsets

BT = 64


def _round64(d: int) -> int:
    return -(-d // 64) * 64


def _pad_last(x: Optional[torch.Tensor], size: int) -> Optional[torch.Tensor]:
    if x is None or x.shape[-1] == size:
        return x
    return F.pad(x, (0, size - x.shape[-1]))


def _pad_state(m: Optional[torch.Tensor], Kp: int, Vp: int) -> Optional[torch.Tensor]:
    if m is None or tuple(m.shape[-2:]) == (Kp, Vp):
        return m
    return F.pad(m, (0, Vp - m.shape[-1], 0, Kp - m.shape[-2]))


def _seq_first(x: Optional[torch.Tensor], head_first: bool) -> Optional[torch.Tensor]:
    if x is None or not head_first:
        return x
    return x.transpose(1, 2)


def _check_chunk_size(T: int, chunk_size: int, offsets) -> None:
    """The kernels walk chunks of 64.  The reference's chunk length ``min(chunk_size, max(16, npow2(T)))``
    (``fla/ops/common/chunk_h.py:300``) is shorter for T <= 32, where a batch of equal-length sequences is a single
    chunk either way (the one stored state is the initial state, the final state is the same)."""
    bt = min(chunk_size, max(16, 1 << (max(T, 1) - 1).bit_length()))
    if bt == BT or (offsets is None and T <= bt):
        return
    raise NotImplementedError("fla_amd chunk_fwd_h / chunk_bwd_dh: the kernels are built for chunks of 64 tokens")


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
    """Per-chunk states ``h`` (the state entering each chunk; ``[B,NT,H,K,V]``, ``[B,H,NT,K,V]`` if ``head_first``)
    and the final state.  ``g`` ``[B,T,H]``, ``gk`` ``[B,T,H,K]``, ``gv`` ``[B,T,H,V]`` are chunk-local cumulative
    log-gates, as in the reference, unless ``gates_are_cumsum=False`` (raw ``gk``; the prefix sum is formed in the
    kernel).  ``fragment_layout=True`` stores ``h`` in the MFMA-fragment order the library's own pipelines read
    (seq-first, head dims that are multiples of 64, no ``gv``)."""
    if gv is not None:
        if gk is not None or g is not None:
            raise NotImplementedError("fla_amd chunk_fwd_h: gv together with g / gk is not covered")
        if fragment_layout or not gates_are_cumsum:
            raise NotImplementedError("fla_amd chunk_fwd_h: gv takes the reference's layout and cumulative gates")
        hT, htT = chunk_fwd_h(k=v, v=k, g=None, gk=gv, gv=None, h0=None if h0 is None else h0.transpose(-1, -2),
                              output_final_state=output_final_state, offsets=offsets, indices=indices,
                              head_first=head_first, chunk_size=chunk_size, states_in_fp32=states_in_fp32,
                              chunk_offsets=chunk_offsets, store_states=store_states)
        return (None if hT is None else hT.transpose(-1, -2).contiguous(),
                None if htT is None else htT.transpose(-1, -2).contiguous())
    k, v, g, gk = (_seq_first(x, head_first) for x in (k, v, g, gk))
    if g is not None:
        # per-head gates run on the per-key kernel: the same log-gate on every key channel
        # (what chunk_simple_gla does at the operator level), added to gk when both are given
        gb = g.float().unsqueeze(-1).expand(*g.shape, k.shape[-1])
        gk = gb if gk is None else gk.float() + gb
    if gk is None:
        raise NotImplementedError("fla_amd chunk_fwd_h: g, gk or gv is required")
    be.require_gpu(k, v, gk)
    B, T, H, K = k.shape
    V = v.shape[-1]
    _check_chunk_size(T, chunk_size, offsets)
    Kp, Vp = _round64(K), _round64(V)
    if fragment_layout and (head_first or (Kp, Vp) != (K, V)):
        raise NotImplementedError("fla_amd chunk_fwd_h: fragment-order states are seq-first with head dims that are "
                                  "multiples of 64")
    if k.dtype not in (torch.bfloat16, torch.float16):
        raise NotImplementedError("fla_amd chunk_fwd_h: k and v must be bf16 or fp16")
    k, gk = _pad_last(k, Kp).contiguous(), _pad_last(gk, Kp).contiguous()
    v = _pad_last(v.to(k.dtype), Vp).contiguous()
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
    h = k.new_empty(B, NT, H, Kp, Vp, dtype=h_dtype) if store_states else None
    ht = k.new_empty(N, H, Kp, Vp, dtype=torch.float32) if output_final_state else None
    if h0 is not None:
        h0 = _pad_state(h0 if h0.dtype == torch.float32 else h0.float(), Kp, Vp).contiguous()
    if gates_are_cumsum and gk.dtype != torch.float32:
        gk = gk.float()
    be.check(be.lib().fla_chunk_gla_fwd_h(
        be.ptr(k), be.ptr(v), be.ptr(gk), int(gates_are_cumsum), be.ptr(h0), be.ptr(h), be.ptr(ht),
        be.ptr(offsets), be.ptr(chunk_offsets), be.dt(k), be.dt(gk), be._DTYPES[h_dtype],
        (be.FLA_H_FRAGMENT_T if transposed_fragments else be.FLA_H_FRAGMENT) if fragment_layout
        else be.FLA_H_ROW_MAJOR,
        B, T, H, Kp, Vp, N, be.stream_of(k)), "fla_chunk_gla_fwd_h")
    if (Kp, Vp) != (K, V):
        h = None if h is None else h[..., :K, :V]
        ht = None if ht is None else ht[..., :K, :V].contiguous()
    if head_first and h is not None:
        h = h.transpose(1, 2)
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
    """Reverse state scan with the reference's arguments (``fla/ops/common/chunk_h.py:338-410``): ``dh`` row-major
    (``[B,NT,HQ,K,V]``, ``[B,HQ,NT,K,V]`` if ``head_first``), the gradient w.r.t. the state leaving every chunk, and
    ``dh0`` (returned when ``h0`` is given, as in the reference).  ``g`` ``[B,T,H]``, ``gk`` ``[B,T,H,K]`` and ``gv``
    ``[B,T,H,V]`` are chunk-cumulative log-gates.  ``q`` and ``do`` may carry ``HQ = NG * H`` heads (grouped queries,
    ``:156-188``): query head ``hq`` decays with the gates of head ``hq // NG`` and has a state gradient of its own.
    ``chunk_gla``'s own backward does not come through here (its scan keeps ``dh`` in fragment order)."""
    if gv is not None:
        if gk is not None or g is not None:
            raise NotImplementedError("fla_amd chunk_bwd_dh: gv together with g / gk is not covered")
        # the transposed problem: dh^T <- diag(e^{gv_last}) dh^T + (do e^{gv})^T (scale q)
        dhT, dh0T = chunk_bwd_dh(q=do, k=v, v=k, g=None, gk=gv, gv=None, do=q,
                                 h0=None if h0 is None else h0.transpose(-1, -2),
                                 dht=None if dht is None else dht.transpose(-1, -2), scale=scale, offsets=offsets,
                                 indices=indices, head_first=head_first, chunk_size=chunk_size,
                                 states_in_fp32=states_in_fp32)
        return dhT.transpose(-1, -2).contiguous(), (None if dh0T is None else dh0T.transpose(-1, -2).contiguous())
    q, k, v, do, g, gk = (_seq_first(x, head_first) for x in (q, k, v, do, g, gk))
    if q.dtype not in (torch.bfloat16, torch.float16) or do.dtype != q.dtype:
        raise NotImplementedError("fla_amd chunk_bwd_dh: q and do must both be bf16 or fp16")
    be.require_gpu(q, do)
    B, T, H, K = k.shape
    V = v.shape[-1]
    HQ = q.shape[2]
    _check_chunk_size(T, chunk_size, offsets)
    if HQ != H:
        if HQ % H or do.shape[2] != HQ:
            raise ValueError(f"chunk_bwd_dh: {HQ} query heads do not group over {H} key/value heads")
        # every query head of a group reads its group's gates
        NG = HQ // H
        g = None if g is None else g.repeat_interleave(NG, dim=2)
        gk = None if gk is None else gk.repeat_interleave(NG, dim=2)
    Kp, Vp = _round64(K), _round64(V)
    qp = _pad_last(q, Kp).contiguous()
    dop = _pad_last(do, Vp).contiguous()
    gp = None if g is None else g.float().contiguous()
    gkp = None if gk is None else _pad_last(gk.float(), Kp).contiguous()
    chunk_offsets = None
    if offsets is None:
        N, NT = B, -(-T // BT)
    else:
        offsets = offsets.to(torch.int64).contiguous()
        chunk_offsets = prepare_chunk_offsets(offsets, BT, device=k.device)
        N = len(offsets) - 1
        NT = int(indices.shape[0]) if indices is not None else int(prepare_chunk_offsets(offsets, BT)[-1])
    dhtp = None if dht is None else _pad_state(dht.float(), Kp, Vp).contiguous()
    dh_dtype = torch.float32 if states_in_fp32 else k.dtype
    dh = k.new_empty(B, NT, HQ, Kp, Vp, dtype=dh_dtype)
    dh0 = k.new_empty(N, HQ, Kp, Vp, dtype=torch.float32) if h0 is not None else None
    be.check(be.lib().fla_chunk_bwd_dh(
        be.ptr(qp), be.ptr(gp), be.ptr(gkp), be.ptr(dop), be.ptr(dhtp), be.ptr(dh), be.ptr(dh0),
        be.ptr(offsets), be.ptr(chunk_offsets), be.dt(qp), be._DTYPES[dh_dtype], B, T, HQ, Kp, Vp, N, float(scale),
        be.stream_of(q)), "fla_chunk_bwd_dh")
    if (Kp, Vp) != (K, V):
        dh = dh[..., :K, :V]
        dh0 = None if dh0 is None else dh0[..., :K, :V]
    if dh0 is not None and HQ != H:
        # the query heads of a group read one state: its gradient is the sum over the group, shaped like h0
        dh0 = dh0.reshape(N, H, HQ // H, K, V).sum(2)
    if head_first:
        dh = dh.transpose(1, 2)
    return dh, dh0
