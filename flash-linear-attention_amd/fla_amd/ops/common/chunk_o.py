"""``chunk_fwd_o`` for scalar-gated models (``fla/ops/common/chunk_o.py:444-495``),
served by ``fla_chunk_fwd_o``."""
from typing import Optional

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
    ``g`` is the fp32 chunk-local cumsum ``[B,T,H]`` or ``None``."""
    if head_first or chunk_size != BT:
        raise NotImplementedError("fla_amd chunk_fwd_o: seq-first, chunk size 64 only")
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
