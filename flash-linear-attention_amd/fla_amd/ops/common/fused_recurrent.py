"""``fused_recurrent`` (``fla/ops/common/fused_recurrent.py:545-574``): the
token-by-token recurrence with optional scalar / per-key / per-value log-gates,
served by ``fla_fused_recurrent_fwd``."""
from typing import Optional, Tuple

import torch

from ... import _backend as be
from ...utils import autocast_custom_bwd, autocast_custom_fwd, contiguous


def fused_recurrent_fwd(q, k, v, g=None, gk=None, gv=None, scale=None, initial_state=None,
                        output_final_state=False, reverse=False, offsets=None, head_first=True,
                        inplace_state=False):
    be.require_gpu(q, k, v)
    if head_first:
        tr = (lambda x: None if x is None else x.transpose(1, 2).contiguous())
        o, ht = fused_recurrent_fwd(tr(q), tr(k), tr(v), tr(g), tr(gk), tr(gv), scale, initial_state,
                                    output_final_state, reverse, offsets, False, inplace_state)
        return o.transpose(1, 2).contiguous(), ht
    B, T, H, K = k.shape
    V = v.shape[-1]
    N = B if offsets is None else len(offsets) - 1
    if K > 256:
        raise NotImplementedError("fla_amd fused_recurrent: key head dims above 256 are not covered")
    qkv_dtype = q.dtype
    k, v = k.to(qkv_dtype), v.to(qkv_dtype)
    gates = [x for x in (g, gk, gv) if x is not None]
    gdt = None
    if gates:
        gdt = gates[0].dtype
        if any(x.dtype != gdt for x in gates) or gdt not in (torch.float32, qkv_dtype):
            gdt = torch.float32
        g, gk, gv = (None if x is None else x.to(gdt) for x in (g, gk, gv))
    if V % 4:
        raise NotImplementedError("fla_amd fused_recurrent: value head dim must be a multiple of 4")
    h0 = None
    if initial_state is not None:
        h0 = initial_state if initial_state.dtype == torch.float32 else initial_state.float()
        h0 = h0.contiguous()
    ht = None
    if output_final_state:
        if inplace_state:
            if h0 is None or h0.data_ptr() != initial_state.data_ptr():
                raise ValueError("inplace_state=True needs a contiguous fp32 initial_state to update")
            ht = h0
        else:
            ht = q.new_empty(N, H, K, V, dtype=torch.float32)
    o = torch.empty_like(v, dtype=qkv_dtype)  # fp32 accumulation, rounded once on store
    if offsets is not None:
        offsets = offsets.to(torch.int64).contiguous()
    gate_code = be.FLA_F32 if gdt is None else be._DTYPES[gdt]
    q, k, v = q.contiguous(), k.contiguous(), v.contiguous()
    g, gk, gv = (None if x is None else x.contiguous() for x in (g, gk, gv))
    be.check(be.lib().fla_fused_recurrent_fwd(
        be.ptr(q), be.ptr(k), be.ptr(v), be.ptr(g), be.ptr(gk), be.ptr(gv), be.ptr(o), be.ptr(h0), be.ptr(ht),
        be.ptr(offsets), be.dt(q), gate_code, be.dt(o), B, T, H, K, V, N, float(scale), int(bool(reverse)),
        be.stream_of(q)), "fla_fused_recurrent_fwd")
    return o, ht


class FusedRecurrentFunction(torch.autograd.Function):
    """Forward: the token-by-token kernel.  Backward: the recurrence equals the chunked operator on
    the same inputs, so the gradients come from ``chunk_gla``'s backward kernels (the reference runs
    a second token-by-token pass, ``fla/ops/common/fused_recurrent.py:381-468``, and a global
    reverse cumsum for the gates, ``:462-467``)."""

    @staticmethod
    @contiguous
    @autocast_custom_fwd
    def forward(ctx, q, k, v, g=None, gk=None, gv=None, scale=None, initial_state=None,
                output_final_state=False, reverse=False, offsets=None, head_first=True, inplace_state=False):
        o, ht = fused_recurrent_fwd(q, k, v, g, gk, gv, scale, initial_state, output_final_state, reverse,
                                    offsets, head_first, inplace_state)
        if any(t is not None and t.requires_grad for t in (q, k, v, g, gk, gv, initial_state)):
            if inplace_state:
                raise ValueError("inplace_state=True overwrites the initial state the backward needs")
            ctx.save_for_backward(q, k, v, g, gk, gv, initial_state, offsets)
            ctx.scale, ctx.reverse, ctx.head_first = scale, reverse, head_first
        return o.to(q.dtype), ht

    @staticmethod
    @contiguous
    @autocast_custom_bwd
    def backward(ctx, do, dht):
        import warnings

        from ..gla.chunk import chunk_gla
        q, k, v, g, gk, gv, h0, offsets = ctx.saved_tensors
        if gv is not None or ctx.reverse:
            raise NotImplementedError("fla_amd fused_recurrent backward: value gates (gv) and reverse=True are not covered")
        leaves = [None if t is None else t.detach().requires_grad_() for t in (q, k, v, g, gk, h0)]
        ql, kl, vl, gl, gkl, h0l = leaves
        with torch.enable_grad(), warnings.catch_warnings():
            warnings.simplefilter("ignore")
            # one per-key log-gate: gk, plus the per-head scalar g broadcast over the key channels
            gate = gkl.float() if gkl is not None else None
            if gl is not None:
                gs = gl.float().unsqueeze(-1).expand(*kl.shape)
                gate = gs if gate is None else gate + gs
            if gate is None:
                gate = torch.zeros(kl.shape, dtype=torch.float32, device=kl.device)
            o, ht = chunk_gla(ql, kl, vl, gate.contiguous(), scale=ctx.scale, initial_state=h0l, output_final_state=True,
                              offsets=offsets, head_first=ctx.head_first)
            outs, grads = [o], [do.to(o.dtype)]
            if dht is not None:
                outs.append(ht)
                grads.append(dht.to(ht.dtype))
            torch.autograd.backward(outs, grads)
        dq, dk, dv, dg, dgk, dh0 = (None if t is None else t.grad for t in leaves)
        return dq, dk, dv, dg, dgk, None, None, dh0, None, None, None, None, None


def fused_recurrent(
    q: torch.Tensor,
    k: torch.Tensor,
    v: torch.Tensor,
    g: Optional[torch.Tensor] = None,
    gk: Optional[torch.Tensor] = None,
    gv: Optional[torch.Tensor] = None,
    scale: Optional[float] = None,
    initial_state: Optional[torch.Tensor] = None,
    output_final_state: bool = False,
    reverse: bool = False,
    offsets: Optional[torch.LongTensor] = None,
    head_first: bool = True,
    inplace_state: bool = False,
) -> Tuple[torch.Tensor, Optional[torch.Tensor]]:
    if scale is None:
        scale = k.shape[-1] ** -0.5
    return FusedRecurrentFunction.apply(q, k, v, g, gk, gv, scale, initial_state, output_final_state,
                                        reverse, offsets, head_first, inplace_state)
