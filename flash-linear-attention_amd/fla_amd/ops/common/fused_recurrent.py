"""``fused_recurrent`` (``fla/ops/common/fused_recurrent.py:545-574``): the
token-by-token recurrence with optional scalar / per-key / per-value log-gates,
served by ``fla_fused_recurrent_fwd`` and ``fla_fused_recurrent_bwd``."""
from typing import Optional, Tuple

import torch

from ... import _backend as be
from ...utils import autocast_custom_bwd, autocast_custom_fwd, contiguous


def fused_recurrent_fwd(q, k, v, g=None, gk=None, gv=None, scale=None, initial_state=None,
                        output_final_state=False, reverse=False, offsets=None, head_first=True,
                        inplace_state=False, o_dtype=None):
    be.require_gpu(q, k, v)
    if head_first:
        tr = (lambda x: None if x is None else x.transpose(1, 2).contiguous())
        o, ht = fused_recurrent_fwd(tr(q), tr(k), tr(v), tr(g), tr(gk), tr(gv), scale, initial_state,
                                    output_final_state, reverse, offsets, False, inplace_state, o_dtype)
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
    o = torch.empty_like(v, dtype=o_dtype or qkv_dtype)  # fp32 accumulation, rounded once on store
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


def _gate_dtype(gates, qkv_dtype):
    gates = [x for x in gates if x is not None]
    if not gates:
        return None
    gdt = gates[0].dtype
    if any(x.dtype != gdt for x in gates) or gdt not in (torch.float32, qkv_dtype):
        gdt = torch.float32
    return gdt


def _per_token(term, B, T, offsets):
    """A per-sequence tensor [N, ...] repeated over the tokens of its sequence: [B, T, ...]."""
    if offsets is None:
        return term.unsqueeze(1)
    lens = offsets[1:] - offsets[:-1]
    ids = torch.repeat_interleave(torch.arange(lens.numel(), device=term.device), lens, output_size=T)
    return term[ids].unsqueeze(0)


def fused_recurrent_bwd(q, k, v, g=None, gk=None, gv=None, o=None, do=None, dht=None, scale=None,
                        initial_state=None, reverse=False, offsets=None, head_first=True, ht=None):
    """Gradients of the recurrence (``fla/ops/common/fused_recurrent.py:381-468``): a token-by-token
    kernel for dq, dk, dv, dh0 (fp32 arithmetic) and whole-sequence reverse cumulative sums for the
    gates.  Returns ``(dq, dk, dv, dg, dgk, dgv, dh0)`` in fp32.  With ``dht`` and gates the final state
    ``ht`` of the forward pass is needed as well: the last cumulative gate also scales the final state,
    which adds ``sum(dht * ht)`` over the ungated dims to every token's gate gradient (the reference
    leaves that term out and refuses the combination, ``:518-525``)."""
    from ..utils.cumsum import chunk_global_cumsum
    be.require_gpu(q, k, v, do)
    if head_first:
        tr = (lambda x: None if x is None else x.transpose(1, 2).contiguous())
        outs = fused_recurrent_bwd(tr(q), tr(k), tr(v), tr(g), tr(gk), tr(gv), tr(o), tr(do), dht, scale,
                                   initial_state, reverse, offsets, False, ht)
        return tuple(None if x is None else x.transpose(1, 2) for x in outs[:6]) + (outs[6],)
    B, T, H, K = k.shape
    V = v.shape[-1]
    N = B if offsets is None else len(offsets) - 1
    if K > 256 or V % 4:
        raise NotImplementedError("fla_amd fused_recurrent backward: K <= 256 and V a multiple of 4")
    qkv_dtype = q.dtype
    q, k, v, do = q.contiguous(), k.to(qkv_dtype).contiguous(), v.to(qkv_dtype).contiguous(), do.to(qkv_dtype).contiguous()
    gdt = _gate_dtype((g, gk, gv), qkv_dtype)
    gg, ggk, ggv = (None if x is None else x.to(gdt).contiguous() for x in (g, gk, gv))
    h0 = None if initial_state is None else initial_state.float().contiguous()
    dht_ = None if dht is None else dht.float().contiguous()
    if offsets is not None:
        offsets = offsets.to(torch.int64).contiguous()
    NV = -(-V // 64)
    dq = q.new_empty(NV, B, T, H, K, dtype=torch.float32)
    dk = q.new_empty(NV, B, T, H, K, dtype=torch.float32)
    dv = q.new_empty(B, T, H, V, dtype=torch.float32)
    dh0 = q.new_empty(N, H, K, V, dtype=torch.float32) if initial_state is not None else None
    be.check(be.lib().fla_fused_recurrent_bwd(
        be.ptr(q), be.ptr(k), be.ptr(v), be.ptr(gg), be.ptr(ggk), be.ptr(ggv), be.ptr(h0), be.ptr(do), be.ptr(dht_),
        be.ptr(dq), be.ptr(dk), be.ptr(dv), be.ptr(dh0), be.ptr(offsets), be.dt(q),
        be.FLA_F32 if gdt is None else be._DTYPES[gdt], B, T, H, K, V, N, float(scale), int(bool(reverse)),
        be.stream_of(q)), "fla_fused_recurrent_bwd")
    dq, dk = (dq[0] if NV == 1 else dq.sum(0)), (dk[0] if NV == 1 else dk.sum(0))
    dg = dgk = dgv = None
    if g is not None or gk is not None:
        dgk_all = chunk_global_cumsum(dq * q.float() - dk * k.float(), reverse=not reverse, offsets=offsets,
                                      head_first=False)
        if dht is not None and ht is not None:
            dgk_all = dgk_all + _per_token((dht_ * ht.float()).sum(-1), B, T, offsets)
        if gk is not None:
            dgk = dgk_all
        if g is not None:
            dg = dgk_all.sum(-1)
    if gv is not None:
        dgv = chunk_global_cumsum(do.float() * o.float() - dv * v.float(), reverse=not reverse, offsets=offsets,
                                  head_first=False)
        if dht is not None and ht is not None:
            dgv = dgv + _per_token((dht_ * ht.float()).sum(-2), B, T, offsets)
    return dq, dk, dv, dg, dgk, dgv, dh0


class FusedRecurrentFunction(torch.autograd.Function):
    """Forward and backward are the token-by-token kernels, in fp32 arithmetic whatever the storage type
    (``fla/ops/common/fused_recurrent.py:471-542``)."""

    @staticmethod
    @contiguous
    @autocast_custom_fwd
    def forward(ctx, q, k, v, g=None, gk=None, gv=None, scale=None, initial_state=None,
                output_final_state=False, reverse=False, offsets=None, head_first=True, inplace_state=False):
        # ctx.needs_input_grad, not the tensors' own flags: the wrapper above may have handed over contiguous
        # copies made under no_grad
        nig = ctx.needs_input_grad
        needs_grad = any(nig[:6]) or nig[7]
        if needs_grad and inplace_state:
            raise ValueError("inplace_state=True overwrites the initial state the backward needs")
        gates_grad = any(nig[3:6])
        gv_grad = gv is not None and nig[5]
        # the gate gradients read the unrounded output (gv) and the final state (a gradient of the final state)
        o, ht = fused_recurrent_fwd(q, k, v, g, gk, gv, scale, initial_state, output_final_state or gates_grad,
                                    reverse, offsets, head_first, inplace_state,
                                    o_dtype=torch.float32 if gv_grad else None)
        if needs_grad:
            ctx.save_for_backward(q, k, v, g, gk, gv, initial_state, offsets,
                                  o if gv_grad else None, ht if gates_grad else None)
            ctx.scale, ctx.reverse, ctx.head_first = scale, reverse, head_first
        return o.to(q.dtype), (ht if output_final_state else None)

    @staticmethod
    @contiguous
    @autocast_custom_bwd
    def backward(ctx, do, dht):
        q, k, v, g, gk, gv, h0, offsets, o, ht = ctx.saved_tensors
        dq, dk, dv, dg, dgk, dgv, dh0 = fused_recurrent_bwd(
            q, k, v, g, gk, gv, o, do, dht, ctx.scale, h0, ctx.reverse, offsets, ctx.head_first, ht=ht)
        cast = lambda x, like: None if (x is None or like is None) else x.to(like.dtype)
        return (cast(dq, q), cast(dk, k), cast(dv, v), cast(dg, g), cast(dgk, gk), cast(dgv, gv), None,
                cast(dh0, h0), None, None, None, None, None)


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
