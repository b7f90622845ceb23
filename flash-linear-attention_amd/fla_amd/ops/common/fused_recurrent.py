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

    @staticmethod
    @contiguous
    @autocast_custom_fwd
    def forward(ctx, q, k, v, g=None, gk=None, gv=None, scale=None, initial_state=None,
                output_final_state=False, reverse=False, offsets=None, head_first=True, inplace_state=False):
        o, ht = fused_recurrent_fwd(q, k, v, g, gk, gv, scale, initial_state, output_final_state, reverse,
                                    offsets, head_first, inplace_state)
        return o.to(q.dtype), ht

    @staticmethod
    @contiguous
    @autocast_custom_bwd
    def backward(ctx, do, dht):
        raise NotImplementedError(
            "fla_amd: the backward of the token-by-token recurrence is not built; "
            "use the chunked operators (chunk_gla, chunk_gated_delta_rule) for training.")


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
