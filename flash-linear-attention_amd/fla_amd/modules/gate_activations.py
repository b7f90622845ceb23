"""Gate pre-activations of the layers that call the chunk operators, as single launches with
backward: ``gla_gate`` (``fla/layers/gla.py:214-217``: ``logsigmoid(x) / normalizer`` with an
optional lower clamp) and ``gdn_gate`` (``fla/layers/gated_deltanet.py:236-237``:
``g = -exp(A_log) * softplus(a + dt_bias)``, ``beta = sigmoid(b)``)."""
from typing import Optional, Tuple

import torch

from .. import _backend as be


def _flat(x: torch.Tensor) -> torch.Tensor:
    return x if x.is_contiguous() else x.contiguous()


def gla_gate_fwd(x: torch.Tensor, normalizer: float = 16.0, clamp_min: Optional[float] = None,
                 output_dtype: Optional[torch.dtype] = torch.float32) -> torch.Tensor:
    """``max(logsigmoid(x) / normalizer, clamp_min)`` in ``output_dtype`` (fp32, or x's own dtype)."""
    be.require_gpu(x)
    x = _flat(x)
    y = torch.empty_like(x, dtype=output_dtype or x.dtype)
    n = x.numel()
    if n % 8:
        raise NotImplementedError("fla_amd gla_gate: the number of elements must be a multiple of 8")
    be.check(be.lib().fla_gate_logsigmoid_fwd(be.ptr(x), be.ptr(y), n, float(normalizer), int(clamp_min is not None),
                                              float(clamp_min or 0.0), be.dt(x), be.dt(y), be.stream_of(x)),
             "fla_gate_logsigmoid_fwd")
    return y


def gla_gate_bwd(x: torch.Tensor, dy: torch.Tensor, normalizer: float = 16.0,
                 clamp_min: Optional[float] = None) -> torch.Tensor:
    """Gradient of :func:`gla_gate_fwd` with respect to ``x`` (in x's dtype)."""
    be.require_gpu(x, dy)
    x, dy = _flat(x), _flat(dy)
    if dy.dtype not in (torch.float32, x.dtype):
        dy = dy.float()
    dx = torch.empty_like(x)
    be.check(be.lib().fla_gate_logsigmoid_bwd(be.ptr(x), be.ptr(dy), be.ptr(dx), x.numel(), float(normalizer),
                                              int(clamp_min is not None), float(clamp_min or 0.0), be.dt(x), be.dt(dy),
                                              be.stream_of(x)), "fla_gate_logsigmoid_bwd")
    return dx


class GLAGateFunction(torch.autograd.Function):

    @staticmethod
    def forward(ctx, x, normalizer, clamp_min, output_dtype):
        ctx.save_for_backward(x)
        ctx.normalizer, ctx.clamp_min = normalizer, clamp_min
        return gla_gate_fwd(x, normalizer, clamp_min, output_dtype)

    @staticmethod
    def backward(ctx, dy):
        x, = ctx.saved_tensors
        return gla_gate_bwd(x, dy, ctx.normalizer, ctx.clamp_min), None, None, None


def gla_gate(x: torch.Tensor, normalizer: float = 16.0, clamp_min: Optional[float] = None,
             output_dtype: Optional[torch.dtype] = torch.float32) -> torch.Tensor:
    """The log forget gate of a GLA layer from the gate projection's output, one launch each way."""
    return GLAGateFunction.apply(x, normalizer, clamp_min, output_dtype)


def gdn_gate_fwd(a, b, A_log, dt_bias) -> Tuple[torch.Tensor, Optional[torch.Tensor]]:
    be.require_gpu(a, A_log)
    a = _flat(a)
    H = a.shape[-1]
    M = a.numel() // H
    if b is not None:
        b = _flat(b).to(a.dtype)
    A_log = A_log.float().contiguous()
    dt_bias = None if dt_bias is None else dt_bias.float().contiguous()
    g = torch.empty_like(a, dtype=torch.float32)
    beta = None if b is None else torch.empty_like(b)
    be.check(be.lib().fla_gdn_gate_fwd(be.ptr(a), be.ptr(b), be.ptr(A_log), be.ptr(dt_bias), be.ptr(g), be.ptr(beta),
                                       M, H, be.dt(a), be.dt(a), be.stream_of(a)), "fla_gdn_gate_fwd")
    return g, beta


def gdn_gate_bwd(a, b, A_log, dt_bias, dg, dbeta):
    """Returns ``(da, db, dA_log, ddt_bias)``; the parameter gradients are fp32 ``[H]``."""
    be.require_gpu(a, dg)
    a = _flat(a)
    H = a.shape[-1]
    M = a.numel() // H
    A_log = A_log.float().contiguous()
    dt_bias = None if dt_bias is None else dt_bias.float().contiguous()
    dg = _flat(dg).float()
    if b is not None:
        b = _flat(b).to(a.dtype)
        dbeta = torch.zeros_like(b) if dbeta is None else _flat(dbeta).to(a.dtype)
    da = torch.empty_like(a)
    db = None if b is None else torch.empty_like(b)
    P = be.lib().fla_gdn_gate_workgroups(M, H)
    part = a.new_empty(P, 2, H, dtype=torch.float32)
    be.check(be.lib().fla_gdn_gate_bwd(be.ptr(a), be.ptr(b), be.ptr(A_log), be.ptr(dt_bias), be.ptr(dg),
                                       be.ptr(dbeta if b is not None else None), be.ptr(da), be.ptr(db), be.ptr(part),
                                       M, H, be.dt(a), be.dt(a), be.stream_of(a)), "fla_gdn_gate_bwd")
    sums = part.sum(0)
    return da, db, sums[0], (None if dt_bias is None else sums[1])


class GDNGateFunction(torch.autograd.Function):

    @staticmethod
    def forward(ctx, a, b, A_log, dt_bias):
        g, beta = gdn_gate_fwd(a, b, A_log, dt_bias)
        ctx.save_for_backward(a, b, A_log, dt_bias)
        return g, beta

    @staticmethod
    def backward(ctx, dg, dbeta):
        a, b, A_log, dt_bias = ctx.saved_tensors
        if dg is None:
            dg = torch.zeros_like(a, dtype=torch.float32)
        da, db, dA, dbias = gdn_gate_bwd(a, b, A_log, dt_bias, dg, dbeta)
        return da, db, dA.to(A_log.dtype), (None if dt_bias is None else dbias.to(dt_bias.dtype))


def gdn_gate(a: torch.Tensor, b: Optional[torch.Tensor], A_log: torch.Tensor,
             dt_bias: Optional[torch.Tensor] = None) -> Tuple[torch.Tensor, Optional[torch.Tensor]]:
    """``(g, beta)`` of a gated DeltaNet layer from the outputs of its ``a`` / ``b`` projections ``[..., H]``
    and the per-head parameters ``A_log``, ``dt_bias`` ``[H]``: ``g`` fp32, ``beta`` in b's dtype."""
    return GDNGateFunction.apply(a, b, A_log, dt_bias)
