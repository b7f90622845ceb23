"""Norm + swish output gate, ``y = norm(x) * weight (+ bias) * o * sigmoid(o)``
(mirror of fla/modules/fused_norm_gate.py:400-505 and the modules at :680-760)."""
from __future__ import annotations

import torch
import torch.nn as nn

from .. import _backend as be


def _rows(x: torch.Tensor) -> torch.Tensor:
    x2 = x.reshape(-1, x.shape[-1])
    return x2 if x2.is_contiguous() else x2.contiguous()


def _f32(t):
    return None if t is None else t.detach().float().contiguous()


def norm_gate_fwd(x, o, weight, bias, eps, is_rms_norm):
    """Rows of ``x``/``o`` [M,N] -> ``(y, mean, rstd)`` (fla/modules/fused_norm_gate.py:186-256)."""
    be.require_gpu(x, o)
    M, N = x.shape
    if N % 8 or N > 2048:
        raise NotImplementedError(f"fla_amd norm gate: last dimension {N} must be a multiple of 8 and at most 2048")
    o = o.to(x.dtype)
    y = torch.empty_like(x)
    mean = None if is_rms_norm else torch.empty(M, dtype=torch.float32, device=x.device)
    rstd = torch.empty(M, dtype=torch.float32, device=x.device)
    if M == 0:
        return y, mean, rstd
    be.check(be.lib().fla_norm_swish_gate_fwd(be.ptr(x), be.ptr(o), be.ptr(_f32(weight)), be.ptr(_f32(bias)), be.ptr(y),
                                              be.ptr(mean), be.ptr(rstd), M, N, float(eps), int(is_rms_norm), be.dt(x),
                                              be.stream_of(x)), "fla_norm_swish_gate_fwd")
    return y, mean, rstd


def norm_gate_bwd(dy, x, o, weight, bias, eps, mean, rstd, is_rms_norm):
    """``(dx, do, dw, db)`` (fla/modules/fused_norm_gate.py:333-397)."""
    M, N = x.shape
    dy = dy.to(x.dtype).contiguous()
    dx, do = torch.empty_like(x), torch.empty_like(x)
    if M == 0:
        zw = None if weight is None else torch.zeros_like(weight)
        zb = None if bias is None else torch.zeros_like(bias)
        return dx, do, zw, zb
    nwg = be.lib().fla_norm_swish_gate_workgroups(M, N)
    dwp = torch.empty(nwg, N, dtype=torch.float32, device=x.device) if weight is not None else None
    dbp = torch.empty(nwg, N, dtype=torch.float32, device=x.device) if bias is not None else None
    be.check(be.lib().fla_norm_swish_gate_bwd(be.ptr(dy), be.ptr(x), be.ptr(o), be.ptr(_f32(weight)), be.ptr(_f32(bias)),
                                              be.ptr(mean), be.ptr(rstd), be.ptr(dx), be.ptr(do), be.ptr(dwp), be.ptr(dbp),
                                              M, N, float(eps), int(is_rms_norm), be.dt(x), be.stream_of(x)),
             "fla_norm_swish_gate_bwd")
    dw = None if dwp is None else dwp.sum(0).to(weight.dtype)
    db = None if dbp is None else dbp.sum(0).to(bias.dtype)
    return dx, do, dw, db


class LayerNormSwishGateFn(torch.autograd.Function):
    """Same argument list as the reference's function (fla/modules/fused_norm_gate.py:400-480).
    The residual / prenorm variants are not covered."""

    @staticmethod
    def forward(ctx, x, o, weight, bias, residual=None, eps=1e-6, prenorm=False, residual_in_fp32=False,
                is_rms_norm=False):
        if residual is not None or prenorm or residual_in_fp32:
            raise NotImplementedError("fla_amd norm gate: residual / prenorm variants are not covered")
        shape = x.shape
        x2, o2 = _rows(x), _rows(o).to(x.dtype)
        y, mean, rstd = norm_gate_fwd(x2, o2, weight, bias, eps, is_rms_norm)
        ctx.save_for_backward(x2, o2, weight, bias, mean, rstd)
        ctx.shape, ctx.o_shape, ctx.o_dtype, ctx.eps, ctx.is_rms_norm = shape, o.shape, o.dtype, eps, is_rms_norm
        return y.reshape(shape)

    @staticmethod
    def backward(ctx, dy, *args):
        x, o, weight, bias, mean, rstd = ctx.saved_tensors
        dx, do, dw, db = norm_gate_bwd(_rows(dy), x, o, weight, bias, ctx.eps, mean, rstd, ctx.is_rms_norm)
        return (dx.reshape(ctx.shape), do.reshape(ctx.o_shape).to(ctx.o_dtype), dw, db, None, None, None, None, None)


def layer_norm_swish_gate_fn(x, o, weight, bias, residual=None, prenorm=False, residual_in_fp32=False, eps=1e-6):
    return LayerNormSwishGateFn.apply(x, o, weight, bias, residual, eps, prenorm, residual_in_fp32, False)


def rms_norm_swish_gate_fn(x, o, weight, bias, residual=None, prenorm=False, residual_in_fp32=False, eps=1e-6):
    return LayerNormSwishGateFn.apply(x, o, weight, bias, residual, eps, prenorm, residual_in_fp32, True)


class _NormSwishGate(nn.Module):
    _fn = None

    def __init__(self, hidden_size, elementwise_affine: bool = True, eps=1e-5):
        super().__init__()
        self.hidden_size = hidden_size
        self.elementwise_affine = elementwise_affine
        self.eps = eps
        if elementwise_affine:
            self.weight = nn.Parameter(torch.ones(hidden_size))
        else:
            self.register_parameter("weight", None)
        self.register_parameter("bias", None)

    def __repr__(self) -> str:
        s = f"{self.__class__.__name__}({self.hidden_size}"
        if not self.elementwise_affine:
            s += f", elementwise_affine={self.elementwise_affine}"
        return s + f", eps={self.eps})"

    def forward(self, x, o, residual=None, prenorm=False, residual_in_fp32=False):
        return type(self)._fn(x, o, self.weight, self.bias, residual=residual, eps=self.eps, prenorm=prenorm,
                              residual_in_fp32=residual_in_fp32)


class FusedLayerNormSwishGate(_NormSwishGate):
    """fla/modules/fused_norm_gate.py:680-722."""
    _fn = staticmethod(layer_norm_swish_gate_fn)


class FusedRMSNormSwishGate(_NormSwishGate):
    """fla/modules/fused_norm_gate.py:725-767."""
    _fn = staticmethod(rms_norm_swish_gate_fn)
