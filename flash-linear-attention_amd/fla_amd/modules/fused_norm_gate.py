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


def norm_gate_fwd(x, o, weight, bias, eps, is_rms_norm, residual=None, residual_dtype=None):
    """Rows of ``x``/``o`` [M,N] -> ``(y, mean, rstd, residual_out)`` (fla/modules/fused_norm_gate.py:103-180).

    With ``residual`` the normalised row is ``x + residual``; that sum is returned as ``residual_out`` (in the
    residual's dtype), as it is when ``residual_dtype`` differs from ``x.dtype``; otherwise ``residual_out`` is ``x``."""
    be.require_gpu(x, o)
    M, N = x.shape
    if N % 8 or N > 2048:
        raise NotImplementedError(f"fla_amd norm gate: last dimension {N} must be a multiple of 8 and at most 2048")
    o = o.to(x.dtype)
    if residual is not None:
        assert residual.shape == (M, N)
        residual_dtype = residual.dtype
        if residual_dtype not in (x.dtype, torch.float32):
            raise NotImplementedError("fla_amd norm gate: the residual is in x's dtype or in fp32")
        residual = residual.contiguous()
    y = torch.empty_like(x)
    keep = residual is not None or (residual_dtype is not None and residual_dtype != x.dtype)
    residual_out = torch.empty(M, N, dtype=residual_dtype, device=x.device) if keep else None
    mean = None if is_rms_norm else torch.empty(M, dtype=torch.float32, device=x.device)
    rstd = torch.empty(M, dtype=torch.float32, device=x.device)
    if M == 0:
        return y, mean, rstd, residual_out if keep else x
    be.check(be.lib().fla_norm_swish_gate_residual_fwd(
        be.ptr(x), be.ptr(o), be.ptr(_f32(weight)), be.ptr(_f32(bias)), be.ptr(residual),
        be.dt(residual) if residual is not None else be.dt(x), be.ptr(y), be.ptr(residual_out),
        be.dt(residual_out) if keep else be.dt(x), be.ptr(mean), be.ptr(rstd), M, N, float(eps), int(is_rms_norm),
        be.dt(x), be.stream_of(x)), "fla_norm_swish_gate_residual_fwd")
    return y, mean, rstd, residual_out if keep else x


def norm_gate_bwd(dy, x, o, weight, bias, eps, mean, rstd, is_rms_norm, dresidual=None, has_residual=False,
                  x_dtype=None):
    """``(dx, do, dw, db, dresidual_in)`` (fla/modules/fused_norm_gate.py:301-400); ``x`` is what the forward
    normalised (its ``residual_out``), ``x_dtype`` the dtype of the forward's ``x`` (and of ``dx``, ``do``)."""
    M, N = x.shape
    x_dtype = x.dtype if x_dtype is None else x_dtype
    dy = dy.to(x_dtype).contiguous()
    dx = torch.empty(M, N, dtype=x_dtype, device=x.device)
    do = torch.empty(M, N, dtype=x_dtype, device=x.device)
    dresidual_in = torch.empty_like(x) if has_residual and dx.dtype != x.dtype else None
    if dresidual is not None:
        dresidual = dresidual.to(x.dtype).contiguous()
    if M == 0:
        zw = None if weight is None else torch.zeros_like(weight)
        zb = None if bias is None else torch.zeros_like(bias)
        return dx, do, zw, zb, (dx if has_residual and dresidual_in is None else dresidual_in)
    nwg = be.lib().fla_norm_swish_gate_workgroups(M, N)
    dwp = torch.empty(nwg, N, dtype=torch.float32, device=x.device) if weight is not None else None
    dbp = torch.empty(nwg, N, dtype=torch.float32, device=x.device) if bias is not None else None
    be.check(be.lib().fla_norm_swish_gate_residual_bwd(
        be.ptr(dy), be.ptr(x), be.dt(x), be.ptr(o), be.ptr(_f32(weight)), be.ptr(_f32(bias)), be.ptr(mean),
        be.ptr(rstd), be.ptr(dresidual), be.ptr(dx), be.ptr(do), be.ptr(dresidual_in), be.ptr(dwp), be.ptr(dbp), M, N,
        float(eps), int(is_rms_norm), be.dt(dx), be.stream_of(x)), "fla_norm_swish_gate_residual_bwd")
    dw = None if dwp is None else dwp.sum(0).to(weight.dtype)
    db = None if dbp is None else dbp.sum(0).to(bias.dtype)
    if has_residual and dresidual_in is None:
        dresidual_in = dx
    return dx, do, dw, db, dresidual_in


class LayerNormSwishGateFn(torch.autograd.Function):
    """Same argument list and return values as the reference's function (fla/modules/fused_norm_gate.py:402-481),
    residual / prenorm variants included."""

    @staticmethod
    def forward(ctx, x, o, weight, bias, residual=None, eps=1e-6, prenorm=False, residual_in_fp32=False,
                is_rms_norm=False):
        shape = x.shape
        x2, o2 = _rows(x), _rows(o).to(x.dtype)
        if residual is not None:
            assert residual.shape == shape
            residual = _rows(residual)
        residual_dtype = residual.dtype if residual is not None else (torch.float32 if residual_in_fp32 else None)
        y, mean, rstd, residual_out = norm_gate_fwd(x2, o2, weight, bias, eps, is_rms_norm, residual, residual_dtype)
        ctx.save_for_backward(residual_out, o2, weight, bias, mean, rstd)
        ctx.shape, ctx.o_shape, ctx.o_dtype, ctx.eps, ctx.is_rms_norm = shape, o.shape, o.dtype, eps, is_rms_norm
        ctx.has_residual, ctx.prenorm, ctx.x_dtype = residual is not None, prenorm, x.dtype
        y = y.reshape(shape)
        return y if not prenorm else (y, residual_out.reshape(shape))

    @staticmethod
    def backward(ctx, dy, *args):
        x, o, weight, bias, mean, rstd = ctx.saved_tensors
        dresidual = _rows(args[0]) if ctx.prenorm else None
        dx, do, dw, db, dres_in = norm_gate_bwd(_rows(dy), x, o, weight, bias, ctx.eps, mean, rstd, ctx.is_rms_norm,
                                                dresidual, ctx.has_residual, ctx.x_dtype)
        return (dx.reshape(ctx.shape), do.reshape(ctx.o_shape).to(ctx.o_dtype), dw, db,
                dres_in.reshape(ctx.shape) if ctx.has_residual else None, None, None, None, None)


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
