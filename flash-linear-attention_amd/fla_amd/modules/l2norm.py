"""l2 normalisation over the last dimension (mirror of fla/modules/l2norm.py:91-199)."""
from typing import Optional

import torch

from .. import _backend as be


def _rows(x: torch.Tensor) -> torch.Tensor:
    x2 = x.reshape(-1, x.shape[-1])
    return x2 if x2.is_contiguous() else x2.contiguous()


def l2norm_fwd(x: torch.Tensor, eps: float = 1e-6, output_dtype: Optional[torch.dtype] = None) -> torch.Tensor:
    """``y = x / sqrt(sum(x^2, -1) + eps)`` (fla/modules/l2norm.py:91-132)."""
    be.require_gpu(x)
    shape = x.shape
    x2 = _rows(x)
    M, N = x2.shape
    if N % 8 or N > 2048:
        raise NotImplementedError(f"fla_amd l2norm: last dimension {N} must be a multiple of 8 and at most 2048")
    y = torch.empty_like(x2, dtype=output_dtype or x.dtype)
    if M == 0:
        return y.reshape(shape)
    be.check(be.lib().fla_l2norm_fwd(be.ptr(x2), be.ptr(y), M, N, float(eps), be.dt(x2), be.dt(y), be.stream_of(x2)),
             "fla_l2norm_fwd")
    return y.reshape(shape)


def l2norm_bwd(x: torch.Tensor, dy: torch.Tensor, eps: float = 1e-6) -> torch.Tensor:
    """``dx = dy*rstd - sum(dy*x)*rstd^3*x`` (fla/modules/l2norm.py:135-166)."""
    be.require_gpu(x, dy)
    shape = x.shape
    x2, dy2 = _rows(x), _rows(dy)
    M, N = x2.shape
    assert dy2.shape == x2.shape
    dx = torch.empty_like(x2)
    if M == 0:
        return dx.reshape(shape)
    be.check(be.lib().fla_l2norm_bwd(be.ptr(x2), be.ptr(dy2), be.ptr(dx), M, N, float(eps), be.dt(x2), be.dt(dy2),
                                     be.stream_of(x2)), "fla_l2norm_bwd")
    return dx.reshape(shape)


class L2NormFunction(torch.autograd.Function):

    @staticmethod
    def forward(ctx, x, eps=1e-6, output_dtype=None):
        y = l2norm_fwd(x, eps, output_dtype)
        ctx.eps = eps
        ctx.save_for_backward(x)
        return y

    @staticmethod
    def backward(ctx, dy, *args):
        x, = ctx.saved_tensors
        return l2norm_bwd(x, dy, ctx.eps), None, None


def l2_norm(x: torch.Tensor, eps: float = 1e-6, output_dtype: Optional[torch.dtype] = None) -> torch.Tensor:
    return L2NormFunction.apply(x, eps, output_dtype)
