"""Row-wise steps either side of the chunk operators in the layers, restated in plain torch
(fp32 by default, fp64 on request) and differentiable by ``torch.autograd``.

* ``l2norm`` follows ``l2norm_fwd_kernel`` (``fla/modules/l2norm.py:18-40``):
  ``y = x / sqrt(sum(x^2, -1) + eps)`` -- eps inside the square root, no mean.
* ``norm_swish_gate`` follows ``layer_norm_fwd_kernel`` of the gated norms
  (``fla/modules/fused_norm_gate.py:144-183``): ``xhat = (x - mean) * rstd`` with
  ``rstd = 1/sqrt(mean(xbar^2) + eps)`` (``mean = 0`` for RMS norm), ``y = xhat * w + b``,
  output ``y * o * sigmoid(o)``.
* ``causal_conv1d`` follows ``ShortConvolution.forward`` without the external package
  (``fla/modules/convolution.py:183-186``): depthwise ``nn.Conv1d`` with left padding
  ``W - 1``, cropped to ``T``, then SiLU; ``causal_conv1d_step`` follows ``step``
  (``:203-210``): roll the cache left, write ``x`` last, ``sum(cache * w) + b``, SiLU.

* ``gla_gate`` follows ``fla/layers/gla.py:214-217`` (``logsigmoid(x) / normalizer``, then an optional
  ``clamp_min``); ``gdn_gate`` follows ``fla/layers/gated_deltanet.py:236-237``
  (``g = -exp(A_log) * softplus(a + dt_bias)`` in fp32, ``beta = sigmoid(b)``).  Both are written from
  the defining formulas (``log(1 / (1 + e^{-x}))``, ``log(1 + e^{x})``) in a numerically stable form and
  pinned against ``torch.nn.functional.logsigmoid`` / ``softplus`` / ``sigmoid``.

Pinned by tests/test_oracle_modules.py: unit norm and scale invariance of ``l2norm``;
``norm_swish_gate`` against ``torch.nn.functional.layer_norm`` / ``rms_norm`` times
``silu``; ``causal_conv1d`` against ``torch.nn.functional.conv1d``, causality, and the
step against the full convolution.

Test infrastructure only.
"""
from typing import Optional

import torch
import torch.nn.functional as F


def l2norm(x: torch.Tensor, eps: float = 1e-6, dtype=torch.float32) -> torch.Tensor:
    x = x.to(dtype)
    return x / torch.sqrt((x * x).sum(-1, keepdim=True) + eps)


def norm_swish_gate(x, o, weight=None, bias=None, eps: float = 1e-5, is_rms_norm: bool = True, dtype=torch.float32,
                    residual=None, prenorm: bool = False):
    """``norm(x + residual) * weight + bias`` times ``o * sigmoid(o)``; with ``prenorm`` also the sum that was
    normalised (fla/modules/fused_norm_gate.py:68-74, :446)."""
    x, o = x.to(dtype), o.to(dtype)
    if residual is not None:
        x = x + residual.to(dtype)
    pre = x
    if not is_rms_norm:
        x = x - x.mean(-1, keepdim=True)
    rstd = 1.0 / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)
    y = x * rstd
    if weight is not None:
        y = y * weight.to(dtype)
    if bias is not None:
        y = y + bias.to(dtype)
    y = y * o * torch.sigmoid(o)
    return (y, pre) if prenorm else y


def causal_conv1d(x, weight, bias=None, activation: Optional[str] = None, dtype=torch.float32):
    """``x`` [B,T,D], ``weight`` [D,W]: ``y[b,t,d] = act(bias[d] + sum_i weight[d,i] x[b,t-(W-1)+i,d])``."""
    x, weight = x.to(dtype), weight.to(dtype)
    B, T, D = x.shape
    W = weight.shape[-1]
    xp = torch.cat([x.new_zeros(B, W - 1, D), x], dim=1)
    y = sum(xp[:, i:i + T] * weight[:, i] for i in range(W))
    if bias is not None:
        y = y + bias.to(dtype)
    if activation in ("silu", "swish"):
        y = y * torch.sigmoid(y)
    return y


def causal_conv1d_step(x, cache, weight, bias=None, activation: Optional[str] = None, dtype=torch.float32):
    """``x`` [B,D], ``cache`` [B,D,W] -> ``(y [B,D], new cache)``; nothing is modified in place."""
    cache = torch.cat([cache[..., 1:].to(dtype), x.to(dtype).unsqueeze(-1)], dim=-1)
    y = (cache * weight.to(dtype)).sum(-1)
    if bias is not None:
        y = y + bias.to(dtype)
    if activation in ("silu", "swish"):
        y = y * torch.sigmoid(y)
    return y, cache


def gla_gate(x, normalizer: float = 16.0, clamp_min: Optional[float] = None, dtype=torch.float32):
    """``log sigmoid(x) / normalizer`` with ``log sigmoid(x) = min(x, 0) - log(1 + e^{-|x|})``, clamped from below."""
    x = x.to(dtype)
    y = (torch.minimum(x, torch.zeros_like(x)) - torch.log1p(torch.exp(-x.abs()))) / normalizer
    if clamp_min is not None:
        y = torch.clamp(y, min=clamp_min)
    return y


def gdn_gate(a, b, A_log, dt_bias=None, dtype=torch.float32):
    """``(g, beta)``: ``g = -e^{A_log} * log(1 + e^{a + dt_bias})`` (the argument itself above 20, where the two
    agree to fp32 precision), ``beta = 1 / (1 + e^{-b})``."""
    x = a.to(dtype)
    if dt_bias is not None:
        x = x + dt_bias.to(dtype)
    sp = torch.where(x > 20, x, torch.log1p(torch.exp(torch.clamp(x, max=20))))
    g = -torch.exp(A_log.to(dtype)) * sp
    beta = None if b is None else 1.0 / (1.0 + torch.exp(-b.to(dtype)))
    return g, beta
