"""Short causal depthwise convolution over time, channels last
(mirror of fla/modules/convolution.py:79-211; no external causal_conv1d package needed)."""
from typing import Optional, Tuple

import torch
import torch.nn as nn
import torch.nn.functional as F

from .. import _backend as be


def _act_flag(activation: Optional[str]) -> int:
    if activation is None:
        return 0
    if activation in ("silu", "swish"):
        return 1
    raise ValueError(f"Activation `{activation}` not supported yet.")


class CausalConv1dFunction(torch.autograd.Function):

    @staticmethod
    def forward(ctx, x, weight, bias, activation):
        be.require_gpu(x)
        x = x.contiguous()
        B, T, D = x.shape
        W = weight.shape[-1]
        if D % 8 or not 2 <= W <= 4:
            raise NotImplementedError(f"fla_amd causal_conv1d: needs channels % 8 == 0 and 2 <= kernel <= 4, got {D}, {W}")
        w32 = weight.detach().reshape(D, W).float().contiguous()
        b32 = None if bias is None else bias.detach().float().contiguous()
        y = torch.empty_like(x)
        silu = _act_flag(activation)
        if x.numel():
            be.check(be.lib().fla_causal_conv1d_fwd(be.ptr(x), be.ptr(w32), be.ptr(b32), be.ptr(y), B, T, D, W, silu,
                                                    be.dt(x), be.stream_of(x)), "fla_causal_conv1d_fwd")
        ctx.save_for_backward(x, w32, b32)
        ctx.silu, ctx.w_shape, ctx.w_dtype = silu, weight.shape, weight.dtype
        ctx.b_dtype = None if bias is None else bias.dtype
        return y

    @staticmethod
    def backward(ctx, dy):
        x, w32, b32 = ctx.saved_tensors
        B, T, D = x.shape
        W = w32.shape[-1]
        dy = dy.to(x.dtype).contiguous()
        dx = torch.empty_like(x)
        parts = be.lib().fla_causal_conv1d_bwd_partials(B, T)
        dw = torch.empty(parts, D, W, dtype=torch.float32, device=x.device)
        db = None if b32 is None else torch.empty(parts, D, dtype=torch.float32, device=x.device)
        if x.numel():
            be.check(be.lib().fla_causal_conv1d_bwd(be.ptr(x), be.ptr(w32), be.ptr(b32), be.ptr(dy), be.ptr(dx),
                                                    be.ptr(dw), be.ptr(db), B, T, D, W, ctx.silu, be.dt(x),
                                                    be.stream_of(x)), "fla_causal_conv1d_bwd")
        return (dx, dw.sum(0).reshape(ctx.w_shape).to(ctx.w_dtype),
                None if db is None else db.sum(0).to(ctx.b_dtype), None)


def causal_conv1d(x: torch.Tensor, weight: torch.Tensor, bias: Optional[torch.Tensor] = None,
                  activation: Optional[str] = None) -> torch.Tensor:
    """``x`` [B,T,D], ``weight`` [D,W] (or the ``nn.Conv1d`` layout [D,1,W]) -> [B,T,D]."""
    return CausalConv1dFunction.apply(x, weight, bias, activation)


def causal_conv1d_update(x: torch.Tensor, cache: torch.Tensor, weight: torch.Tensor,
                         bias: Optional[torch.Tensor] = None, activation: Optional[str] = None) -> torch.Tensor:
    """Single-token step: ``x`` [B,D]; ``cache`` [B,D,W] is shifted and updated in place."""
    be.require_gpu(x, cache)
    B, D = x.shape
    W = weight.shape[-1]
    if not 2 <= W <= 4:
        raise NotImplementedError(f"fla_amd causal_conv1d_update: kernel size {W} not in 2..4")
    assert cache.shape == (B, D, W) and cache.is_contiguous() and cache.dtype == x.dtype
    x = x.contiguous()
    w32 = weight.detach().reshape(D, W).float().contiguous()
    b32 = None if bias is None else bias.detach().float().contiguous()
    y = torch.empty_like(x)
    be.check(be.lib().fla_causal_conv1d_update(be.ptr(x), be.ptr(cache), be.ptr(w32), be.ptr(b32), be.ptr(y), B, D, W,
                                               _act_flag(activation), be.dt(x), be.stream_of(x)),
             "fla_causal_conv1d_update")
    return y


class ShortConvolution(nn.Conv1d):
    """Same constructor, parameters (``weight`` [D,1,W]) and ``forward`` contract as the
    reference's module (fla/modules/convolution.py:79-211).  ``use_fast_conv1d`` is accepted
    and ignored: the HIP kernels are the only path."""

    def __init__(self, hidden_size: int, kernel_size: int, bias: bool = False, activation: Optional[str] = 'silu',
                 use_fast_conv1d: Optional[bool] = True):
        super().__init__(in_channels=hidden_size, out_channels=hidden_size, kernel_size=kernel_size,
                         groups=hidden_size, bias=bias, padding=kernel_size - 1)
        self.hidden_size = hidden_size
        self.activation = None
        if activation is not None:
            assert activation in ['silu', 'swish'], f"Activation `{activation}` not supported yet."
            self.activation = activation
        self.use_fast_conv1d = use_fast_conv1d

    def forward(self, x: torch.Tensor, mask: Optional[torch.Tensor] = None, cache: Optional[torch.Tensor] = None,
                output_final_state: bool = False) -> Tuple[torch.Tensor, torch.Tensor]:
        """``x`` [B,T,D]; ``cache`` [B,D,W] is updated in place; returns ``(y [B,T,D], cache)``."""
        batch_size, _, hidden_size = x.shape
        if mask is not None:
            x = x.mul_(mask.unsqueeze(-1))
        if output_final_state and cache is None:
            cache = x.new_zeros(batch_size, hidden_size, self.kernel_size[0])
        if cache is not None and x.shape[1] == 1:
            return self.step(x, cache)
        if cache is not None:
            cache.copy_(F.pad(x.transpose(1, 2), (self.kernel_size[0] - x.shape[1], 0)))
        y = causal_conv1d(x, self.weight, self.bias, self.activation)
        return y, cache

    def step(self, x: torch.Tensor, cache: torch.Tensor):
        assert x.shape[1] == 1, "Only support decoding with 1 token at a time for now"
        y = causal_conv1d_update(x.squeeze(1), cache, self.weight, self.bias, self.activation)
        return y.unsqueeze(1), cache

    @property
    def state_size(self) -> int:
        return self.hidden_size * self.kernel_size[0]
