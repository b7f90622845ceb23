"""Token-by-token (naive) recurrences: the golden reference of the path.

All functions take seq-first tensors ``[B, T, H, D]`` (``[1, T_total, H, D]``
plus ``offsets`` for packed variable-length batches), compute in the dtype
given by ``dtype`` (fp32 by default, fp64 for gradient checks) on whatever
device the inputs live on, and are differentiable by ``torch.autograd``.

* ``naive_recurrent_gla`` follows the recurrence of ``naive_recurrent_gla``
  (``fla/ops/gla/naive.py:22-37``): ``h <- h * exp(gk)[:, None] + k v^T``,
  ``o = (scale * q)^T h``.  The reference is head-first and hard-codes
  ``scale = K ** -0.5`` (``naive.py:24``); here the layout is seq-first and the
  scale is an argument with the same default.  The optional ``g`` (one scalar
  per head) and ``gv`` (per value channel) gates and ``reverse`` follow the
  recurrent kernel (``fla/ops/common/fused_recurrent.py:98-114``).
* ``naive_recurrent_gated_delta_rule`` follows ``recurrent_gated_delta_rule_ref``
  (``tests/ops/test_gated_delta.py:57-66``): decay the state, read the old
  value for ``k``, write ``beta * (v - old)``, then read with ``q``.  ``beta``
  may be ``[B, T, H]`` or per value channel ``[B, T, H, V]``
  (``fla/ops/gated_delta_rule/fused_recurrent.py:89-93``).

Test infrastructure only.
"""
from typing import Optional, Sequence, Tuple

import torch


def _spans(B: int, T: int, offsets: Optional[Sequence[int]]):
    if offsets is None:
        return [(b, 0, T) for b in range(B)]
    assert B == 1, "packed batches have batch size 1"
    offs = [int(x) for x in offsets]
    return [(0, offs[i], offs[i + 1]) for i in range(len(offs) - 1)]


def naive_recurrent_gla(
    q: torch.Tensor, k: torch.Tensor, v: torch.Tensor,
    gk: Optional[torch.Tensor] = None,
    scale: Optional[float] = None,
    initial_state: Optional[torch.Tensor] = None,
    output_final_state: bool = False,
    offsets: Optional[Sequence[int]] = None,
    g: Optional[torch.Tensor] = None,
    gv: Optional[torch.Tensor] = None,
    reverse: bool = False,
    dtype: torch.dtype = torch.float32,
) -> Tuple[torch.Tensor, Optional[torch.Tensor]]:
    cast = (lambda x: None if x is None else x.to(dtype))
    q, k, v, gk, g, gv = map(cast, (q, k, v, gk, g, gv))
    B, T, H, K = k.shape
    V = v.shape[-1]
    if scale is None:
        scale = K ** -0.5
    spans = _spans(B, T, offsets)
    o = torch.zeros(B, T, H, V, dtype=dtype, device=q.device)
    finals = []
    for n, (b, bos, eos) in enumerate(spans):
        h = torch.zeros(H, K, V, dtype=dtype, device=q.device)
        if initial_state is not None:
            h = h + initial_state[n].to(dtype)
        steps = range(eos - 1, bos - 1, -1) if reverse else range(bos, eos)
        outs = {}
        for t in steps:
            if gk is not None:
                h = h * gk[b, t].exp()[:, :, None]
            if gv is not None:
                h = h * gv[b, t].exp()[:, None, :]
            if g is not None:
                h = h * g[b, t].exp()[:, None, None]
            h = h + k[b, t][:, :, None] * v[b, t][:, None, :]
            outs[t] = torch.einsum('hk,hkv->hv', q[b, t] * scale, h)
        if eos > bos:
            o[b, bos:eos] = torch.stack([outs[t] for t in range(bos, eos)], 0)
        finals.append(h)
    ht = torch.stack(finals, 0) if output_final_state else None
    return o, ht


def naive_recurrent_gated_delta_rule(
    q: torch.Tensor, k: torch.Tensor, v: torch.Tensor,
    g: Optional[torch.Tensor], beta: Optional[torch.Tensor],
    scale: Optional[float] = None,
    initial_state: Optional[torch.Tensor] = None,
    output_final_state: bool = False,
    offsets: Optional[Sequence[int]] = None,
    dtype: torch.dtype = torch.float32,
) -> Tuple[torch.Tensor, Optional[torch.Tensor]]:
    cast = (lambda x: None if x is None else x.to(dtype))
    q, k, v, g, beta = map(cast, (q, k, v, g, beta))
    B, T, H, K = k.shape
    V = v.shape[-1]
    if scale is None:
        scale = K ** -0.5
    spans = _spans(B, T, offsets)
    o = torch.zeros(B, T, H, V, dtype=dtype, device=q.device)
    finals = []
    for n, (b, bos, eos) in enumerate(spans):
        S = torch.zeros(H, K, V, dtype=dtype, device=q.device)
        if initial_state is not None:
            S = S + initial_state[n].to(dtype)
        outs = []
        for t in range(bos, eos):
            if g is not None:
                S = S * g[b, t].exp()[:, None, None]
            old = torch.einsum('hk,hkv->hv', k[b, t], S)
            delta = v[b, t] - old
            if beta is not None:
                bt = beta[b, t]
                delta = delta * (bt[:, None] if bt.dim() == 1 else bt)
            S = S + k[b, t][:, :, None] * delta[:, None, :]
            outs.append(torch.einsum('hk,hkv->hv', q[b, t] * scale, S))
        if eos > bos:
            o[b, bos:eos] = torch.stack(outs, 0)
        finals.append(S)
    ht = torch.stack(finals, 0) if output_final_state else None
    return o, ht
