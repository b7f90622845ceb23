"""``fused_recurrent_gated_delta_rule`` with the reference's signature
(``fla/ops/gated_delta_rule/fused_recurrent.py:210-315``), served by
``fla_fused_recurrent_gated_delta_rule_fwd``."""
from typing import Optional, Tuple

import torch

from ... import _backend as be
from ...utils import check_varlen_args, contiguous, resolve_offsets

L2NORM_EPS = 1e-6   # the eps of fla.modules.l2norm


def fused_recurrent_gated_delta_rule_fwd(q, k, v, g, beta, scale, initial_state, output_final_state,
                                         offsets=None, head_first=True, inplace_state=False, l2norm_eps=None):
    """``l2norm_eps``: q and k arrive un-normalised and the step normalises the rows it loads
    (``x / sqrt(sum x^2 + eps)``, what ``l2_norm`` in front of the operator computes)."""
    be.require_gpu(q, k, v)
    if head_first:
        tr = (lambda x: None if x is None else x.transpose(1, 2).contiguous())
        o, ht = fused_recurrent_gated_delta_rule_fwd(tr(q), tr(k), tr(v), tr(g), tr(beta), scale, initial_state,
                                                     output_final_state, offsets, False, inplace_state, l2norm_eps)
        return o.transpose(1, 2).contiguous(), ht
    B, T, H, K = k.shape
    V = v.shape[-1]
    N = B if offsets is None else len(offsets) - 1
    if K > 256:
        raise NotImplementedError("fla_amd fused_recurrent_gated_delta_rule: key head dims above 256 are not covered")
    if V % 4:
        raise NotImplementedError("fla_amd fused_recurrent_gated_delta_rule: value head dim must be a multiple of 4")
    k, v = k.to(q.dtype), v.to(q.dtype)
    # per-head scalars are tiny: always hand them over in fp32
    g = None if g is None else g.float().contiguous()
    beta_per_value = int(beta is not None and beta.dim() == v.dim())
    beta = None if beta is None else beta.float().contiguous()
    h0 = None
    if initial_state is not None:
        h0 = (initial_state if initial_state.dtype == torch.float32 else initial_state.float()).contiguous()
    ht = None
    if output_final_state:
        if inplace_state:
            if h0 is None or h0.data_ptr() != initial_state.data_ptr():
                raise ValueError("inplace_state=True needs a contiguous fp32 initial_state to update")
            ht = h0
        else:
            ht = q.new_empty(N, H, K, V, dtype=torch.float32)
    o = torch.empty_like(v)  # the reference returns o in q's dtype (q.new_empty, :133)
    if offsets is not None:
        offsets = offsets.to(torch.int64).contiguous()
    q, k, v = q.contiguous(), k.contiguous(), v.contiguous()
    if l2norm_eps is not None:
        be.check(be.lib().fla_fused_recurrent_gated_delta_rule_fwd_l2norm(
            be.ptr(q), be.ptr(k), be.ptr(v), be.ptr(g), be.ptr(beta), be.ptr(o), be.ptr(h0), be.ptr(ht),
            be.ptr(offsets), be.dt(q), be.FLA_F32, be.dt(o), beta_per_value, B, T, H, K, V, N, float(scale),
            float(l2norm_eps), be.stream_of(q)), "fla_fused_recurrent_gated_delta_rule_fwd_l2norm")
        return o, ht
    be.check(be.lib().fla_fused_recurrent_gated_delta_rule_fwd(
        be.ptr(q), be.ptr(k), be.ptr(v), be.ptr(g), be.ptr(beta), be.ptr(o), be.ptr(h0), be.ptr(ht),
        be.ptr(offsets), be.dt(q), be.FLA_F32, be.dt(o), beta_per_value, B, T, H, K, V, N, float(scale),
        be.stream_of(q)), "fla_fused_recurrent_gated_delta_rule_fwd")
    return o, ht


class FusedRecurrentFunction(torch.autograd.Function):

    @staticmethod
    @contiguous
    def forward(ctx, q, k, v, g, beta, scale, initial_state, output_final_state, offsets=None, head_first=True,
                inplace_state=False, l2norm_eps=None):
        return fused_recurrent_gated_delta_rule_fwd(q, k, v, g, beta, scale, initial_state, output_final_state,
                                                    offsets, head_first, inplace_state, l2norm_eps)

    @staticmethod
    @contiguous
    def backward(ctx, do, dht):
        # same behaviour as the reference (fused_recurrent.py:203-208)
        raise NotImplementedError("Backward pass is not implemented yet and we do not have plans to implement it "
                                  "because we haven't figured out how to compute dg without materializing the full "
                                  "hidden states for all time steps.")


def fused_recurrent_gated_delta_rule(
    q: torch.Tensor,
    k: torch.Tensor,
    v: torch.Tensor,
    g: torch.Tensor,
    beta: torch.Tensor = None,
    scale: float = None,
    initial_state: torch.Tensor = None,
    output_final_state: bool = False,
    offsets: Optional[torch.LongTensor] = None,
    head_first: bool = True,
    cu_seqlens: Optional[torch.LongTensor] = None,
    inplace_state: bool = False,
    use_qk_l2norm_in_kernel: bool = False,
) -> Tuple[torch.Tensor, Optional[torch.Tensor]]:
    r"""
    Args mirror the reference: q, k ``[B,H,T,K]`` (``[B,T,H,K]`` if not
    ``head_first``), v ``[.., V]``, ``g`` and ``beta`` ``[B,H,T]`` / ``[B,T,H]``
    (``beta`` may also be per value channel, or ``None`` meaning 1), ``scale``
    (default ``K ** -0.5``, must be positive), ``initial_state`` ``[N,H,K,V]``.

    Extensions: ``cu_seqlens`` (synonym of ``offsets``), ``inplace_state``
    (final state written over a contiguous fp32 ``initial_state``),
    ``use_qk_l2norm_in_kernel`` (q and k arrive raw and are l2-normalised by the step itself,
    as ``chunk_gated_delta_rule`` offers, ``fla/ops/gated_delta_rule/chunk.py:189-215``: two
    launches fewer per decode step).
    """
    offsets = resolve_offsets(offsets, cu_seqlens)
    check_varlen_args(q, offsets, head_first, initial_state)
    if scale is None:
        scale = k.shape[-1] ** -0.5
    else:
        assert scale > 0, "scale must be positive"
    if beta is None:
        beta = torch.ones_like(q[..., 0])
    l2norm_eps = L2NORM_EPS if use_qk_l2norm_in_kernel else None
    if not (torch.is_grad_enabled() and any(t is not None and t.requires_grad
                                            for t in (q, k, v, g, beta, initial_state))):
        # decode loops: no autograd node to build, and the host time of a step is of the order of its device time
        return fused_recurrent_gated_delta_rule_fwd(q, k, v, g, beta, scale, initial_state, output_final_state,
                                                    offsets, head_first, inplace_state, l2norm_eps)
    return FusedRecurrentFunction.apply(q, k, v, g, beta, scale, initial_state, output_final_state, offsets,
                                        head_first, inplace_state, l2norm_eps)
