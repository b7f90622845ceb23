"""``chunk_gla`` with the reference's signature (``fla/ops/gla/chunk.py:1409-1495``).

Forward on the device (chunk size 64): one launch, ``fla_chunk_gla_fwd_fused`` (prefix sums of the
gates, gated scores, output and state scan in one pass; the per-chunk states stay on the chip;
chunks whose gates left the range of the single-reference-point scores are flagged and their
output rows recomputed exactly by the same launch after its last chunk).  The two-kernel form (``fla_chunk_gla_fwd_h`` ->
``fla_chunk_gla_fwd_o``) serves the reference-shaped internal entry points ``chunk_gla_fwd`` /
``chunk_fwd_h`` / ``chunk_gla_fwd_o_gk``.
"""
import os
import threading
import warnings
from typing import Optional, Tuple

import torch
import torch.nn.functional as F

from ... import _backend as be
from ...utils import VarlenPlan, check_varlen_args, contiguous, empty_batch_result, resolve_offsets
from ..common.chunk_h import chunk_fwd_h
from ..utils.cumsum import chunk_local_cumsum, chunk_local_cumsum_inverse

BT = 64
_SUPPORTED_KV = {(64, 64), (128, 128), (64, 128), (128, 64)}

# A forward pass that will be differentiated has the fused launch write the state entering every
# chunk (one more [K, V] tile in the q/k/v dtype per chunk and head) and keeps it for the backward
# pass, which the reference starts by recomputing those states (fla/ops/gla/chunk.py:1239-1253).
# FLA_AMD_RECOMPUTE_STATES=1 (or setting this flag to False) restores the reference's behaviour.
KEEP_STATES_FOR_BACKWARD = os.environ.get("FLA_AMD_RECOMPUTE_STATES", "0") in ("", "0")
# With the states, a differentiated forward (per-key gates, V <= 128) also keeps k^ = k e^{G_last - G} and the score tile
# of every chunk (1.5 more tensors of k's size), from which the backward's reverse state scan forms dv on its way.
KEEP_KHAT_AND_SCORES = os.environ.get("FLA_AMD_GLA_FUSED_DV", "1") not in ("", "0")
# fp32 q/k/v run through the fp16 chunk kernels, as the reference runs them through its chunk kernels with fp32 operands
# on the matrix pipe at reduced precision (tests/ops/test_gla.py:149-201): q, k and v are divided by a power of two >= their
# largest magnitude (exact; found on the device, no synchronisation) and rounded to fp16, gates and states stay fp32, and
# the results are scaled back.  About 5e-4 relative error - the reference's own fp32 tests allow 4e-3 (:195-201).
# FLA_AMD_FP32_EXACT=1 takes the fp32 token-by-token kernels instead: exact to 1e-4, serial in time (10.5 ms against
# 1.0 ms at B=8, T=4096, H=16, D=128).
FP32_INPUTS_EXACT = os.environ.get("FLA_AMD_FP32_EXACT", "0") not in ("", "0")


def _pow2_scale(x: torch.Tensor) -> torch.Tensor:
    """A power of two >= max|x| as a tensor of one element on x's device (1 for an all-zero tensor); one pass over x."""
    lo, hi = torch.aminmax(x.detach())
    amax = torch.maximum(-lo, hi).float().reshape(1)
    return torch.where(amax > 0, torch.exp2(torch.ceil(torch.log2(amax.clamp_min(1e-37)))), torch.ones_like(amax))


def _scaled_half(x: torch.Tensor, s: torch.Tensor) -> torch.Tensor:
    """x / s rounded to fp16 in one pass (s a power of two: the division is exact)."""
    return torch.mul(x.detach(), 1.0 / s, out=torch.empty_like(x, dtype=torch.float16))


class _ScaledFp16ChunkGla(torch.autograd.Function):
    """fp32 q, k, v through the fp16 chunk kernels with every fp16 tensor - inputs, and in the backward pass the
    cotangent of o - divided by a power of two that brings it to at most 1 (the operator is linear in each of q, k,
    v, and its gradients are linear in the cotangents, so the scales factor out exactly)."""

    @staticmethod
    def forward(ctx, q, k, v, g, initial_state, scale, output_final_state, offsets, head_first):
        sq, sk, sv = _pow2_scale(q), _pow2_scale(k), _pow2_scale(v)
        skv = sk * sv
        need = ctx.needs_input_grad
        with torch.enable_grad():
            leaves = [_scaled_half(q, sq).requires_grad_(need[0]), _scaled_half(k, sk).requires_grad_(need[1]),
                      _scaled_half(v, sv).requires_grad_(need[2]), g.detach().float().requires_grad_(need[3]),
                      None if initial_state is None else (initial_state.detach().float() / skv).requires_grad_(need[4])]
            o_h, ht_h = chunk_gla(leaves[0], leaves[1], leaves[2], leaves[3], scale=scale, initial_state=leaves[4],
                                  output_final_state=output_final_state, offsets=offsets, head_first=head_first)
        ctx.inner = (leaves, o_h, ht_h)
        ctx.scales = (sq, sk, sv)
        ctx.in_dtypes = (g.dtype, None if initial_state is None else initial_state.dtype)
        o = o_h.detach() * (sq * skv)      # (a one-element fp32 tensor promotes the product to fp32)
        ht = None if ht_h is None else ht_h.detach() * skv
        return o, ht

    @staticmethod
    def backward(ctx, do, dht):
        leaves, o_h, ht_h = ctx.inner
        sq, sk, sv = ctx.scales
        skv = sk * sv
        co = do.float() * (sq * skv)
        ch = None if (dht is None or ht_h is None) else dht.float() * skv
        wanted = [i for i, x in enumerate(leaves) if x is not None and x.requires_grad]
        targets = [leaves[i] for i in wanted]
        res = [None] * 5

        def accumulate(grads, c):
            back = (c / sq, c / sk, c / sv, c, c / skv)
            for i, gr in zip(wanted, grads):
                if gr is not None:
                    term = gr.float() * back[i]
                    res[i] = term if res[i] is None else res[i] + term

        # The two cotangents live on unrelated scales (that of o carries q's scale, that of the final state does not),
        # and the gradients are linear in them: one pass each, every pass with its cotangent brought to at most 1.
        c = _pow2_scale(co)
        cots = [(co / c).half()] + ([torch.zeros_like(ht_h)] if ht_h is not None else [])
        outs = [o_h] + ([ht_h] if ht_h is not None else [])
        accumulate(torch.autograd.grad(outs, targets, cots, allow_unused=True, retain_graph=ch is not None), c)
        if ch is not None:
            c = _pow2_scale(ch)
            accumulate(torch.autograd.grad([o_h, ht_h], targets, [torch.zeros_like(o_h), ch / c], allow_unused=True), c)
        if res[3] is not None:
            res[3] = res[3].to(ctx.in_dtypes[0])
        if res[4] is not None:
            res[4] = res[4].to(ctx.in_dtypes[1])
        return res[0], res[1], res[2], res[3], res[4], None, None, None, None


def _chunk_gla_fp32_via_fp16(q, k, v, g, scale, initial_state, output_final_state, offsets, head_first):
    if torch.is_grad_enabled() and any(x is not None and x.requires_grad for x in (q, k, v, g, initial_state)):
        return _ScaledFp16ChunkGla.apply(q, k, v, g, initial_state, scale, output_final_state, offsets, head_first)
    sq, sk, sv = _pow2_scale(q), _pow2_scale(k), _pow2_scale(v)
    skv = sk * sv
    h0 = None if initial_state is None else initial_state.float() / skv
    o, ht = chunk_gla(_scaled_half(q, sq), _scaled_half(k, sk), _scaled_half(v, sv), g.float(), scale=scale,
                      initial_state=h0, output_final_state=output_final_state, offsets=offsets, head_first=head_first)
    return o * (sq * skv), None if ht is None else ht * skv


def _pad_dim(x: Optional[torch.Tensor], size: int) -> Optional[torch.Tensor]:
    if x is None or x.shape[-1] == size:
        return x
    return F.pad(x, (0, size - x.shape[-1]))


def _round64(d: int) -> int:
    return -(-d // 64) * 64


def _piece_chunk_size(T: int, chunk_size: int) -> int:
    """The reference's chunk length for a launch over T tokens (``fla/ops/gla/chunk.py:995``)."""
    if chunk_size != BT:
        raise NotImplementedError("fla_amd: the chunk kernels are built for chunk_size=64")
    return min(chunk_size, max(16, 1 << (max(T, 1) - 1).bit_length()))


def _piece_k(K: int) -> int:
    if K > 256:
        raise NotImplementedError("fla_amd: the chunk-parallel GLA stages are built for K <= 256")
    return 64 if K <= 64 else 128 if K <= 128 else 256


def _seq_first(x: Optional[torch.Tensor], head_first: bool) -> Optional[torch.Tensor]:
    """[B, H, T|NT, ...] -> [B, T|NT, H, ...] (a copy) for head-first callers."""
    if x is None or not head_first:
        return x
    return x.transpose(1, 2).contiguous()


def _pad_state(m: torch.Tensor, Kp: int, Vp: int) -> torch.Tensor:
    K, V = m.shape[-2:]
    if (K, V) == (Kp, Vp):
        return m.contiguous()
    return F.pad(m, (0, Vp - V, 0, Kp - K)).contiguous()


def _check_piece_dtypes(x: torch.Tensor, A: torch.Tensor, m: torch.Tensor, g: torch.Tensor):
    if x.dtype not in (torch.bfloat16, torch.float16):
        raise NotImplementedError("fla_amd: q/k/v/do must be bf16 or fp16")
    for name, t in (("A", A), ("the states", m)):
        if t.dtype not in (torch.float32, x.dtype):
            raise NotImplementedError(f"fla_amd: {name} must be fp32 or of the q/k/v dtype")
    if g.dtype != torch.float32:
        raise NotImplementedError("fla_amd: the cumulative gates must be fp32")


def _chunk_gla_fwd_o_gk_plain(q, v, g, A, h, scale, offsets, indices, head_first, chunk_size):
    """``chunk_gla_fwd_o_gk`` on the reference's operands (``fla/ops/gla/chunk.py:941-979``):
    scores ``A`` [B,T,H,BT] and row-major states ``h`` [B,NT,H,K,V] as the caller computed them."""
    q, v, g, A, h = (_seq_first(t, head_first) for t in (q, v, g, A, h))
    B, T, H, K = q.shape
    V = v.shape[-1]
    bt = _piece_chunk_size(T, chunk_size)
    _check_piece_dtypes(q, A, h, g)
    Kp, Vp = _piece_k(K), _round64(V)
    qp, gp = _pad_dim(q, Kp).contiguous(), _pad_dim(g, Kp).contiguous()
    vp, Ap, hp = _pad_dim(v, Vp).contiguous(), _pad_dim(A, BT).contiguous(), _pad_state(h, Kp, Vp)
    NT = 0 if offsets is None else indices.shape[0]
    o = torch.empty_like(vp)
    be.check(be.lib().fla_chunk_gla_fwd_o_gk(
        be.ptr(qp), be.ptr(vp), be.ptr(gp), be.ptr(Ap), be.ptr(hp), be.ptr(o), be.ptr(offsets), be.ptr(indices), NT,
        be.dt(qp), be.dt(Ap), be.dt(hp), B, T, H, Kp, Vp, float(scale), be.stream_of(q)), "fla_chunk_gla_fwd_o_gk")
    o = o[..., :V]
    return o.transpose(1, 2) if head_first else o


def chunk_gla_fwd_o_gk(q, v, g, A, h, scale, offsets=None, indices=None, head_first=True, chunk_size=64,
                       *, k=None, gates_are_cumsum=True, A_out=None):
    """Output stage ``o = (scale q e^{g}) h + tril(A) v`` (``fla/ops/gla/chunk.py:941-979``).

    Called as the reference calls it (``k`` not given), ``A`` and the row-major ``h`` are read as
    they are.  The operator's own pipeline passes ``k=``: the device kernel then recomputes the
    scores from ``q, k, g`` and takes ``h`` in MFMA-fragment order (seq-first only); that form scores a
    chunk with one reference point and has no range guard, so it is exact only while the chunk-cumulative
    log-gate stays within +-80 (bf16) or +-8 (fp16) - ``chunk_gla`` itself goes through the guarded
    fused launch."""
    if k is None:
        return _chunk_gla_fwd_o_gk_plain(q, v, g, A, h, scale, offsets, indices, head_first, chunk_size)
    if head_first or chunk_size != BT:
        raise NotImplementedError("fla_amd chunk_gla_fwd_o_gk with k=: seq-first, chunk size 64 only")
    B, T, H, K = q.shape
    V = v.shape[-1]
    NT = 0
    if offsets is not None:
        NT = indices.shape[0]
    o = torch.empty_like(v)
    be.check(be.lib().fla_chunk_gla_fwd_o(
        be.ptr(q), be.ptr(k), be.ptr(v), be.ptr(g), int(gates_are_cumsum), be.ptr(h), be.ptr(o), be.ptr(A_out),
        be.ptr(offsets), be.ptr(indices), NT, be.dt(q), be.dt(g), B, T, H, K, V, float(scale),
        be.stream_of(q)), "fla_chunk_gla_fwd_o")
    return o


def chunk_gla_bwd_dA(v, do, scale, offsets=None, indices=None, head_first=True, chunk_size=64):
    """``dA = scale tril(do v^T)``, fp32 [B,T,H,BT] (``fla/ops/gla/chunk.py:982-1015``)."""
    v, do = _seq_first(v, head_first), _seq_first(do, head_first)
    B, T, H, V = v.shape
    bt = _piece_chunk_size(T, chunk_size)
    if v.dtype not in (torch.bfloat16, torch.float16) or do.dtype != v.dtype:
        raise NotImplementedError("fla_amd chunk_gla_bwd_dA: v and do must both be bf16 or fp16")
    if V > 256:
        raise NotImplementedError("fla_amd chunk_gla_bwd_dA: V <= 256")
    Vp = _piece_k(V)
    vp, dop = _pad_dim(v, Vp).contiguous(), _pad_dim(do, Vp).contiguous()
    NT = 0 if offsets is None else indices.shape[0]
    dA = v.new_empty(B, T, H, BT, dtype=torch.float32)
    be.check(be.lib().fla_chunk_gla_bwd_dA(
        be.ptr(vp), be.ptr(dop), be.ptr(dA), be.ptr(offsets), be.ptr(indices), NT, be.dt(vp), B, T, H, Vp,
        float(scale), be.stream_of(v)), "fla_chunk_gla_bwd_dA")
    dA = dA[..., :bt]
    return dA.transpose(1, 2) if head_first else dA


def chunk_gla_bwd_dv(k, g, A, do, dh, offsets=None, indices=None, head_first=True, chunk_size=64):
    """``dv = triu(A^T) do + (k e^{g_last-g}) dh`` with row-major ``dh`` [B,NT,H,K,V]
    (``fla/ops/gla/chunk.py:1018-1054``)."""
    k, g, A, do, dh = (_seq_first(t, head_first) for t in (k, g, A, do, dh))
    B, T, H, K = k.shape
    V = do.shape[-1]
    _piece_chunk_size(T, chunk_size)
    _check_piece_dtypes(k, A, dh, g)
    Kp, Vp = _piece_k(K), _round64(V)
    kp, gp = _pad_dim(k, Kp).contiguous(), _pad_dim(g, Kp).contiguous()
    dop, Ap, dhp = _pad_dim(do, Vp).contiguous(), _pad_dim(A, BT).contiguous(), _pad_state(dh, Kp, Vp)
    NT = 0 if offsets is None else indices.shape[0]
    dv = torch.empty_like(dop)
    be.check(be.lib().fla_chunk_gla_bwd_dv(
        be.ptr(kp), be.ptr(gp), be.ptr(Ap), be.ptr(dop), be.ptr(dhp), be.ptr(dv), be.ptr(offsets), be.ptr(indices), NT,
        be.dt(kp), be.dt(Ap), be.dt(dhp), B, T, H, Kp, Vp, be.stream_of(k)), "fla_chunk_gla_bwd_dv")
    dv = dv[..., :V]
    return dv.transpose(1, 2) if head_first else dv


# Workspaces of the range guard for forward passes whose flags nobody keeps: one pair per (device, stream, dtype,
# host thread), grown to the largest call seen and reused by every later call (launches on one stream are ordered,
# so the next call may overwrite them; two host threads never share a pair).  The state hand-over buffer holds one
# [K, V] tile per (chunk, head) - 268 MB at B=8, T=4096, H=16, K=V=128 in 16 bits - and stays allocated; a forward
# that hands its flags to a backward pass gets fresh ones.
_GUARD_WS = {}


def _guard_workspaces(q, chunks, H, KV, keep):
    if keep:
        return q.new_empty(chunks, H, dtype=torch.int32), q.new_empty(chunks, H, KV)
    key = (q.device, torch.cuda.current_stream(q.device).cuda_stream, q.dtype, threading.get_ident())
    ws = _GUARD_WS.get(key)
    n_flags, n_state = chunks * H, chunks * H * KV
    if ws is None or ws[0].numel() < n_flags or ws[1].numel() < n_state:
        if ws is None and len(_GUARD_WS) >= 16:
            _GUARD_WS.clear()
        ws = _GUARD_WS[key] = (q.new_empty(max(n_flags, 0 if ws is None else ws[0].numel()), dtype=torch.int32),
                               q.new_empty(max(n_state, 0 if ws is None else ws[1].numel())))
    return ws


def chunk_gla_fwd_fused(q, k, v, g, scale, initial_state, output_final_state, offsets=None, exact_guard=True,
                        return_flags=False, states_out=None, head_gates=False, first_launch_only=False,
                        gate_logits=None):
    """Forward through ``fla_chunk_gla_fwd_fused``: seq-first, K in {64,128}, V % 64 == 0.
    With ``exact_guard`` (needs V <= 128) chunks whose cumulative log-gate leaves the
    single-reference range are detected on the device and recomputed exactly; ``return_flags``
    also returns the int32 ``[chunks, H]`` flags (for the backward pass).  With a list
    ``states_out`` the launch also writes the state entering every chunk (transposed fragment
    order, what the backward kernels read) and appends it, followed (per-key gates only) by the gated queries
    ``q e^{G}`` ``[B,T,H,K]`` and the chunk decays ``e^{G_last}`` ``[chunks,H,K]`` the backward's reverse state scan
    streams (``fla_chunk_gla_fwd_fused_kept``).  ``head_gates``: ``g`` is one fp32 log-gate
    per (token, head), ``[B,T,H]`` (``fla_chunk_simple_gla_fwd_fused``).  ``gate_logits = (normalizer, clamp_min)``:
    ``g`` is the gate projection's output and the kernel forms ``logsigmoid(g) / normalizer`` (clamped from below
    unless ``clamp_min`` is None) itself (``fla_chunk_gla_fwd_fused_logits``; no kept states, per-key gates)."""
    B, T, H, K = q.shape
    V = v.shape[-1]
    plan = VarlenPlan(offsets, BT) if offsets is not None else None
    N = B if plan is None else plan.N
    o = torch.empty_like(v)
    ht = q.new_empty(N, H, K, V, dtype=torch.float32) if output_final_state else None
    h0 = None
    if initial_state is not None:
        h0 = (initial_state if initial_state.dtype == torch.float32 else initial_state.float()).contiguous()
    wide = hwide = None
    if exact_guard and V <= 128:
        chunks = plan.NT if plan is not None else B * (-(-T // BT))
        wide, hwide = _guard_workspaces(q, chunks, H, K * V, keep=return_flags)
    tail = (be.ptr(None if plan is None else plan.offsets), be.ptr(None if plan is None else plan.indices),
            be.ptr(None if plan is None else plan.chunk_offsets), be.ptr(None if plan is None else plan.seq_order),
            0 if plan is None else plan.NT,
            be.dt(q), be.dt(g), B, T, H, K, V, N, float(scale), be.stream_of(q))
    head = (be.ptr(q), be.ptr(k), be.ptr(v), be.ptr(g), be.ptr(h0), be.ptr(o), be.ptr(ht), be.ptr(wide), be.ptr(hwide))
    if gate_logits is not None:
        if head_gates or states_out is not None or first_launch_only:
            raise ValueError("gate logits: per-key gates, forward without kept states")
        normalizer, clamp_min = gate_logits
        be.check(be.lib().fla_chunk_gla_fwd_fused_logits(*head, *tail[:-1], float(normalizer), int(clamp_min is not None),
                                                         float(clamp_min or 0.0), tail[-1]),
                 "fla_chunk_gla_fwd_fused_logits")
    elif head_gates:
        if g.dtype != torch.float32 or g.shape != q.shape[:3]:
            raise ValueError("head gates must be fp32 [B, T, H]")
        hT = qg = decay = kh = sc = None
        if states_out is not None:
            nt = plan.NT if plan is not None else -(-T // BT)
            hT = q.new_empty(B, nt, H, K, V)
            states_out.append(hT)
            if V <= 256:
                qg = torch.empty_like(q)
                decay = q.new_empty(B, nt, H, K, dtype=torch.float32)
                states_out.extend((qg, decay))
                if KEEP_KHAT_AND_SCORES and V <= 128:
                    kh = q.new_empty(B, nt, H, K, BT)
                    sc = q.new_empty(B, nt, H, BT, BT)
                    states_out.extend((kh, sc))
        be.check(be.lib().fla_chunk_simple_gla_fwd_fused(*head, be.ptr(hT), be.ptr(qg), be.ptr(decay), be.ptr(kh), be.ptr(sc), *tail[:5],
                                                         be.dt(q), *tail[7:]), "fla_chunk_simple_gla_fwd_fused")
    elif states_out is not None:
        nt = plan.NT if plan is not None else -(-T // BT)
        hT = q.new_empty(B, nt, H, K, V)
        if V <= 256:
            qg = torch.empty_like(q)
            decay = q.new_empty(B, nt, H, K, dtype=torch.float32)
            kh = sc = None
            if KEEP_KHAT_AND_SCORES and V <= 128:
                kh = q.new_empty(B, nt, H, K, BT)
                sc = q.new_empty(B, nt, H, BT, BT)
            be.check(be.lib().fla_chunk_gla_fwd_fused_kept(*head, be.ptr(hT), be.ptr(qg), be.ptr(decay), be.ptr(kh),
                                                           be.ptr(sc), *tail), "fla_chunk_gla_fwd_fused_kept")
            states_out.extend((hT, qg, decay) if kh is None else (hT, qg, decay, kh, sc))
        else:
            be.check(be.lib().fla_chunk_gla_fwd_fused_states(*head, be.ptr(hT), *tail), "fla_chunk_gla_fwd_fused_states")
            states_out.append(hT)
    elif first_launch_only:   # benchmark hook: the scan without the recomputation of flagged chunks
        be.check(be.lib().fla_chunk_gla_fwd_fused_first_launch(*head, *tail), "fla_chunk_gla_fwd_fused_first_launch")
    else:
        be.check(be.lib().fla_chunk_gla_fwd_fused(*head, *tail), "fla_chunk_gla_fwd_fused")
    if return_flags:
        return o, ht, wide
    return o, ht


def _gla_forward(q, k, v, g, scale, initial_state, output_final_state, offsets, want_A=False, fused=True,
                 flags_out=None, states_out=None):
    """Seq-first forward on 64-aligned head dims.  Returns (o, ht, A); with a list ``flags_out`` the
    gate-range flags of the fused kernel are appended to it, with a list ``states_out`` the per-chunk
    states it kept for the backward pass."""
    if fused and not want_A and q.shape[-1] in (64, 128):
        if flags_out is None:
            o, ht = chunk_gla_fwd_fused(q, k, v, g, scale, initial_state, output_final_state, offsets,
                                        states_out=states_out)
            return o, ht, None
        o, ht, wide = chunk_gla_fwd_fused(q, k, v, g, scale, initial_state, output_final_state, offsets,
                                          return_flags=True, states_out=states_out)
        flags_out.append(wide)
        return o, ht, None
    plan = VarlenPlan(offsets, BT) if offsets is not None else None
    B, T, H, K = q.shape
    h, ht = chunk_fwd_h(
        k=k, v=v, g=None, gk=g, gv=None, h0=initial_state, output_final_state=output_final_state,
        offsets=None if plan is None else plan.offsets,
        indices=None if plan is None else plan.indices,
        head_first=False, chunk_size=BT, gates_are_cumsum=False, fragment_layout=True,
        chunk_offsets=None if plan is None else plan.chunk_offsets)
    A = q.new_empty(B, T, H, BT, dtype=torch.float32) if want_A else None
    o = chunk_gla_fwd_o_gk(q, v, g, None, h, scale,
                           offsets=None if plan is None else plan.offsets,
                           indices=None if plan is None else plan.indices,
                           head_first=False, chunk_size=BT, k=k, gates_are_cumsum=False, A_out=A)
    return o, ht, A


def _internal_layout(head_first, *tensors):
    """Seq-first, contiguous copies of the operands of an internal entry point."""
    return tuple(None if t is None else (t.transpose(1, 2) if head_first else t).contiguous() for t in tensors)


def _check_internal(q, k, v, T, offsets=None):
    """Returns the reference's chunk length for the call, ``min(64, max(16, npow2(T)))`` (``fla/ops/gla/chunk.py:1350``).
    The kernels walk chunks of 64; for T <= 32 a batch of equal-length sequences is one chunk either way (same
    cumulative gates, states and outputs; the score tile has 16 or 32 columns instead of 64)."""
    bt = min(BT, max(16, 1 << (max(T, 1) - 1).bit_length()))
    if bt != BT and offsets is not None:
        raise NotImplementedError("fla_amd chunk_gla_fwd / chunk_gla_bwd: packed batches of 32 tokens or fewer are "
                                  "chunked by 16 or 32 in the reference; the kernels are built for chunks of 64")
    if q.dtype not in (torch.bfloat16, torch.float16) or k.dtype != q.dtype or v.dtype != q.dtype:
        raise NotImplementedError("fla_amd chunk_gla_fwd / chunk_gla_bwd: q, k, v must share one 16-bit dtype")
    if (q.shape[-1], v.shape[-1]) not in _SUPPORTED_KV:
        raise NotImplementedError(f"fla_amd chunk_gla_fwd / chunk_gla_bwd: head dims {q.shape[-1]}, {v.shape[-1]} "
                                  f"outside the built tiles {sorted(_SUPPORTED_KV)}")
    return bt


def chunk_gla_fwd(q, k, v, g, g_cumsum, scale, initial_state, output_final_state,
                  offsets=None, indices=None, head_first=True, chunk_size=64):
    """Reference-shaped forward (``fla/ops/gla/chunk.py:1156-1214``) for internal callers
    (GSA calls it with ``g=None, g_cumsum=...``, ``fla/ops/gsa/chunk.py:622-636``): returns
    ``(g_cumsum, A, h, ht, o)`` in the caller's layout, ``h`` row-major ``[B,NT,H,K,V]`` in the q/k/v dtype,
    ``A`` fp32 ``[B,T,H,64]``.  ``o``, ``h`` and ``ht`` are exact for any gate (``o`` comes from the guarded
    fused launch); ``A`` is scored with one reference point per chunk, i.e. exact while the chunk-cumulative
    log-gate stays within +-80 (bf16) / +-8 (fp16) - the backward entry below does not read it."""
    q, k, v, g, g_cumsum = _internal_layout(head_first, q, k, v, g, g_cumsum)
    B, T, H, K = q.shape
    bt = _check_internal(q, k, v, T, offsets)
    plan = VarlenPlan(offsets, BT) if offsets is not None else None
    offs = None if plan is None else plan.offsets
    idx = None if plan is None else plan.indices
    co = None if plan is None else plan.chunk_offsets
    if g_cumsum is None:
        g_cumsum = chunk_local_cumsum(g, BT, offsets=offs, indices=idx, head_first=False)
    elif g_cumsum.dtype != torch.float32:
        g_cumsum = g_cumsum.float()
    if g is None:
        g = chunk_local_cumsum_inverse(g_cumsum, BT, offsets=offs, indices=idx, head_first=False)
    h, ht = chunk_fwd_h(k=k, v=v, g=None, gk=g_cumsum, gv=None, h0=initial_state,
                        output_final_state=output_final_state, offsets=offs, indices=idx, head_first=False,
                        chunk_size=BT, chunk_offsets=co)
    # the scores depend on q, k and the gates only: the score launch also forms an output from whatever
    # states it is given, which is discarded here (the row-major states stand in for the fragment-order ones,
    # same size), and o comes from the guarded fused launch instead
    A = q.new_empty(B, T, H, BT, dtype=torch.float32)
    chunk_gla_fwd_o_gk(q, v, g_cumsum, None, h, scale, offsets=offs, indices=idx, head_first=False,
                       chunk_size=BT, k=k, gates_are_cumsum=True, A_out=A)
    o, _ = chunk_gla_fwd_fused(q, k, v, g if g.dtype in (torch.float32, q.dtype) else g.float(), scale, initial_state,
                               False, offsets)
    if bt != BT:
        A = A[..., :bt]
    if head_first:
        g_cumsum, A, o = (x.transpose(1, 2) for x in (g_cumsum, A, o))
        h = h.transpose(1, 2)
    return g_cumsum, A, h, ht, o


def chunk_gla_bwd_device(q, k, v, g, scale, initial_state, do, dht, offsets, wide=None, hT=None, qg=None,
                         decay=None, head_gates=False, kh=None, scores=None):
    """Backward on prepared tensors (seq-first, 16-bit, 64-aligned head dims).
    Returns ``(dq, dk, dv, dg, dh0)``; without ``hT`` (the states a forward pass kept) it
    recomputes the per-chunk states as the reference does (``fla/ops/gla/chunk.py:1239-1253``).  ``qg``, ``decay``:
    the gated queries and chunk decays of ``fla_chunk_gla_fwd_fused_kept``, if the forward kept them.  ``wide``: the forward's
    gate-range flags (int32 ``[chunks, H]``); flagged chunks get their intra-chunk terms
    from the exact kernel.  Without it the result is exact only while the chunk-cumulative
    log-gate stays within +-80.  ``head_gates``: ``g`` is one fp32 log-gate per (token, head), ``[B, T, H]``, and
    ``dg`` comes back in that shape (``fla_chunk_simple_gla_bwd`` when the forward kept its gated queries; otherwise
    the gates are broadcast over the key channels and the per-key gradient is summed afterwards)."""
    plan = VarlenPlan(offsets, BT) if offsets is not None else None
    offs = None if plan is None else plan.offsets
    idx = None if plan is None else plan.indices
    co = None if plan is None else plan.chunk_offsets
    B, T, H, K = q.shape
    V = v.shape[-1]
    N = B if plan is None else plan.N
    NT = 0 if plan is None else plan.NT
    kept = qg is not None and decay is not None and float(scale) != 0.0 and hT is not None
    g_head = None
    if head_gates and not kept:
        g_head, g = g, g.unsqueeze(-1).expand(*g.shape, K).contiguous()
    if hT is None:
        hT, _ = chunk_fwd_h(k=k, v=v, g=None, gk=g, gv=None, h0=initial_state, output_final_state=False,
                            offsets=offs, indices=idx, head_first=False, chunk_size=BT, gates_are_cumsum=False,
                            fragment_layout=True, transposed_fragments=True, chunk_offsets=co)
    dhtf = torch.empty_like(hT)
    dq, dk, dv = torch.empty_like(q), torch.empty_like(k), torch.empty_like(v)
    if kept and head_gates:
        dg = q.new_zeros(B, T, H, dtype=torch.float32)   # the kernels add their slices' sums to it
    else:
        dg = q.new_empty(B, T, H, K, dtype=torch.float32)
    dh0 = q.new_empty(N, H, K, V, dtype=torch.float32) if initial_state is not None else None
    if dht is not None:
        dht = (dht if dht.dtype == torch.float32 else dht.float()).contiguous()
    tail = (be.ptr(dh0), be.ptr(wide), be.ptr(offs),
            be.ptr(idx), be.ptr(co), NT, be.dt(q), be.dt(g), B, T, H, K, V, N, float(scale), be.stream_of(q))
    outs = (be.ptr(dhtf), be.ptr(dq), be.ptr(dk), be.ptr(dv), be.ptr(dg))
    head = (be.ptr(q), be.ptr(k), be.ptr(v), be.ptr(g), be.ptr(do), be.ptr(dht), be.ptr(hT))
    if kept and head_gates:
        be.check(be.lib().fla_chunk_simple_gla_bwd(*head, be.ptr(qg), be.ptr(decay), be.ptr(kh), be.ptr(scores), *outs,
                                                   *tail[:7], *tail[8:]),
                 "fla_chunk_simple_gla_bwd")
    elif kept:
        be.check(be.lib().fla_chunk_gla_bwd_kept(*head, be.ptr(qg), be.ptr(decay), be.ptr(kh), be.ptr(scores), *outs,
                                                 *tail), "fla_chunk_gla_bwd_kept")
    else:
        be.check(be.lib().fla_chunk_gla_bwd(*head, *outs, *tail), "fla_chunk_gla_bwd")
    if g_head is not None:
        dg = dg.sum(-1)
    return dq, dk, dv, dg, dh0


def _gate_range_flags(g_cumsum: torch.Tensor, dtype: torch.dtype) -> torch.Tensor:
    """int32 ``[B * NT, H]``: 1 where a chunk's cumulative log-gates leave the range in which the kernels score a
    chunk with one reference point (|G| <= 80 for bf16 operands, 8 for fp16) - what the fused forward's staging
    waves flag on their way - from seq-first cumulative gates ``[B, T, H, K]`` of equal-length sequences."""
    B, T, H, K = g_cumsum.shape
    limit = 80.0 if dtype == torch.bfloat16 else 8.0
    peak = g_cumsum.abs().amax(-1)                                    # [B, T, H]
    pad = -T % BT
    if pad:
        peak = F.pad(peak, (0, 0, 0, pad))
    return (peak.view(B, -1, BT, H).amax(2) > limit).to(torch.int32).view(-1, H).contiguous()


def chunk_gla_bwd(q, k, v, g, g_cumsum, scale, initial_state, h, A, do, dht,
                  offsets=None, indices=None, head_first=True, chunk_size=64):
    """Reference-shaped backward (``fla/ops/gla/chunk.py:1217-1320``) for internal callers (GSA:
    ``g=None, g_cumsum=..., h=..., A=...``, ``fla/ops/gsa/chunk.py:741-757``): returns ``(dq, dk, dv, dg, dh0)`` in
    the caller's layout, ``dg`` the gradient of the raw gates (the chunk-local reverse cumulative sum already
    applied, as ``chunk_gla_bwd_kernel_inter`` leaves it, ``fla/ops/gla/chunk.py:818-823``).  Either ``g`` or
    ``g_cumsum`` may be ``None``.  Row-major states ``h`` (fp32 or the q/k/v dtype) of equal-length sequences are
    used as given, together with ``g_cumsum``; otherwise the per-chunk states and the gate-range flags come from one
    run of the fused forward launch.  The scores are recomputed on chip (``A`` is accepted and not read); exact for
    any gate."""
    q, k, v, g, g_cumsum, do = _internal_layout(head_first, q, k, v, g, g_cumsum, do)
    _check_internal(q, k, v, q.shape[1], offsets)
    if g is None:
        if g_cumsum is None:
            raise ValueError("chunk_gla_bwd needs g or g_cumsum")
        plan = VarlenPlan(offsets, BT) if offsets is not None else None
        g = chunk_local_cumsum_inverse(g_cumsum, BT, offsets=None if plan is None else plan.offsets,
                                       indices=None if plan is None else plan.indices, head_first=False)
    elif g.dtype not in (torch.float32, q.dtype):
        g = g.float()
    do = do.to(q.dtype).contiguous()
    if h is not None and g_cumsum is not None and offsets is None and h.dtype in (torch.float32, q.dtype):
        # the caller's states (row-major, the state entering every chunk) are re-ordered for the kernels instead of
        # being recomputed; the chunks whose cumulative gates leave the range of the single-reference-point scores
        # are read off the cumulative gates the caller holds
        from ..common.chunk_o import states_to_fragments
        hT = states_to_fragments(h.transpose(1, 2) if head_first else h, q.dtype, transposed=True)
        wide = _gate_range_flags(g_cumsum, q.dtype)
        dq, dk, dv, dg, dh0 = chunk_gla_bwd_device(q, k, v, g, scale, initial_state, do, dht, offsets, wide, hT=hT)
    else:
        states = []
        _, _, wide = chunk_gla_fwd_fused(q, k, v, g, scale, initial_state, False, offsets, return_flags=True,
                                         states_out=states)
        dq, dk, dv, dg, dh0 = chunk_gla_bwd_device(q, k, v, g, scale, initial_state, do, dht, offsets, wide,
                                                   hT=states[0],
                                                   qg=states[1] if len(states) > 1 else None,
                                                   decay=states[2] if len(states) > 2 else None,
                                                   kh=states[3] if len(states) > 4 else None,
                                                   scores=states[4] if len(states) > 4 else None)
    if head_first:
        dq, dk, dv, dg = (x.transpose(1, 2) for x in (dq, dk, dv, dg))
    return dq, dk, dv, dg, dh0


class ChunkGLAFunction(torch.autograd.Function):

    @staticmethod
    @contiguous
    def forward(ctx, q, k, v, g, scale, initial_state, output_final_state, offsets, head_first):
        be.require_gpu(q, k, v, g)
        in_dtypes = (q.dtype, k.dtype, v.dtype, g.dtype)
        if head_first:
            q, k, v, g = (x.transpose(1, 2).contiguous() for x in (q, k, v, g))
        if q.dtype not in (torch.bfloat16, torch.float16):
            raise NotImplementedError(f"fla_amd chunk_gla kernels: q must be bf16 or fp16, got {q.dtype}")
        k, v = k.to(q.dtype), v.to(q.dtype)
        if g.dtype not in (torch.float32, q.dtype):
            g = g.float()
        K, V = q.shape[-1], v.shape[-1]
        KP, VP = _round64(K), _round64(V)
        if (KP, VP) not in _SUPPORTED_KV:
            raise NotImplementedError(f"fla_amd chunk_gla: head dims K={K}, V={V} are outside the built tiles "
                                      f"{sorted(_SUPPORTED_KV)} (after rounding up to multiples of 64)")
        h0 = initial_state
        if (KP, VP) != (K, V):
            q, k, g = _pad_dim(q, KP), _pad_dim(k, KP), _pad_dim(g, KP)
            v = _pad_dim(v, VP)
            if h0 is not None:
                h0 = F.pad(h0, (0, VP - V, 0, KP - K))
        needs_grad = any(ctx.needs_input_grad)
        flags = [] if needs_grad else None   # the backward pass reads the guard's flags
        states = [] if KEEP_STATES_FOR_BACKWARD and needs_grad else None
        o, ht, _ = _gla_forward(q, k, v, g, scale, h0, output_final_state, offsets, flags_out=flags,
                                states_out=states)
        # the inputs, the small table of chunks whose gates need the exact intra-chunk arithmetic, and
        # (unless recomputation is asked for) the per-chunk states the fused launch wrote on its way
        kept = tuple(states) + (None,) * (5 - len(states)) if states else (None,) * 5
        ctx.save_for_backward(q, k, v, g, h0, offsets, flags[0] if flags else None, *kept)
        ctx.scale, ctx.head_first, ctx.dims, ctx.in_dtypes = scale, head_first, (K, V, KP, VP), in_dtypes
        ctx.h0_dtype = None if initial_state is None else initial_state.dtype
        if (KP, VP) != (K, V):
            o = o[..., :V]
            if ht is not None:
                ht = ht[..., :K, :V].contiguous()
        o = o.to(in_dtypes[2])
        if head_first:
            o = o.transpose(1, 2).contiguous()
        return o, ht

    @staticmethod
    @contiguous
    def backward(ctx, do, dht):
        q, k, v, g, h0, offsets, wide, hT, qg, decay, kh, scores = ctx.saved_tensors
        K, V, KP, VP = ctx.dims
        if ctx.head_first:
            do = do.transpose(1, 2)
        do = do.to(q.dtype)
        if VP != V:
            do = F.pad(do, (0, VP - V))
        do = do.contiguous()
        if dht is not None and (KP, VP) != (K, V):
            dht = F.pad(dht, (0, VP - V, 0, KP - K))
        dq, dk, dv, dg, dh0 = chunk_gla_bwd_device(q, k, v, g, ctx.scale, h0, do, dht, offsets, wide, hT=hT, qg=qg,
                                                   decay=decay, kh=kh, scores=scores)
        if (KP, VP) != (K, V):
            dq, dk, dg, dv = dq[..., :K], dk[..., :K], dg[..., :K], dv[..., :V]
            if dh0 is not None:
                dh0 = dh0[..., :K, :V]
        if ctx.head_first:
            dq, dk, dv, dg = (x.transpose(1, 2) for x in (dq, dk, dv, dg))
        qd, kd, vd, gd = ctx.in_dtypes
        if dh0 is not None:
            dh0 = dh0.to(ctx.h0_dtype)
        return dq.to(qd), dk.to(kd), dv.to(vd), dg.to(gd), None, dh0, None, None, None


def _direct_launch_ok(q, k, v, g, initial_state, head_first) -> bool:
    """True when a call can go straight to the fused launch: no operand takes part in autograd, and every
    operand already has the layout, dtype and head dims the kernel reads (seq-first, contiguous, one 16-bit
    dtype, fp32 or 16-bit gates, fp32 state, built tile sizes).  Anything else takes the autograd function,
    which converts and pads."""
    if head_first or q.dtype not in (torch.bfloat16, torch.float16) or k.dtype != q.dtype or v.dtype != q.dtype:
        return False
    if g.dtype != torch.float32 and g.dtype != q.dtype:
        return False
    if (q.shape[-1], v.shape[-1]) not in _SUPPORTED_KV:
        return False
    if torch.is_grad_enabled() and (q.requires_grad or k.requires_grad or v.requires_grad or g.requires_grad or
                                    (initial_state is not None and initial_state.requires_grad)):
        return False
    if not (q.is_cuda and k.is_cuda and v.is_cuda and g.is_cuda and q.is_contiguous() and k.is_contiguous()
            and v.is_contiguous() and g.is_contiguous()):
        return False
    return initial_state is None or (initial_state.dtype == torch.float32 and initial_state.is_contiguous())


def _chunk_gla_fp32(q, k, v, g, scale, initial_state, output_final_state, offsets, head_first):
    """fp32 q/k/v (the reference runs and tests the operator in fp32, ``tests/ops/test_gla.py:29-87``): the
    chunk kernels multiply 16-bit operands, so fp32 callers are served by the token-by-token kernels, which
    evaluate the same recurrence in fp32 forward and backward (slower - serial in time - but to fp32
    accuracy).  Key dims above 256 and value dims that are not multiples of 4 are split / padded."""
    from ..common.fused_recurrent import fused_recurrent
    K, V = q.shape[-1], v.shape[-1]
    if K > 256:
        o_sum, states = None, []
        for k0 in range(0, K, 256):
            ks = slice(k0, k0 + 256)
            h0 = None if initial_state is None else initial_state[..., ks, :]
            o, ht = _chunk_gla_fp32(q[..., ks], k[..., ks], v, g[..., ks], scale, h0, output_final_state, offsets,
                                    head_first)
            o_sum = o if o_sum is None else o_sum + o
            states.append(ht)
        return o_sum, (torch.cat(states, dim=-2) if output_final_state else None)
    Vp = -(-V // 4) * 4
    h0 = initial_state
    if Vp != V:
        v = F.pad(v, (0, Vp - V))
        h0 = None if h0 is None else F.pad(h0, (0, Vp - V))
    o, ht = fused_recurrent(q, k.float(), v.float(), gk=g.float(), scale=scale, initial_state=h0,
                            output_final_state=output_final_state, offsets=offsets, head_first=head_first)
    if Vp != V:
        o = o[..., :V]
        ht = None if ht is None else ht[..., :V]
    return o, ht


def chunk_gla(
    q: torch.Tensor,
    k: torch.Tensor,
    v: torch.Tensor,
    g: torch.Tensor,
    scale: Optional[int] = None,
    initial_state: torch.Tensor = None,
    output_final_state: bool = False,
    offsets: Optional[torch.LongTensor] = None,
    head_first: bool = True,
    cu_seqlens: Optional[torch.LongTensor] = None,
    gate_logit_normalizer: Optional[float] = None,
    gate_clamp_min: Optional[float] = None,
) -> Tuple[torch.Tensor, torch.Tensor]:
    r"""
    Args:
        q, k: ``[B, H, T, K]`` if ``head_first`` else ``[B, T, H, K]``.
        v: ``[B, H, T, V]`` / ``[B, T, H, V]``.
        g: log forget gates applied to keys, same shape as ``k``.
        scale: score scale, default ``K ** -0.5``.
        initial_state: ``[N, H, K, V]`` for ``N`` sequences, or ``None``.
        output_final_state: also return the fp32 final state ``[N, H, K, V]``.
        offsets (synonym ``cu_seqlens``): int64 ``[N+1]`` sequence boundaries of a
            packed batch (batch size 1, seq-first only).
        head_first: layout switch; seq-first is the native layout.
        gate_logit_normalizer (extension, default off): when given, ``g`` is the output of the layer's gate
            projection and the log-gates are ``logsigmoid(g) / gate_logit_normalizer``, clamped from below at
            ``gate_clamp_min`` if that is given (``fla/layers/gla.py:214-217``).  A forward that is not
            differentiated applies that inside the fused launch (no fp32 gate tensor is written or read);
            otherwise it is one elementwise launch in front of the operator, with its backward.

    Returns ``(o, final_state)``.
    """
    offsets = resolve_offsets(offsets, cu_seqlens)
    if gate_logit_normalizer is not None:
        from ...modules.gate_activations import gla_gate
        if (q.numel() and q.dtype != torch.float32 and q.shape[-1] in (64, 128) and v.shape[-1] <= 128
                and _direct_launch_ok(q, k, v, g, initial_state, head_first)):
            check_varlen_args(q, offsets, head_first, initial_state)
            return chunk_gla_fwd_fused(q, k, v, g, q.shape[-1] ** -0.5 if scale is None else scale, initial_state,
                                       output_final_state, offsets,
                                       gate_logits=(gate_logit_normalizer, gate_clamp_min))
        g = gla_gate(g, gate_logit_normalizer, gate_clamp_min,
                     output_dtype=torch.float32 if q.dtype != torch.float32 else None)
    check_varlen_args(q, offsets, head_first, initial_state)
    if scale is None:
        scale = q.shape[-1] ** -0.5
    if q.numel() == 0:
        return empty_batch_result(q.transpose(1, 2) if head_first else q, v, offsets, initial_state, output_final_state)
    if q.dtype == torch.float32:
        if FP32_INPUTS_EXACT:
            return _chunk_gla_fp32(q, k, v, g, scale, initial_state, output_final_state, offsets, head_first)
        return _chunk_gla_fp32_via_fp16(q, k, v, g, scale, initial_state, output_final_state, offsets, head_first)
    K, V = q.shape[-1], v.shape[-1]
    if K > 128:
        # every key channel carries its own row of the state and o sums over them: wider key heads
        # run as slabs of 128 channels whose outputs are added (in fp32)
        o_sum, states = None, []
        for k0 in range(0, K, 128):
            ks = slice(k0, k0 + 128)
            h0 = None if initial_state is None else initial_state[..., ks, :]
            o, ht = chunk_gla(q[..., ks], k[..., ks], v, g[..., ks], scale=scale, initial_state=h0,
                              output_final_state=output_final_state, offsets=offsets, head_first=head_first)
            o_sum = o.float() if o_sum is None else o_sum + o.float()
            states.append(ht)
        return o_sum.to(v.dtype), (torch.cat(states, dim=-2) if output_final_state else None)
    if V > 128:
        # value columns are independent in the recurrence: wider heads run as slabs of 128 columns
        # (autograd sums the slabs' gradients of q, k and g)
        outs, states = [], []
        for v0 in range(0, V, 128):
            h0 = None if initial_state is None else initial_state[..., v0:v0 + 128]
            o, ht = ChunkGLAFunction.apply(q, k, v[..., v0:v0 + 128], g, scale, h0, output_final_state, offsets,
                                           head_first)
            outs.append(o)
            states.append(ht)
        return torch.cat(outs, dim=-1), (torch.cat(states, dim=-1) if output_final_state else None)
    if _direct_launch_ok(q, k, v, g, initial_state, head_first):
        # nothing to differentiate and nothing to convert: no autograd node, no copies
        return chunk_gla_fwd_fused(q, k, v, g, scale, initial_state, output_final_state, offsets)
    o, final_state = ChunkGLAFunction.apply(q, k, v, g, scale, initial_state, output_final_state, offsets, head_first)
    return o, final_state
