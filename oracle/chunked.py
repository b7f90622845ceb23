"""fp32 chunked forms of the two operators, exposing every intermediate.

These restate the chunk algebra the kernels implement so that each kernel can
be checked on its own:

* GLA (``fla/ops/gla/chunk.py:1156-1214`` for the pipeline order;
  ``fla/ops/common/chunk_h.py:73-137`` for "the stored state is the one
  ENTERING the chunk" and ``G_last`` = last valid row;
  ``fla/ops/gla/chunk.py:29-97,113-170`` for ``A``; ``:320-393`` for ``o``):
  ``G`` = chunk-local cumsum of ``gk``;
  ``A_ij = s * sum_k q_ik k_jk exp(G_ik - G_jk)`` for ``j <= i``;
  ``o_i = (s q_i * exp(G_i))^T h_c + sum_{j<=i} A_ij v_j``;
  ``h_{c+1} = diag(exp(G_last)) h_c + sum_j (k_j * exp(G_last - G_j)) v_j^T``.
* gated delta rule (``fla/ops/gated_delta_rule/wy_fast.py:150-208`` for
  ``Aw, Au``; ``:250-317`` for ``w, u``; ``fla/ops/common/chunk_delta_h.py:71-119``
  for the scan; ``fla/ops/common/chunk_o.py:68-101`` for ``o``):
  ``M = strict_lower(diag(beta) K K^T)``, ``Aw = (I + M)^-1``,
  ``Au = (I + M * Gamma)^-1`` with ``Gamma_ij = exp(gamma_i - gamma_j)``;
  ``w = Aw (beta * K)``, ``u = Au (beta * V)``;
  ``v_new = u - (w * exp(gamma)) h_c``;
  ``o = s (exp(gamma) * (Q h_c) + tril(Q K^T * Gamma) v_new)``;
  ``h_{c+1} = exp(gamma_last) h_c + (K * exp(gamma_last - gamma))^T v_new``.

No rounding to bf16 anywhere: this is the exact-arithmetic target, so kernel
intermediates are compared with a tolerance, final outputs against the naive
recurrences.  Chunks never straddle sequences; tail chunks are short.

The three ``gla_*`` functions at the end restate single stages of the GLA pipeline on the
operands the reference's internal callers pass (scores ``A`` and row-major per-chunk states):
``fla/ops/gla/chunk.py:320-393`` (output), ``:582-624`` (dA), ``:642-710`` (dv).  ``chunk_fwd_h`` restates the state
scan of ``fla/ops/common/chunk_h.py:29-137`` for any mix of per-head, per-key and per-value gates (pinned by the
token-by-token recurrence), ``chunk_bwd_dh`` the reverse
state scan of ``fla/ops/common/chunk_h.py:146-262`` (same gates; pinned by autograd through the state chain), ``chunk_bwd_dv_local`` the intra-chunk dv of the
per-head-gate operators (``fla/ops/common/chunk_o.py:379-441``).  They are pinned
by the recurrence (output stage on ``chunked_gla``'s intermediates) and by autograd through the
chunk step (dA, dv, dh) in ``tests/test_oracle_pins.py``.

The ``gdr_*`` / ``chunk_bwd_dqkwg`` / ``chunk_bwd_dv`` / ``*_wy_repr`` functions after them restate the stages of
the delta rule's backward on the reference's operands (``fla/ops/gated_delta_rule/chunk.py:76-177`` for the
order; ``fla/ops/common/chunk_delta_h.py:136-237``, ``chunk_o.py:118-265,294-375``,
``gated_delta_rule/wy_fast.py:250-317,440-562`` for the stages).  Pinned by autograd through one chunk step and
through the WY map, and by their composition against autograd through the naive recurrence.

Test infrastructure only.
"""
from typing import Dict, Optional, Sequence

import torch

from .recurrent import _spans


def _chunks(bos: int, eos: int, BT: int):
    return [(s, min(s + BT, eos)) for s in range(bos, eos, BT)]


def chunked_gla(q, k, v, gk, scale=None, initial_state=None, chunk_size=64,
                offsets: Optional[Sequence[int]] = None,
                dtype=torch.float32) -> Dict[str, torch.Tensor]:
    q, k, v, gk = (x.to(dtype) for x in (q, k, v, gk))
    B, T, H, K = k.shape
    V = v.shape[-1]
    BT = chunk_size
    if scale is None:
        scale = K ** -0.5
    spans = _spans(B, T, offsets)
    G = torch.zeros_like(gk)
    A = torch.zeros(B, T, H, BT, dtype=dtype)
    o = torch.zeros(B, T, H, V, dtype=dtype)
    hs, finals = [], []
    for n, (b, bos, eos) in enumerate(spans):
        h = torch.zeros(H, K, V, dtype=dtype)
        if initial_state is not None:
            h = h + initial_state[n].to(dtype)
        for s, e in _chunks(bos, eos, BT):
            L = e - s
            Gc = torch.cumsum(gk[b, s:e], 0)                    # [L,H,K]
            G[b, s:e] = Gc
            hs.append(h)
            qc, kc, vc = q[b, s:e], k[b, s:e], v[b, s:e]
            # A_ij = s * sum_k q_ik k_jk exp(G_ik - G_jk), j <= i
            diff = Gc[:, None] - Gc[None, :]                    # [L,L,H,K]
            mask = torch.tril(torch.ones(L, L, dtype=torch.bool))
            diff = torch.where(mask[:, :, None, None], diff, torch.full_like(diff, -float('inf')))
            Ac = scale * torch.einsum('ihk,jhk,ijhk->ihj', qc, kc, diff.exp())
            A[b, s:e, :, :L] = Ac
            o[b, s:e] = (torch.einsum('ihk,hkv->ihv', scale * qc * Gc.exp(), h)
                         + torch.einsum('ihj,jhv->ihv', Ac, vc))
            Glast = Gc[-1]                                      # [H,K]
            kd = kc * (Glast[None] - Gc).exp()
            h = h * Glast.exp()[:, :, None] + torch.einsum('jhk,jhv->hkv', kd, vc)
        finals.append(h)
    if offsets is None:
        NT = -(-T // BT)
        h_all = torch.stack(hs, 0).reshape(B, NT, H, K, V) if hs else torch.zeros(B, 0, H, K, V)
    else:
        h_all = torch.stack(hs, 0)[None]
    return dict(g_cumsum=G, A=A, h=h_all, o=o, ht=torch.stack(finals, 0))


def chunked_gated_delta_rule(q, k, v, g, beta, scale=None, initial_state=None, chunk_size=64,
                             offsets: Optional[Sequence[int]] = None,
                             dtype=torch.float32) -> Dict[str, torch.Tensor]:
    q, k, v, beta = (x.to(dtype) for x in (q, k, v, beta))
    B, T, H, K = k.shape
    V = v.shape[-1]
    BT = chunk_size
    g = torch.zeros(B, T, H, dtype=dtype) if g is None else g.to(dtype)
    if scale is None:
        scale = K ** -0.5
    spans = _spans(B, T, offsets)
    gam = torch.zeros_like(g)
    Aw = torch.zeros(B, T, H, BT, dtype=dtype)
    Au = torch.zeros(B, T, H, BT, dtype=dtype)
    Aqk = torch.zeros(B, T, H, BT, dtype=dtype)
    w = torch.zeros_like(k)
    u = torch.zeros_like(v)
    v_new = torch.zeros_like(v)
    o = torch.zeros_like(v)
    hs, finals = [], []
    for n, (b, bos, eos) in enumerate(spans):
        h = torch.zeros(H, K, V, dtype=dtype)
        if initial_state is not None:
            h = h + initial_state[n].to(dtype)
        for s, e in _chunks(bos, eos, BT):
            L = e - s
            gc = torch.cumsum(g[b, s:e], 0)                     # [L,H]
            gam[b, s:e] = gc
            qc, kc, vc, bc = q[b, s:e], k[b, s:e], v[b, s:e], beta[b, s:e]
            kb = kc * bc[..., None]
            vb = vc * bc[..., None]
            eye = torch.eye(L, dtype=dtype)
            strict = torch.tril(torch.ones(L, L, dtype=dtype), -1)
            lower = torch.tril(torch.ones(L, L, dtype=dtype))
            M = torch.einsum('ihk,jhk->hij', kb, kc) * strict    # [H,L,L]
            Gam = ((gc[:, None] - gc[None, :]).permute(2, 0, 1) * lower).exp() * lower
            aw = torch.linalg.solve_triangular(eye + M, eye.expand(H, L, L), upper=False)
            au = torch.linalg.solve_triangular(eye + M * Gam, eye.expand(H, L, L), upper=False)
            Aw[b, s:e, :, :L] = aw.permute(1, 0, 2)
            Au[b, s:e, :, :L] = au.permute(1, 0, 2)
            wc = torch.einsum('hij,jhk->ihk', aw, kb)
            uc = torch.einsum('hij,jhv->ihv', au, vb)
            w[b, s:e], u[b, s:e] = wc, uc
            hs.append(h)
            eg = gc.exp()                                       # [L,H]
            vn = uc - torch.einsum('ihk,hkv->ihv', wc * eg[..., None], h)
            v_new[b, s:e] = vn
            P = torch.einsum('ihk,jhk->hij', qc, kc) * Gam       # tril by Gam's mask
            Aqk[b, s:e, :, :L] = scale * P.permute(1, 0, 2)
            o[b, s:e] = scale * (eg[..., None] * torch.einsum('ihk,hkv->ihv', qc, h)
                                 + torch.einsum('hij,jhv->ihv', P, vn))
            glast = gc[-1]                                      # [H]
            kd = kc * (glast[None] - gc).exp()[..., None]
            h = h * glast.exp()[:, None, None] + torch.einsum('jhk,jhv->hkv', kd, vn)
        finals.append(h)
    if offsets is None:
        NT = -(-T // BT)
        h_all = torch.stack(hs, 0).reshape(B, NT, H, K, V) if hs else torch.zeros(B, 0, H, K, V)
    else:
        h_all = torch.stack(hs, 0)[None]
    return dict(g_cumsum=gam, Aw=Aw, Au=Au, Aqk=Aqk, w=w, u=u, h=h_all, v_new=v_new, o=o,
                ht=torch.stack(finals, 0))


def _chunk_list(B, T, BT, offsets):
    """(global chunk index, batch row, first token, end token) in the order the states are stored."""
    out = []
    for b, bos, eos in _spans(B, T, offsets):
        for s, e in _chunks(bos, eos, BT):
            out.append((len(out), b, s, e))
    return out


def _state_of(m, c, B, offsets):
    """State of global chunk c from [B, NT, H, K, V] (equal lengths) or [1, NT_total, H, K, V]."""
    if offsets is None:
        NT = m.shape[1]
        return m[c // NT, c % NT]
    return m[0, c]


def gla_fwd_o_gk(q, v, g_cumsum, A, h, scale, chunk_size=64, offsets=None, dtype=torch.float32):
    """o_i = (s q_i e^{G_i})^T h_c + sum_{j<=i} A_ij v_j   (fla/ops/gla/chunk.py:353-393)."""
    q, v, G, A, h = (x.to(dtype) for x in (q, v, g_cumsum, A, h))
    B, T, H, _ = q.shape
    o = torch.zeros(B, T, H, v.shape[-1], dtype=dtype)
    for c, b, s, e in _chunk_list(B, T, chunk_size, offsets):
        L = e - s
        Ac = torch.tril(A[b, s:e, :, :L].permute(1, 0, 2)).permute(1, 0, 2)        # [i, H, j], j <= i
        o[b, s:e] = (torch.einsum('ihk,hkv->ihv', scale * q[b, s:e] * G[b, s:e].exp(), _state_of(h, c, B, offsets))
                     + torch.einsum('ihj,jhv->ihv', Ac, v[b, s:e]))
    return o


def gla_bwd_dA(v, do, scale, chunk_size=64, offsets=None, dtype=torch.float32):
    """dA_ij = s * (do_i . v_j) for j <= i, else 0   (fla/ops/gla/chunk.py:607-624)."""
    v, do = v.to(dtype), do.to(dtype)
    B, T, H, _ = v.shape
    dA = torch.zeros(B, T, H, chunk_size, dtype=dtype)
    for c, b, s, e in _chunk_list(B, T, chunk_size, offsets):
        L = e - s
        d = scale * torch.einsum('ihv,jhv->hij', do[b, s:e], v[b, s:e])
        dA[b, s:e, :, :L] = torch.tril(d).permute(1, 0, 2)
    return dA


def gla_bwd_dv(k, g_cumsum, A, do, dh, chunk_size=64, offsets=None, dtype=torch.float32):
    """dv_j = sum_{i>=j} A_ij do_i + (k_j e^{G_last-G_j})^T dh_c, dh_c the gradient w.r.t. the state
    LEAVING chunk c   (fla/ops/gla/chunk.py:681-710)."""
    k, G, A, do, dh = (x.to(dtype) for x in (k, g_cumsum, A, do, dh))
    B, T, H, _ = k.shape
    dv = torch.zeros(B, T, H, do.shape[-1], dtype=dtype)
    for c, b, s, e in _chunk_list(B, T, chunk_size, offsets):
        L = e - s
        Ac = torch.tril(A[b, s:e, :, :L].permute(1, 0, 2))                          # [H, i, j], j <= i
        kd = k[b, s:e] * (G[b, e - 1][None] - G[b, s:e]).exp()
        dv[b, s:e] = (torch.einsum('hij,ihv->jhv', Ac, do[b, s:e])
                      + torch.einsum('jhk,hkv->jhv', kd, _state_of(dh, c, B, offsets)))
    return dv


def chunk_fwd_h(k, v, g=None, gk=None, gv=None, h0=None, chunk_size=64, offsets=None, dtype=torch.float32):
    """The state entering every chunk and the final state, for any mix of chunk-cumulative log-gates g [B,T,H],
    gk [B,T,H,K], gv [B,T,H,V]:  h_next = e^{g_last} diag(e^{gk_last}) h diag(e^{gv_last})
    + (k e^{gk_last - gk})^T (v e^{g_last - g} e^{gv_last - gv})   (fla/ops/common/chunk_h.py:73-137).
    Returns h in storage order ([B,NT,H,K,V] / [1,NT_total,H,K,V]) and ht [N,H,K,V]."""
    k, v = k.to(dtype), v.to(dtype)
    B, T, H, K = k.shape
    V = v.shape[-1]
    out, ht = [], []
    for n, (b, bos, eos) in enumerate(_spans(B, T, offsets)):
        h = torch.zeros(H, K, V, dtype=dtype) if h0 is None else h0[n].to(dtype).clone()
        for s, e in _chunks(bos, eos, chunk_size):
            out.append(h)
            kt, vt = k[b, s:e], v[b, s:e]
            if g is not None:
                gg = g[b, s:e].to(dtype)
                vt = vt * (gg[-1][None] - gg).exp()[..., None]
                h = h * gg[-1].exp()[:, None, None]
            if gk is not None:
                gg = gk[b, s:e].to(dtype)
                kt = kt * (gg[-1][None] - gg).exp()
                h = h * gg[-1].exp()[:, :, None]
            if gv is not None:
                gg = gv[b, s:e].to(dtype)
                vt = vt * (gg[-1][None] - gg).exp()
                h = h * gg[-1].exp()[:, None, :]
            h = h + torch.einsum('thk,thv->hkv', kt, vt)
        ht.append(h)
    if offsets is None:
        NT = -(-T // chunk_size)
        hs = torch.stack(out, 0).reshape(B, NT, H, K, V) if out else torch.zeros(B, 0, H, K, V, dtype=dtype)
    else:
        hs = torch.stack(out, 0)[None]
    return hs, torch.stack(ht, 0)


def chunk_bwd_dh(q, g, gk, do, dht, scale, chunk_size=64, offsets=None, dtype=torch.float32, gv=None):
    """For c = last .. 0:  dh[c] = dH;  dH = e^{g_last} diag(e^{gk_last}) dH diag(e^{gv_last})
    + (s q e^{g} e^{gk})^T (do e^{gv}), from dH = dht.
    g [B,T,H], gk [B,T,H,K] and gv [B,T,H,V] are chunk-cumulative log-gates, each may be None.  Returns dh in the
    storage order of the states ([B,NT,H,K,V] / [1,NT_total,H,K,V]) and dh0 [N,H,K,V]
    (fla/ops/common/chunk_h.py:202-262)."""
    q, do = q.to(dtype), do.to(dtype)
    B, T, H, K = q.shape
    V = do.shape[-1]
    spans = _spans(B, T, offsets)
    out, dh0 = [], []
    for n, (b, bos, eos) in enumerate(spans):
        dH = torch.zeros(H, K, V, dtype=dtype) if dht is None else dht[n].to(dtype).clone()
        seq = []
        for s, e in reversed(_chunks(bos, eos, chunk_size)):
            seq.append(dH)
            qt = scale * q[b, s:e]
            dot = do[b, s:e]
            decay = torch.ones(H, K, dtype=dtype)
            if g is not None:
                qt = qt * g[b, s:e].to(dtype).exp()[..., None]
                decay = decay * g[b, e - 1].to(dtype).exp()[:, None]
            if gk is not None:
                qt = qt * gk[b, s:e].to(dtype).exp()
                decay = decay * gk[b, e - 1].to(dtype).exp()
            dH = dH * decay[:, :, None]
            if gv is not None:
                dot = dot * gv[b, s:e].to(dtype).exp()
                dH = dH * gv[b, e - 1].to(dtype).exp()[:, None, :]
            dH = dH + torch.einsum('thk,thv->hkv', qt, dot)
        out.extend(reversed(seq))
        dh0.append(dH)
    if offsets is None:
        NT = -(-T // chunk_size)
        dh = torch.stack(out, 0).reshape(B, NT, H, K, V) if out else torch.zeros(B, 0, H, K, V, dtype=dtype)
    else:
        dh = torch.stack(out, 0)[None]
    return dh, torch.stack(dh0, 0)


def chunk_bwd_dv_local(q, k, g_cumsum, do, scale, chunk_size=64, offsets=None, dtype=torch.float32):
    """dv_j = sum_{i>=j} s (k_j . q_i) e^{g_i-g_j} do_i within each chunk; g_cumsum [B,T,H] or None
    (fla/ops/common/chunk_o.py:419-441)."""
    q, k, do = q.to(dtype), k.to(dtype), do.to(dtype)
    B, T, H, _ = k.shape
    dv = torch.zeros(B, T, H, do.shape[-1], dtype=dtype)
    for c, b, s, e in _chunk_list(B, T, chunk_size, offsets):
        A = scale * torch.einsum('jhk,ihk->hji', k[b, s:e], q[b, s:e])               # [H, j, i]
        if g_cumsum is not None:
            gc = g_cumsum[b, s:e].to(dtype)                                           # [L, H]
            x = gc.t()[:, None, :] - gc.t()[:, :, None]                               # g_i - g_j
            A = A * torch.where(x <= 0, x.exp(), torch.zeros_like(x))                 # safe_exp (fla/ops/utils/exp.py:9-10)
        dv[b, s:e] = torch.einsum('hji,ihv->jhv', torch.triu(A), do[b, s:e])
    return dv


def _gates_of(g_cumsum, b, s, e, H, dtype):
    """(gamma [L,H], Gamma [H,L,L] lower triangular) of one chunk; zeros / ones without a gate."""
    L = e - s
    gc = torch.zeros(L, H, dtype=dtype) if g_cumsum is None else g_cumsum[b, s:e].to(dtype)
    lower = torch.tril(torch.ones(L, L, dtype=dtype))
    Gam = ((gc[:, None] - gc[None, :]).permute(2, 0, 1) * lower).exp() * lower
    return gc, Gam


def fwd_recompute_w_u(k, v, beta, Aw, Au, chunk_size=64, offsets=None, dtype=torch.float32):
    """w = Aw (beta k), u = Au (beta v) per chunk; Aw, Au [B,T,H,BT]
    (fla/ops/gated_delta_rule/wy_fast.py:250-317)."""
    k, v, beta, Aw, Au = (x.to(dtype) for x in (k, v, beta, Aw, Au))
    B, T, H, _ = k.shape
    w, u = torch.zeros_like(k), torch.zeros_like(v)
    for c, b, s, e in _chunk_list(B, T, chunk_size, offsets):
        L = e - s
        w[b, s:e] = torch.einsum('ihj,jhk->ihk', Aw[b, s:e, :, :L], k[b, s:e] * beta[b, s:e, :, None])
        u[b, s:e] = torch.einsum('ihj,jhv->ihv', Au[b, s:e, :, :L], v[b, s:e] * beta[b, s:e, :, None])
    return w, u


def chunk_bwd_dv(q, k, g_cumsum, do, dh, scale, chunk_size=64, offsets=None, dtype=torch.float32):
    """dv_j = sum_{i>=j} s (k_j . q_i) e^{g_i-g_j} do_i + (k_j e^{g_last-g_j})^T dh_c
    (fla/ops/common/chunk_o.py:294-375)."""
    dv = chunk_bwd_dv_local(q, k, g_cumsum, do, scale, chunk_size, offsets, dtype)
    k, dh = k.to(dtype), dh.to(dtype)
    B, T, H, _ = k.shape
    for c, b, s, e in _chunk_list(B, T, chunk_size, offsets):
        gc, _ = _gates_of(g_cumsum, b, s, e, H, dtype)
        kd = k[b, s:e] * (gc[-1][None] - gc).exp()[..., None]
        dv[b, s:e] += torch.einsum('jhk,hkv->jhv', kd, _state_of(dh, c, B, offsets))
    return dv


def gdr_bwd_dhu(q, k, w, g_cumsum, dht, do, dv, scale, chunk_size=64, offsets=None, dtype=torch.float32):
    """For c = last .. 0:  dh[c] = dH;  dv2 = dv + (k e^{g_last-g}) dH;
    dH = e^{g_last} dH + (s q e^g)^T do - (w e^g)^T dv2, from dH = dht.  Returns (dh, dh0, dv2)
    (fla/ops/common/chunk_delta_h.py:136-237)."""
    q, k, w, do, dv = (x.to(dtype) for x in (q, k, w, do, dv))
    B, T, H, K = q.shape
    V = do.shape[-1]
    dv2 = torch.zeros_like(dv)
    out, dh0 = [], []
    for n, (b, bos, eos) in enumerate(_spans(B, T, offsets)):
        dH = torch.zeros(H, K, V, dtype=dtype) if dht is None else dht[n].to(dtype).clone()
        seq = []
        for s, e in reversed(_chunks(bos, eos, chunk_size)):
            seq.append(dH)
            gc, _ = _gates_of(g_cumsum, b, s, e, H, dtype)
            eg = gc.exp()[..., None]
            kd = k[b, s:e] * (gc[-1][None] - gc).exp()[..., None]
            d2 = dv[b, s:e] + torch.einsum('jhk,hkv->jhv', kd, dH)
            dv2[b, s:e] = d2
            dH = (dH * gc[-1].exp()[:, None, None]
                  + torch.einsum('thk,thv->hkv', scale * q[b, s:e] * eg, do[b, s:e])
                  - torch.einsum('thk,thv->hkv', w[b, s:e] * eg, d2))
        out.extend(reversed(seq))
        dh0.append(dH)
    if offsets is None:
        NT = -(-T // chunk_size)
        dh = torch.stack(out, 0).reshape(B, NT, H, K, V) if out else torch.zeros(B, 0, H, K, V, dtype=dtype)
    else:
        dh = torch.stack(out, 0)[None]
    return dh, torch.stack(dh0, 0), dv2


def chunk_bwd_dqkwg(q, k, v, g_cumsum, do, h, dh, dv, w, scale, chunk_size=64, offsets=None, dtype=torch.float32):
    """Per chunk, with ds = s tril((do v^T) * Gamma):
      dq = s e^g (do h^T) + ds k;   dk = e^{g_last-g} (v dh^T) + ds^T q;   dw = -e^g (dv h^T);
      dg_i = sum_k (q dq - k dk + w dw)_ik + [i last] (sum_jk (k * dk_inter)_jk + e^{g_last} <h, dh>)
    (fla/ops/common/chunk_o.py:118-265; the reference forms the intra-chunk part of dg from ds * (q k^T), whose
    row minus column sums equal sum_k q dq_intra - k dk_intra).  v is v_new for the delta rule; dv / w None
    for the operators without a correction term.  Returns (dq, dk, dw, dg), dg w.r.t. the cumulative gate."""
    q, k, v, do, h, dh = (x.to(dtype) for x in (q, k, v, do, h, dh))
    B, T, H, K = k.shape
    dq, dk = torch.zeros_like(q), torch.zeros_like(k)
    dw = None if w is None else torch.zeros_like(k)
    dg = torch.zeros(B, T, H, dtype=dtype)
    for c, b, s, e in _chunk_list(B, T, chunk_size, offsets):
        gc, Gam = _gates_of(g_cumsum, b, s, e, H, dtype)
        eg = gc.exp()[..., None]
        ed = (gc[-1][None] - gc).exp()[..., None]
        hc, dhc = _state_of(h, c, B, offsets), _state_of(dh, c, B, offsets)
        qc, kc, vc, doc = q[b, s:e], k[b, s:e], v[b, s:e], do[b, s:e]
        ds = scale * torch.einsum('ihv,jhv->hij', doc, vc) * Gam
        dqc = scale * eg * torch.einsum('ihv,hkv->ihk', doc, hc) + torch.einsum('hij,jhk->ihk', ds, kc)
        dk_inter = ed * torch.einsum('jhv,hkv->jhk', vc, dhc)
        dkc = dk_inter + torch.einsum('hij,ihk->jhk', ds, qc)
        row = (qc * dqc - kc * dkc).sum(-1)
        if w is not None:
            dwc = -eg * torch.einsum('ihv,hkv->ihk', dv[b, s:e].to(dtype), hc)
            dw[b, s:e] = dwc
            row = row + (w[b, s:e].to(dtype) * dwc).sum(-1)
        row[-1] += (kc * dk_inter).sum((0, 2)) + gc[-1].exp() * (hc * dhc).sum((1, 2))
        dq[b, s:e], dk[b, s:e], dg[b, s:e] = dqc, dkc, row
    return dq, dk, dw, (None if g_cumsum is None else dg)


def bwd_prepare_wy_repr(k, v, g_cumsum, beta, Aw, dw, du, chunk_size=64, offsets=None, dtype=torch.float32):
    """Gradient through w = Aw kb, u = Au vb with kb = beta k, vb = beta v, M = strict_lower(kb k^T),
    Aw = (I + M)^-1, Au = Aw * Gamma:
      d(kb) = Aw^T dw, d(vb) = Au^T du, dAw = strict_lower(dw kb^T) + strict_lower(du vb^T) * Gamma,
      dM = -strict_lower(Aw^T dAw Aw^T), d(kb) += dM k, dk = beta d(kb) + dM^T kb, dv = beta d(vb),
      dbeta = sum d(kb) k + sum d(vb) v, dg_i = rowsum_i(X) - colsum_i(X), X = strict_lower(du vb^T) * Au
    (fla/ops/gated_delta_rule/wy_fast.py:440-562, there with both inverses as inputs).  Returns (dk, dv, dbeta, dg)."""
    k, v, beta, Aw, dw, du = (x.to(dtype) for x in (k, v, beta, Aw, dw, du))
    B, T, H, _ = k.shape
    dk, dv = torch.zeros_like(k), torch.zeros_like(v)
    dbeta, dg = torch.zeros(B, T, H, dtype=dtype), torch.zeros(B, T, H, dtype=dtype)
    for c, b, s, e in _chunk_list(B, T, chunk_size, offsets):
        L = e - s
        gc, Gam = _gates_of(g_cumsum, b, s, e, H, dtype)
        strict = torch.tril(torch.ones(L, L, dtype=dtype), -1)
        aw = torch.tril(Aw[b, s:e, :, :L].permute(1, 0, 2))                    # [H, i, j]
        au = aw * Gam
        kc, vc, bc = k[b, s:e], v[b, s:e], beta[b, s:e]
        kb, vb = kc * bc[..., None], vc * bc[..., None]
        dkb = torch.einsum('hij,ihk->jhk', aw, dw[b, s:e])
        dvb = torch.einsum('hij,ihv->jhv', au, du[b, s:e])
        X0 = torch.einsum('ihv,jhv->hij', du[b, s:e], vb) * strict
        dAw = torch.einsum('ihk,jhk->hij', dw[b, s:e], kb) * strict + X0 * Gam
        dM = -(aw.transpose(1, 2) @ dAw @ aw.transpose(1, 2)) * strict
        dkb = dkb + torch.einsum('hij,jhk->ihk', dM, kc)
        dk[b, s:e] = bc[..., None] * dkb + torch.einsum('hij,ihk->jhk', dM, kb)
        dv[b, s:e] = bc[..., None] * dvb
        dbeta[b, s:e] = (dkb * kc).sum(-1) + (dvb * vc).sum(-1)
        X = X0 * au
        dg[b, s:e] = (X.sum(2) - X.sum(1)).t()
    return dk, dv, dbeta, dg
