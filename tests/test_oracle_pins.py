"""CPU: pin the oracle against facts that do not come from the oracle itself -
closed forms, special cases that reduce to library routines, brute force on
tiny inputs, the one integer known answer the reference holds, and gradcheck."""
import math

import numpy as np
import pytest
import torch
import torch.nn.functional as F

from oracle import bookkeeping, chunked, cumsum, recurrent

D = torch.float64


def _rand(*shape, seed=0):
    return torch.randn(*shape, generator=torch.Generator().manual_seed(seed), dtype=D)


# ---------------------------------------------------------------- bookkeeping (integer, bit exact)
def _known_answer():
    import json
    import os
    with open(os.path.join(os.path.dirname(__file__), "golden", "chunk_indices_known_answer.json")) as f:
        return json.load(f)


def test_chunk_indices_known_answer():
    # the reference's stored known answer (fla/ops/gla/chunk.py:1352-1355), kept as a fixture
    ka = _known_answer()
    idx = bookkeeping.prepare_chunk_indices(ka["offsets"], ka["chunk_size"])
    assert idx.dtype == np.int64
    assert idx.tolist() == ka["indices"]
    assert ka["offsets"] == [0, 100, 356] and ka["chunk_size"] == 64
    assert bookkeeping.prepare_chunk_offsets(ka["offsets"], ka["chunk_size"]).tolist() == [0, 2, 6]


@pytest.mark.parametrize("bt", [16, 32, 64])
def test_chunk_indices_bruteforce(bt):
    rng = np.random.default_rng(bt)
    for _ in range(50):
        lens = rng.integers(0, 400, size=rng.integers(1, 9))
        offs = np.concatenate([[0], np.cumsum(lens)])
        idx = bookkeeping.prepare_chunk_indices(offs, bt)
        co = bookkeeping.prepare_chunk_offsets(offs, bt)
        # every token position maps to exactly one (sequence, chunk) row, rows are in token order
        expect = []
        for n, length in enumerate(lens):
            seen = sorted({t // bt for t in range(int(length))})
            expect += [[n, c] for c in seen]
        assert idx.tolist() == expect
        assert co[-1] == len(expect) and all(co[n] == sum(1 for r in expect if r[0] < n) for n in range(len(lens)))


@pytest.mark.parametrize("T,bt", [(1, 16), (16, 16), (17, 32), (33, 64), (64, 64), (65, 64), (4096, 64)])
def test_gla_chunk_size_rule(T, bt):
    assert bookkeeping.gla_chunk_size(T) == bt


# ---------------------------------------------------------------- cumsum
@pytest.mark.parametrize("reverse", [False, True])
def test_cumsum_bruteforce(reverse):
    g = _rand(1, 23, 2, 3, seed=1).float()
    offs = [0, 5, 5, 23]
    out = cumsum.chunk_local_cumsum(g, 4, reverse=reverse, offsets=offs)
    for n in range(3):
        bos, eos = offs[n], offs[n + 1]
        for t in range(bos, eos):
            c0 = bos + ((t - bos) // 4) * 4
            c1 = min(c0 + 4, eos)
            rows = range(t, c1) if reverse else range(c0, t + 1)
            acc = torch.zeros(2, 3)
            for r in rows:
                acc = acc + g[0, r]
            torch.testing.assert_close(out[0, t], acc, rtol=1e-6, atol=1e-6)


# ---------------------------------------------------------------- GLA recurrence
def test_gla_scalar_closed_form():
    T = 9
    q, k, v, g = (_rand(1, T, 1, 1, seed=s) for s in range(4))
    g = -g.abs()
    o, ht = recurrent.naive_recurrent_gla(q, k, v, g, scale=0.7, output_final_state=True, dtype=D)
    G = [sum(g[0, :t + 1, 0, 0].tolist()) for t in range(T)]
    for t in range(T):
        want = 0.7 * q[0, t, 0, 0].item() * sum(
            k[0, j, 0, 0].item() * v[0, j, 0, 0].item() * math.exp(G[t] - G[j]) for j in range(t + 1))
        assert abs(o[0, t, 0, 0].item() - want) < 1e-12
    want_h = sum(k[0, j, 0, 0].item() * v[0, j, 0, 0].item() * math.exp(G[-1] - G[j]) for j in range(T))
    assert abs(ht[0, 0, 0, 0].item() - want_h) < 1e-12


def test_gla_zero_gates_is_causal_linear_attention():
    B, T, H, K, V = 2, 11, 2, 5, 3
    q, k, v = _rand(B, T, H, K, seed=1), _rand(B, T, H, K, seed=2), _rand(B, T, H, V, seed=3)
    o, _ = recurrent.naive_recurrent_gla(q, k, v, torch.zeros_like(k), dtype=D)
    scores = torch.einsum('bihk,bjhk->bhij', q, k).tril() * K ** -0.5   # default scale K^-0.5 (naive.py:24)
    want = torch.einsum('bhij,bjhv->bihv', scores, v)
    torch.testing.assert_close(o, want, rtol=1e-12, atol=1e-12)


def test_gla_bruteforce_all_gates_and_reverse():
    B, T, H, K, V = 1, 6, 2, 3, 2
    q, k, v = _rand(B, T, H, K, seed=1), _rand(B, T, H, K, seed=2), _rand(B, T, H, V, seed=3)
    gk, gv, g = -_rand(B, T, H, K, seed=4).abs(), -_rand(B, T, H, V, seed=5).abs(), -_rand(B, T, H, seed=6).abs()
    h0 = _rand(B, H, K, V, seed=7)
    for reverse in (False, True):
        o, ht = recurrent.naive_recurrent_gla(q, k, v, gk, scale=1.3, initial_state=h0, output_final_state=True,
                                              g=g, gv=gv, reverse=reverse, dtype=D)
        order = list(range(T))[::-1] if reverse else list(range(T))
        for h in range(H):
            for pos, t in enumerate(order):
                for c in range(V):
                    want = 0.0
                    for a in range(K):
                        # contribution of the initial state and of every earlier (in processing order) token
                        dec_all = sum(gk[0, m, h, a].item() + gv[0, m, h, c].item() + g[0, m, h].item()
                                      for m in order[:pos + 1])
                        tot = h0[0, h, a, c].item() * math.exp(dec_all)
                        for pj, j in enumerate(order[:pos + 1]):
                            dec = sum(gk[0, m, h, a].item() + gv[0, m, h, c].item() + g[0, m, h].item()
                                      for m in order[pj + 1:pos + 1])
                            tot += k[0, j, h, a].item() * v[0, j, h, c].item() * math.exp(dec)
                        want += 1.3 * q[0, t, h, a].item() * tot
                    assert abs(o[0, t, h, c].item() - want) < 1e-10


def test_gla_segment_chaining_and_varlen():
    B, T, H, K, V = 1, 20, 2, 4, 3
    q, k, v = _rand(B, T, H, K, seed=1), _rand(B, T, H, K, seed=2), _rand(B, T, H, V, seed=3)
    gk = -_rand(B, T, H, K, seed=4).abs()
    h0 = _rand(2, H, K, V, seed=5)
    o, ht = recurrent.naive_recurrent_gla(q, k, v, gk, initial_state=h0[:1], output_final_state=True, dtype=D)
    o1, h1 = recurrent.naive_recurrent_gla(q[:, :7], k[:, :7], v[:, :7], gk[:, :7], initial_state=h0[:1],
                                           output_final_state=True, dtype=D)
    o2, h2 = recurrent.naive_recurrent_gla(q[:, 7:], k[:, 7:], v[:, 7:], gk[:, 7:], initial_state=h1,
                                           output_final_state=True, dtype=D)
    torch.testing.assert_close(torch.cat([o1, o2], 1), o, rtol=1e-12, atol=1e-12)
    torch.testing.assert_close(h2, ht, rtol=1e-12, atol=1e-12)
    # packed batch == per-sequence runs
    ov, hv = recurrent.naive_recurrent_gla(q, k, v, gk, initial_state=h0, output_final_state=True,
                                           offsets=[0, 7, 20], dtype=D)
    oa, ha = recurrent.naive_recurrent_gla(q[:, :7], k[:, :7], v[:, :7], gk[:, :7], initial_state=h0[:1],
                                           output_final_state=True, dtype=D)
    ob, hb = recurrent.naive_recurrent_gla(q[:, 7:], k[:, 7:], v[:, 7:], gk[:, 7:], initial_state=h0[1:],
                                           output_final_state=True, dtype=D)
    torch.testing.assert_close(ov, torch.cat([oa, ob], 1), rtol=1e-12, atol=1e-12)
    torch.testing.assert_close(hv, torch.cat([ha, hb], 0), rtol=1e-12, atol=1e-12)


# ---------------------------------------------------------------- gated delta rule recurrence
def test_gdr_beta_zero_is_pure_decay():
    B, T, H, K, V = 1, 7, 2, 4, 3
    q, k, v = _rand(B, T, H, K, seed=1), _rand(B, T, H, K, seed=2), _rand(B, T, H, V, seed=3)
    g = -_rand(B, T, H, seed=4).abs()
    h0 = _rand(B, H, K, V, seed=5)
    o, ht = recurrent.naive_recurrent_gated_delta_rule(q, k, v, g, torch.zeros(B, T, H, dtype=D), scale=1.0,
                                                       initial_state=h0, output_final_state=True, dtype=D)
    dec = g.cumsum(1).exp()
    torch.testing.assert_close(ht, h0 * dec[:, -1, :, None, None], rtol=1e-12, atol=1e-12)
    want = torch.einsum('bthk,bhkv->bthv', q, h0) * dec[..., None]
    torch.testing.assert_close(o, want, rtol=1e-12, atol=1e-12)


def test_gdr_orthonormal_keys_exact_overwrite():
    H, K, V = 2, 6, 4
    T = K
    Q, _ = torch.linalg.qr(_rand(H, K, K, seed=1))          # orthonormal rows per head
    k = Q.permute(1, 0, 2)[None]                            # [1,T,H,K], k_t orthonormal across t
    v, q = _rand(1, T, H, V, seed=2), _rand(1, T, H, K, seed=3)
    h0 = _rand(1, H, K, V, seed=4)
    _, S = recurrent.naive_recurrent_gated_delta_rule(q, k, v, torch.zeros(1, T, H, dtype=D),
                                                      torch.ones(1, T, H, dtype=D), initial_state=h0,
                                                      output_final_state=True, dtype=D)
    read = torch.einsum('thk,hkv->thv', k[0], S[0])         # S^T k_i must return v_i for every i
    torch.testing.assert_close(read, v[0], rtol=1e-10, atol=1e-10)


def test_gdr_single_step_closed_form():
    H, K, V = 3, 5, 4
    q, k, v = _rand(1, 1, H, K, seed=1), _rand(1, 1, H, K, seed=2), _rand(1, 1, H, V, seed=3)
    beta, g = torch.rand(1, 1, H, dtype=D), -torch.rand(1, 1, H, dtype=D)
    o, _ = recurrent.naive_recurrent_gated_delta_rule(q, k, v, g, beta, scale=0.3, dtype=D)
    want = 0.3 * (q * k).sum(-1, keepdim=True) * beta[..., None] * v
    torch.testing.assert_close(o, want, rtol=1e-12, atol=1e-12)


def test_gdr_dense_transition_matrices():
    """S_t = (I - beta k k^T) e^{g} S_{t-1} + beta k v^T with every transition materialised."""
    B, T, H, K, V = 1, 8, 2, 4, 3
    q, k, v = _rand(B, T, H, K, seed=1), F.normalize(_rand(B, T, H, K, seed=2), dim=-1), _rand(B, T, H, V, seed=3)
    g, beta = -_rand(B, T, H, seed=4).abs(), torch.rand(B, T, H, dtype=D)
    bv = torch.rand(B, T, H, V, dtype=D)
    h0 = _rand(B, H, K, V, seed=5)
    for b_in in (beta, bv):
        o, ht = recurrent.naive_recurrent_gated_delta_rule(q, k, v, g, b_in, scale=0.5, initial_state=h0,
                                                           output_final_state=True, dtype=D)
        for h in range(H):
            S = h0[0, h].numpy().copy()
            for t in range(T):
                kk = k[0, t, h].numpy()
                bcol = np.broadcast_to(b_in[0, t, h].numpy(), (V,))
                Sd = math.exp(g[0, t, h].item()) * S
                # per-value beta: column c uses its own beta
                S = Sd - np.outer(kk, (kk @ Sd) * bcol) + np.outer(kk, v[0, t, h].numpy() * bcol)
                np.testing.assert_allclose(o[0, t, h].numpy(), 0.5 * q[0, t, h].numpy() @ S, rtol=1e-10, atol=1e-12)
            np.testing.assert_allclose(ht[0, h].numpy(), S, rtol=1e-10, atol=1e-12)


# ---------------------------------------------------------------- chunked forms
@pytest.mark.parametrize("offsets", [None, [0, 40, 41, 150]])
def test_chunked_gla_equals_recurrence(offsets):
    B, T, H, K, V = (2 if offsets is None else 1), 150, 2, 8, 6
    N = B if offsets is None else len(offsets) - 1
    q, k, v = _rand(B, T, H, K, seed=1), _rand(B, T, H, K, seed=2), _rand(B, T, H, V, seed=3)
    gk = F.logsigmoid(_rand(B, T, H, K, seed=4))
    h0 = _rand(N, H, K, V, seed=5)
    o, ht = recurrent.naive_recurrent_gla(q, k, v, gk, initial_state=h0, output_final_state=True, offsets=offsets,
                                          dtype=D)
    r = chunked.chunked_gla(q, k, v, gk, initial_state=h0, offsets=offsets, dtype=D)
    torch.testing.assert_close(r['o'], o, rtol=1e-10, atol=1e-10)
    torch.testing.assert_close(r['ht'], ht, rtol=1e-10, atol=1e-10)
    torch.testing.assert_close(r['g_cumsum'].float(), cumsum.chunk_local_cumsum(gk, 64, offsets=offsets),
                               rtol=1e-5, atol=1e-5)
    # per-chunk state h[c] equals the recurrence's state after c*64 tokens of that sequence
    if offsets is None:
        _, h64 = recurrent.naive_recurrent_gla(q[:, :64], k[:, :64], v[:, :64], gk[:, :64], initial_state=h0,
                                               output_final_state=True, dtype=D)
        torch.testing.assert_close(r['h'][:, 1], h64, rtol=1e-10, atol=1e-10)
        torch.testing.assert_close(r['h'][:, 0], h0, rtol=0, atol=0)


@pytest.mark.parametrize("offsets", [None, [0, 40, 41, 150]])
def test_chunked_gdr_equals_recurrence(offsets):
    B, T, H, K, V = (2 if offsets is None else 1), 150, 2, 8, 6
    N = B if offsets is None else len(offsets) - 1
    q, k, v = _rand(B, T, H, K, seed=1), F.normalize(_rand(B, T, H, K, seed=2), dim=-1), _rand(B, T, H, V, seed=3)
    g, beta = F.logsigmoid(_rand(B, T, H, seed=4)), torch.rand(B, T, H, dtype=D)
    h0 = _rand(N, H, K, V, seed=5)
    o, ht = recurrent.naive_recurrent_gated_delta_rule(q, k, v, g, beta, initial_state=h0, output_final_state=True,
                                                       offsets=offsets, dtype=D)
    r = chunked.chunked_gated_delta_rule(q, k, v, g, beta, initial_state=h0, offsets=offsets, dtype=D)
    torch.testing.assert_close(r['o'], o, rtol=1e-9, atol=1e-9)
    torch.testing.assert_close(r['ht'], ht, rtol=1e-9, atol=1e-9)


def test_wy_inverse_identities():
    """Aw (I + M) = I, and Au = Aw * Gamma elementwise (so one inverse suffices)."""
    B, T, H, K, V = 1, 64, 2, 16, 8
    q, k, v = _rand(B, T, H, K, seed=1), F.normalize(_rand(B, T, H, K, seed=2), dim=-1), _rand(B, T, H, V, seed=3)
    g, beta = F.logsigmoid(_rand(B, T, H, seed=4)), torch.rand(B, T, H, dtype=D)
    r = chunked.chunked_gated_delta_rule(q, k, v, g, beta, dtype=D)
    gam = g[0].cumsum(0)
    for h in range(H):
        kb = k[0, :, h] * beta[0, :, h, None]
        M = (kb @ k[0, :, h].T).tril(-1)
        Aw, Au = r['Aw'][0, :, h], r['Au'][0, :, h]
        torch.testing.assert_close(Aw @ (torch.eye(64, dtype=D) + M), torch.eye(64, dtype=D), rtol=1e-9, atol=1e-9)
        Gam = (gam[:, h, None] - gam[None, :, h]).exp().tril()
        torch.testing.assert_close(Au, Aw * Gam, rtol=1e-9, atol=1e-9)
        torch.testing.assert_close(r['w'][0, :, h], Aw @ kb, rtol=1e-9, atol=1e-9)


# ---------------------------------------------------------------- gradients of the oracle (autograd)
def test_oracle_gradcheck():
    B, T, H, K, V = 1, 5, 1, 3, 2
    q, k, v = (_rand(B, T, H, n, seed=s).requires_grad_() for s, n in ((1, K), (2, K), (3, V)))
    gk = (-_rand(B, T, H, K, seed=4).abs()).requires_grad_()
    h0 = _rand(B, H, K, V, seed=5).requires_grad_()
    f = lambda q, k, v, gk, h0: recurrent.naive_recurrent_gla(q, k, v, gk, initial_state=h0,
                                                              output_final_state=True, dtype=D)
    assert torch.autograd.gradcheck(f, (q, k, v, gk, h0), atol=1e-6)
    g = (-_rand(B, T, H, seed=6).abs()).requires_grad_()
    beta = torch.rand(B, T, H, dtype=D).requires_grad_()
    f2 = lambda q, k, v, g, beta, h0: recurrent.naive_recurrent_gated_delta_rule(
        q, k, v, g, beta, initial_state=h0, output_final_state=True, dtype=D)
    assert torch.autograd.gradcheck(f2, (q, k, v, g, beta, h0), atol=1e-6)


# ---------------------------------------------------------------- single GLA stages on the reference's internal operands
@pytest.mark.parametrize("offsets", [None, [0, 40, 41, 150]])
def test_gla_stage_output_on_chunked_intermediates_equals_recurrence(offsets):
    B, T, H, K, V = (2 if offsets is None else 1), 150, 2, 8, 6
    q, k, v = _rand(B, T, H, K, seed=11), _rand(B, T, H, K, seed=12), _rand(B, T, H, V, seed=13)
    gk = F.logsigmoid(_rand(B, T, H, K, seed=14))
    o, _ = recurrent.naive_recurrent_gla(q, k, v, gk, offsets=offsets, dtype=D)
    r = chunked.chunked_gla(q, k, v, gk, offsets=offsets, dtype=D)
    # garbage above the diagonal of A must not matter (the stage masks it)
    A = r['A'] + torch.triu(torch.ones(64, 64, dtype=D), 1)[torch.arange(T) % 64 if offsets is None else _pos_in_chunk(offsets, T)][None, :, None, :]
    got = chunked.gla_fwd_o_gk(q, v, r['g_cumsum'], A, r['h'], K ** -0.5, offsets=offsets, dtype=D)
    torch.testing.assert_close(got, o, rtol=1e-10, atol=1e-10)


def _pos_in_chunk(offsets, T):
    pos = torch.zeros(T, dtype=torch.long)
    for bos, eos in zip(offsets[:-1], offsets[1:]):
        pos[bos:eos] = torch.arange(eos - bos) % 64
    return pos


@pytest.mark.parametrize("offsets", [None, [0, 40, 41, 150]])
def test_gla_stage_gradients_match_autograd_through_the_chunk_step(offsets):
    """dA and dv are the gradients of  sum(do * o) + sum(dh_next * h_next)  w.r.t. the unscaled scores
    and v, where o = (s q e^G) h + tril(s S) v and h_next = e^{G_last} h + (k e^{G_last - G})^T v
    (the chunk step that chunked_gla, pinned against the recurrence, is built from)."""
    B, T, H, K, V = (2 if offsets is None else 1), 150, 2, 8, 6
    q, k = _rand(B, T, H, K, seed=21), _rand(B, T, H, K, seed=22)
    v = _rand(B, T, H, V, seed=23).requires_grad_()
    G = cumsum.chunk_local_cumsum(F.logsigmoid(_rand(B, T, H, K, seed=24)), 64, offsets=offsets).to(D)
    S = _rand(B, T, H, 64, seed=25).requires_grad_()
    do = _rand(B, T, H, V, seed=26)
    spans = recurrent._spans(B, T, offsets)
    chunks = [(b, s, min(s + 64, eos)) for b, bos, eos in spans for s in range(bos, eos, 64)]
    NT = len(chunks)
    h = _rand(NT, H, K, V, seed=27)
    dh_next = _rand(NT, H, K, V, seed=28)
    scale = 0.37
    loss = 0.
    for c, (b, s, e) in enumerate(chunks):
        L = e - s
        Ac = torch.tril((scale * S[b, s:e, :, :L]).permute(1, 0, 2))                    # [H, i, j]
        o = (torch.einsum('ihk,hkv->ihv', scale * q[b, s:e] * G[b, s:e].exp(), h[c])
             + torch.einsum('hij,jhv->ihv', Ac, v[b, s:e]))
        kd = k[b, s:e] * (G[b, e - 1][None] - G[b, s:e]).exp()
        h_next = h[c] * G[b, e - 1].exp()[:, :, None] + torch.einsum('jhk,jhv->hkv', kd, v[b, s:e])
        loss = loss + (do[b, s:e] * o).sum() + (dh_next[c] * h_next).sum()
    gv, gS = torch.autograd.grad(loss, [v, S])
    states = dh_next.reshape(B, NT // B, H, K, V) if offsets is None else dh_next[None]
    dv = chunked.gla_bwd_dv(k, G, (scale * S).detach(), do, states, offsets=offsets, dtype=D)
    dA = chunked.gla_bwd_dA(v.detach(), do, scale, offsets=offsets, dtype=D)
    torch.testing.assert_close(dv, gv, rtol=1e-10, atol=1e-10)
    # autograd leaves the entries of S above the diagonal (and beyond a short chunk) at zero, as dA does
    torch.testing.assert_close(dA, gS, rtol=1e-10, atol=1e-10)


@pytest.mark.parametrize("offsets", [None, [0, 40, 41, 150]])
@pytest.mark.parametrize("gates", ["gk", "g", "both", "none", "gv", "all"])
def test_chunk_bwd_dh_matches_autograd_through_the_state_chain(offsets, gates):
    """dh[c] is the gradient of  sum(do * o) + sum(dht * ht)  w.r.t. the state leaving chunk c (taken with a
    zero tap added to every state), dh0 the one w.r.t. the initial state; only the inter-chunk part of o sees
    the states:  o = ((s q e^{g} e^{gk}) h) e^{gv},
    h_next = e^{g_last} diag(e^{gk_last}) h diag(e^{gv_last}) + (k e^{gk_last - gk})^T (v e^{g_last - g} e^{gv_last - gv})."""
    B, T, H, K, V = (2 if offsets is None else 1), 150, 2, 8, 6
    N = B if offsets is None else len(offsets) - 1
    q, k, v = _rand(B, T, H, K, seed=31), _rand(B, T, H, K, seed=32), _rand(B, T, H, V, seed=33)
    gk = cumsum.chunk_local_cumsum(F.logsigmoid(_rand(B, T, H, K, seed=34)), 64, offsets=offsets).to(D)
    g = cumsum.chunk_local_cumsum(F.logsigmoid(_rand(B, T, H, seed=35)), 64, offsets=offsets).to(D)
    gv = cumsum.chunk_local_cumsum(F.logsigmoid(_rand(B, T, H, V, seed=39)), 64, offsets=offsets).to(D)
    if gates not in ("gk", "both", "all"):
        gk = None
    if gates not in ("g", "both", "all"):
        g = None
    if gates not in ("gv", "all"):
        gv = None
    do, dht = _rand(B, T, H, V, seed=36), _rand(N, H, K, V, seed=37)
    h0 = _rand(N, H, K, V, seed=38).requires_grad_()
    scale = 0.41
    taps, loss, entering, finals = [], 0., [], []
    for n, (b, bos, eos) in enumerate(recurrent._spans(B, T, offsets)):
        h = h0[n]
        for s in range(bos, eos, 64):
            e = min(s + 64, eos)
            entering.append(h.detach())
            lg = torch.zeros(e - s, H, K, dtype=D)
            lv = torch.zeros(e - s, H, V, dtype=D)
            if g is not None:
                lg = lg + g[b, s:e][..., None]
            if gk is not None:
                lg = lg + gk[b, s:e]
            if gv is not None:
                lv = lv + gv[b, s:e]
            o = torch.einsum('thk,hkv->thv', scale * q[b, s:e] * lg.exp(), h) * lv.exp()
            loss = loss + (do[b, s:e] * o).sum()
            kd = k[b, s:e] * (lg[-1][None] - lg).exp()
            vd = v[b, s:e] * (lv[-1][None] - lv).exp()
            tap = torch.zeros(H, K, V, dtype=D, requires_grad=True)
            taps.append(tap)
            h = h * lg[-1].exp()[:, :, None] * lv[-1].exp()[:, None, :] + torch.einsum('thk,thv->hkv', kd, vd) + tap
        loss = loss + (dht[n] * h).sum()
        finals.append(h.detach())
    grads = torch.autograd.grad(loss, [h0] + taps)
    dh, dh0 = chunked.chunk_bwd_dh(q, g, gk, do, dht, scale, offsets=offsets, dtype=D, gv=gv)
    torch.testing.assert_close(dh0, grads[0], rtol=1e-10, atol=1e-10)
    torch.testing.assert_close(dh.reshape(-1, H, K, V), torch.stack(grads[1:], 0), rtol=1e-10, atol=1e-10)
    # the forward states of the same chain, as chunk_fwd_h restates them
    hs, ht = chunked.chunk_fwd_h(k, v, g, gk, gv, h0.detach(), offsets=offsets, dtype=D)
    torch.testing.assert_close(hs.reshape(-1, H, K, V), torch.stack(entering, 0), rtol=1e-10, atol=1e-10)
    torch.testing.assert_close(ht, torch.stack(finals, 0), rtol=1e-10, atol=1e-10)


@pytest.mark.parametrize("offsets", [None, [0, 40, 41, 150]])
@pytest.mark.parametrize("gates", ["gk", "gv", "g", "all"])
def test_chunk_fwd_h_final_state_matches_the_recurrence(offsets, gates):
    """The chunked state scan ends where the token-by-token recurrence ends, for every kind of gate (the chunk
    form takes cumulative gates, the recurrence raw ones), and its stored states are the recurrence's states at
    the chunk boundaries (checked through a run that stops there)."""
    B, T, H, K, V = (2 if offsets is None else 1), 150, 2, 8, 6
    N = B if offsets is None else len(offsets) - 1
    q, k, v = _rand(B, T, H, K, seed=51), _rand(B, T, H, K, seed=52), _rand(B, T, H, V, seed=53)
    raw = dict(gk=F.logsigmoid(_rand(B, T, H, K, seed=54)), g=F.logsigmoid(_rand(B, T, H, seed=55)),
               gv=F.logsigmoid(_rand(B, T, H, V, seed=56)))
    use = {"gk": ("gk",), "gv": ("gv",), "g": ("g",), "all": ("gk", "g", "gv")}[gates]
    raw = {n: (x if n in use else None) for n, x in raw.items()}
    def local_cumsum(x):   # in the test's own precision (the oracle's cumsum returns fp32, like the reference's)
        out = torch.empty_like(x)
        for b, bos, eos in recurrent._spans(B, T, offsets):
            for s in range(bos, eos, 64):
                out[b, s:min(s + 64, eos)] = torch.cumsum(x[b, s:min(s + 64, eos)], 0)
        return out

    cum = {n: (None if x is None else local_cumsum(x)) for n, x in raw.items()}
    h0 = _rand(N, H, K, V, seed=57)
    hs, ht = chunked.chunk_fwd_h(k, v, cum["g"], cum["gk"], cum["gv"], h0, offsets=offsets, dtype=D)
    _, rht = recurrent.naive_recurrent_gla(q, k, v, gk=raw["gk"], g=raw["g"], gv=raw["gv"], initial_state=h0,
                                           output_final_state=True, offsets=offsets, dtype=D)
    torch.testing.assert_close(ht, rht, rtol=1e-10, atol=1e-10)
    if offsets is None:
        # the state entering chunk 1 is the final state of a run over the first 64 tokens
        cut = lambda x: None if x is None else x[:, :64]
        _, r64 = recurrent.naive_recurrent_gla(q[:, :64], k[:, :64], v[:, :64], gk=cut(raw["gk"]), g=cut(raw["g"]),
                                               gv=cut(raw["gv"]), initial_state=h0, output_final_state=True, dtype=D)
        torch.testing.assert_close(hs[:, 1], r64, rtol=1e-10, atol=1e-10)
        torch.testing.assert_close(hs[:, 0], h0, rtol=0, atol=0)


@pytest.mark.parametrize("offsets", [None, [0, 40, 41, 150]])
@pytest.mark.parametrize("gated", [True, False])
def test_chunk_bwd_dv_local_matches_autograd_of_the_intra_chunk_output(offsets, gated):
    """dv_local is the gradient w.r.t. v of  sum(do * o_intra),  o_intra_i = s sum_{j<=i} (q_i . k_j) e^{g_i-g_j} v_j
    (the intra-chunk term of chunk_fwd_o, fla/ops/common/chunk_o.py:86-101)."""
    B, T, H, K, V = (2 if offsets is None else 1), 150, 2, 8, 6
    q, k = _rand(B, T, H, K, seed=41), _rand(B, T, H, K, seed=42)
    v = _rand(B, T, H, V, seed=43).requires_grad_()
    do = _rand(B, T, H, V, seed=44)
    g = cumsum.chunk_local_cumsum(F.logsigmoid(_rand(B, T, H, seed=45)), 64, offsets=offsets).to(D) if gated else None
    scale, loss = 0.29, 0.
    for b, bos, eos in recurrent._spans(B, T, offsets):
        for s in range(bos, eos, 64):
            e = min(s + 64, eos)
            A = scale * torch.einsum('ihk,jhk->hij', q[b, s:e], k[b, s:e])
            if gated:
                A = A * (g[b, s:e].t()[:, :, None] - g[b, s:e].t()[:, None, :]).exp()
            loss = loss + (do[b, s:e] * torch.einsum('hij,jhv->ihv', torch.tril(A), v[b, s:e])).sum()
    gv, = torch.autograd.grad(loss, [v])
    got = chunked.chunk_bwd_dv_local(q, k, g, do, scale, offsets=offsets, dtype=D)
    torch.testing.assert_close(got, gv, rtol=1e-10, atol=1e-10)


# ---------------------------------------------------------------- stages of the delta rule's backward
def _gdr_chunks(B, T, offsets):
    return [(n, b, s, min(s + 64, eos)) for n, (b, bos, eos) in enumerate(recurrent._spans(B, T, offsets))
            for s in range(bos, eos, 64)]


def _local_cumsum64(x, B, T, offsets, reverse=False):
    out = torch.zeros_like(x)
    for _, b, s, e in _gdr_chunks(B, T, offsets):
        blk = x[b, s:e]
        out[b, s:e] = blk.flip(0).cumsum(0).flip(0) if reverse else blk.cumsum(0)
    return out


@pytest.mark.parametrize("offsets", [None, [0, 40, 41, 150]])
@pytest.mark.parametrize("gated", [True, False])
def test_gdr_backward_stages_match_autograd_through_the_chunk_step(offsets, gated):
    """With q, k, w, u and the cumulative gate as independent leaves, the chunk step
      v_new = u - (w e^g) h,  o = s (e^g (q h) + tril(q k^T * Gamma) v_new),  h_next = e^{g_last} h + (k e^{g_last-g})^T v_new
    chained over the chunks has, for  sum(do * o) + sum(dht * ht):  d/du = dv2 and d/d(state leaving a chunk) = dh
    (reverse scan), d/dq, d/dk, d/dw, d/dg = the outputs of chunk_bwd_dqkwg, d/dh0 = dh0."""
    B, T, H, K, V = (2 if offsets is None else 1), 150, 2, 8, 6
    N = B if offsets is None else len(offsets) - 1
    q, k, w = (_rand(B, T, H, K, seed=s).requires_grad_() for s in (51, 52, 53))
    u = _rand(B, T, H, V, seed=54).requires_grad_()
    G = None
    if gated:
        G = _local_cumsum64(F.logsigmoid(_rand(B, T, H, seed=55)), B, T, offsets).requires_grad_()
    do, dht = _rand(B, T, H, V, seed=56), _rand(N, H, K, V, seed=57)
    h0 = (0.3 * _rand(N, H, K, V, seed=58)).requires_grad_()
    scale = 0.33
    taps, hs, vns, loss = [], [], torch.zeros(B, T, H, V, dtype=D), 0.
    h, last_n = None, -1
    for n, b, s, e in _gdr_chunks(B, T, offsets):
        if n != last_n:
            if last_n >= 0:
                loss = loss + (dht[last_n] * h).sum()
            h, last_n = h0[n], n
        L = e - s
        gc = torch.zeros(L, H, dtype=D) if G is None else G[b, s:e]
        lower = torch.tril(torch.ones(L, L, dtype=D))
        Gam = ((gc[:, None] - gc[None, :]).permute(2, 0, 1) * lower).exp() * lower
        eg = gc.exp()[..., None]
        hs.append(h.detach())
        vn = u[b, s:e] - torch.einsum('ihk,hkv->ihv', w[b, s:e] * eg, h)
        vns[b, s:e] = vn.detach()
        P = torch.einsum('ihk,jhk->hij', q[b, s:e], k[b, s:e]) * Gam
        o = scale * (eg * torch.einsum('ihk,hkv->ihv', q[b, s:e], h) + torch.einsum('hij,jhv->ihv', P, vn))
        loss = loss + (do[b, s:e] * o).sum()
        tap = torch.zeros(H, K, V, dtype=D, requires_grad=True)
        taps.append(tap)
        kd = k[b, s:e] * (gc[-1][None] - gc).exp()[..., None]
        h = h * gc[-1].exp()[:, None, None] + torch.einsum('jhk,jhv->hkv', kd, vn) + tap
    loss = loss + (dht[last_n] * h).sum()
    leaves = [q, k, w, u, h0] + ([G] if gated else [])
    grads = torch.autograd.grad(loss, leaves + taps)
    gq, gk, gw, gu, gh0 = grads[:5]
    gtaps = torch.stack(grads[len(leaves):], 0)
    states = torch.stack(hs, 0)
    states = states.reshape(B, -1, H, K, V) if offsets is None else states[None]
    Gd = None if G is None else G.detach()
    qd, kd_, wd = q.detach(), k.detach(), w.detach()
    dvl = chunked.chunk_bwd_dv_local(qd, kd_, Gd, do, scale, offsets=offsets, dtype=D)
    dh, dh0, dv2 = chunked.gdr_bwd_dhu(qd, kd_, wd, Gd, dht, do, dvl, scale, offsets=offsets, dtype=D)
    dq, dk, dw, dg = chunked.chunk_bwd_dqkwg(qd, kd_, vns, Gd, do, states, dh, dv2, wd, scale, offsets=offsets, dtype=D)
    tol = dict(rtol=1e-9, atol=1e-9)
    torch.testing.assert_close(dv2, gu, **tol)
    torch.testing.assert_close(dh.reshape(-1, H, K, V), gtaps, **tol)
    torch.testing.assert_close(dh0, gh0, **tol)
    torch.testing.assert_close(dq, gq, **tol)
    torch.testing.assert_close(dk, gk, **tol)
    torch.testing.assert_close(dw, gw, **tol)
    if gated:
        torch.testing.assert_close(dg, grads[5], **tol)
    else:
        assert dg is None


@pytest.mark.parametrize("offsets", [None, [0, 40, 41, 150]])
def test_bwd_prepare_wy_repr_matches_autograd_through_the_wy_map(offsets):
    """(dk, dv, dbeta, dg) are the gradients of  sum(dw * w) + sum(du * u)  with w = (I + M)^-1 (beta k),
    u = (I + M * Gamma)^-1 (beta v), M = strict_lower(diag(beta) k k^T), both inverses by triangular solves."""
    B, T, H, K, V = (2 if offsets is None else 1), 150, 2, 8, 6
    k = F.normalize(_rand(B, T, H, K, seed=61), dim=-1).requires_grad_()
    v = _rand(B, T, H, V, seed=62).requires_grad_()
    beta = torch.rand(B, T, H, dtype=D, generator=torch.Generator().manual_seed(63)).requires_grad_()
    G = _local_cumsum64(F.logsigmoid(_rand(B, T, H, seed=64)), B, T, offsets).requires_grad_()
    dw, du = _rand(B, T, H, K, seed=65), _rand(B, T, H, V, seed=66)
    Aw = torch.zeros(B, T, H, 64, dtype=D)
    Au = torch.zeros(B, T, H, 64, dtype=D)
    loss = 0.
    for _, b, s, e in _gdr_chunks(B, T, offsets):
        L = e - s
        gc = G[b, s:e]
        eye = torch.eye(L, dtype=D)
        strict, lower = torch.tril(torch.ones(L, L, dtype=D), -1), torch.tril(torch.ones(L, L, dtype=D))
        kb, vb = k[b, s:e] * beta[b, s:e, :, None], v[b, s:e] * beta[b, s:e, :, None]
        M = torch.einsum('ihk,jhk->hij', kb, k[b, s:e]) * strict
        Gam = ((gc[:, None] - gc[None, :]).permute(2, 0, 1) * lower).exp() * lower
        aw = torch.linalg.solve_triangular(eye + M, eye.expand(H, L, L), upper=False)
        au = torch.linalg.solve_triangular(eye + M * Gam, eye.expand(H, L, L), upper=False)
        Aw[b, s:e, :, :L], Au[b, s:e, :, :L] = aw.detach().permute(1, 0, 2), au.detach().permute(1, 0, 2)
        loss = loss + (dw[b, s:e] * torch.einsum('hij,jhk->ihk', aw, kb)).sum()
        loss = loss + (du[b, s:e] * torch.einsum('hij,jhv->ihv', au, vb)).sum()
    gk, gv, gb, gG = torch.autograd.grad(loss, [k, v, beta, G])
    dk, dv, dbeta, dg = chunked.bwd_prepare_wy_repr(k.detach(), v.detach(), G.detach(), beta.detach(), Aw, dw, du,
                                                    offsets=offsets, dtype=D)
    tol = dict(rtol=1e-9, atol=1e-9)
    torch.testing.assert_close(dk, gk, **tol)
    torch.testing.assert_close(dv, gv, **tol)
    torch.testing.assert_close(dbeta, gb, **tol)
    torch.testing.assert_close(dg, gG, **tol)
    # the second inverse is the first one rescaled: what lets the stage take Aw alone
    torch.testing.assert_close(Au, Aw * _gamma_rows(G.detach(), B, T, offsets), **tol)


def _gamma_rows(G, B, T, offsets):
    """e^{g_i - g_j} for j <= i laid out like Aw: [B, T, H, 64], zero elsewhere."""
    out = torch.zeros(B, T, G.shape[-1], 64, dtype=D)
    for _, b, s, e in _gdr_chunks(B, T, offsets):
        L = e - s
        gc = G[b, s:e]
        lower = torch.tril(torch.ones(L, L, dtype=D))
        out[b, s:e, :, :L] = (((gc[:, None] - gc[None, :]) * lower[..., None]).exp() * lower[..., None]).permute(0, 2, 1)
    return out


@pytest.mark.parametrize("offsets", [None, [0, 40, 41, 150]])
def test_gdr_backward_stages_compose_to_autograd_through_the_recurrence(offsets):
    """The reference's order (fla/ops/gated_delta_rule/chunk.py:76-177) on the oracle's stages: recompute w, u and
    the states, dv_local, reverse scan, dq/dk/dw/dg, WY gradient, dk and dg summed, reverse chunk-local cumsum of dg;
    against autograd through the token-by-token recurrence."""
    B, T, H, K, V = (2 if offsets is None else 1), 150, 2, 8, 6
    N = B if offsets is None else len(offsets) - 1
    q = _rand(B, T, H, K, seed=71).requires_grad_()
    k = F.normalize(_rand(B, T, H, K, seed=72), dim=-1).requires_grad_()
    v = _rand(B, T, H, V, seed=73).requires_grad_()
    g = F.logsigmoid(_rand(B, T, H, seed=74)).requires_grad_()
    beta = torch.rand(B, T, H, dtype=D, generator=torch.Generator().manual_seed(75)).requires_grad_()
    h0 = (0.3 * _rand(N, H, K, V, seed=76)).requires_grad_()
    do, dht = _rand(B, T, H, V, seed=77), _rand(N, H, K, V, seed=78)
    scale = K ** -0.5
    o, ht = recurrent.naive_recurrent_gated_delta_rule(q, k, v, g, beta, scale=scale, initial_state=h0,
                                                       output_final_state=True, offsets=offsets, dtype=D)
    want = torch.autograd.grad((do * o).sum() + (dht * ht).sum(), [q, k, v, g, beta, h0])
    qd, kd, vd, gd, bd = (x.detach() for x in (q, k, v, g, beta))
    r = chunked.chunked_gated_delta_rule(qd, kd, vd, gd, bd, scale=scale, initial_state=h0.detach(), offsets=offsets, dtype=D)
    G = r['g_cumsum']
    w, u = chunked.fwd_recompute_w_u(kd, vd, bd, r['Aw'], r['Au'], offsets=offsets, dtype=D)
    torch.testing.assert_close(w, r['w'], rtol=1e-10, atol=1e-10)
    torch.testing.assert_close(u, r['u'], rtol=1e-10, atol=1e-10)
    dvl = chunked.chunk_bwd_dv_local(qd, kd, G, do, scale, offsets=offsets, dtype=D)
    dh, dh0, dv2 = chunked.gdr_bwd_dhu(qd, kd, w, G, dht, do, dvl, scale, offsets=offsets, dtype=D)
    dq, dk, dw, dg = chunked.chunk_bwd_dqkwg(qd, kd, r['v_new'], G, do, r['h'], dh, dv2, w, scale, offsets=offsets, dtype=D)
    dk2, dv, db, dg2 = chunked.bwd_prepare_wy_repr(kd, vd, G, bd, r['Aw'], dw, dv2, offsets=offsets, dtype=D)
    dg = _local_cumsum64(dg + dg2, B, T, offsets, reverse=True)
    tol = dict(rtol=1e-8, atol=1e-8)
    for name, got, ref in zip("dq dk dv dg dbeta dh0".split(), (dq, dk + dk2, dv, dg, db, dh0), want):
        torch.testing.assert_close(got, ref, msg=lambda m, name=name: f"{name}: {m}", **tol)


@pytest.mark.parametrize("offsets", [None, [0, 40, 41, 150]])
@pytest.mark.parametrize("gated", [True, False])
def test_chunk_bwd_dv_matches_autograd_of_the_scalar_gated_chunk_step(offsets, gated):
    """dv is the gradient w.r.t. v of  sum(do * o) + sum(dh * h_next)  for  o_i = s sum_{j<=i} (q_i . k_j) e^{g_i-g_j} v_j
    (+ a term without v)  and  h_next = e^{g_last} h + (k e^{g_last-g})^T v."""
    B, T, H, K, V = (2 if offsets is None else 1), 150, 2, 8, 6
    q, k = _rand(B, T, H, K, seed=81), _rand(B, T, H, K, seed=82)
    v = _rand(B, T, H, V, seed=83).requires_grad_()
    do = _rand(B, T, H, V, seed=84)
    g = _local_cumsum64(F.logsigmoid(_rand(B, T, H, seed=85)), B, T, offsets) if gated else None
    chunks = _gdr_chunks(B, T, offsets)
    dh = _rand(len(chunks), H, K, V, seed=86)
    scale, loss = 0.29, 0.
    for c, (_, b, s, e) in enumerate(chunks):
        gc = torch.zeros(e - s, H, dtype=D) if g is None else g[b, s:e]
        A = scale * torch.einsum('ihk,jhk->hij', q[b, s:e], k[b, s:e]) * (gc.t()[:, :, None] - gc.t()[:, None, :]).exp()
        loss = loss + (do[b, s:e] * torch.einsum('hij,jhv->ihv', torch.tril(A), v[b, s:e])).sum()
        kd = k[b, s:e] * (gc[-1][None] - gc).exp()[..., None]
        loss = loss + (dh[c] * torch.einsum('jhk,jhv->hkv', kd, v[b, s:e])).sum()
    gv, = torch.autograd.grad(loss, [v])
    states = dh.reshape(B, -1, H, K, V) if offsets is None else dh[None]
    got = chunked.chunk_bwd_dv(q, k, g, do, states, scale, offsets=offsets, dtype=D)
    torch.testing.assert_close(got, gv, rtol=1e-10, atol=1e-10)
