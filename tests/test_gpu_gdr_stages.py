"""GPU: the stages of the delta rule's backward under the reference's internal signatures
(``chunk_gated_delta_rule_bwd_dhu`` of ``fla/ops/common/chunk_delta_h.py:323``, ``chunk_bwd_dqkwg`` /
``chunk_bwd_dv`` of ``fla/ops/common/chunk_o.py:602,499``, ``bwd_prepare_wy_repr`` / ``fwd_recompute_w_u`` of
``fla/ops/gated_delta_rule/wy_fast.py:565,320``) with row-major per-chunk states, against the fp32 oracle
evaluated on the same 16-bit operands.

Tolerances (rel-L2): 8e-3 on dq, dk, dv, dw, w, u, dh, dh0 and 2e-2 on dbeta, dg, the reference's own bounds for
the whole backward (``tests/ops/test_gated_delta.py:220-294``)."""
import pytest
import torch

from helpers import assert_close, gdr_inputs, random_offsets

pytestmark = pytest.mark.gpu

TOL, TOL_G = 8e-3, 2e-2


def _case(B, T, H, K, V, varlen, seed, dtype=torch.bfloat16, gated=True):
    """Inputs, the oracle's forward intermediates rounded to the storage type, and random cotangents."""
    from oracle import chunked
    N = 4 if varlen else B
    offs = random_offsets(T, N, torch.Generator().manual_seed(seed), min_len=1) if varlen else None
    q, k, v, g, beta, h0 = gdr_inputs(1 if varlen else B, T, H, K, V, seed=seed, dtype=dtype, N=N, h0_std=0.5)
    if not gated:
        g = None
    ol = None if offs is None else offs.tolist()
    scale = K ** -0.5
    r = chunked.chunked_gated_delta_rule(q, k, v, g, beta, scale=scale, initial_state=h0, offsets=ol)
    gen = torch.Generator().manual_seed(seed + 1)
    rd = lambda x: x.to(dtype)
    c = dict(q=q, k=k, v=v, g=g, beta=beta, h0=h0, offs=offs, ol=ol, scale=scale, N=N,
             G=r["g_cumsum"] if gated else None, Aw=rd(r["Aw"]), Au=rd(r["Au"]), w=rd(r["w"]), u=rd(r["u"]),
             v_new=rd(r["v_new"]), h=rd(r["h"]),
             do=torch.randn(v.shape, generator=gen).to(dtype), dht=torch.randn(N, H, K, V, generator=gen) * 0.1)
    return c


def _dev(device):
    return lambda x: None if x is None else x.to(device)


SHAPES = [
    # B, T, H, K, V
    (2, 256, 3, 128, 128),
    (2, 200, 2, 64, 64),
    (1, 300, 2, 128, 64),
    (2, 130, 2, 64, 128),
    (2, 150, 2, 256, 128),
    (2, 40, 2, 128, 128),
]


@pytest.mark.parametrize("B,T,H,K,V", SHAPES)
@pytest.mark.parametrize("varlen", [False, True])
def test_fwd_recompute_w_u_reference_operands(device, B, T, H, K, V, varlen):
    from fla_amd.ops.gated_delta_rule.wy_fast import fwd_recompute_w_u
    from oracle import chunked
    if varlen and T < 64:
        pytest.skip("packed case covered at the longer shapes")
    c = _case(B, T, H, K, V, varlen, seed=T + K)
    d = _dev(device)
    print(f"fwd_recompute_w_u B={B} T={T} H={H} K={K} V={V} varlen={varlen}", flush=True)
    w, u = fwd_recompute_w_u(d(c["k"]), d(c["v"]), d(c["beta"]), d(c["Aw"]), d(c["Au"]), offsets=d(c["offs"]),
                             head_first=False)
    torch.cuda.synchronize()
    rw, ru = chunked.fwd_recompute_w_u(c["k"], c["v"], c["beta"], c["Aw"], c["Au"], offsets=c["ol"])
    assert w.dtype == c["k"].dtype and u.dtype == c["v"].dtype
    assert_close("w", rw, w, TOL)
    assert_close("u", ru, u, TOL)


@pytest.mark.parametrize("B,T,H,K,V", SHAPES)
@pytest.mark.parametrize("varlen", [False, True])
@pytest.mark.parametrize("gated", [True, False])
def test_chunk_gated_delta_rule_bwd_dhu_reference_operands(device, B, T, H, K, V, varlen, gated):
    from fla_amd.ops.common.chunk_delta_h import chunk_gated_delta_rule_bwd_dhu
    from oracle import chunked
    if varlen and T < 64:
        pytest.skip("packed case covered at the longer shapes")
    c = _case(B, T, H, K, V, varlen, seed=T + K + 1, gated=gated)
    d = _dev(device)
    dvl = chunked.chunk_bwd_dv_local(c["q"], c["k"], c["G"], c["do"], c["scale"], offsets=c["ol"]).to(c["v"].dtype)
    print(f"bwd_dhu B={B} T={T} H={H} K={K} V={V} varlen={varlen} gated={gated}", flush=True)
    dh, dh0, dv2 = chunk_gated_delta_rule_bwd_dhu(d(c["q"]), d(c["k"]), d(c["w"]), d(c["G"]), d(c["h0"]), d(c["dht"]),
                                                  d(c["do"]), d(dvl), c["scale"], offsets=d(c["offs"]), head_first=False)
    torch.cuda.synchronize()
    rdh, rdh0, rdv2 = chunked.gdr_bwd_dhu(c["q"], c["k"], c["w"], c["G"], c["dht"], c["do"], dvl, c["scale"],
                                          offsets=c["ol"])
    assert dh.dtype == c["q"].dtype and dh0.dtype == torch.float32 and dv2.dtype == c["v"].dtype
    assert_close("dh", rdh, dh, TOL)
    assert_close("dh0", rdh0, dh0, TOL)
    assert_close("dv2", rdv2, dv2, TOL)
    # without an initial state the reference returns no dh0
    _, none0, _ = chunk_gated_delta_rule_bwd_dhu(d(c["q"]), d(c["k"]), d(c["w"]), d(c["G"]), None, None, d(c["do"]),
                                                 d(dvl), c["scale"], offsets=d(c["offs"]), head_first=False)
    assert none0 is None


@pytest.mark.parametrize("B,T,H,K,V", SHAPES)
@pytest.mark.parametrize("varlen", [False, True])
@pytest.mark.parametrize("gated", [True, False])
def test_chunk_bwd_dqkwg_reference_operands(device, B, T, H, K, V, varlen, gated):
    from fla_amd.ops.common.chunk_o import chunk_bwd_dqkwg
    from oracle import chunked
    if varlen and T < 64:
        pytest.skip("packed case covered at the longer shapes")
    c = _case(B, T, H, K, V, varlen, seed=T + K + 2, gated=gated)
    d = _dev(device)
    dt = c["q"].dtype
    dvl = chunked.chunk_bwd_dv_local(c["q"], c["k"], c["G"], c["do"], c["scale"], offsets=c["ol"]).to(dt)
    dh, _, dv2 = chunked.gdr_bwd_dhu(c["q"], c["k"], c["w"], c["G"], c["dht"], c["do"], dvl, c["scale"], offsets=c["ol"])
    dh, dv2 = dh.to(dt), dv2.to(dt)
    print(f"bwd_dqkwg B={B} T={T} H={H} K={K} V={V} varlen={varlen} gated={gated}", flush=True)
    dq, dk, dw, dg = chunk_bwd_dqkwg(d(c["q"]), d(c["k"]), d(c["v_new"]), d(c["G"]), d(c["do"]), d(c["h"]), d(dh),
                                     dv=d(dv2), w=d(c["w"]), offsets=d(c["offs"]), scale=c["scale"], head_first=False)
    torch.cuda.synchronize()
    rq, rk, rw, rg = chunked.chunk_bwd_dqkwg(c["q"], c["k"], c["v_new"], c["G"], c["do"], c["h"], dh, dv2, c["w"],
                                             c["scale"], offsets=c["ol"])
    assert_close("dq", rq, dq, TOL)
    assert_close("dk", rk, dk, TOL)
    assert_close("dw", rw, dw, TOL)
    if gated:
        assert dg.dtype == torch.float32
        assert_close("dg", rg, dg, TOL_G)
    else:
        assert dg is None
    # the form the operators without a correction term use: no w, no dv, fp32 states
    dq2, dk2, dw2, _ = chunk_bwd_dqkwg(d(c["q"]), d(c["k"]), d(c["v_new"]), d(c["G"]), d(c["do"]), d(c["h"].float()),
                                       d(dh.float()), offsets=d(c["offs"]), scale=c["scale"], head_first=False)
    torch.cuda.synchronize()
    assert dw2 is None
    assert torch.equal(dq2, dq) and torch.equal(dk2, dk)


@pytest.mark.parametrize("B,T,H,K,V", SHAPES)
@pytest.mark.parametrize("varlen", [False, True])
@pytest.mark.parametrize("gated", [True, False])
def test_bwd_prepare_wy_repr_reference_operands(device, B, T, H, K, V, varlen, gated):
    from fla_amd.ops.gated_delta_rule.wy_fast import bwd_prepare_wy_repr
    from oracle import chunked
    if varlen and T < 64:
        pytest.skip("packed case covered at the longer shapes")
    c = _case(B, T, H, K, V, varlen, seed=T + K + 3, gated=gated)
    d = _dev(device)
    gen = torch.Generator().manual_seed(T)
    dw = torch.randn(c["k"].shape, generator=gen).to(c["k"].dtype)
    du = torch.randn(c["v"].shape, generator=gen).to(c["v"].dtype)
    print(f"bwd_prepare_wy_repr B={B} T={T} H={H} K={K} V={V} varlen={varlen} gated={gated}", flush=True)
    dk, dv, db, dg = bwd_prepare_wy_repr(d(c["k"]), d(c["v"]), d(c["G"]), d(c["beta"]), d(c["Aw"]), d(c["Au"]), d(dw),
                                         d(du), offsets=d(c["offs"]), indices=None, head_first=False, chunk_size=64)
    torch.cuda.synchronize()
    rk, rv, rb, rg = chunked.bwd_prepare_wy_repr(c["k"], c["v"], c["G"], c["beta"], c["Aw"], dw, du, offsets=c["ol"])
    assert db.dtype == torch.float32 and dg.dtype == torch.float32
    assert_close("dk", rk, dk, TOL)
    assert_close("dv", rv, dv, TOL)
    assert_close("dbeta", rb, db, TOL_G)
    assert_close("dg", rg, dg, TOL_G)   # without a gate: the gradient w.r.t. a gate of zeros


@pytest.mark.parametrize("B,T,H,K,V", [(2, 256, 3, 128, 128), (2, 200, 2, 64, 64), (2, 150, 2, 100, 50)])
@pytest.mark.parametrize("varlen", [False, True])
@pytest.mark.parametrize("gated", [True, False])
def test_chunk_bwd_dv_reference_operands(device, B, T, H, K, V, varlen, gated):
    """The generic dv stage (intra-chunk part + state part) with row-major dh, fp32 or 16-bit."""
    from fla_amd.ops.common.chunk_o import chunk_bwd_dv
    from oracle import chunked, cumsum
    import torch.nn.functional as F
    gen = torch.Generator().manual_seed(T + V)
    offs = random_offsets(T, 4, gen, min_len=1) if varlen else None
    ol = None if offs is None else offs.tolist()
    Bq = 1 if varlen else B
    q = torch.randn(Bq, T, H, K, generator=gen).bfloat16()
    k = torch.randn(Bq, T, H, K, generator=gen).bfloat16()
    do = torch.randn(Bq, T, H, V, generator=gen).bfloat16()
    g = cumsum.chunk_local_cumsum(F.logsigmoid(torch.randn(Bq, T, H, generator=gen)), 64, offsets=ol) if gated else None
    NT = (-(-T // 64)) if offs is None else int(sum(-(-(b - a) // 64) for a, b in zip(ol[:-1], ol[1:])))
    dh = torch.randn(Bq, NT, H, K, V, generator=gen) * 0.1
    d = _dev(device)
    print(f"chunk_bwd_dv B={B} T={T} H={H} K={K} V={V} varlen={varlen} gated={gated}", flush=True)
    dv = chunk_bwd_dv(d(q), d(k), d(g), d(do), d(dh), K ** -0.5, offsets=d(offs), head_first=False)
    torch.cuda.synchronize()
    assert dv.shape == do.shape and dv.dtype == do.dtype
    assert_close("dv", chunked.chunk_bwd_dv(q, k, g, do, dh, K ** -0.5, offsets=ol), dv, 1e-2)


@pytest.mark.parametrize("varlen", [False, True])
def test_gdr_stages_compose_to_the_operators_backward(device, varlen):
    """The reference's order of calls (fla/ops/gated_delta_rule/chunk.py:76-177) on the stage functions, every
    intermediate in the reference's layout, against the operator's own backward and the recurrence's autograd."""
    from fla_amd.ops.common.chunk_delta_h import chunk_gated_delta_rule_bwd_dhu, chunk_gated_delta_rule_fwd_h
    from fla_amd.ops.common.chunk_o import chunk_bwd_dqkwg, chunk_bwd_dv_local
    from fla_amd.ops.gated_delta_rule import chunk_gated_delta_rule
    from fla_amd.ops.gated_delta_rule.wy_fast import bwd_prepare_wy_repr, fwd_prepare_wy_repr, fwd_recompute_w_u
    from fla_amd.ops.utils.cumsum import chunk_local_cumsum
    from fla_amd.utils import VarlenPlan
    B, T, H, K, V = 2, 300, 2, 128, 128
    c = _case(B, T, H, K, V, varlen, seed=91)
    d = _dev(device)
    q, k, v, g, beta, h0, do, dht = (d(c[n]) for n in ("q", "k", "v", "g", "beta", "h0", "do", "dht"))
    offs = d(c["offs"])
    idx = None if offs is None else VarlenPlan(offs, 64).indices
    scale = c["scale"]
    print(f"gdr stages composed varlen={varlen}", flush=True)
    G = chunk_local_cumsum(g, 64, offsets=offs, indices=idx, head_first=False)
    _, _, Aw, Au = fwd_prepare_wy_repr(k, v, beta, G, offsets=offs, indices=idx, head_first=False)
    w, u = fwd_recompute_w_u(k, v, beta, Aw, Au, offsets=offs, indices=idx, head_first=False)
    h, v_new, _ = chunk_gated_delta_rule_fwd_h(k=k, w=w, u=u, g=G, initial_state=h0, output_final_state=False,
                                               offsets=offs, indices=idx, head_first=False, chunk_size=64)
    dv = chunk_bwd_dv_local(q, k, G, do, None, scale, offsets=offs, indices=idx, head_first=False)
    dh, dh0, dv = chunk_gated_delta_rule_bwd_dhu(q, k, w, G, h0, dht, do, dv, scale, offsets=offs, head_first=False)
    dq, dk, dw, dg = chunk_bwd_dqkwg(q, k, v_new, G, do, h, dh, dv=dv, w=w, offsets=offs, indices=idx, scale=scale,
                                     head_first=False)
    dk2, dv, db, dg2 = bwd_prepare_wy_repr(k, v, G, beta, Aw, Au, dw, dv, offs, idx, False, 64)
    dk = dk + dk2
    dg = chunk_local_cumsum(dg + dg2, 64, reverse=True, offsets=offs, indices=idx, head_first=False)
    torch.cuda.synchronize()
    leaves = [x.detach().clone().requires_grad_() for x in (q, k, v, g, beta, h0)]
    o, ht = chunk_gated_delta_rule(*leaves[:5], scale=scale, initial_state=leaves[5], output_final_state=True,
                                   offsets=offs, head_first=False)
    ((o.float() * do.float()).sum() + (ht * dht).sum()).backward()
    torch.cuda.synchronize()
    names = ("dq", "dk", "dv", "dg", "dbeta", "dh0")
    for name, got, leaf, tol in zip(names, (dq, dk, dv, dg, db, dh0), leaves, (TOL, TOL, TOL, TOL_G, TOL_G, TOL)):
        assert_close(name + " vs operator", leaf.grad.float().cpu(), got.float().cpu(), tol)
    from oracle import recurrent
    cl = [c[n].float().requires_grad_() for n in ("q", "k", "v", "g", "beta", "h0")]
    ro, rht = recurrent.naive_recurrent_gated_delta_rule(*cl[:5], scale=scale, initial_state=cl[5],
                                                         output_final_state=True, offsets=c["ol"])
    want = torch.autograd.grad((c["do"].float() * ro).sum() + (c["dht"] * rht).sum(), cl)
    for name, got, ref, tol in zip(names, (dq, dk, dv, dg, db, dh0), want, (TOL, TOL, TOL, TOL_G, TOL_G, TOL)):
        assert_close(name + " vs recurrence", ref, got, tol)


def test_gdr_stages_head_first_and_fp16(device):
    """head_first operands ([B,H,T,..], states [B,H,NT,K,V]) and fp16 storage give what the seq-first bf16 path gives."""
    from fla_amd.ops.common.chunk_delta_h import chunk_gated_delta_rule_bwd_dhu
    from fla_amd.ops.common.chunk_o import chunk_bwd_dqkwg
    from fla_amd.ops.gated_delta_rule.wy_fast import bwd_prepare_wy_repr, fwd_recompute_w_u
    from oracle import chunked
    B, T, H, K, V = 2, 200, 3, 64, 128
    c = _case(B, T, H, K, V, False, seed=17, dtype=torch.float16)
    d = _dev(device)
    tr = lambda x: None if x is None else d(x).transpose(1, 2).contiguous()
    dt = torch.float16
    dvl = chunked.chunk_bwd_dv_local(c["q"], c["k"], c["G"], c["do"], c["scale"]).to(dt)
    print("gdr stages head-first fp16", flush=True)
    w, u = fwd_recompute_w_u(tr(c["k"]), tr(c["v"]), tr(c["beta"]), tr(c["Aw"]), tr(c["Au"]), head_first=True)
    rw, ru = chunked.fwd_recompute_w_u(c["k"], c["v"], c["beta"], c["Aw"], c["Au"])
    assert_close("w", rw, w.transpose(1, 2), TOL)
    assert_close("u", ru, u.transpose(1, 2), TOL)
    dh, dh0, dv2 = chunk_gated_delta_rule_bwd_dhu(tr(c["q"]), tr(c["k"]), tr(c["w"]), tr(c["G"]), d(c["h0"]), d(c["dht"]),
                                                  tr(c["do"]), tr(dvl), c["scale"], head_first=True)
    rdh, rdh0, rdv2 = chunked.gdr_bwd_dhu(c["q"], c["k"], c["w"], c["G"], c["dht"], c["do"], dvl, c["scale"])
    assert dh.shape == (B, H, rdh.shape[1], K, V)
    assert_close("dh", rdh, dh.transpose(1, 2), TOL)
    assert_close("dh0", rdh0, dh0, TOL)
    assert_close("dv2", rdv2, dv2.transpose(1, 2), TOL)
    dq, dk, dw, dg = chunk_bwd_dqkwg(tr(c["q"]), tr(c["k"]), tr(c["v_new"]), tr(c["G"]), tr(c["do"]), tr(c["h"]), dh,
                                     dv=dv2, w=tr(c["w"]), scale=c["scale"], head_first=True)
    rq, rk, rww, rg = chunked.chunk_bwd_dqkwg(c["q"], c["k"], c["v_new"], c["G"], c["do"], c["h"], rdh.to(dt), rdv2.to(dt),
                                              c["w"], c["scale"])
    assert_close("dq", rq, dq.transpose(1, 2), TOL)
    assert_close("dk", rk, dk.transpose(1, 2), TOL)
    assert_close("dw", rww, dw.transpose(1, 2), TOL)
    assert_close("dg", rg, dg.transpose(1, 2), TOL_G)
    dk2, dv, db, dg2 = bwd_prepare_wy_repr(tr(c["k"]), tr(c["v"]), tr(c["G"]), tr(c["beta"]), tr(c["Aw"]), tr(c["Au"]), dw,
                                           dv2, None, None, True, 64)
    r2 = chunked.bwd_prepare_wy_repr(c["k"], c["v"], c["G"], c["beta"], c["Aw"], rww.to(dt), rdv2.to(dt))
    for name, ref, got, tol in zip(("dk2", "dv", "dbeta", "dg2"), r2, (dk2, dv, db, dg2), (TOL, TOL, TOL_G, TOL_G)):
        assert_close(name, ref, got.transpose(1, 2), tol)


@pytest.mark.parametrize("K,V", [(128, 128), (64, 96), (256, 32)])
@pytest.mark.parametrize("transposed", [False, True])
def test_fragments_to_states_inverts_states_to_fragments(device, K, V, transposed):
    from fla_amd.ops.common.chunk_o import fragments_to_states, states_to_fragments
    h = torch.randn(3, 5, 2, K, V, generator=torch.Generator().manual_seed(K + V)).to(device)
    for dt in (torch.bfloat16, torch.float16):
        fr = states_to_fragments(h, dt, transposed=transposed)
        back = fragments_to_states(fr, dt, transposed=transposed)
        back32 = fragments_to_states(fr, torch.float32, transposed=transposed)
        torch.cuda.synchronize()
        assert torch.equal(back, h.to(dt))
        assert torch.equal(back32, h.to(dt).float())


def test_gdr_stage_argument_errors(device):
    from fla_amd.ops.common.chunk_delta_h import chunk_gated_delta_rule_bwd_dhu
    from fla_amd.ops.common.chunk_o import chunk_bwd_dqkwg
    from fla_amd.ops.gated_delta_rule.wy_fast import bwd_prepare_wy_repr, fwd_recompute_w_u
    x = torch.zeros(1, 64, 1, 64, device=device, dtype=torch.bfloat16)
    s = torch.zeros(1, 64, 1, device=device)
    A = torch.zeros(1, 64, 1, 64, device=device, dtype=torch.bfloat16)
    m = torch.zeros(1, 1, 1, 64, 64, device=device)
    with pytest.raises(NotImplementedError):
        chunk_gated_delta_rule_bwd_dhu(x, x, x, s, None, None, x, x, 1.0, head_first=False, chunk_size=32)
    with pytest.raises(NotImplementedError):
        chunk_bwd_dqkwg(x.float(), x.float(), x.float(), s, x.float(), m, m, head_first=False)
    with pytest.raises(NotImplementedError):
        fwd_recompute_w_u(x[..., :48], x, s, A, A, head_first=False)
    with pytest.raises(NotImplementedError):
        bwd_prepare_wy_repr(x, x[..., :48], s, s, A, A, x, x[..., :48], None, None, False, 64)


def test_head_first_forms_of_the_forward_stages(device):
    """fwd_prepare_wy_repr, chunk_gated_delta_rule_fwd_h and chunk_fwd_o take head-first operands as the
    reference's do by default ([B,H,T,*], states [B,H,NT,K,V]): bit-identical to the seq-first results, transposed."""
    from fla_amd.ops.common.chunk_delta_h import chunk_gated_delta_rule_fwd_h
    from fla_amd.ops.common.chunk_o import chunk_fwd_o
    from fla_amd.ops.gated_delta_rule.wy_fast import fwd_prepare_wy_repr
    from fla_amd.ops.utils import chunk_local_cumsum
    B, T, H, K, V = 2, 200, 3, 128, 128
    q, k, v, g, beta, h0 = (x.to(device) for x in gdr_inputs(B, T, H, K, V, seed=77))
    gc = chunk_local_cumsum(g, 64, head_first=False)
    hf = lambda x: x.transpose(1, 2).contiguous()
    print("head-first forward stages", flush=True)
    w, u, Aw, Au = fwd_prepare_wy_repr(k, v, beta, gc, head_first=False)
    w2, u2, Aw2, Au2 = fwd_prepare_wy_repr(hf(k), hf(v), hf(beta), hf(gc), head_first=True)
    for a, b in ((w, w2), (u, u2), (Aw, Aw2), (Au, Au2)):
        assert torch.equal(a, b.transpose(1, 2))
    h, v_new, ht = chunk_gated_delta_rule_fwd_h(k, w, u, gc, h0, True, head_first=False)
    h2, v_new2, ht2 = chunk_gated_delta_rule_fwd_h(hf(k), hf(w), hf(u), hf(gc), h0, True, head_first=True)
    assert tuple(h2.shape) == (B, H, -(-T // 64), K, V)
    assert torch.equal(h, h2.transpose(1, 2)) and torch.equal(v_new, v_new2.transpose(1, 2)) and torch.equal(ht, ht2)
    o = chunk_fwd_o(q, k, v_new, h, gc, K ** -0.5, head_first=False)
    o2 = chunk_fwd_o(hf(q), hf(k), v_new2, h2, hf(gc), K ** -0.5, head_first=True)
    torch.cuda.synchronize()
    assert torch.equal(o, o2.transpose(1, 2))
