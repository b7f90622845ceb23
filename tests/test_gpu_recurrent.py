"""GPU: token-by-token recurrences (prefill and the T=1 decode step) against the
fp32 naive recurrences of the oracle on the same seeded inputs."""
import pytest
import torch
import torch.nn.functional as F

from helpers import assert_close, gdr_inputs, gla_inputs, random_offsets, rel_l2

pytestmark = pytest.mark.gpu


# shapes follow the reference ladder (tests/ops/test_gla.py:29-87): fp32, h0 ~ N(0,1)
@pytest.mark.parametrize("T", [1, 7, 300])
@pytest.mark.parametrize("D", [32, 64, 100, 128])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_fused_recurrent_gla(device, T, D, dtype):
    from fla_amd.ops.gla import fused_recurrent_gla
    from oracle.recurrent import naive_recurrent_gla
    B, H = 2, 3
    q, k, v, g, h0 = gla_inputs(B, T, H, D, D, seed=3, dtype=dtype, normalizer=1.0, h0_std=1.0)
    print(f"recurrent gla T={T} D={D} {dtype}", flush=True)
    o, ht = fused_recurrent_gla(q.to(device), k.to(device), v.to(device), g.to(device), initial_state=h0.to(device),
                                output_final_state=True, head_first=False)
    ro, rht = naive_recurrent_gla(q, k, v, g, initial_state=h0, output_final_state=True)
    tol = 1e-5 if dtype == torch.float32 else 5e-3
    assert o.dtype == dtype and ht.dtype == torch.float32
    assert_close("o", ro, o, tol)
    assert_close("ht", rht, ht, 1e-5)


def test_fused_recurrent_gla_variants(device):
    """g / gv gates, reverse, head-first, no initial state, K != V."""
    from fla_amd.ops.common.fused_recurrent import fused_recurrent
    from oracle.recurrent import naive_recurrent_gla
    gen = torch.Generator().manual_seed(4)
    B, T, H, K, V = 2, 37, 2, 64, 128
    q, k, v = torch.randn(B, T, H, K, generator=gen), torch.randn(B, T, H, K, generator=gen), torch.randn(B, T, H, V, generator=gen)
    gk = F.logsigmoid(torch.randn(B, T, H, K, generator=gen))
    gv = F.logsigmoid(torch.randn(B, T, H, V, generator=gen))
    g = F.logsigmoid(torch.randn(B, T, H, generator=gen))
    for kwargs in [dict(g=g), dict(gv=gv), dict(gk=gk, gv=gv, g=g), dict(gk=gk, reverse=True), dict()]:
        print(f"recurrent variants {list(kwargs)}", flush=True)
        dev = {n: (x.to(device) if torch.is_tensor(x) else x) for n, x in kwargs.items()}
        o, ht = fused_recurrent(q.to(device), k.to(device), v.to(device), output_final_state=True, head_first=False, **dev)
        ro, rht = naive_recurrent_gla(q, k, v, output_final_state=True, **kwargs)
        assert_close("o", ro, o, 1e-5)
        assert_close("ht", rht, ht, 1e-5)
    tr = lambda x: x.transpose(1, 2).contiguous().to(device)
    o, ht = fused_recurrent(tr(q), tr(k), tr(v), gk=tr(gk), output_final_state=True, head_first=True)
    ro, rht = naive_recurrent_gla(q, k, v, gk, output_final_state=True)
    assert_close("o head-first", ro.transpose(1, 2), o, 1e-5)
    assert_close("ht head-first", rht, ht, 1e-5)


@pytest.mark.parametrize("T,N", [(64, 2), (300, 4), (1000, 5)])
def test_fused_recurrent_gla_varlen(device, T, N):
    from fla_amd.ops.gla import fused_recurrent_gla
    from oracle.recurrent import naive_recurrent_gla
    gen = torch.Generator().manual_seed(5)
    offs = random_offsets(T, N, gen)
    q, k, v, g, h0 = gla_inputs(1, T, 2, 64, 64, seed=5, dtype=torch.float32, normalizer=1.0, N=N, h0_std=1.0)
    print(f"recurrent gla varlen offs={offs.tolist()}", flush=True)
    o, ht = fused_recurrent_gla(q.to(device), k.to(device), v.to(device), g.to(device), initial_state=h0.to(device),
                                output_final_state=True, offsets=offs.to(device), head_first=False)
    ro, rht = naive_recurrent_gla(q, k, v, g, initial_state=h0, output_final_state=True, offsets=offs.tolist())
    assert_close("o", ro, o, 1e-5)
    assert_close("ht", rht, ht, 1e-5)


# reference ladder: tests/ops/test_gated_delta.py:161-217 (bf16, k L2-normalised, h0 ~ N(0,1), tol 0.002)
@pytest.mark.parametrize("T", [1, 7, 63, 300])
@pytest.mark.parametrize("H", [2, 16])
@pytest.mark.parametrize("D", [64, 100, 128, 200])
def test_fused_recurrent_gated_delta_rule(device, T, H, D):
    from fla_amd.ops.gated_delta_rule import fused_recurrent_gated_delta_rule
    from oracle.recurrent import naive_recurrent_gated_delta_rule
    q, k, v, g, beta, h0 = gdr_inputs(2, T, H, D, D, seed=6, h0_std=1.0)
    print(f"recurrent gdr T={T} H={H} D={D}", flush=True)
    o, ht = fused_recurrent_gated_delta_rule(q.to(device), k.to(device), v.to(device), g.to(device), beta.to(device),
                                             initial_state=h0.to(device), output_final_state=True, head_first=False)
    ro, rht = naive_recurrent_gated_delta_rule(q, k, v, g, beta, initial_state=h0, output_final_state=True)
    assert o.dtype == q.dtype
    assert_close("o", ro, o, 5e-3)
    assert_close("ht", rht, ht, 2e-3)


def test_fused_recurrent_gated_delta_rule_variants(device):
    """fp32 inputs, per-value beta, beta=None, varlen, scale argument."""
    from fla_amd.ops.gated_delta_rule import fused_recurrent_gated_delta_rule
    from oracle.recurrent import naive_recurrent_gated_delta_rule
    gen = torch.Generator().manual_seed(7)
    T, H, K, V, N = 200, 3, 64, 128, 3
    q, k, v, g, beta, h0 = gdr_inputs(1, T, H, K, V, seed=7, dtype=torch.float32, N=N, h0_std=1.0)
    offs = random_offsets(T, N, gen)
    bv = torch.rand(1, T, H, V, generator=gen)
    for name, b in [("scalar", beta), ("per-value", bv), ("none", None)]:
        print(f"gdr variants beta={name}", flush=True)
        o, ht = fused_recurrent_gated_delta_rule(q.to(device), k.to(device), v.to(device), g.to(device),
                                                 None if b is None else b.to(device), scale=0.3,
                                                 initial_state=h0.to(device), output_final_state=True,
                                                 offsets=offs.to(device), head_first=False)
        ro, rht = naive_recurrent_gated_delta_rule(q, k, v, g, b, scale=0.3, initial_state=h0,
                                                   output_final_state=True, offsets=offs.tolist())
        assert_close("o", ro, o, 1e-5)
        assert_close("ht", rht, ht, 1e-5)


@pytest.mark.parametrize("T,D,varlen", [(1, 128, False), (37, 128, False), (5, 64, False), (3, 100, False), (40, 128, True)])
def test_fused_recurrent_gated_delta_rule_l2norm_in_kernel(device, T, D, varlen):
    """use_qk_l2norm_in_kernel on raw q, k == l2_norm in front of the operator (the layer's form,
    fla/layers/gated_deltanet.py:234-237), and both match the oracle on normalised rows."""
    from fla_amd.modules import l2_norm
    from fla_amd.ops.gated_delta_rule import fused_recurrent_gated_delta_rule
    from oracle.recurrent import naive_recurrent_gated_delta_rule
    torch.manual_seed(5)
    B, H = (1, 3) if varlen else (2, 3)
    offsets = torch.tensor([0, 7, 8, T], device=device) if varlen else None
    N = 3 if varlen else B
    q = (torch.randn(B, T, H, D, device=device) * 3).bfloat16()
    k = (torch.randn(B, T, H, D, device=device) * 0.2).bfloat16()
    v = torch.randn(B, T, H, D, device=device).bfloat16()
    g = F.logsigmoid(torch.randn(B, T, H, device=device))
    beta = torch.rand(B, T, H, device=device)
    h0 = torch.randn(N, H, D, D, device=device) * 0.1
    o1, ht1 = fused_recurrent_gated_delta_rule(q, k, v, g, beta, initial_state=h0, output_final_state=True,
                                               offsets=offsets, head_first=False, use_qk_l2norm_in_kernel=True)
    # (the stand-alone kernel takes rows that are multiples of 8 elements)
    nrm = l2_norm if D % 8 == 0 else (lambda x: F.normalize(x.float(), dim=-1, eps=1e-6).to(x.dtype))
    qn, kn = nrm(q), nrm(k)
    o2, ht2 = fused_recurrent_gated_delta_rule(qn, kn, v, g, beta, initial_state=h0, output_final_state=True,
                                               offsets=offsets, head_first=False)
    # the separate launches round the normalised rows to bf16, the fused step keeps them in fp32
    assert rel_l2(o1, o2) < 6e-3 and rel_l2(ht1, ht2) < 6e-3
    qf, kf = q.float(), k.float()
    qr = (qf / torch.sqrt((qf * qf).sum(-1, keepdim=True) + 1e-6)).cpu()
    kr = (kf / torch.sqrt((kf * kf).sum(-1, keepdim=True) + 1e-6)).cpu()
    o_ref, ht_ref = naive_recurrent_gated_delta_rule(qr, kr, v.float().cpu(), g.cpu(), beta.cpu(), initial_state=h0.cpu(),
                                                     output_final_state=True,
                                                     offsets=None if offsets is None else offsets.cpu())
    assert rel_l2(o1.float().cpu(), o_ref) < 5e-3
    assert rel_l2(ht1.cpu(), ht_ref) < 1e-4


@pytest.mark.parametrize("op", ["gla", "gdr"])
def test_decode_inplace_matches_out_of_place(device, op):
    """T=1 decode steps: the in-place state update equals the out-of-place one, and a
    run of single steps equals one recurrent call over the whole span."""
    from fla_amd.ops.gated_delta_rule import fused_recurrent_gated_delta_rule
    from fla_amd.ops.gla import fused_recurrent_gla
    B, H, D, steps = 4, 4, 128, 5
    if op == "gla":
        q, k, v, g, h0 = gla_inputs(B, steps, H, D, D, seed=8, normalizer=1.0)
        args = [x.to(device) for x in (q, k, v, g)]
        fn = fused_recurrent_gla
    else:
        q, k, v, g, beta, h0 = gdr_inputs(B, steps, H, D, D, seed=8)
        args = [x.to(device) for x in (q, k, v, g, beta)]
        fn = fused_recurrent_gated_delta_rule
    h0 = h0.to(device)
    o_all, ht_all = fn(*args, initial_state=h0, output_final_state=True, head_first=False)
    state_a = h0.clone()   # out-of-place chain
    state_b = h0.clone()   # in-place chain
    for t in range(steps):
        step = [x[:, t:t + 1].contiguous() for x in args]
        o_a, state_a = fn(*step, initial_state=state_a, output_final_state=True, head_first=False)
        o_b, ret = fn(*step, initial_state=state_b, output_final_state=True, head_first=False, inplace_state=True)
        assert ret.data_ptr() == state_b.data_ptr()
        assert torch.equal(o_a, o_b) and torch.equal(state_a, state_b)
        assert torch.equal(o_a, o_all[:, t:t + 1])
    assert torch.equal(state_b, ht_all)


# ---------------------------------------------------------------- backward of fused_recurrent_gla
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("T,D,head_first", [(1, 128, False), (20, 64, False), (64, 128, True), (100, 100, False)])
def test_fused_recurrent_gla_backward(device, dtype, T, D, head_first):
    """Gradients of the token-by-token operator (the layers' path for sequences of at most 64
    tokens) against autograd through the naive recurrence, at the reference's tolerance for this
    operator (tests/ops/test_gla.py:66-87 uses 0.005 in fp32)."""
    from fla_amd.ops.gla import fused_recurrent_gla
    from oracle.recurrent import naive_recurrent_gla
    B, H = 2, 2
    q, k, v, g, h0 = gla_inputs(B, T, H, D, D, seed=40 + T, dtype=dtype, normalizer=4.0, h0_std=1.0)
    gen = torch.Generator().manual_seed(6)
    do = torch.randn(B, T, H, D, generator=gen).to(dtype)
    dht = torch.randn(B, H, D, D, generator=gen) * 0.1
    print(f"fused_recurrent_gla backward {dtype} T={T} D={D} head_first={head_first}", flush=True)
    tr = (lambda x: x.transpose(1, 2).contiguous()) if head_first else (lambda x: x)
    leaves = [tr(x.to(device)).detach().requires_grad_() for x in (q, k, v, g)]
    h0l = h0.to(device).requires_grad_()
    o, ht = fused_recurrent_gla(*leaves, initial_state=h0l, output_final_state=True, head_first=head_first)
    ((o.float() * tr(do.to(device)).float()).sum() + (ht * dht.to(device)).sum()).backward()
    refs = [x.detach().float().requires_grad_() for x in (q, k, v, g)]
    rh0 = h0.clone().requires_grad_()
    ro, rht = naive_recurrent_gla(*refs, initial_state=rh0, output_final_state=True)
    ((ro * do.float()).sum() + (rht * dht).sum()).backward()
    for name, r, x, tol in zip(("dq", "dk", "dv", "dg"), refs, leaves, (8e-3, 8e-3, 8e-3, 1e-2)):
        assert x.grad.dtype == x.dtype
        assert_close(name, r.grad, tr(x.grad), tol)
    assert_close("dh0", rh0.grad, h0l.grad, 8e-3)


@pytest.mark.parametrize("reverse", [False, True])
@pytest.mark.parametrize("gates", ["g", "gk", "gv", "gk+gv", "g+gk+gv", "none"])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_fused_recurrent_backward_all_gates(device, gates, reverse, dtype):
    """dq, dk, dv, every gate gradient and dh0 of the token-by-token operator, with a gradient of the final
    state as well, against autograd through the fp32 naive recurrence (fla/ops/common/fused_recurrent.py:381-468
    covers g, gk, gv and reverse).  fp32 inputs: both sides are fp32 recurrences, 1e-4; bf16 inputs: the output is
    rounded once, the rest is fp32."""
    from fla_amd.ops.common.fused_recurrent import fused_recurrent
    from oracle.recurrent import naive_recurrent_gla
    B, T, H, K, V = 2, 70, 2, 64, 128
    gen = torch.Generator().manual_seed(8 + len(gates))
    q, k = (torch.randn(B, T, H, K, generator=gen).to(dtype) for _ in range(2))
    v = torch.randn(B, T, H, V, generator=gen).to(dtype)
    gd = {"g": F.logsigmoid(torch.randn(B, T, H, generator=gen)) / 4 if "g" in gates.split("+") else None,
          "gk": F.logsigmoid(torch.randn(B, T, H, K, generator=gen)) / 4 if "gk" in gates else None,
          "gv": F.logsigmoid(torch.randn(B, T, H, V, generator=gen)) / 4 if "gv" in gates else None}
    h0 = torch.randn(B, H, K, V, generator=gen)
    do = torch.randn(B, T, H, V, generator=gen).to(dtype)
    dht = torch.randn(B, H, K, V, generator=gen) * 0.1
    print(f"fused_recurrent backward gates={gates} reverse={reverse} {dtype}", flush=True)
    mk = lambda x: None if x is None else x.to(device).requires_grad_()
    ql, kl, vl, h0l = mk(q), mk(k), mk(v), mk(h0)
    gl = {n: mk(x) for n, x in gd.items()}
    o, ht = fused_recurrent(ql, kl, vl, g=gl["g"], gk=gl["gk"], gv=gl["gv"], initial_state=h0l, output_final_state=True,
                            reverse=reverse, head_first=False)
    ((o.float() * do.to(device).float()).sum() + (ht * dht.to(device)).sum()).backward()
    rq, rk, rv, rh0 = (x.float().requires_grad_() for x in (q, k, v, h0))
    rg = {n: None if x is None else x.clone().requires_grad_() for n, x in gd.items()}
    ro, rht = naive_recurrent_gla(rq, rk, rv, rg["gk"], g=rg["g"], gv=rg["gv"], initial_state=rh0,
                                  output_final_state=True, reverse=reverse)
    ((ro * do.float()).sum() + (rht * dht).sum()).backward()
    tol = 1e-4 if dtype == torch.float32 else 8e-3
    assert_close("o", ro, o, 1e-5 if dtype == torch.float32 else 5e-3)
    for name, r, x in (("dq", rq, ql), ("dk", rk, kl), ("dv", rv, vl), ("dh0", rh0, h0l)):
        assert x.grad.dtype == x.dtype
        assert_close(name, r.grad, x.grad, tol)
    for n in ("g", "gk", "gv"):
        if gd[n] is not None:
            assert_close("d" + n, rg[n].grad, gl[n].grad, 5e-4 if dtype == torch.float32 else 2e-2)


@pytest.mark.parametrize("reverse", [False, True])
def test_fused_recurrent_backward_packed_and_head_first(device, reverse):
    from fla_amd.ops.common.fused_recurrent import fused_recurrent
    from oracle.recurrent import naive_recurrent_gla
    T, N, H, K, V = 90, 4, 2, 100, 64
    gen = torch.Generator().manual_seed(77)
    offs = torch.tensor([0, 1, 40, 40, 90])
    q, k = (torch.randn(1, T, H, K, generator=gen) for _ in range(2))
    v = torch.randn(1, T, H, V, generator=gen)
    gk = F.logsigmoid(torch.randn(1, T, H, K, generator=gen)) / 4
    gv = F.logsigmoid(torch.randn(1, T, H, V, generator=gen)) / 4
    h0 = torch.randn(N, H, K, V, generator=gen)
    do = torch.randn(1, T, H, V, generator=gen)
    dht = torch.randn(N, H, K, V, generator=gen) * 0.1
    print(f"fused_recurrent backward packed reverse={reverse}", flush=True)
    leaves = [x.to(device).requires_grad_() for x in (q, k, v, gk, gv, h0)]
    o, ht = fused_recurrent(leaves[0], leaves[1], leaves[2], gk=leaves[3], gv=leaves[4], initial_state=leaves[5],
                            output_final_state=True, reverse=reverse, offsets=offs.to(device), head_first=False)
    ((o * do.to(device)).sum() + (ht * dht.to(device)).sum()).backward()
    refs = [x.clone().requires_grad_() for x in (q, k, v, gk, gv, h0)]
    ro, rht = naive_recurrent_gla(refs[0], refs[1], refs[2], refs[3], gv=refs[4], initial_state=refs[5],
                                  output_final_state=True, reverse=reverse, offsets=offs.tolist())
    ((ro * do).sum() + (rht * dht).sum()).backward()
    for name, r, x in zip(("dq", "dk", "dv", "dgk", "dgv", "dh0"), refs, leaves):
        assert_close(name, r.grad, x.grad, 5e-4)
    # head-first, equal lengths, per-head gate
    B, T2 = 2, 33
    q, k, v = (torch.randn(B, H, T2, 64, generator=gen) for _ in range(3))
    g = F.logsigmoid(torch.randn(B, H, T2, generator=gen))
    do = torch.randn(B, H, T2, 64, generator=gen)
    leaves = [x.to(device).requires_grad_() for x in (q, k, v, g)]
    o, _ = fused_recurrent(leaves[0], leaves[1], leaves[2], g=leaves[3], reverse=reverse, head_first=True)
    (o * do.to(device)).sum().backward()
    refs = [x.transpose(1, 2).clone().requires_grad_() for x in (q, k, v, g)]
    ro, _ = naive_recurrent_gla(refs[0], refs[1], refs[2], None, g=refs[3], reverse=reverse)
    (ro * do.transpose(1, 2)).sum().backward()
    for name, r, x in zip(("dq", "dk", "dv", "dg"), refs, leaves):
        assert_close(name + " head-first", r.grad, x.grad.transpose(1, 2), 5e-4)


def test_fused_recurrent_inplace_state_refused_before_launch(device):
    """A state that would be overwritten while a backward needs it is refused before anything runs."""
    from fla_amd.ops.common.fused_recurrent import fused_recurrent
    q = torch.randn(1, 1, 1, 64, device=device).requires_grad_()
    state = torch.ones(1, 1, 64, 64, device=device)
    with pytest.raises(ValueError, match="inplace_state"):
        fused_recurrent(q, q.detach(), q.detach(), initial_state=state, output_final_state=True, head_first=False,
                        inplace_state=True)
    torch.cuda.synchronize()
    assert torch.equal(state, torch.ones_like(state))


# ---------------------------------------------------------------- prefill + decode through the Cache
@pytest.mark.parametrize("op", ["gla", "gdr"])
def test_cache_prefill_then_decode(device, op):
    """A layer's call pattern (fla/layers/gla.py:232-263, gated_deltanet.py:241-275): chunk operator on the
    prompt, state into the Cache, then single-token steps that read it back.  With in-place steps the
    Cache holds one buffer from the first step to the last."""
    from fla_amd.models import Cache
    from fla_amd.ops.gated_delta_rule import chunk_gated_delta_rule, fused_recurrent_gated_delta_rule
    from fla_amd.ops.gla import chunk_gla, fused_recurrent_gla
    from oracle.recurrent import naive_recurrent_gated_delta_rule, naive_recurrent_gla
    B, H, D, Tp, steps = 2, 2, 128, 150, 6
    T = Tp + steps
    if op == "gla":
        q, k, v, g, _ = gla_inputs(B, T, H, D, D, seed=91)
        cpu = (q, k, v, g)
        chunk, step_fn = chunk_gla, fused_recurrent_gla
        ro, rht = naive_recurrent_gla(q, k, v, g, output_final_state=True)
    else:
        q, k, v, g, beta, _ = gdr_inputs(B, T, H, D, D, seed=91)
        cpu = (q, k, v, g, beta)
        chunk, step_fn = chunk_gated_delta_rule, fused_recurrent_gated_delta_rule
        ro, rht = naive_recurrent_gated_delta_rule(q, k, v, g, beta, output_final_state=True)
    args = [x.to(device) for x in cpu]
    print(f"cache prefill+decode {op}", flush=True)
    cache = Cache()
    o_p, ht = chunk(*[x[:, :Tp].contiguous() for x in args], initial_state=None, output_final_state=True,
                    head_first=False)
    cache.update(recurrent_state=ht, layer_idx=0, offset=Tp)
    outs = [o_p]
    ptr = cache[0]['recurrent_state'].data_ptr()
    for t in range(Tp, T):
        state = cache[0]['recurrent_state']
        o_t, new_state = step_fn(*[x[:, t:t + 1].contiguous() for x in args], initial_state=state,
                                 output_final_state=True, head_first=False, inplace_state=True)
        cache.update(recurrent_state=new_state, layer_idx=0, offset=1)
        outs.append(o_t)
        assert cache[0]['recurrent_state'].data_ptr() == ptr
    assert cache.get_seq_length() == T
    assert_close("o", ro, torch.cat(outs, 1), 1e-2)
    assert_close("ht", rht, cache[0]['recurrent_state'], 5e-3)
