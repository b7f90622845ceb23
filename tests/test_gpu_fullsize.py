"""GPU: the four measured workloads at their full sizes.

The fp32 naive recurrence cannot walk these shapes in full, so each workload is checked (a) against
the oracle on a slice of the same seeded inputs - (sequence, head) pairs are independent in every
kernel, so the full-size launch must reproduce on those pairs what the oracle computes from the
slice alone - and (b) through properties that do not depend on size: a run split at a chunk
boundary with the state handed over equals the whole run, a packed batch equals its sequences run
one by one, the chunked operator equals the token-by-token one, the operators are linear in v (and
the gradients in do), the in-place decode step equals the out-of-place one.
Tolerances: rel-L2 1e-2 on outputs and gradients, 5e-3 on states (bf16 inputs); exact where the two
sides run the same arithmetic."""
import pytest
import torch
import torch.nn.functional as F

from helpers import assert_close, rel_l2

pytestmark = pytest.mark.gpu


def _config1(device, B=8, T=4096, H=16, D=128):
    g = torch.Generator(device=device).manual_seed(0)
    q, k, v = (torch.randn(B, T, H, D, device=device, generator=g).bfloat16() for _ in range(3))
    gk = F.logsigmoid(torch.randn(B, T, H, D, device=device, generator=g)) / 16
    h0 = torch.randn(B, H, D, D, device=device, generator=g) * 0.1
    return q, k, v, gk, h0


def test_config1_chunk_gla_forward_full_size(device):
    from fla_amd.ops.gla import chunk_gla, fused_recurrent_gla
    from oracle.recurrent import naive_recurrent_gla
    q, k, v, gk, h0 = _config1(device)
    print("config 1: chunk_gla forward B=8 T=4096 H=16 D=128", flush=True)
    o, ht = chunk_gla(q, k, v, gk, initial_state=h0, output_final_state=True, head_first=False)
    torch.cuda.synchronize()
    assert torch.isfinite(o.float()).all() and torch.isfinite(ht).all()
    # (a) oracle on three (batch, head) pairs of the same inputs
    for b, h in ((0, 0), (3, 7), (7, 15)):
        sl = lambda x: x[b:b + 1, :, h:h + 1].float().cpu()
        ro, rht = naive_recurrent_gla(sl(q), sl(k), sl(v), sl(gk), initial_state=h0[b:b + 1, h:h + 1].cpu(),
                                      output_final_state=True)
        assert_close(f"o[{b},{h}]", ro, o[b:b + 1, :, h:h + 1], 1e-2)
        assert_close(f"ht[{b},{h}]", rht, ht[b:b + 1, h:h + 1], 5e-3)
    # (b1) split at a chunk boundary with the state handed over: same arithmetic, same bits
    Ts = 1984
    o1, s1 = chunk_gla(q[:, :Ts].contiguous(), k[:, :Ts].contiguous(), v[:, :Ts].contiguous(), gk[:, :Ts].contiguous(),
                       initial_state=h0, output_final_state=True, head_first=False)
    o2, s2 = chunk_gla(q[:, Ts:].contiguous(), k[:, Ts:].contiguous(), v[:, Ts:].contiguous(), gk[:, Ts:].contiguous(),
                       initial_state=s1, output_final_state=True, head_first=False)
    assert torch.equal(torch.cat([o1, o2], 1), o) and torch.equal(s2, ht)
    # (b2) batch elements are independent: a permuted batch gives the permuted result
    perm = torch.tensor([5, 2, 7, 0, 3, 6, 1, 4], device=device)
    op, hp = chunk_gla(q[perm], k[perm], v[perm], gk[perm], initial_state=h0[perm], output_final_state=True,
                       head_first=False)
    assert torch.equal(op, o[perm]) and torch.equal(hp, ht[perm])
    # (b3) the token-by-token kernel computes the same operator
    orr, hr = fused_recurrent_gla(q, k, v, gk, initial_state=h0, output_final_state=True, head_first=False)
    assert_close("chunk vs recurrent o", orr, o, 1e-2)
    assert_close("chunk vs recurrent ht", hr, ht, 5e-3)
    # (b4) linear in v (zero initial state): o(v1 + 2 v2) = o(v1) + 2 o(v2)
    v2 = torch.randn_like(v)
    oa, _ = chunk_gla(q, k, v, gk, head_first=False)
    ob, _ = chunk_gla(q, k, v2, gk, head_first=False)
    oc, _ = chunk_gla(q, k, (v.float() + 2 * v2.float()).bfloat16(), gk, head_first=False)
    assert_close("linearity in v", oa.float() + 2 * ob.float(), oc, 1e-2)


def _config2(device, T=32768, H=16, D=128, N=12):
    g = torch.Generator().manual_seed(0)
    lens = torch.randint(256, 6001, (N,), generator=g).double()
    lens = (lens / lens.sum() * T).round().long()
    lens[-1] += T - lens.sum()
    offs = torch.cat([torch.zeros(1, dtype=torch.long), lens.cumsum(0)])
    gd = torch.Generator(device=device).manual_seed(0)
    q = torch.randn(1, T, H, D, device=device, generator=gd).bfloat16()
    k = F.normalize(torch.randn(1, T, H, D, device=device, generator=gd), dim=-1).bfloat16()
    v = torch.randn(1, T, H, D, device=device, generator=gd).bfloat16()
    gl = F.logsigmoid(torch.randn(1, T, H, device=device, generator=gd))
    beta = torch.randn(1, T, H, device=device, generator=gd).sigmoid()
    return q, k, v, gl, beta, offs


def test_config2_chunk_gated_delta_rule_varlen_full_size(device):
    from fla_amd.ops.gated_delta_rule import chunk_gated_delta_rule, fused_recurrent_gated_delta_rule
    from oracle.recurrent import naive_recurrent_gated_delta_rule
    q, k, v, gl, beta, offs = _config2(device)
    lens = (offs[1:] - offs[:-1]).tolist()
    print(f"config 2: chunk_gated_delta_rule packed T=32768, lengths {lens}", flush=True)
    o, ht = chunk_gated_delta_rule(q, k, v, gl, beta, output_final_state=True, offsets=offs.to(device),
                                   head_first=False)
    torch.cuda.synchronize()
    assert torch.isfinite(o.float()).all() and torch.isfinite(ht).all() and ht.shape[0] == len(lens)
    # (a) oracle on the two shortest sequences, two heads each
    order = sorted(range(len(lens)), key=lambda n: lens[n])[:2]
    for n in order:
        s, e = int(offs[n]), int(offs[n + 1])
        for h in (1, 14):
            sl = lambda x: x[:, s:e, h:h + 1].float().cpu()
            ro, rht = naive_recurrent_gated_delta_rule(sl(q), sl(k), sl(v), gl[:, s:e, h:h + 1].cpu(),
                                                       beta[:, s:e, h:h + 1].cpu(), output_final_state=True)
            assert_close(f"o[seq {n}, head {h}]", ro, o[:, s:e, h:h + 1], 1e-2)
            assert_close(f"ht[seq {n}, head {h}]", rht, ht[n:n + 1, h:h + 1], 5e-3)
    # (a2) and on the longest sequence, the one whose serial chain bounds the launch, for one head
    n = max(range(len(lens)), key=lambda i: lens[i])
    s, e, h = int(offs[n]), int(offs[n + 1]), 7
    sl = lambda x: x[:, s:e, h:h + 1].float().cpu()
    ro, rht = naive_recurrent_gated_delta_rule(sl(q), sl(k), sl(v), gl[:, s:e, h:h + 1].cpu(),
                                               beta[:, s:e, h:h + 1].cpu(), output_final_state=True)
    assert_close(f"o[longest seq {n} ({e - s} tokens), head {h}]", ro, o[:, s:e, h:h + 1], 1e-2)
    assert_close(f"ht[longest seq {n}, head {h}]", rht, ht[n:n + 1, h:h + 1], 5e-3)
    # (b1) the packed batch equals its sequences run one by one
    for n in range(len(lens)):
        s, e = int(offs[n]), int(offs[n + 1])
        on, hn = chunk_gated_delta_rule(q[:, s:e].contiguous(), k[:, s:e].contiguous(), v[:, s:e].contiguous(),
                                        gl[:, s:e].contiguous(), beta[:, s:e].contiguous(), output_final_state=True,
                                        head_first=False)
        assert torch.equal(on, o[:, s:e]) and torch.equal(hn[0], ht[n]), f"sequence {n}"
    # (b2) the token-by-token kernel computes the same operator
    orr, hr = fused_recurrent_gated_delta_rule(q, k, v, gl, beta, output_final_state=True, offsets=offs.to(device),
                                               head_first=False)
    assert_close("chunk vs recurrent o", orr, o, 1e-2)
    assert_close("chunk vs recurrent ht", hr, ht, 5e-3)
    # (b3) beta = 0 writes nothing: the output is zero and the states stay zero
    oz, hz = chunk_gated_delta_rule(q, k, v, gl, torch.zeros_like(beta), output_final_state=True,
                                    offsets=offs.to(device), head_first=False)
    assert float(oz.float().abs().max()) == 0.0 and float(hz.abs().max()) == 0.0


@pytest.mark.parametrize("op", ["gla", "gdr"])
def test_config3_decode_step_full_size(device, op):
    from fla_amd.ops.gated_delta_rule import fused_recurrent_gated_delta_rule
    from fla_amd.ops.gla import fused_recurrent_gla
    from oracle.recurrent import naive_recurrent_gated_delta_rule, naive_recurrent_gla
    B, H, D, steps = 256, 32, 128, 4
    g = torch.Generator(device=device).manual_seed(0)
    S0 = torch.randn(B, H, D, D, device=device, generator=g) * 0.1
    q, v = (torch.randn(B, steps, H, D, device=device, generator=g).bfloat16() for _ in range(2))
    kf = torch.randn(B, steps, H, D, device=device, generator=g)
    print(f"config 3: decode {op} B=256 H=32 D=128, {steps} steps", flush=True)
    if op == "gla":
        k = kf.bfloat16()
        gate = F.logsigmoid(torch.randn(B, steps, H, D, device=device, generator=g))
        args, fn = (q, k, v, gate), fused_recurrent_gla
        ref = lambda sl, s0: naive_recurrent_gla(sl(q).float(), sl(k).float(), sl(v).float(), sl(gate),
                                                 initial_state=s0, output_final_state=True)
    else:
        k = F.normalize(kf, dim=-1).bfloat16()
        gate = F.logsigmoid(torch.randn(B, steps, H, device=device, generator=g))
        beta = torch.randn(B, steps, H, device=device, generator=g).sigmoid()
        args, fn = (q, k, v, gate, beta), fused_recurrent_gated_delta_rule
        ref = lambda sl, s0: naive_recurrent_gated_delta_rule(sl(q).float(), sl(k).float(), sl(v).float(), sl(gate),
                                                              sl(beta), initial_state=s0, output_final_state=True)
    state_in, state_out = S0.clone(), S0.clone()
    outs = []
    for t in range(steps):
        step = [x[:, t:t + 1].contiguous() for x in args]
        o_a, state_out = fn(*step, initial_state=state_out, output_final_state=True, head_first=False)
        o_b, ret = fn(*step, initial_state=state_in, output_final_state=True, head_first=False, inplace_state=True)
        assert ret.data_ptr() == state_in.data_ptr()
        assert torch.equal(o_a, o_b) and torch.equal(state_in, state_out)      # in place == out of place
        outs.append(o_b)
    o_all, s_all = fn(*args, initial_state=S0, output_final_state=True, head_first=False)
    assert torch.equal(torch.cat(outs, 1), o_all) and torch.equal(s_all, state_in)   # steps == one call
    for b, h in ((0, 0), (100, 17), (255, 31)):
        sl = lambda x: x[b:b + 1, :, h:h + 1].cpu()
        ro, rs = ref(sl, S0[b:b + 1, h:h + 1].cpu())
        assert_close(f"o[{b},{h}]", ro, o_all[b:b + 1, :, h:h + 1], 1e-2)
        assert_close(f"state[{b},{h}]", rs, state_in[b:b + 1, h:h + 1], 1e-5)


@pytest.mark.parametrize("op", ["gla", "gdr"])
def test_config3_decode_1000_steps_full_size(device, op):
    """1000 consecutive in-place decode steps at B=256, H=32, D=128 (what bench.py times): on three (b, h) slices the
    outputs and the final state equal one fused_recurrent call over the same 1000 tokens to fp32 round-off, and the
    fp32 naive recurrence within the operator's tolerances."""
    from fla_amd.ops.gated_delta_rule import fused_recurrent_gated_delta_rule
    from fla_amd.ops.gla import fused_recurrent_gla
    from oracle.recurrent import naive_recurrent_gated_delta_rule, naive_recurrent_gla
    B, H, D, steps = 256, 32, 128, 1000
    g = torch.Generator(device=device).manual_seed(3)
    S = torch.randn(B, H, D, D, device=device, generator=g) * 0.1
    S0 = S.clone()
    q, v = (torch.randn(B, steps, H, D, device=device, generator=g).bfloat16() for _ in range(2))
    print(f"config 3: {steps} in-place decode steps, {op}", flush=True)
    if op == "gla":
        k = torch.randn(B, steps, H, D, device=device, generator=g).bfloat16()
        gate = F.logsigmoid(torch.randn(B, steps, H, D, device=device, generator=g))
        args, fn = (q, k, v, gate), fused_recurrent_gla
        ref = lambda a, s0: naive_recurrent_gla(a[0].float(), a[1].float(), a[2].float(), a[3], initial_state=s0,
                                                output_final_state=True)
    else:
        k = F.normalize(torch.randn(B, steps, H, D, device=device, generator=g), dim=-1).bfloat16()
        gate = F.logsigmoid(torch.randn(B, steps, H, device=device, generator=g))
        beta = torch.randn(B, steps, H, device=device, generator=g).sigmoid()
        args, fn = (q, k, v, gate, beta), fused_recurrent_gated_delta_rule
        ref = lambda a, s0: naive_recurrent_gated_delta_rule(a[0].float(), a[1].float(), a[2].float(), a[3], a[4],
                                                             initial_state=s0, output_final_state=True)
    picks = ((0, 0), (100, 17), (255, 31))
    kept = {p: [] for p in picks}
    with torch.no_grad():
        for t in range(steps):
            step = [x[:, t:t + 1].contiguous() for x in args]
            o, ret = fn(*step, initial_state=S, output_final_state=True, head_first=False, inplace_state=True)
            for b, h in picks:
                kept[(b, h)].append(o[b:b + 1, :, h:h + 1])
    assert ret.data_ptr() == S.data_ptr() and torch.isfinite(S).all()
    for b, h in picks:
        a = [x[b:b + 1, :, h:h + 1].contiguous() for x in args]
        o_all, s_all = fn(*a, initial_state=S0[b:b + 1, h:h + 1].contiguous(), output_final_state=True,
                          head_first=False)
        o_steps = torch.cat(kept[(b, h)], 1)
        # (the launcher picks its slab width from the batch, so the two runs may add in a different order: equal to
        # fp32 round-off, not bit for bit; the bit-exact step-by-step check at one batch size is the 4-step test above)
        assert_close(f"o[{b},{h}] steps vs one call", o_all, o_steps, 2e-3)
        assert_close(f"state[{b},{h}] steps vs one call", s_all, S[b:b + 1, h:h + 1], 1e-5)
        ro, rs = ref([x.cpu() for x in a], S0[b:b + 1, h:h + 1].cpu())
        assert_close(f"o[{b},{h}]", ro, o_steps, 1e-2)
        assert_close(f"state[{b},{h}]", rs, S[b:b + 1, h:h + 1], 1e-4)


@pytest.mark.parametrize("op", ["gla", "gdr"])
def test_config4_backward_full_size(device, op):
    from fla_amd.ops.gated_delta_rule import chunk_gated_delta_rule
    from fla_amd.ops.gla import chunk_gla
    from oracle.recurrent import naive_recurrent_gated_delta_rule, naive_recurrent_gla
    B, T, H, D = 4, 4096, 16, 128
    g = torch.Generator(device=device).manual_seed(0)
    q, v = (torch.randn(B, T, H, D, device=device, generator=g).bfloat16() for _ in range(2))
    kf = torch.randn(B, T, H, D, device=device, generator=g)
    h0 = torch.randn(B, H, D, D, device=device, generator=g) * 0.1
    do = torch.randn(B, T, H, D, device=device, generator=g).bfloat16()
    dht = torch.randn(B, H, D, D, device=device, generator=g) * 0.1
    print(f"config 4: {op} forward + backward B=4 T=4096 H=16 D=128", flush=True)
    if op == "gla":
        k = kf.bfloat16()
        gate = F.logsigmoid(torch.randn(B, T, H, D, device=device, generator=g)) / 16
        extra, names = (), ("dq", "dk", "dv", "dg")
        run = lambda *a, **kw: chunk_gla(*a, **kw)
        naive = naive_recurrent_gla
    else:
        k = F.normalize(kf, dim=-1).bfloat16()
        gate = F.logsigmoid(torch.randn(B, T, H, device=device, generator=g))
        extra, names = (torch.randn(B, T, H, device=device, generator=g).sigmoid(),), ("dq", "dk", "dv", "dg", "dbeta")
        run = lambda *a, **kw: chunk_gated_delta_rule(*a, **kw)
        naive = naive_recurrent_gated_delta_rule
    inputs = (q, k, v, gate) + extra

    def grads(do_, dht_):
        leaves = [x.detach().clone().requires_grad_() for x in inputs]
        h0l = h0.detach().clone().requires_grad_()
        o, ht = run(*leaves, initial_state=h0l, output_final_state=True, head_first=False)
        torch.autograd.backward((o, ht), (do_, dht_))
        return [x.grad for x in leaves] + [h0l.grad]

    got = grads(do, dht)
    torch.cuda.synchronize()
    assert all(torch.isfinite(x.float()).all() for x in got)
    # (a) autograd through the fp32 recurrence on one (batch, head) pair of the same inputs
    b, h = 2, 9
    sl = lambda x: x[b:b + 1, :, h:h + 1].float().cpu()
    leaves = [sl(x).requires_grad_() for x in inputs]
    h0l = h0[b:b + 1, h:h + 1].cpu().clone().requires_grad_()
    ro, rht = naive(*leaves, initial_state=h0l, output_final_state=True)
    torch.autograd.backward((ro, rht), (sl(do), dht[b:b + 1, h:h + 1].cpu()))
    tols = dict(dq=1e-2, dk=1e-2, dv=1e-2, dg=2e-2, dbeta=2e-2)
    for name, r, x in zip(names, leaves, got):
        assert_close(f"{name}[{b},{h}]", r.grad, x[b:b + 1, :, h:h + 1], tols[name])
    assert_close(f"dh0[{b},{h}]", h0l.grad, got[-1][b:b + 1, h:h + 1], 1e-2)
    # (b) the gradients are linear in (do, dht)
    do2 = torch.randn_like(do)
    dht2 = torch.randn_like(dht) * 0.1
    g2 = grads(do2, dht2)
    g3 = grads((do.float() - 0.5 * do2.float()).bfloat16(), dht - 0.5 * dht2)
    for name, a, c, d in zip(names + ("dh0",), got, g2, g3):
        assert_close(f"linearity {name}", a.float() - 0.5 * c.float(), d, 1.5e-2)


def test_config4_row_major_stage_pipeline_reproduces_the_operator(device):
    """At config 4's size, the stages that take the reference's internal operands (scores A [B,T,H,64],
    row-major fp32 states) rebuild chunk_gla's output and its gradient w.r.t. v from separately computed
    pieces: h from chunk_fwd_h, A from the output kernel's A_out, dh from chunk_bwd_dh.  Different kernels,
    layouts and summation orders on the two sides, so the bar is the bf16 tolerance (1e-2), not equality."""
    from fla_amd.ops.common.chunk_h import chunk_bwd_dh, chunk_fwd_h
    from fla_amd.ops.gla import chunk_gla
    from fla_amd.ops.gla.chunk import chunk_gla_bwd_dA, chunk_gla_bwd_dv, chunk_gla_fwd_o_gk
    from fla_amd.ops.utils.cumsum import chunk_local_cumsum
    B, T, H, D = 4, 4096, 16, 128
    q, k, v, gk, h0 = _config1(device, B=B)
    gen = torch.Generator(device=device).manual_seed(3)
    do = torch.randn(B, T, H, D, device=device, generator=gen).bfloat16()
    dht = torch.randn(B, H, D, D, device=device, generator=gen) * 0.1
    scale = D ** -0.5
    print("config 4: row-major stage pipeline vs chunk_gla, B=4 T=4096 H=16 D=128", flush=True)
    vl = v.clone().requires_grad_()
    o_ref, ht_ref = chunk_gla(q, k, vl, gk, initial_state=h0, output_final_state=True, head_first=False)
    torch.autograd.backward((o_ref, ht_ref), (do, dht))
    kw = dict(head_first=False, chunk_size=64)
    G = chunk_local_cumsum(gk, 64, head_first=False)
    h, ht = chunk_fwd_h(k, v, None, G, None, h0, True, states_in_fp32=True, **kw)
    A = torch.empty(B, T, H, 64, device=device, dtype=torch.float32)
    h_frag, _ = chunk_fwd_h(k, v, None, G, None, h0, False, fragment_layout=True, **kw)
    chunk_gla_fwd_o_gk(q, v, G, None, h_frag, scale, k=k, A_out=A, **kw)
    o = chunk_gla_fwd_o_gk(q, v, G, A, h, scale, **kw)
    dh, dh0 = chunk_bwd_dh(q, k, v, None, G, None, do, h0, dht, scale, states_in_fp32=True, **kw)
    dv = chunk_gla_bwd_dv(k, G, A, do, dh, **kw)
    dA = chunk_gla_bwd_dA(v, do, scale, **kw)
    torch.cuda.synchronize()
    assert_close("o", o_ref.float(), o, 1e-2)
    assert_close("ht", ht_ref, ht, 5e-3)
    assert_close("dv", vl.grad.float(), dv, 1e-2)
    # dA against a plain matrix product on one chunk of three (batch, head) pairs
    for b, hh, c in ((0, 0, 0), (2, 7, 31), (3, 15, 63)):
        sl = slice(c * 64, c * 64 + 64)
        ref = torch.tril(do[b, sl, hh].float() @ v[b, sl, hh].float().t()) * scale
        assert_close(f"dA[{b},{hh},{c}]", ref, dA[b, sl, hh], 5e-3)
