"""GPU: the operators that are pure compositions of the hot-path kernels
(``chunk_delta_rule``, ``chunk_simple_gla``, ``fused_recurrent_simple_gla``) against the
fp32 naive recurrences, forward and backward."""
import pytest
import torch
import torch.nn.functional as F

from helpers import assert_close, gdr_inputs, gla_inputs, random_offsets

pytestmark = pytest.mark.gpu

TOL_O, TOL_HT, TOL_G = 1e-2, 5e-3, 2e-2


def _dev(device):
    return lambda x: None if x is None else x.to(device)


# reference ladder: tests/ops/test_delta.py (T in {63, 300, 1000}-style lengths, packed batches)
@pytest.mark.parametrize("T,K,V", [(63, 128, 128), (300, 128, 128), (1000, 128, 128), (300, 256, 256), (150, 200, 100)])
@pytest.mark.parametrize("varlen", [False, True])
def test_chunk_delta_rule(device, T, K, V, varlen):
    from fla_amd.ops.delta_rule import chunk_delta_rule
    from oracle.recurrent import naive_recurrent_gated_delta_rule
    N = 3
    offs = random_offsets(T, N, torch.Generator().manual_seed(T), min_len=1) if varlen else None
    q, k, v, _, beta, h0 = gdr_inputs(1 if varlen else 2, T, 2, K, V, seed=T, N=N if varlen else None)
    dev = _dev(device)
    print(f"chunk_delta_rule T={T} K={K} V={V} varlen={varlen}", flush=True)
    do = torch.randn(v.shape, generator=torch.Generator().manual_seed(1)).to(v.dtype)
    dht = torch.randn(h0.shape, generator=torch.Generator().manual_seed(2)) * 0.1
    # device
    leaves = [dev(x).detach().requires_grad_() for x in (q, k, v, beta)]
    h0l = dev(h0).detach().requires_grad_()
    o, ht = chunk_delta_rule(*leaves, initial_state=h0l, output_final_state=True, offsets=dev(offs), head_first=False)
    torch.autograd.backward((o, ht), (dev(do), dev(dht)))
    torch.cuda.synchronize()
    # oracle
    rl = [x.detach().float().requires_grad_() for x in (q, k, v, beta)]
    rh0 = h0.detach().float().requires_grad_()
    ro, rht = naive_recurrent_gated_delta_rule(rl[0], rl[1], rl[2], None, rl[3], initial_state=rh0,
                                               output_final_state=True,
                                               offsets=None if offs is None else offs.tolist())
    ((ro * do.float()).sum() + (rht * dht).sum()).backward()
    assert_close("o", ro, o, TOL_O)
    assert_close("ht", rht, ht, TOL_HT)
    for name, a, b in zip(("dq", "dk", "dv", "dbeta"), rl, leaves):
        assert_close(name, a.grad, b.grad, TOL_G)
    assert_close("dh0", rh0.grad, h0l.grad, TOL_G)


@pytest.mark.parametrize("T", [64, 300, 1000])
@pytest.mark.parametrize("varlen", [False, True])
def test_chunk_simple_gla(device, T, varlen):
    from fla_amd.ops.simple_gla import chunk_simple_gla
    from oracle.recurrent import naive_recurrent_gla
    N, H, K, V = 3, 2, 128, 64
    B = 1 if varlen else 2
    gen = torch.Generator().manual_seed(T + 7)
    offs = random_offsets(T, N, gen, min_len=1) if varlen else None
    q = torch.randn(B, T, H, K, generator=gen).bfloat16()
    k = torch.randn(B, T, H, K, generator=gen).bfloat16()
    v = torch.randn(B, T, H, V, generator=gen).bfloat16()
    g = F.logsigmoid(torch.randn(B, T, H, generator=gen))
    h0 = torch.randn(N if varlen else B, H, K, V, generator=gen) * 0.1
    do = torch.randn(B, T, H, V, generator=gen).bfloat16()
    dht = torch.randn(h0.shape, generator=gen) * 0.1
    dev = _dev(device)
    print(f"chunk_simple_gla T={T} varlen={varlen}", flush=True)
    leaves = [dev(x).detach().requires_grad_() for x in (q, k, v, g)]
    h0l = dev(h0).detach().requires_grad_()
    o, ht = chunk_simple_gla(*leaves, initial_state=h0l, output_final_state=True, cu_seqlens=dev(offs),
                             head_first=False)
    torch.autograd.backward((o, ht), (dev(do), dev(dht)))
    torch.cuda.synchronize()
    rl = [x.detach().float().requires_grad_() for x in (q, k, v, g)]
    rh0 = h0.detach().float().requires_grad_()
    ro, rht = naive_recurrent_gla(rl[0], rl[1], rl[2], None, g=rl[3], initial_state=rh0, output_final_state=True,
                                  offsets=None if offs is None else offs.tolist())
    ((ro * do.float()).sum() + (rht * dht).sum()).backward()
    assert_close("o", ro, o, TOL_O)
    assert_close("ht", rht, ht, TOL_HT)
    # the head-wise gate gradient is the sum over the 128 key channels of the channel-wise one; the
    # terms largely cancel, so its relative error is a few times that of a single channel
    for name, a, b, tol in zip(("dq", "dk", "dv", "dg"), rl, leaves, (TOL_G, TOL_G, TOL_G, 4e-2)):
        assert_close(name, a.grad, b.grad, tol)
    assert_close("dh0", rh0.grad, h0l.grad, TOL_G)


@pytest.mark.parametrize("T", [1, 100])
def test_fused_recurrent_simple_gla(device, T):
    from fla_amd.ops.simple_gla import fused_recurrent_simple_gla
    from oracle.recurrent import naive_recurrent_gla
    B, H, K, V = 2, 3, 128, 128
    gen = torch.Generator().manual_seed(T)
    q = torch.randn(B, T, H, K, generator=gen)
    k = torch.randn(B, T, H, K, generator=gen)
    v = torch.randn(B, T, H, V, generator=gen)
    g = F.logsigmoid(torch.randn(B, T, H, generator=gen))
    h0 = torch.randn(B, H, K, V, generator=gen) * 0.1
    dev = _dev(device)
    print(f"fused_recurrent_simple_gla T={T}", flush=True)
    o, ht = fused_recurrent_simple_gla(dev(q), dev(k), dev(v), dev(g), initial_state=dev(h0), output_final_state=True,
                                       head_first=False)
    torch.cuda.synchronize()
    ro, rht = naive_recurrent_gla(q, k, v, None, g=g, initial_state=h0, output_final_state=True)
    assert_close("o", ro, o, 1e-5)
    assert_close("ht", rht, ht, 1e-5)


@pytest.mark.parametrize("K,V", [(128, 256), (256, 128), (192, 320)])
def test_chunk_gla_wide_heads(device, K, V):
    """Head dims above the built 128-wide tiles: key channels and value columns are independent
    in the GLA recurrence, so the operator runs slabs of 128 (the reference allows K <= 256)."""
    from fla_amd.ops.gla import chunk_gla
    from oracle.recurrent import naive_recurrent_gla
    B, T, H = 2, 150, 2
    q, k, v, g, h0 = gla_inputs(B, T, H, K, V, seed=K + V, h0_std=1.0)
    gen = torch.Generator().manual_seed(3)
    do = torch.randn(B, T, H, V, generator=gen).bfloat16()
    dht = torch.randn(B, H, K, V, generator=gen) * 0.1
    dev = _dev(device)
    print(f"chunk_gla wide heads K={K} V={V}", flush=True)
    leaves = [dev(x).requires_grad_() for x in (q, k, v, g)]
    h0l = dev(h0).requires_grad_()
    o, ht = chunk_gla(*leaves, initial_state=h0l, output_final_state=True, head_first=False)
    ((o.float() * dev(do).float()).sum() + (ht * dev(dht)).sum()).backward()
    refs = [x.float().requires_grad_() for x in (q, k, v, g)]
    rh0 = h0.clone().requires_grad_()
    ro, rht = naive_recurrent_gla(*refs, initial_state=rh0, output_final_state=True)
    ((ro * do.float()).sum() + (rht * dht).sum()).backward()
    assert_close("o", ro, o, 1e-2)
    assert_close("ht", rht, ht, 5e-3)
    for name, a, b in zip(("dq", "dk", "dv", "dg"), refs, leaves):
        assert_close(name, a.grad, b.grad, 1e-2)
    assert_close("dh0", rh0.grad, h0l.grad, TOL_G)


def test_chunk_gdr_wide_values(device):
    """Value head dims above 128 for the gated delta rule (independent per value column)."""
    from fla_amd.ops.gated_delta_rule import chunk_gated_delta_rule
    from oracle.recurrent import naive_recurrent_gated_delta_rule
    B, T, H, K, V = 2, 150, 2, 128, 256
    q, k, v, g, beta, h0 = gdr_inputs(B, T, H, K, V, seed=77, h0_std=1.0)
    gen = torch.Generator().manual_seed(4)
    do = torch.randn(B, T, H, V, generator=gen).bfloat16()
    dev = _dev(device)
    print("chunk_gated_delta_rule V=256", flush=True)
    leaves = [dev(x).requires_grad_() for x in (q, k, v, g, beta)]
    h0l = dev(h0).requires_grad_()
    o, ht = chunk_gated_delta_rule(*leaves, initial_state=h0l, output_final_state=True, head_first=False)
    (o.float() * dev(do).float()).sum().backward()
    refs = [x.float().requires_grad_() for x in (q, k, v, g, beta)]
    rh0 = h0.clone().requires_grad_()
    ro, rht = naive_recurrent_gated_delta_rule(*refs, initial_state=rh0, output_final_state=True)
    (ro * do.float()).sum().backward()
    assert_close("o", ro, o, 1e-2)
    assert_close("ht", rht, ht, 5e-3)
    for name, a, b, tol in zip(("dq", "dk", "dv", "dg", "dbeta"), refs, leaves, (8e-3, 8e-3, 8e-3, 2e-2, 2e-2)):
        assert_close(name, a.grad, b.grad, tol)
    assert_close("dh0", rh0.grad, h0l.grad, 8e-3)


@pytest.mark.parametrize("B,T,H,K,V,varlen", [
    (2, 150, 2, 256, 128, False),
    (1, 200, 2, 200, 200, False),   # the reference's own test dims: padded to 256 keys, two value slabs
    (1, 300, 2, 256, 64, True),
])
def test_chunk_gdr_wide_keys(device, B, T, H, K, V, varlen):
    """Key head dims up to 256 (the default of the reference's GatedDeltaNet layer), forward and
    backward through the chunk kernels."""
    from fla_amd.ops.gated_delta_rule import chunk_gated_delta_rule
    from oracle.recurrent import naive_recurrent_gated_delta_rule
    q, k, v, g, beta, h0 = gdr_inputs(B, T, H, K, V, seed=78, h0_std=1.0)
    offsets = torch.tensor([0, 70, 71, 199, T]) if varlen else None
    N = B if offsets is None else len(offsets) - 1
    gen = torch.Generator().manual_seed(5)
    h0 = torch.randn(N, H, K, V, generator=gen)
    do = torch.randn(B, T, H, V, generator=gen).bfloat16()
    dht = torch.randn(N, H, K, V, generator=gen) * 0.1
    dev = _dev(device)
    print(f"chunk_gated_delta_rule K={K} V={V} varlen={varlen}", flush=True)
    leaves = [dev(x).requires_grad_() for x in (q, k, v, g, beta)]
    h0l = dev(h0).requires_grad_()
    o, ht = chunk_gated_delta_rule(*leaves, initial_state=h0l, output_final_state=True, head_first=False,
                                   offsets=None if offsets is None else dev(offsets))
    ((o.float() * dev(do).float()).sum() + (ht * dev(dht)).sum()).backward()
    refs = [x.float().requires_grad_() for x in (q, k, v, g, beta)]
    rh0 = h0.clone().requires_grad_()
    ro, rht = naive_recurrent_gated_delta_rule(*refs, initial_state=rh0, output_final_state=True, offsets=offsets)
    ((ro * do.float()).sum() + (rht * dht).sum()).backward()
    assert_close("o", ro, o, 1e-2)
    assert_close("ht", rht, ht, 5e-3)
    for name, a, b, tol in zip(("dq", "dk", "dv", "dg", "dbeta"), refs, leaves, (8e-3, 8e-3, 8e-3, 2e-2, 2e-2)):
        assert_close(name, a.grad, b.grad, tol)
    assert_close("dh0", rh0.grad, h0l.grad, 8e-3)


def test_chunk_gdr_keys_above_256_refused(device):
    from fla_amd.ops.gated_delta_rule import chunk_gated_delta_rule
    q, k, v, g, beta, _ = gdr_inputs(1, 64, 1, 320, 64, seed=3, h0_std=1.0)
    dev = _dev(device)
    with pytest.raises(NotImplementedError):
        chunk_gated_delta_rule(dev(q), dev(k), dev(v), dev(g), dev(beta), head_first=False)


@pytest.mark.parametrize("op", ["gla", "gdr"])
def test_packed_batch_with_empty_sequence(device, op):
    """A packed batch may contain a sequence of length zero: it has no chunks, its final state is its
    initial state and the gradient of that state passes straight through."""
    from fla_amd.ops.gated_delta_rule import chunk_gated_delta_rule
    from fla_amd.ops.gla import chunk_gla
    from oracle.recurrent import naive_recurrent_gated_delta_rule, naive_recurrent_gla
    T, H, D = 200, 2, 128
    offs = torch.tensor([0, 70, 70, 199, 200])          # the second sequence is empty, the last has one token
    N = 4
    gen = torch.Generator().manual_seed(21)
    do = torch.randn(1, T, H, D, generator=gen).bfloat16()
    dht = torch.randn(N, H, D, D, generator=gen) * 0.1
    dev = _dev(device)
    print(f"packed batch with an empty sequence: {op}", flush=True)
    if op == "gla":
        q, k, v, g, h0 = gla_inputs(1, T, H, D, D, seed=22, N=N, h0_std=1.0)
        cpu, fn, naive = (q, k, v, g), chunk_gla, naive_recurrent_gla
    else:
        q, k, v, g, beta, h0 = gdr_inputs(1, T, H, D, D, seed=22, N=N, h0_std=1.0)
        cpu, fn, naive = (q, k, v, g, beta), chunk_gated_delta_rule, naive_recurrent_gated_delta_rule
    leaves = [dev(x).requires_grad_() for x in cpu]
    h0l = dev(h0).requires_grad_()
    o, ht = fn(*leaves, initial_state=h0l, output_final_state=True, offsets=dev(offs), head_first=False)
    ((o.float() * dev(do).float()).sum() + (ht * dev(dht)).sum()).backward()
    torch.cuda.synchronize()
    refs = [x.float().requires_grad_() for x in cpu]
    rh0 = h0.clone().requires_grad_()
    ro, rht = naive(*refs, initial_state=rh0, output_final_state=True, offsets=offs.tolist())
    ((ro * do.float()).sum() + (rht * dht).sum()).backward()
    assert_close("o", ro, o, 1e-2)
    assert_close("ht", rht, ht, 5e-3)
    assert torch.equal(ht[1].cpu(), h0[1]) and torch.equal(h0l.grad[1].cpu(), dht[1])
    for name, a, b in zip(("dq", "dk", "dv", "dg", "dbeta"), refs, leaves):
        assert_close(name, a.grad, b.grad, 2e-2)
    assert_close("dh0", rh0.grad, h0l.grad, 1e-2)


# the forward that is not differentiated reads the per-head gates as they are (no [B,T,H,K] gate tensor)
@pytest.mark.parametrize("T,K,V", [(64, 128, 128), (300, 128, 64), (1000, 64, 128), (37, 64, 64)])
@pytest.mark.parametrize("varlen", [False, True])
@pytest.mark.parametrize("gate_scale", [1.0, 40.0])   # 40: chunk-cumulative gates far beyond the single-reference range
@pytest.mark.parametrize("route", ["scan", "fused"])   # the plain scan kernel (default) / the GLA kernel's per-head-gate form
def test_chunk_simple_gla_forward_per_head_gate_kernel(device, T, K, V, varlen, gate_scale, route, monkeypatch):
    import fla_amd.ops.simple_gla.chunk as sg_mod
    from fla_amd.ops.simple_gla import chunk_simple_gla
    from oracle.recurrent import naive_recurrent_gla
    monkeypatch.setattr(sg_mod, "SCAN_FORWARD", route == "scan")
    N, H = 3, 3
    B = 1 if varlen else 2
    gen = torch.Generator().manual_seed(T + K + int(gate_scale))
    offs = random_offsets(T, N, gen, min_len=1) if varlen else None
    q = torch.randn(B, T, H, K, generator=gen).bfloat16()
    k = torch.randn(B, T, H, K, generator=gen).bfloat16()
    v = torch.randn(B, T, H, V, generator=gen).bfloat16()
    g = F.logsigmoid(torch.randn(B, T, H, generator=gen)) * gate_scale
    h0 = torch.randn(N if varlen else B, H, K, V, generator=gen) * 0.1
    dev = _dev(device)
    print(f"chunk_simple_gla no-grad T={T} K={K} V={V} varlen={varlen} gate x{gate_scale} route={route}", flush=True)
    with torch.no_grad():
        o, ht = chunk_simple_gla(dev(q), dev(k), dev(v), dev(g), initial_state=dev(h0), output_final_state=True,
                                 cu_seqlens=dev(offs), head_first=False)
        # the general route (gates broadcast over the key channels) on the same inputs
        from fla_amd.ops.gla import chunk_gla
        o2, ht2 = chunk_gla(dev(q), dev(k), dev(v), dev(g)[..., None].expand(B, T, H, K).contiguous(),
                            initial_state=dev(h0), output_final_state=True, offsets=dev(offs), head_first=False)
    torch.cuda.synchronize()
    ro, rht = naive_recurrent_gla(q.float(), k.float(), v.float(), None, g=g, initial_state=h0,
                                  output_final_state=True, offsets=None if offs is None else offs.tolist())
    assert_close("o", ro, o, TOL_O)
    assert_close("ht", rht, ht, TOL_HT)
    if route == "fused":
        assert torch.equal(o, o2) and torch.equal(ht, ht2)   # same arithmetic as the per-key-gate launch
    else:
        assert_close("o vs the per-key-gate launch", o2, o, TOL_O)
        assert_close("ht vs the per-key-gate launch", ht2, ht, TOL_HT)


def test_chunk_simple_gla_per_head_gate_kernel_fp16_and_gradients(device):
    """fp16 operands through the per-head-gate launch, forward and backward (the states it keeps feed the GLA
    backward kernels), against the fp32 recurrence."""
    from fla_amd.ops.simple_gla import chunk_simple_gla
    from oracle.recurrent import naive_recurrent_gla
    B, T, H, K, V = 2, 200, 2, 64, 128
    gen = torch.Generator().manual_seed(77)
    q = (torch.randn(B, T, H, K, generator=gen) * 0.5).half()
    k = (torch.randn(B, T, H, K, generator=gen) * 0.5).half()
    v = torch.randn(B, T, H, V, generator=gen).half()
    g = F.logsigmoid(torch.randn(B, T, H, generator=gen))
    h0 = torch.randn(B, H, K, V, generator=gen) * 0.1
    do = torch.randn(B, T, H, V, generator=gen).half()
    dht = torch.randn(B, H, K, V, generator=gen) * 0.1
    dev = _dev(device)
    leaves = [dev(x).detach().requires_grad_() for x in (q, k, v, g)]
    h0l = dev(h0).detach().requires_grad_()
    o, ht = chunk_simple_gla(*leaves, initial_state=h0l, output_final_state=True, head_first=False)
    torch.autograd.backward((o, ht), (dev(do), dev(dht)))
    torch.cuda.synchronize()
    rl = [x.detach().float().requires_grad_() for x in (q, k, v, g)]
    rh0 = h0.detach().float().requires_grad_()
    ro, rht = naive_recurrent_gla(rl[0], rl[1], rl[2], None, g=rl[3], initial_state=rh0, output_final_state=True)
    ((ro * do.float()).sum() + (rht * dht).sum()).backward()
    assert o.dtype == torch.float16
    assert_close("o", ro, o, TOL_O)
    assert_close("ht", rht, ht, TOL_HT)
    for name, a, b in zip(("dq", "dk", "dv", "dg"), rl, leaves):
        assert_close(name, a.grad, b.grad, TOL_G)
    assert_close("dh0", rh0.grad, h0l.grad, TOL_G)


@pytest.mark.parametrize("varlen", [False, True])
def test_chunk_simple_gla_strong_gates_backward_reproducible(device, varlen, monkeypatch):
    """Gates strong enough that chunks leave the single-reference range (their intra-chunk terms come from the
    exact kernel): the per-head gate gradient, which the backward kernels accumulate from their key slices, is
    the same bit for bit on a second run, agrees with the form that writes per-key gradients and sums them
    afterwards (the backward that recomputes the states), and both meet the fp32 recurrence."""
    import fla_amd.ops.gla.chunk as gla_mod
    from fla_amd.ops.simple_gla import chunk_simple_gla
    from oracle.recurrent import naive_recurrent_gla
    N, H, K, V, T = 3, 2, 128, 128, 333
    B = 1 if varlen else 2
    gen = torch.Generator().manual_seed(91)
    offs = random_offsets(T, N, gen, min_len=1) if varlen else None
    q = torch.randn(B, T, H, K, generator=gen).bfloat16()
    k = torch.randn(B, T, H, K, generator=gen).bfloat16()
    v = torch.randn(B, T, H, V, generator=gen).bfloat16()
    g = -2.5 * torch.rand(B, T, H, generator=gen)       # about -80 per chunk: most chunks are flagged
    h0 = torch.randn(N if varlen else B, H, K, V, generator=gen) * 0.1
    do = torch.randn(B, T, H, V, generator=gen).bfloat16()
    dht = torch.randn(h0.shape, generator=gen) * 0.1
    dev = _dev(device)
    print(f"chunk_simple_gla strong gates varlen={varlen}", flush=True)

    def run():
        leaves = [dev(x).detach().requires_grad_() for x in (q, k, v, g)]
        h0l = dev(h0).detach().requires_grad_()
        o, ht = chunk_simple_gla(*leaves, initial_state=h0l, output_final_state=True, cu_seqlens=dev(offs),
                                 head_first=False)
        torch.autograd.backward((o, ht), (dev(do), dev(dht)))
        torch.cuda.synchronize()
        return [x.grad for x in leaves] + [h0l.grad]

    first, second = run(), run()
    for a, b in zip(first, second):
        assert torch.equal(a, b)
    monkeypatch.setattr(gla_mod, "KEEP_STATES_FOR_BACKWARD", False)
    rec = run()
    rl = [x.detach().float().requires_grad_() for x in (q, k, v, g)]
    rh0 = h0.detach().float().requires_grad_()
    ro, rht = naive_recurrent_gla(rl[0], rl[1], rl[2], None, g=rl[3], initial_state=rh0, output_final_state=True,
                                  offsets=None if offs is None else offs.tolist())
    ((ro * do.float()).sum() + (rht * dht).sum()).backward()
    refs = [x.grad for x in rl] + [rh0.grad]
    for name, r, a, b, tol in zip(("dq", "dk", "dv", "dg", "dh0"), refs, first, rec, (TOL_G, TOL_G, TOL_G, 4e-2, TOL_G)):
        assert_close(f"{name} (kept)", r, a, tol)
        assert_close(f"{name} (recomputed)", r, b, tol)
