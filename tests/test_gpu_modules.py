"""GPU: the row-wise steps either side of the chunk operators (l2 norm, gated norms, short causal
convolution and its single-token step), forward and backward, against the torch restatements in
oracle/modules.py.  Tolerances (rel-L2): 1e-5 for fp32 storage; for 16-bit storage the outputs are
rounded once to bf16/fp16, 4e-3 forward and 8e-3 for gradients (the bar of the chunk operators)."""
import pytest
import torch

from helpers import assert_close

pytestmark = pytest.mark.gpu


def _tols(dtype):
    return (1e-5, 1e-5) if dtype == torch.float32 else (4e-3, 8e-3)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("N", [64, 128, 200, 256, 512, 1024])
def test_l2norm(device, dtype, N):
    from fla_amd.modules import l2_norm
    from oracle.modules import l2norm
    gen = torch.Generator().manual_seed(N)
    x = (torch.randn(3, 37, 2, N, generator=gen) * 1.5).to(dtype)
    dy = torch.randn(3, 37, 2, N, generator=gen).to(dtype)
    print(f"l2_norm {dtype} N={N}", flush=True)
    xd = x.to(device).requires_grad_()
    y = l2_norm(xd)
    y.backward(dy.to(device))
    xr = x.float().requires_grad_()
    yr = l2norm(xr)
    yr.backward(dy.float())
    ft, bt = _tols(dtype)
    assert y.dtype == dtype and xd.grad.dtype == dtype
    assert_close("y", yr, y, ft)
    assert_close("dx", xr.grad, xd.grad, bt)


def test_l2norm_output_dtype_and_empty(device):
    from fla_amd.modules import l2_norm
    from oracle.modules import l2norm
    x = torch.randn(5, 128).bfloat16()
    y = l2_norm(x.to(device), output_dtype=torch.float32)
    assert y.dtype == torch.float32
    assert_close("y", l2norm(x), y, 1e-5)
    assert l2_norm(torch.empty(0, 128, device=device)).shape == (0, 128)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("is_rms", [True, False])
@pytest.mark.parametrize("N,affine", [(128, True), (128, False), (64, True), (256, True), (1024, True), (1536, True)])
def test_norm_swish_gate(device, dtype, is_rms, N, affine):
    from fla_amd.modules import FusedLayerNormSwishGate, FusedRMSNormSwishGate
    from oracle.modules import norm_swish_gate
    gen = torch.Generator().manual_seed(N + is_rms)
    shape = (2, 300, 3, N) if N <= 256 else (2, 77, N)
    x = (torch.randn(*shape, generator=gen) * 2 + 0.3).to(dtype)
    o = torch.randn(*shape, generator=gen).to(dtype)
    dy = torch.randn(*shape, generator=gen).to(dtype)
    w = torch.randn(N, generator=gen) * 0.5 + 1.0
    print(f"norm gate {dtype} rms={is_rms} N={N} affine={affine}", flush=True)
    mod = (FusedRMSNormSwishGate if is_rms else FusedLayerNormSwishGate)(N, elementwise_affine=affine, eps=1e-5).to(device)
    if affine:
        with torch.no_grad():
            mod.weight.copy_(w)
    xd, od = x.to(device).requires_grad_(), o.to(device).requires_grad_()
    y = mod(xd, od)
    y.backward(dy.to(device))
    xr, orr = x.float().requires_grad_(), o.float().requires_grad_()
    wr = w.clone().requires_grad_() if affine else None
    yr = norm_swish_gate(xr, orr, wr, None, eps=1e-5, is_rms_norm=is_rms)
    yr.backward(dy.float())
    ft, bt = _tols(dtype)
    assert y.dtype == dtype
    assert_close("y", yr, y, ft)
    assert_close("dx", xr.grad, xd.grad, bt)
    assert_close("do", orr.grad, od.grad, bt)
    if affine:
        assert_close("dw", wr.grad, mod.weight.grad, 2e-3 if dtype != torch.float32 else 1e-5)


def test_norm_swish_gate_with_bias_function(device):
    from fla_amd.modules import layer_norm_swish_gate_fn
    from oracle.modules import norm_swish_gate
    gen = torch.Generator().manual_seed(5)
    N = 128
    x, o, dy = (torch.randn(4, 50, N, generator=gen) for _ in range(3))
    w, b = torch.randn(N, generator=gen), torch.randn(N, generator=gen)
    leaves = [t.to(device).requires_grad_() for t in (x, o, w, b)]
    y = layer_norm_swish_gate_fn(*leaves, eps=1e-6)
    y.backward(dy.to(device))
    refs = [t.clone().requires_grad_() for t in (x, o, w, b)]
    yr = norm_swish_gate(*refs, eps=1e-6, is_rms_norm=False)
    yr.backward(dy)
    assert_close("y", yr, y, 1e-5)
    for name, r, d in zip(("dx", "do", "dw", "db"), refs, leaves):
        assert_close(name, r.grad, d.grad, 1e-5)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("is_rms", [True, False])
@pytest.mark.parametrize("res_kind,prenorm,in_fp32", [("same", False, False), ("same", True, False), ("fp32", True, False),
                                                     (None, True, True), (None, True, False), ("fp32", False, False)])
def test_norm_swish_gate_residual_prenorm(device, dtype, is_rms, res_kind, prenorm, in_fp32):
    """The residual / prenorm forms of the reference's function (fla/modules/fused_norm_gate.py:402-481): the sum
    x + residual is normalised, prenorm returns it, and gradients reach x, o, the weight and the residual."""
    from fla_amd.modules import layer_norm_swish_gate_fn, rms_norm_swish_gate_fn
    from oracle.modules import norm_swish_gate
    gen = torch.Generator().manual_seed(11)
    N, shape = 128, (3, 70, 2, 128)
    x = (torch.randn(*shape, generator=gen) * 2 + 0.3).to(dtype)
    o = torch.randn(*shape, generator=gen).to(dtype)
    dy = torch.randn(*shape, generator=gen).to(dtype)
    dpre = torch.randn(*shape, generator=gen)
    w = torch.randn(N, generator=gen) * 0.5 + 1.0
    res = None if res_kind is None else torch.randn(*shape, generator=gen).to(dtype if res_kind == "same" else torch.float32)
    print(f"norm gate residual {dtype} rms={is_rms} res={res_kind} prenorm={prenorm} fp32={in_fp32}", flush=True)
    fn = rms_norm_swish_gate_fn if is_rms else layer_norm_swish_gate_fn
    xd, od, wd = x.to(device).requires_grad_(), o.to(device).requires_grad_(), w.to(device).requires_grad_()
    rd = None if res is None else res.to(device).requires_grad_()
    out = fn(xd, od, wd, None, residual=rd, prenorm=prenorm, residual_in_fp32=in_fp32, eps=1e-5)
    xr, orr, wr = x.float().requires_grad_(), o.float().requires_grad_(), w.clone().requires_grad_()
    rr = None if res is None else res.float().requires_grad_()
    ref = norm_swish_gate(xr, orr, wr, None, eps=1e-5, is_rms_norm=is_rms, residual=rr, prenorm=prenorm)
    ft, bt = _tols(dtype)
    if prenorm:
        y, pre = out
        yr, prer = ref
        want = res.dtype if res is not None else (torch.float32 if in_fp32 else dtype)
        assert pre.dtype == want and pre.shape == x.shape
        assert_close("residual_out", prer, pre, ft)
        (y.float() * dy.to(device).float()).sum().add((pre.float() * dpre.to(device)).sum()).backward()
        ((yr * dy.float()).sum() + (prer * dpre).sum()).backward()
    else:
        y, yr = out, ref
        y.backward(dy.to(device))
        yr.backward(dy.float())
    assert y.dtype == dtype
    assert_close("y", yr, y, ft)
    assert_close("dx", xr.grad, xd.grad, bt)
    assert_close("do", orr.grad, od.grad, bt)
    assert_close("dw", wr.grad, wd.grad, 2e-3 if dtype != torch.float32 else 1e-5)
    if res is not None:
        assert rd.grad.dtype == res.dtype
        assert_close("dresidual", rr.grad, rd.grad, bt)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("W", [2, 3, 4])
@pytest.mark.parametrize("T,D,bias,act", [(1, 64, False, "silu"), (5, 64, True, "silu"), (64, 200, False, None),
                                          (300, 512, True, "silu"), (1000, 2048, False, "silu")])
def test_causal_conv1d(device, dtype, W, T, D, bias, act):
    from fla_amd.modules import ShortConvolution
    from oracle.modules import causal_conv1d
    gen = torch.Generator().manual_seed(T + W)
    B = 2
    x = torch.randn(B, T, D, generator=gen).to(dtype)
    dy = torch.randn(B, T, D, generator=gen).to(dtype)
    print(f"short conv {dtype} W={W} T={T} D={D} bias={bias} act={act}", flush=True)
    conv = ShortConvolution(D, W, bias=bias, activation=act).to(device)
    w = conv.weight.detach().cpu().reshape(D, W).clone()
    b = conv.bias.detach().cpu().clone() if bias else None
    xd = x.to(device).requires_grad_()
    # with a cache a single token takes the (non-differentiable) decode step, as in the reference
    y, cache = conv(xd, output_final_state=T > 1)
    y.backward(dy.to(device))
    xr = x.float().requires_grad_()
    wr = w.clone().requires_grad_()
    br = b.clone().requires_grad_() if bias else None
    yr = causal_conv1d(xr, wr, br, act)
    yr.backward(dy.float())
    ft, bt = _tols(dtype)
    assert y.dtype == dtype and y.shape == x.shape
    assert_close("y", yr, y, ft)
    assert_close("dx", xr.grad, xd.grad, bt)
    # weight/bias gradients are fp32 sums over B*T terms of 16-bit inputs
    assert_close("dw", wr.grad, conv.weight.grad.reshape(D, W), 2e-3 if dtype != torch.float32 else 2e-5)
    if bias:
        assert_close("db", br.grad, conv.bias.grad, 2e-3 if dtype != torch.float32 else 2e-5)
    # final state: the last W inputs, zero-padded on the left, [B,D,W]
    if T > 1:
        ref_cache = torch.nn.functional.pad(x.transpose(1, 2), (W - T, 0))
        assert torch.equal(cache.cpu(), ref_cache)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("W", [2, 4])
def test_short_convolution_step(device, dtype, W):
    """Prefill T tokens then decode 3 more one at a time == one pass over T+3 tokens."""
    from fla_amd.modules import ShortConvolution
    gen = torch.Generator().manual_seed(9)
    B, T, D = 3, 20, 256
    x = torch.randn(B, T + 3, D, generator=gen).to(dtype).to(device)
    conv = ShortConvolution(D, W, bias=True, activation="silu").to(device).to(dtype)
    with torch.no_grad():
        full, _ = conv(x)
        y, cache = conv(x[:, :T].contiguous(), output_final_state=True)
        outs = [y]
        for t in range(T, T + 3):
            yt, cache = conv(x[:, t:t + 1].contiguous(), cache=cache)
            outs.append(yt)
    got = torch.cat(outs, dim=1)
    assert_close("y", full, got, 1e-6 if dtype == torch.float32 else 4e-3)
    assert torch.equal(cache, x[:, -W:].transpose(1, 2))


@pytest.mark.parametrize("dtype,out_dtype", [(torch.bfloat16, torch.float32), (torch.float16, torch.float32),
                                             (torch.float32, torch.float32), (torch.bfloat16, torch.bfloat16)])
@pytest.mark.parametrize("normalizer,clamp_min", [(16.0, None), (1.0, None), (0.05, None), (16.0, -0.05)])
def test_gla_gate(device, dtype, out_dtype, normalizer, clamp_min):
    """logsigmoid(x) / normalizer (+ clamp) of fla/layers/gla.py:214-217, forward and backward."""
    from fla_amd.modules import gla_gate
    from oracle.modules import gla_gate as ref_gate
    gen = torch.Generator().manual_seed(11)
    x = (torch.randn(2, 129, 4, 64, generator=gen) * 3).to(dtype)
    x[0, 0, 0, :8] = torch.tensor([-90.0, -30.0, -12.0, 0.0, 12.0, 30.0, 90.0, 1e-3]).to(dtype)
    dy = torch.randn(2, 129, 4, 64, generator=gen)
    print(f"gla_gate {dtype}->{out_dtype} normalizer={normalizer} clamp={clamp_min}", flush=True)
    xd = x.to(device).requires_grad_()
    y = gla_gate(xd, normalizer, clamp_min, output_dtype=out_dtype)
    y.backward(dy.to(device).to(out_dtype))
    xr = x.double().requires_grad_()
    yr = ref_gate(xr, normalizer, clamp_min, dtype=torch.float64)
    yr.backward(dy.to(out_dtype).double())
    assert y.dtype == out_dtype and xd.grad.dtype == dtype
    assert_close("y", yr, y, 1e-5 if out_dtype == torch.float32 else 4e-3)
    # tiny values far on the positive side must keep their relative accuracy too (they are e^{-x}, not 0)
    if out_dtype == torch.float32 and clamp_min is None:
        big = x.double() > 10
        assert_close("y(x > 10)", yr[big], y.detach().cpu()[big], 1e-5)
    assert_close("dx", xr.grad, xd.grad, 1e-5 if dtype == torch.float32 else 4e-3)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("H,with_b,with_bias", [(16, True, True), (6, True, True), (32, False, True), (7, True, False)])
def test_gdn_gate(device, dtype, H, with_b, with_bias):
    """g = -exp(A_log) softplus(a + dt_bias), beta = sigmoid(b) of fla/layers/gated_deltanet.py:236-237,
    forward and backward incl. the per-head parameter gradients; run twice for bit-equal gradients."""
    from fla_amd.modules import gdn_gate
    from oracle.modules import gdn_gate as ref_gate
    gen = torch.Generator().manual_seed(H)
    a = (torch.randn(3, 211, H, generator=gen) * 4).to(dtype)
    a[0, 0, 0], a[0, 0, 1] = 35.0, -60.0
    b = (torch.randn(3, 211, H, generator=gen) * 2).to(dtype) if with_b else None
    A_log = torch.randn(H, generator=gen)
    dt_bias = torch.randn(H, generator=gen) if with_bias else None
    dg = torch.randn(3, 211, H, generator=gen)
    dbeta = torch.randn(3, 211, H, generator=gen).to(dtype) if with_b else None
    print(f"gdn_gate {dtype} H={H} b={with_b} bias={with_bias}", flush=True)

    def run():
        leaves = [t.to(device).requires_grad_() if t is not None else None for t in (a, b, A_log, dt_bias)]
        g, beta = gdn_gate(*leaves)
        outs, grads = [g], [dg.to(device)]
        if with_b:
            outs.append(beta)
            grads.append(dbeta.to(device))
        torch.autograd.backward(outs, grads)
        return g, beta, [None if t is None else t.grad for t in leaves]

    g, beta, grads = run()
    _, _, grads2 = run()
    for x, y in zip(grads, grads2):
        assert (x is None and y is None) or torch.equal(x, y)
    leaves = [t.double().requires_grad_() if t is not None else None for t in (a, b, A_log, dt_bias)]
    gr, br = ref_gate(*leaves, dtype=torch.float64)
    outs, gs = [gr], [dg.double()]
    if with_b:
        outs.append(br)
        gs.append(dbeta.double())
    torch.autograd.backward(outs, gs)
    ft, bt = _tols(dtype)
    assert g.dtype == torch.float32
    assert_close("g", gr, g, 1e-5)
    if with_b:
        assert beta.dtype == dtype
        assert_close("beta", br, beta, ft)
        assert_close("db", leaves[1].grad, grads[1], bt)
    assert_close("da", leaves[0].grad, grads[0], bt)
    assert_close("dA_log", leaves[2].grad, grads[2], 1e-4)
    if with_bias:
        assert_close("ddt_bias", leaves[3].grad, grads[3], 1e-4)
