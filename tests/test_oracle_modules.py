"""CPU: the torch restatements of the row-wise steps (oracle/modules.py) against library routines
and the invariants that fix them."""
import pytest
import torch
import torch.nn.functional as F

from oracle.modules import causal_conv1d, causal_conv1d_step, gdn_gate, gla_gate, l2norm, norm_swish_gate


def test_l2norm_unit_norm_and_scale_invariance():
    gen = torch.Generator().manual_seed(0)
    x = torch.randn(5, 7, 64, generator=gen, dtype=torch.float64)
    y = l2norm(x, eps=0.0, dtype=torch.float64)
    torch.testing.assert_close(y.norm(dim=-1), torch.ones(5, 7, dtype=torch.float64))
    torch.testing.assert_close(l2norm(3.7 * x, eps=0.0, dtype=torch.float64), y)
    # eps sits inside the square root: a zero row maps to zero, and the norm of a unit row is 1/sqrt(1+eps)
    assert l2norm(torch.zeros(1, 8), eps=1e-6).abs().max() == 0
    e = torch.zeros(1, 8, dtype=torch.float64)
    e[0, 3] = 1.0
    torch.testing.assert_close(l2norm(e, eps=0.25, dtype=torch.float64)[0, 3], torch.tensor(1 / 1.25 ** 0.5, dtype=torch.float64))


@pytest.mark.parametrize("is_rms", [True, False])
@pytest.mark.parametrize("affine", [True, False])
def test_norm_swish_gate_against_library(is_rms, affine):
    gen = torch.Generator().manual_seed(1)
    N = 48
    x = torch.randn(6, N, generator=gen, dtype=torch.float64) * 2 + 0.5
    o = torch.randn(6, N, generator=gen, dtype=torch.float64)
    w = torch.randn(N, generator=gen, dtype=torch.float64) if affine else None
    b = torch.randn(N, generator=gen, dtype=torch.float64) if affine else None
    got = norm_swish_gate(x, o, w, b, eps=1e-5, is_rms_norm=is_rms, dtype=torch.float64)
    if is_rms:
        ref = F.rms_norm(x, (N,), w, eps=1e-5)
        if b is not None:
            ref = ref + b
    else:
        ref = F.layer_norm(x, (N,), w, b, eps=1e-5)
    torch.testing.assert_close(got, ref * F.silu(o))
    # residual: the row that is normalised is the sum, and prenorm hands that sum back
    r = torch.randn(6, N, generator=gen, dtype=torch.float64)
    y2, pre = norm_swish_gate(x - r, o, w, b, eps=1e-5, is_rms_norm=is_rms, dtype=torch.float64, residual=r, prenorm=True)
    torch.testing.assert_close(y2, got)
    torch.testing.assert_close(pre, x)


@pytest.mark.parametrize("W", [2, 3, 4])
@pytest.mark.parametrize("act", [None, "silu"])
def test_causal_conv1d_against_library(W, act):
    gen = torch.Generator().manual_seed(2)
    B, T, D = 2, 11, 6
    x = torch.randn(B, T, D, generator=gen, dtype=torch.float64)
    w = torch.randn(D, W, generator=gen, dtype=torch.float64)
    b = torch.randn(D, generator=gen, dtype=torch.float64)
    got = causal_conv1d(x, w, b, act, dtype=torch.float64)
    ref = F.conv1d(x.transpose(1, 2), w.unsqueeze(1), b, padding=W - 1, groups=D)[..., :T].transpose(1, 2)
    if act:
        ref = F.silu(ref)
    torch.testing.assert_close(got, ref)
    # causality: changing the future leaves the past alone
    x2 = x.clone()
    x2[:, 7:] += 1.0
    torch.testing.assert_close(causal_conv1d(x2, w, b, act, dtype=torch.float64)[:, :7], got[:, :7])
    # the last tap multiplies the current input
    imp = torch.zeros(1, 5, D, dtype=torch.float64)
    imp[0, 2] = 1.0
    resp = causal_conv1d(imp, w, None, None, dtype=torch.float64)
    torch.testing.assert_close(resp[0, 2], w[:, W - 1])
    if W > 1:
        torch.testing.assert_close(resp[0, 3], w[:, W - 2])


def test_causal_conv1d_step_matches_full_convolution():
    gen = torch.Generator().manual_seed(3)
    B, T, D, W = 2, 9, 6, 4
    x = torch.randn(B, T, D, generator=gen, dtype=torch.float64)
    w = torch.randn(D, W, generator=gen, dtype=torch.float64)
    b = torch.randn(D, generator=gen, dtype=torch.float64)
    full = causal_conv1d(x, w, b, "silu", dtype=torch.float64)
    cache = torch.zeros(B, D, W, dtype=torch.float64)
    for t in range(T):
        y, cache = causal_conv1d_step(x[:, t], cache, w, b, "silu", dtype=torch.float64)
        torch.testing.assert_close(y, full[:, t])
    torch.testing.assert_close(cache, x[:, -W:].transpose(1, 2))


@pytest.mark.parametrize("normalizer", [16.0, 1.0, 0.05])
def test_gla_gate_against_library(normalizer):
    gen = torch.Generator().manual_seed(7)
    x = torch.cat([torch.randn(4, 33, generator=gen, dtype=torch.float64) * 3,
                   torch.tensor([[-800.0, -40.0, 0.0, 40.0, 800.0] + [0.5] * 28], dtype=torch.float64)])
    ref = F.logsigmoid(x) / normalizer
    torch.testing.assert_close(gla_gate(x, normalizer, dtype=torch.float64), ref)
    # a gate is a log-probability: never positive, 0 only in the limit, log(1/2)/normalizer at 0
    assert gla_gate(x, normalizer, dtype=torch.float64).max() <= 0
    torch.testing.assert_close(gla_gate(torch.zeros(1, dtype=torch.float64), normalizer, dtype=torch.float64),
                               torch.tensor([-0.6931471805599453 / normalizer], dtype=torch.float64))
    torch.testing.assert_close(gla_gate(x, normalizer, clamp_min=-0.3, dtype=torch.float64), ref.clamp_min(-0.3))
    # and its derivative: sigmoid(-x) / normalizer where the clamp is open, 0 where it binds
    xg = x.clone().requires_grad_()
    gla_gate(xg, normalizer, clamp_min=-0.3, dtype=torch.float64).sum().backward()
    want = torch.sigmoid(-x) / normalizer * (ref >= -0.3)
    torch.testing.assert_close(xg.grad, want)


def test_gdn_gate_against_library():
    gen = torch.Generator().manual_seed(8)
    H = 6
    a = torch.randn(3, 17, H, generator=gen, dtype=torch.float64) * 4
    a[0, 0, 0], a[0, 0, 1] = 35.0, -60.0          # either side of softplus' linear switch
    b = torch.randn(3, 17, H, generator=gen, dtype=torch.float64) * 3
    A_log = torch.randn(H, generator=gen, dtype=torch.float64)
    dt_bias = torch.randn(H, generator=gen, dtype=torch.float64)
    g, beta = gdn_gate(a, b, A_log, dt_bias, dtype=torch.float64)
    torch.testing.assert_close(g, -A_log.exp() * F.softplus(a + dt_bias))
    torch.testing.assert_close(beta, torch.sigmoid(b))
    assert g.max() <= 0 and 0 <= beta.min() and beta.max() <= 1
    g2, none = gdn_gate(a, None, A_log, None, dtype=torch.float64)
    assert none is None
    torch.testing.assert_close(g2, -A_log.exp() * F.softplus(a))
