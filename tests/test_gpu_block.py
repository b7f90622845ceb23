"""GPU: the operator together with the steps either side of it, as the reference's GatedDeltaNet
layer strings them (fla/layers/gated_deltanet.py:200-262: short convolutions with SiLU on q, k, v;
l2 norm of q, k; chunk_gated_delta_rule; gated RMS norm of the output), forward and backward through
every autograd function of this package at once, against the same chain built from the oracle."""
import pytest
import torch
import torch.nn.functional as F

from helpers import assert_close

pytestmark = pytest.mark.gpu


def _block_device(mods, x, gate, g, beta, H, D):
    from fla_amd.modules import l2_norm
    from fla_amd.ops.gated_delta_rule import chunk_gated_delta_rule
    cq, ck, cv, norm = mods
    B, T, _ = x.shape
    q, _ = cq(x)
    k, _ = ck(x)
    v, _ = cv(x)
    q, k, v = (t.view(B, T, H, D) for t in (q, k, v))
    o, _ = chunk_gated_delta_rule(l2_norm(q), l2_norm(k), v, g, beta, head_first=False)
    return norm(o, gate.view(B, T, H, D))


def _block_oracle(ws, nw, x, gate, g, beta, H, D):
    from oracle.modules import causal_conv1d, l2norm, norm_swish_gate
    from oracle.recurrent import naive_recurrent_gated_delta_rule
    B, T, _ = x.shape
    q, k, v = (causal_conv1d(x, w, None, "silu").view(B, T, H, D) for w in ws)
    o, _ = naive_recurrent_gated_delta_rule(l2norm(q), l2norm(k), v, g, beta)
    return norm_swish_gate(o, gate.view(B, T, H, D), nw, None, eps=1e-5, is_rms_norm=True)


def test_gated_deltanet_style_block(device):
    from fla_amd.modules import FusedRMSNormSwishGate, ShortConvolution
    torch.manual_seed(1)
    B, T, H, D, W = 2, 200, 2, 128, 4
    x = torch.randn(B, T, H * D).bfloat16()
    gate = torch.randn(B, T, H * D).bfloat16()
    g = F.logsigmoid(torch.randn(B, T, H))
    beta = torch.rand(B, T, H).sigmoid()
    dy = torch.randn(B, T, H, D).bfloat16()
    convs = [ShortConvolution(H * D, W, activation="silu") for _ in range(3)]
    norm = FusedRMSNormSwishGate(D)
    with torch.no_grad():
        norm.weight.copy_(torch.rand(D) + 0.5)
    ws = [c.weight.detach().reshape(H * D, W).clone().requires_grad_() for c in convs]
    nw = norm.weight.detach().clone().requires_grad_()
    mods = [m.to(device) for m in convs] + [norm.to(device)]
    print("GatedDeltaNet-style block", flush=True)
    leaves = [t.to(device).requires_grad_() for t in (x, gate, g, beta)]
    y = _block_device(mods, *leaves, H, D)
    y.backward(dy.to(device))
    refs = [t.float().requires_grad_() for t in (x, gate, g, beta)]
    yr = _block_oracle(ws, nw, *refs, H, D)
    yr.backward(dy.float())
    assert_close("y", yr, y, 1e-2)
    # gradients pass through three rounded 16-bit tensors on the device path
    for name, r, d, tol in zip(("dx", "dgate", "dg", "dbeta"), refs, leaves, (2e-2, 1e-2, 3e-2, 3e-2)):
        assert_close(name, r.grad, d.grad, tol)
    for i, (w, c) in enumerate(zip(ws, mods[:3])):
        assert_close(f"dconv{i}", w.grad, c.weight.grad.reshape(H * D, W), 2e-2)
    assert_close("dnorm_w", nw.grad, mods[3].weight.grad, 1e-2)
