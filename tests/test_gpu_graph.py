"""GPU: the single-token decode path under HIP graph capture (serving loops replay one captured
step per token).  A captured step -- short convolution step, l2 norm, the recurrent state update
in place, gated output norm -- is replayed several times with eager work and synchronisations
in between, and every replay is compared with the same step run eagerly."""
import pytest
import torch
import torch.nn.functional as F

from helpers import assert_close

pytestmark = pytest.mark.gpu


def _decode_step(mods, x, gate_in, g, beta, state, conv_cache):
    """One token through conv step -> l2 norm -> gated delta rule update -> gated RMS norm."""
    from fla_amd.modules import l2_norm
    from fla_amd.ops.gated_delta_rule import fused_recurrent_gated_delta_rule
    conv, norm = mods
    B, _, HD = x.shape
    H = state.shape[1]
    D = HD // H
    y, _ = conv(x, cache=conv_cache)                       # [B,1,H*D], cache updated in place
    q = l2_norm(y.view(B, 1, H, D))
    k = l2_norm(torch.roll(y, 1, dims=-1).view(B, 1, H, D))
    v = y.view(B, 1, H, D)
    o, _ = fused_recurrent_gated_delta_rule(q, k, v, g, beta, initial_state=state, output_final_state=True,
                                            head_first=False, inplace_state=True)
    return norm(o, gate_in.view(B, 1, H, D))


def test_decode_step_graph_replay(device):
    from fla_amd.modules import FusedRMSNormSwishGate, ShortConvolution
    torch.manual_seed(0)
    B, H, D, W, steps = 4, 4, 128, 4, 5
    conv = ShortConvolution(H * D, W, activation="silu").to(device).bfloat16()
    norm = FusedRMSNormSwishGate(D).to(device)
    mods = (conv, norm)
    xs = torch.randn(steps, B, 1, H * D, device=device).bfloat16()
    gates = torch.randn(steps, B, 1, H * D, device=device).bfloat16()
    gs = F.logsigmoid(torch.randn(steps, B, 1, H, device=device))
    betas = torch.rand(steps, B, 1, H, device=device)
    state0 = torch.randn(B, H, D, D, device=device) * 0.1

    with torch.no_grad():
        # eager run
        state_e, cache_e = state0.clone(), torch.zeros(B, H * D, W, device=device, dtype=torch.bfloat16)
        eager = [_decode_step(mods, xs[t], gates[t], gs[t], betas[t], state_e, cache_e).clone() for t in range(steps)]
        torch.cuda.synchronize()

        # captured step on static buffers
        sx, sgate, sg, sbeta = xs[0].clone(), gates[0].clone(), gs[0].clone(), betas[0].clone()
        state_g, cache_g = state0.clone(), torch.zeros_like(cache_e)
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):          # warm-up outside capture (lazy initialisation)
            _decode_step(mods, sx, sgate, sg, sbeta, state_g.clone(), cache_g.clone())
        torch.cuda.current_stream().wait_stream(side)
        graph = torch.cuda.CUDAGraph()
        print("capturing decode step", flush=True)
        with torch.cuda.graph(graph):
            out = _decode_step(mods, sx, sgate, sg, sbeta, state_g, cache_g)
        # the capture itself did not run the kernels: state and cache are still the initial ones
        state_g.copy_(state0)
        cache_g.zero_()
        for t in range(steps):
            sx.copy_(xs[t]); sgate.copy_(gates[t]); sg.copy_(gs[t]); sbeta.copy_(betas[t])
            graph.replay()
            torch.cuda.synchronize()
            assert_close(f"replay {t}", eager[t], out, 1e-6)
            _ = (xs[t].float() @ xs[t].float().transpose(-1, -2)).sum().item()   # unrelated eager work between replays
        assert_close("state", state_e, state_g, 1e-6)
        assert torch.equal(cache_e, cache_g)
