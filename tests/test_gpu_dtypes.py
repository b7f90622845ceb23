"""GPU: storage types other than the default (bf16 q/k/v, fp32 gates, fp32 state): fp16 q/k/v,
gates / beta / initial state in the q/k/v type, as the reference's own tests build them
(tests/ops/test_gla.py:110-121 draws g and h0 in the test dtype; tests/ops/test_gated_delta.py:180-192
draws beta in it).  Forward and backward against the fp32 naive recurrences."""
import pytest
import torch

from helpers import assert_close, gdr_inputs, gla_inputs, random_offsets
from test_gpu_gdr import NAMES as GDR_NAMES, TOLS as GDR_TOLS, _grads_dev as gdr_grads_dev, _grads_ref as gdr_grads_ref
from test_gpu_gla import _grads_dev as gla_grads_dev, _grads_ref as gla_grads_ref

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("varlen", [False, True])
def test_chunk_gla_storage_types(device, dtype, varlen):
    """q, k, v, g, h0 and the incoming gradients all in `dtype`."""
    T, H, K, V = 300, 2, 128, 128
    gen = torch.Generator().manual_seed(3)
    offs = random_offsets(T, 3, gen, min_len=1) if varlen else None
    B, N = (1, 3) if varlen else (2, 2)
    q, k, v, g, h0 = gla_inputs(B, T, H, K, V, seed=71, dtype=dtype, normalizer=16.0, N=N, h0_std=1.0)
    g, h0 = g.to(dtype), h0.to(dtype)
    do = torch.randn(B, T, H, V, generator=gen).to(dtype)
    dht = (torch.randn(N, H, K, V, generator=gen) * 0.1)
    print(f"chunk_gla storage {dtype} varlen={varlen}", flush=True)
    got = gla_grads_dev(device, q, k, v, g, h0, do, dht, offsets=offs)
    ref = gla_grads_ref(q, k, v, g, h0, do, dht, offsets=None if offs is None else offs.tolist())
    # gradients of tensors stored in 16 bits are rounded once more on the way out
    for name, r, x, tol in zip(("dq", "dk", "dv", "dg", "dh0"), ref, got, (8e-3, 8e-3, 8e-3, 1.2e-2, 8e-3)):
        assert x.dtype == dtype, (name, x.dtype)
        assert_close(name, r, x, tol)

    from fla_amd.ops.gla import chunk_gla
    from oracle.recurrent import naive_recurrent_gla
    dev = lambda x: None if x is None else x.to(device)
    o, ht = chunk_gla(dev(q), dev(k), dev(v), dev(g), initial_state=dev(h0), output_final_state=True,
                      offsets=dev(offs), head_first=False)
    ro, rht = naive_recurrent_gla(q, k, v, g, initial_state=h0, output_final_state=True,
                                  offsets=None if offs is None else offs.tolist())
    assert o.dtype == dtype and ht.dtype == torch.float32
    assert_close("o", ro, o, 1e-2)
    assert_close("ht", rht, ht, 5e-3)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("varlen", [False, True])
def test_chunk_gdr_storage_types(device, dtype, varlen):
    """q, k, v, beta and the incoming gradient in `dtype`; log-gates and state fp32 as in the reference's test."""
    T, H, K, V = 300, 2, 128, 128
    gen = torch.Generator().manual_seed(4)
    offs = random_offsets(T, 3, gen, min_len=1) if varlen else None
    B, N = (1, 3) if varlen else (2, 2)
    q, k, v, g, beta, h0 = gdr_inputs(B, T, H, K, V, seed=72, dtype=dtype, N=N, h0_std=1.0)
    beta = beta.to(dtype)
    do = torch.randn(B, T, H, V, generator=gen).to(dtype)
    dht = torch.randn(N, H, K, V, generator=gen) * 0.1
    print(f"chunk_gdr storage {dtype} varlen={varlen}", flush=True)
    got = gdr_grads_dev(device, q, k, v, g, beta, h0, do, dht, offsets=offs)
    ref = gdr_grads_ref(q, k, v, g, beta, h0, do, dht, offsets=None if offs is None else offs.tolist())
    for name, r, x, tol in zip(GDR_NAMES, ref, got, GDR_TOLS):
        assert_close(name, r, x, tol)
    assert got[0].dtype == dtype and got[4].dtype == dtype and got[3].dtype == torch.float32

    from fla_amd.ops.gated_delta_rule import chunk_gated_delta_rule
    from oracle.recurrent import naive_recurrent_gated_delta_rule
    dev = lambda x: None if x is None else x.to(device)
    o, ht = chunk_gated_delta_rule(dev(q), dev(k), dev(v), dev(g), dev(beta), initial_state=dev(h0),
                                   output_final_state=True, offsets=dev(offs), head_first=False)
    ro, rht = naive_recurrent_gated_delta_rule(q, k, v, g, beta, initial_state=h0, output_final_state=True,
                                               offsets=None if offs is None else offs.tolist())
    assert o.dtype == dtype and ht.dtype == torch.float32
    assert_close("o", ro, o, 1e-2)
    assert_close("ht", rht, ht, 5e-3)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16, torch.float32])
def test_fused_recurrent_storage_types(device, dtype):
    """The decode step and a short prefill in every storage type the reference's tests use
    (tests/ops/test_gla.py:33 runs fused_recurrent_gla in fp32)."""
    from fla_amd.ops.gla import fused_recurrent_gla
    from fla_amd.ops.gated_delta_rule import fused_recurrent_gated_delta_rule
    from oracle.recurrent import naive_recurrent_gated_delta_rule, naive_recurrent_gla
    dev = lambda x: None if x is None else x.to(device)
    tol = 1e-4 if dtype == torch.float32 else 1e-2
    for T in (1, 40):
        q, k, v, g, h0 = gla_inputs(2, T, 3, 128, 128, seed=73 + T, dtype=dtype, normalizer=4.0, h0_std=1.0)
        print(f"fused_recurrent_gla {dtype} T={T}", flush=True)
        o, ht = fused_recurrent_gla(dev(q), dev(k), dev(v), gk=dev(g.to(dtype)), initial_state=dev(h0),
                                    output_final_state=True, head_first=False)
        ro, rht = naive_recurrent_gla(q, k, v, g.to(dtype), initial_state=h0, output_final_state=True)
        assert_close("o", ro, o, tol)
        assert_close("ht", rht, ht, 5e-3 if dtype != torch.float32 else 1e-5)
        q, k, v, g, beta, h0 = gdr_inputs(2, T, 3, 128, 128, seed=74 + T, dtype=dtype, h0_std=1.0)
        print(f"fused_recurrent_gated_delta_rule {dtype} T={T}", flush=True)
        o, ht = fused_recurrent_gated_delta_rule(dev(q), dev(k), dev(v), dev(g), dev(beta.to(dtype)), initial_state=dev(h0),
                                                 output_final_state=True, head_first=False)
        ro, rht = naive_recurrent_gated_delta_rule(q, k, v, g, beta.to(dtype), initial_state=h0, output_final_state=True)
        assert_close("o", ro, o, tol)
        assert_close("ht", rht, ht, 5e-3 if dtype != torch.float32 else 1e-5)


def test_chunk_gla_fp16_strong_gates(device):
    """fp16 ends at 65504: with chunk-cumulative log-gates beyond about -8 the factor e^{-G} on k no longer fits,
    so such chunks must take the exact pairwise arithmetic (bf16 only needs it beyond -80).  Forward and backward
    against the fp32 recurrence, 1e-2 / 2e-2 as for the other dtypes."""
    import torch.nn.functional as F
    from fla_amd.ops.gla import chunk_gla
    from helpers import assert_close
    from oracle.recurrent import naive_recurrent_gla
    B, T, H, K, V = 2, 256, 2, 128, 128
    gen = torch.Generator().manual_seed(5)
    q = (torch.randn(B, T, H, K, generator=gen) * 0.5).half()
    k = (torch.randn(B, T, H, K, generator=gen) * 0.5).half()
    v = torch.randn(B, T, H, V, generator=gen).half()
    g = F.logsigmoid(torch.randn(B, T, H, K, generator=gen))          # about -0.8 per step: -50 over a chunk
    do = torch.randn(B, T, H, V, generator=gen).half()
    leaves = [x.to(device).detach().requires_grad_() for x in (q, k, v, g)]
    o, ht = chunk_gla(*leaves, output_final_state=True, head_first=False)
    o.backward(do.to(device))
    torch.cuda.synchronize()
    rl = [x.detach().float().requires_grad_() for x in (q, k, v, g)]
    ro, rht = naive_recurrent_gla(*rl, output_final_state=True)
    (ro * do.float()).sum().backward()
    assert_close("o", ro, o, 1e-2)
    assert_close("ht", rht, ht, 5e-3)
    for name, a, b in zip(("dq", "dk", "dv", "dg"), rl, leaves):
        assert_close(name, a.grad, b.grad, 2e-2)


@pytest.mark.parametrize("T,D,head_first,varlen", [(130, 64, False, False), (300, 100, True, False), (200, 128, False, True),
                                                   (64, 300, False, False)])
def test_chunk_gla_fp32_inputs(device, monkeypatch, T, D, head_first, varlen):
    """fp32 q, k, v on the exact route (FLA_AMD_FP32_EXACT=1; tests/ops/test_gla.py:29-87 and :149-201 run the operator in
    fp32): forward and backward to fp32 accuracy, rel-L2 <= 1e-4, against the fp32 naive recurrence - no rounding of
    the inputs to 16 bits."""
    import torch.nn.functional as F
    import fla_amd.ops.gla.chunk as mod
    from fla_amd.ops.gla import chunk_gla
    monkeypatch.setattr(mod, "FP32_INPUTS_EXACT", True)
    from helpers import assert_close
    from oracle.recurrent import naive_recurrent_gla
    B, H = (1, 2) if varlen else (2, 2)
    N = 3 if varlen else B
    gen = torch.Generator().manual_seed(T + D)
    q, k, v = (torch.randn(B, T, H, D, generator=gen) for _ in range(3))
    g = F.logsigmoid(torch.randn(B, T, H, D, generator=gen)) / 4
    h0 = torch.randn(N, H, D, D, generator=gen)
    do = torch.randn(B, T, H, D, generator=gen)
    dht = torch.randn(N, H, D, D, generator=gen) * 0.1
    offs = torch.tensor([0, 17, 90, T]) if varlen else None
    print(f"chunk_gla fp32 T={T} D={D} head_first={head_first} varlen={varlen}", flush=True)
    tr = (lambda x: x.transpose(1, 2).contiguous()) if head_first else (lambda x: x)
    leaves = [tr(x).to(device).requires_grad_() for x in (q, k, v, g)]
    h0l = h0.to(device).requires_grad_()
    import warnings
    with warnings.catch_warnings(record=True) as record:
        warnings.simplefilter("always")
        o, ht = chunk_gla(*leaves, initial_state=h0l, output_final_state=True, head_first=head_first,
                          offsets=None if offs is None else offs.to(device))
    assert not [w for w in record if "rounded" in str(w.message)]
    assert o.dtype == torch.float32 and ht.dtype == torch.float32
    ((o * tr(do).to(device)).sum() + (ht * dht.to(device)).sum()).backward()
    rl = [x.clone().requires_grad_() for x in (q, k, v, g)]
    rh0 = h0.clone().requires_grad_()
    ro, rht = naive_recurrent_gla(*rl, initial_state=rh0, output_final_state=True,
                                  offsets=None if offs is None else offs.tolist())
    ((ro * do).sum() + (rht * dht).sum()).backward()
    assert_close("o", ro, tr(o) if head_first else o, 1e-4)
    assert_close("ht", rht, ht, 1e-4)
    for name, a, b in zip(("dq", "dk", "dv", "dg"), rl, leaves):
        assert_close(name, a.grad, tr(b.grad) if head_first else b.grad, 2e-4)
    assert_close("dh0", rh0.grad, h0l.grad, 1e-4)


@pytest.mark.parametrize("T,D,varlen,magnitude", [(300, 128, False, 1.0), (257, 100, True, 1.0), (130, 64, False, 3e5),
                                                   (130, 64, False, 1e-6)])
def test_chunk_gla_fp32_inputs_default_route(device, T, D, varlen, magnitude):
    """The default route for fp32 q, k, v (scaled by powers of two into fp16's range, chunk kernels, fp32 gates and
    states): forward and backward inside the tolerances of the reference's own fp32 tests (tests/ops/test_gla.py:195-201:
    4e-3 on o, 5e-3 on the rest), fp32 tensors in and out - also for magnitudes far outside what fp16 holds."""
    import torch.nn.functional as F
    import fla_amd.ops.gla.chunk as mod
    from helpers import assert_close
    from oracle.recurrent import naive_recurrent_gla
    B, H = (1, 2) if varlen else (2, 2)
    N = 3 if varlen else B
    gen = torch.Generator().manual_seed(T + D)
    q, k, v = (torch.randn(B, T, H, D, generator=gen) * magnitude for _ in range(3))
    g = F.logsigmoid(torch.randn(B, T, H, D, generator=gen))
    h0 = torch.randn(N, H, D, D, generator=gen) * magnitude ** 2
    do = torch.randn(B, T, H, D, generator=gen)
    dht = torch.randn(N, H, D, D, generator=gen) * 0.1
    offs = torch.tensor([0, 17, 90, T]) if varlen else None
    print(f"chunk_gla fp32 default route T={T} D={D} varlen={varlen} magnitude={magnitude}", flush=True)
    leaves = [x.to(device).requires_grad_() for x in (q, k, v, g)]
    h0l = h0.to(device).requires_grad_()
    o, ht = mod.chunk_gla(*leaves, initial_state=h0l, output_final_state=True, head_first=False,
                          offsets=None if offs is None else offs.to(device))
    assert o.dtype == torch.float32 and ht.dtype == torch.float32
    ((o * do.to(device)).sum() + (ht * dht.to(device)).sum()).backward()
    rl = [x.clone().requires_grad_() for x in (q, k, v, g)]
    rh0 = h0.clone().requires_grad_()
    ro, rht = naive_recurrent_gla(*rl, initial_state=rh0, output_final_state=True,
                                  offsets=None if offs is None else offs.tolist())
    ((ro * do).sum() + (rht * dht).sum()).backward()
    assert_close("o", ro, o, 4e-3)
    assert_close("ht", rht, ht, 5e-3)
    for name, a, b in zip(("dq", "dk", "dv", "dg"), rl, leaves):
        assert b.grad.dtype == torch.float32
        assert_close(name, a.grad, b.grad, 5e-3)
    assert_close("dh0", rh0.grad, h0l.grad, 5e-3)
