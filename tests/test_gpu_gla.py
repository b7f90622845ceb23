"""GPU: chunk_gla forward against the fp32 naive recurrence (tolerances of the
north star: rel-L2 <= 1e-2 on o, <= 5e-3 on the final state, bf16 inputs)."""
import pytest
import torch

from helpers import assert_close, gla_inputs, random_offsets

pytestmark = pytest.mark.gpu

TOL_O, TOL_HT = 1e-2, 5e-3


def _run(device, q, k, v, g, h0, offsets=None, head_first=False, scale=None):
    from fla_amd.ops.gla import chunk_gla
    dev = lambda x: None if x is None else x.to(device)
    if head_first:
        q, k, v, g = (x.transpose(1, 2).contiguous() for x in (q, k, v, g))
    o, ht = chunk_gla(dev(q), dev(k), dev(v), dev(g), scale=scale, initial_state=dev(h0), output_final_state=True,
                      offsets=dev(offsets), head_first=head_first)
    torch.cuda.synchronize()
    if head_first:
        o = o.transpose(1, 2)
    return o, ht


def test_chunk_gla_config0(device):
    """The CPU-runnable reference shape (B=2, T=256, H=4, K=V=64, zero initial state), bf16 storage."""
    from oracle.recurrent import naive_recurrent_gla
    q, k, v, g, _ = gla_inputs(2, 256, 4, 64, 64, seed=0, h0=False)
    print("chunk_gla config0", flush=True)
    o, ht = _run(device, q, k, v, g, None)
    ro, rht = naive_recurrent_gla(q, k, v, g, output_final_state=True)
    assert o.dtype == torch.bfloat16 and ht.dtype == torch.float32
    assert_close("o", ro, o, TOL_O)
    assert_close("ht", rht, ht, TOL_HT)


@pytest.mark.parametrize("T", [1, 63, 64, 65, 130, 300, 1024])
@pytest.mark.parametrize("K,V", [(128, 128), (64, 64), (64, 128), (128, 64)])
def test_chunk_gla_shapes(device, T, K, V):
    from oracle.recurrent import naive_recurrent_gla
    q, k, v, g, h0 = gla_inputs(2, T, 3, K, V, seed=T + K, normalizer=16.0)
    print(f"chunk_gla T={T} K={K} V={V}", flush=True)
    o, ht = _run(device, q, k, v, g, h0)
    ro, rht = naive_recurrent_gla(q, k, v, g, initial_state=h0, output_final_state=True)
    assert_close("o", ro, o, TOL_O)
    assert_close("ht", rht, ht, TOL_HT)


@pytest.mark.parametrize("normalizer", [1.0, 16.0, 20.0])
@pytest.mark.parametrize("gate_dtype", [torch.float32, torch.bfloat16])
def test_chunk_gla_gates(device, normalizer, gate_dtype):
    """Gate magnitudes of the reference sweep (tests/ops/test_gla.py:90-146) that stay
    inside the single-reference-point range, in fp32 and in bf16 storage."""
    from oracle.recurrent import naive_recurrent_gla
    q, k, v, g, h0 = gla_inputs(2, 300, 4, 128, 128, seed=11, normalizer=normalizer, h0_std=1.0)
    g = g.to(gate_dtype)
    print(f"chunk_gla normalizer={normalizer} gates {gate_dtype}", flush=True)
    o, ht = _run(device, q, k, v, g, h0)
    ro, rht = naive_recurrent_gla(q, k, v, g, initial_state=h0, output_final_state=True)
    assert_close("o", ro, o, TOL_O)
    assert_close("ht", rht, ht, TOL_HT)


def test_chunk_gla_head_first_scale_and_odd_dims(device):
    from oracle.recurrent import naive_recurrent_gla
    q, k, v, g, h0 = gla_inputs(2, 200, 2, 100, 100, seed=12)
    print("chunk_gla head-first D=100 scale=0.2", flush=True)
    o, ht = _run(device, q, k, v, g, h0, head_first=True, scale=0.2)
    ro, rht = naive_recurrent_gla(q, k, v, g, scale=0.2, initial_state=h0, output_final_state=True)
    assert_close("o", ro, o, TOL_O)
    assert_close("ht", rht, ht, TOL_HT)


@pytest.mark.parametrize("T,N", [(64, 2), (300, 4), (1000, 5), (2048, 4)])
def test_chunk_gla_varlen(device, T, N):
    """Packed batches (tests/ops/test_gla.py:149-201): equals the per-sequence recurrence."""
    from oracle.recurrent import naive_recurrent_gla
    gen = torch.Generator().manual_seed(T)
    offs = random_offsets(T, N, gen, min_len=1)
    q, k, v, g, h0 = gla_inputs(1, T, 4, 128, 128, seed=13, N=N, h0_std=1.0)
    print(f"chunk_gla varlen T={T} offs={offs.tolist()}", flush=True)
    o, ht = _run(device, q, k, v, g, h0, offsets=offs)
    ro, rht = naive_recurrent_gla(q, k, v, g, initial_state=h0, output_final_state=True, offsets=offs.tolist())
    assert_close("o", ro, o, TOL_O)
    assert_close("ht", rht, ht, TOL_HT)


def test_chunk_gla_intermediates(device):
    """The reference-shaped internal forward: g_cumsum, A, per-chunk h against the fp32 chunked oracle."""
    from fla_amd.ops.gla.chunk import chunk_gla_fwd
    from oracle.chunked import chunked_gla
    q, k, v, g, h0 = gla_inputs(2, 200, 2, 128, 128, seed=14)
    dev = lambda x: x.to(device)
    print("chunk_gla_fwd intermediates", flush=True)
    gc, A, h, ht, o = chunk_gla_fwd(dev(q), dev(k), dev(v), dev(g), None, 128 ** -0.5, dev(h0), True,
                                    head_first=False, chunk_size=64)
    ref = chunked_gla(q, k, v, g, initial_state=h0)
    torch.testing.assert_close(gc.cpu(), ref['g_cumsum'], rtol=1e-5, atol=1e-5)
    assert_close("A", ref['A'], A, 1e-2)
    assert_close("h", ref['h'], h, 5e-3)
    assert_close("ht", ref['ht'], ht, TOL_HT)
    assert_close("o", ref['o'], o, TOL_O)
    assert (A.cpu().reshape(2, 200, 2, 64)[:, 0, :, 1:] == 0).all()  # strictly upper part is zero


def test_chunk_gla_segment_chaining(device):
    """run(T1) -> ht -> run(T2, h0=ht) equals run(T1+T2)."""
    q, k, v, g, h0 = gla_inputs(2, 320, 2, 128, 128, seed=15)
    print("chunk_gla chaining", flush=True)
    o_full, ht_full = _run(device, q, k, v, g, h0)
    cut = 192
    o1, h1 = _run(device, q[:, :cut], k[:, :cut], v[:, :cut], g[:, :cut], h0)
    o2, h2 = _run(device, q[:, cut:], k[:, cut:], v[:, cut:], g[:, cut:], h1.cpu())
    assert_close("o chained", o_full.float(), torch.cat([o1, o2], 1).float(), 4e-3)
    assert_close("ht chained", ht_full, h2, 1e-5)


# ---------------------------------------------------------------- backward
def _grads_ref(q, k, v, g, h0, do, dht, offsets=None, scale=None):
    """Autograd through the fp32 naive recurrence (tests/ops/test_gla.py:59-64)."""
    from oracle.recurrent import naive_recurrent_gla
    leaves = [x.detach().float().requires_grad_() for x in (q, k, v, g)]
    h0l = None if h0 is None else h0.detach().float().requires_grad_()
    o, ht = naive_recurrent_gla(*leaves, scale=scale, initial_state=h0l, output_final_state=True, offsets=offsets)
    loss = (o * do.float()).sum() + (ht * dht.float()).sum()
    loss.backward()
    return [x.grad for x in leaves] + [None if h0l is None else h0l.grad]


def _grads_dev(device, q, k, v, g, h0, do, dht, offsets=None, scale=None, head_first=False):
    from fla_amd.ops.gla import chunk_gla
    dev = lambda x: None if x is None else x.to(device)
    tr = (lambda x: x.transpose(1, 2).contiguous()) if head_first else (lambda x: x)
    leaves = [tr(dev(x)).detach().requires_grad_() for x in (q, k, v, g)]
    h0l = None if h0 is None else dev(h0).detach().requires_grad_()
    o, ht = chunk_gla(*leaves, scale=scale, initial_state=h0l, output_final_state=True, offsets=dev(offsets),
                      head_first=head_first)
    loss = (o.float() * tr(dev(do)).float()).sum() + (ht * dev(dht)).sum()
    loss.backward()
    torch.cuda.synchronize()
    return [tr(x.grad) for x in leaves] + [None if h0l is None else h0l.grad]


@pytest.mark.parametrize("T", [64, 130, 300])
@pytest.mark.parametrize("K,V", [(128, 128), (64, 64), (64, 128), (128, 64)])
def test_chunk_gla_backward(device, T, K, V):
    """Gradients against autograd through the naive recurrence
    (reference tolerances: tests/ops/test_gla.py:90-146 uses 0.005 on bf16 grads)."""
    B, H = 2, 2
    q, k, v, g, h0 = gla_inputs(B, T, H, K, V, seed=31 + T, normalizer=16.0, h0_std=1.0)
    gen = torch.Generator().manual_seed(5)
    do = torch.randn(B, T, H, V, generator=gen).bfloat16()
    dht = torch.randn(B, H, K, V, generator=gen) * 0.1
    print(f"chunk_gla backward T={T} K={K} V={V}", flush=True)
    got = _grads_dev(device, q, k, v, g, h0, do, dht)
    ref = _grads_ref(q, k, v, g, h0, do, dht)
    for name, r, x, tol in zip(("dq", "dk", "dv", "dg", "dh0"), ref, got, (8e-3, 8e-3, 8e-3, 1e-2, 5e-3)):
        assert_close(name, r, x, tol)
    assert got[0].dtype == torch.bfloat16 and got[3].dtype == torch.float32


def test_chunk_gla_backward_varlen_headfirst_odd(device):
    gen = torch.Generator().manual_seed(6)
    T, N, H, D = 500, 4, 2, 100
    offs = random_offsets(T, N, gen, min_len=1)
    q, k, v, g, h0 = gla_inputs(1, T, H, D, D, seed=41, N=N, normalizer=4.0, h0_std=1.0)
    do = torch.randn(1, T, H, D, generator=gen).bfloat16()
    dht = torch.randn(N, H, D, D, generator=gen) * 0.1
    print(f"chunk_gla backward varlen offs={offs.tolist()}", flush=True)
    got = _grads_dev(device, q, k, v, g, h0, do, dht, offsets=offs)
    ref = _grads_ref(q, k, v, g, h0, do, dht, offsets=offs.tolist())
    for name, r, x, tol in zip(("dq", "dk", "dv", "dg", "dh0"), ref, got, (8e-3, 8e-3, 8e-3, 1e-2, 5e-3)):
        assert_close(name, r, x, tol)
    # head-first, bf16 gates, no initial state
    q, k, v, g, _ = gla_inputs(2, 150, 2, 64, 64, seed=42, h0=False)
    g = g.bfloat16()
    do = torch.randn(2, 150, 2, 64, generator=gen).bfloat16()
    dht = torch.randn(2, 2, 64, 64, generator=gen) * 0.1
    got = _grads_dev(device, q, k, v, g, None, do, dht, head_first=True)
    ref = _grads_ref(q, k, v, g, None, do, dht)
    for name, r, x, tol in zip(("dq", "dk", "dv", "dg"), ref, got, (8e-3, 8e-3, 8e-3, 2e-2)):
        assert_close(name, r, x, tol)
    assert got[3].dtype == torch.bfloat16


@pytest.mark.parametrize("normalizer", [0.05, 0.3])
@pytest.mark.parametrize("T", [100, 300])
def test_chunk_gla_extreme_gates(device, normalizer, T):
    """Gate magnitudes of the reference sweep (normalizer 0.05, tests/ops/test_gla.py:90-146) where the
    chunk-cumulative log-gate runs into the hundreds: the device-side range guard routes those
    chunks through the exact pairwise path."""
    from oracle.recurrent import naive_recurrent_gla
    q, k, v, g, h0 = gla_inputs(2, T, 2, 128, 128, seed=71, normalizer=normalizer, h0_std=1.0)
    print(f"chunk_gla extreme gates normalizer={normalizer} T={T} min g={g.min().item():.1f}", flush=True)
    o, ht = _run(device, q, k, v, g, h0)
    ro, rht = naive_recurrent_gla(q, k, v, g, initial_state=h0, output_final_state=True)
    assert_close("o", ro, o, TOL_O)
    assert_close("ht", rht, ht, TOL_HT)


def test_chunk_gla_extreme_gates_mixed_varlen(device):
    """Only some chunks (and some channels) leave the safe range; packed batch, K != V."""
    from oracle.recurrent import naive_recurrent_gla
    gen = torch.Generator().manual_seed(72)
    T, N = 700, 3
    offs = random_offsets(T, N, gen, min_len=70)
    q, k, v, g, h0 = gla_inputs(1, T, 2, 64, 128, seed=72, N=N, normalizer=16.0)
    g[:, 200:330, :, :17] *= 400.0      # a stretch of very strong decay on a few channels
    print(f"chunk_gla mixed extreme gates offs={offs.tolist()}", flush=True)
    o, ht = _run(device, q, k, v, g, h0, offsets=offs)
    ro, rht = naive_recurrent_gla(q, k, v, g, initial_state=h0, output_final_state=True, offsets=offs.tolist())
    assert_close("o", ro, o, TOL_O)
    assert_close("ht", rht, ht, TOL_HT)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("varlen", [False, True])
def test_chunk_gla_many_heads(device, dtype, varlen):
    """More than 128 (sequence, head) pairs at K = V = 128: the forward without kept states runs one
    workgroup per head over all 128 value columns.  Ragged lengths, an initial state, and a stretch of
    gates strong enough to send some chunks through the exact pairwise path."""
    from oracle.recurrent import naive_recurrent_gla
    gen = torch.Generator().manual_seed(73)
    if varlen:
        T, N, H = 1100, 9, 16
        offs = random_offsets(T, N, gen, min_len=1)
        q, k, v, g, h0 = gla_inputs(1, T, H, 128, 128, seed=73, N=N, normalizer=16.0)
    else:
        T, N, H = 203, 5, 32
        offs = None
        q, k, v, g, h0 = gla_inputs(N, T, H, 128, 128, seed=74, normalizer=16.0)
    g[:, 70:140, 3:7, :9] *= 40.0 if dtype == torch.float16 else 400.0
    q, k, v = (x.to(dtype).float() for x in (q, k, v))
    print(f"chunk_gla {N * H} heads {dtype} offs={None if offs is None else offs.tolist()}", flush=True)
    from fla_amd.ops.gla import chunk_gla
    dev = lambda x: None if x is None else x.to(device)
    o, ht = chunk_gla(dev(q).to(dtype), dev(k).to(dtype), dev(v).to(dtype), dev(g), initial_state=dev(h0),
                      output_final_state=True, offsets=dev(offs), head_first=False)
    torch.cuda.synchronize()
    ro, rht = naive_recurrent_gla(q, k, v, g, initial_state=h0, output_final_state=True,
                                  offsets=None if offs is None else offs.tolist())
    assert o.dtype == dtype
    assert_close("o", ro, o, TOL_O)
    assert_close("ht", rht, ht, TOL_HT)


@pytest.mark.parametrize("normalizer", [0.05, 0.3])
def test_chunk_gla_backward_extreme_gates(device, normalizer):
    """Backward with gates far outside the single-reference range (the reference sweeps
    normalizer 0.05 for the gradients too, tests/ops/test_gla.py:90-146): the flagged chunks get
    their intra-chunk terms from the exact pairwise kernel."""
    B, T, H, K, V = 2, 200, 2, 128, 128
    q, k, v, g, h0 = gla_inputs(B, T, H, K, V, seed=81, normalizer=normalizer, h0_std=1.0)
    gen = torch.Generator().manual_seed(8)
    do = torch.randn(B, T, H, V, generator=gen).bfloat16()
    dht = torch.randn(B, H, K, V, generator=gen) * 0.1
    print(f"chunk_gla backward extreme gates normalizer={normalizer} min g={g.min().item():.1f}", flush=True)
    got = _grads_dev(device, q, k, v, g, h0, do, dht)
    ref = _grads_ref(q, k, v, g, h0, do, dht)
    for name, r, x, tol in zip(("dq", "dk", "dv", "dg", "dh0"), ref, got, (1e-2, 1e-2, 1e-2, 2e-2, 5e-3)):
        assert_close(name, r, x, tol)


def test_chunk_gla_backward_extreme_gates_mixed_varlen(device):
    """Only some chunks and channels are flagged; packed batch, K != V."""
    gen = torch.Generator().manual_seed(82)
    T, N = 500, 3
    offs = random_offsets(T, N, gen, min_len=70)
    q, k, v, g, h0 = gla_inputs(1, T, 2, 64, 128, seed=82, N=N, normalizer=16.0)
    g[:, 150:290, :, :17] *= 400.0
    do = torch.randn(1, T, 2, 128, generator=gen).bfloat16()
    dht = torch.randn(N, 2, 64, 128, generator=gen) * 0.1
    print(f"chunk_gla backward mixed extreme gates offs={offs.tolist()}", flush=True)
    got = _grads_dev(device, q, k, v, g, h0, do, dht, offsets=offs)
    ref = _grads_ref(q, k, v, g, h0, do, dht, offsets=offs.tolist())
    for name, r, x, tol in zip(("dq", "dk", "dv", "dg", "dh0"), ref, got, (1e-2, 1e-2, 1e-2, 2e-2, 5e-3)):
        assert_close(name, r, x, tol)


def test_chunk_gla_internal_fwd_bwd_signatures(device):
    """The reference-shaped internal entry points other operators build on (chunk_gla_fwd /
    chunk_gla_bwd, fla/ops/gla/chunk.py:1156-1320): same gradients as the public operator."""
    from fla_amd.ops.gla.chunk import chunk_gla_bwd, chunk_gla_fwd
    B, T, H, D = 2, 200, 2, 128
    q, k, v, g, h0 = gla_inputs(B, T, H, D, D, seed=33, h0_std=1.0)
    gen = torch.Generator().manual_seed(9)
    do = torch.randn(B, T, H, D, generator=gen).bfloat16()
    dht = torch.randn(B, H, D, D, generator=gen) * 0.1
    dev = lambda x: x.to(device)
    print("chunk_gla_fwd / chunk_gla_bwd internal signatures", flush=True)
    gc, A, h, ht, o = chunk_gla_fwd(dev(q), dev(k), dev(v), dev(g), None, D ** -0.5, dev(h0), True, head_first=False)
    dq, dk, dv, dg, dh0 = chunk_gla_bwd(dev(q), dev(k), dev(v), dev(g), gc, D ** -0.5, dev(h0), h, A, dev(do), dev(dht),
                                        head_first=False)
    ref = _grads_ref(q, k, v, g, h0, do, dht)
    for name, r, x, tol in zip(("dq", "dk", "dv", "dg", "dh0"), ref, (dq, dk, dv, dg, dh0), (8e-3, 8e-3, 8e-3, 1e-2, 5e-3)):
        assert_close(name, r, x, tol)


@pytest.mark.parametrize("head_first", [False, True])
@pytest.mark.parametrize("varlen", [False, True])
def test_chunk_gla_internal_entries_as_gsa_calls_them(device, head_first, varlen):
    """chunk_gla_fwd / chunk_gla_bwd with GSA's argument lists (fla/ops/gsa/chunk.py:622-636 and :741-757):
    g=None, g_cumsum = the chunk-local cumulative gates, the saved h and A handed back to the backward,
    either layout, keyword arguments throughout."""
    from fla_amd.ops.gla.chunk import chunk_gla_bwd, chunk_gla_fwd
    from fla_amd.utils import prepare_chunk_indices
    from oracle.chunked import chunked_gla
    from oracle.cumsum import chunk_local_cumsum as ref_cumsum
    if varlen and head_first:
        pytest.skip("packed batches are seq-first")
    B, T, H, K, V = (1, 300, 2, 128, 64) if varlen else (2, 200, 2, 128, 64)
    N = 3 if varlen else B
    offs = torch.tensor([0, 70, 71, 300]) if varlen else None
    q, k, v, g, h0 = gla_inputs(B, T, H, K, V, seed=35, h0_std=1.0, N=N)
    gen = torch.Generator().manual_seed(10)
    do = torch.randn(B, T, H, V, generator=gen).bfloat16()
    dht = torch.randn(N, H, K, V, generator=gen) * 0.1
    gc = ref_cumsum(g, 64, offsets=None if offs is None else offs.tolist())
    tr = (lambda x: x.transpose(1, 2).contiguous()) if head_first else (lambda x: x)
    dev = lambda x: None if x is None else x.to(device)
    print(f"chunk_gla_fwd / bwd, GSA calling form, head_first={head_first} varlen={varlen}", flush=True)
    doffs = dev(offs)
    idx = None if offs is None else prepare_chunk_indices(doffs, 64)
    A, h, ht, o = chunk_gla_fwd(q=dev(tr(q)), k=dev(tr(k)), v=dev(tr(v)), g=None, g_cumsum=dev(tr(gc)), scale=K ** -0.5,
                                initial_state=dev(h0), output_final_state=True, offsets=doffs, indices=idx,
                                head_first=head_first, chunk_size=64)[1:]
    ref = chunked_gla(q, k, v, g, initial_state=h0, offsets=None if offs is None else offs.tolist())
    assert_close("o", ref['o'], tr(o) if head_first else o, TOL_O)
    assert_close("ht", ref['ht'], ht, TOL_HT)
    assert_close("A", ref['A'], tr(A) if head_first else A, 1e-2)
    assert_close("h", ref['h'], h.transpose(1, 2) if head_first else h, 5e-3)
    dq, dk, dv, dg, dh0 = chunk_gla_bwd(q=dev(tr(q)), k=dev(tr(k)), v=dev(tr(v)), g=None, g_cumsum=dev(tr(gc)),
                                        scale=K ** -0.5, initial_state=dev(h0), h=h, A=A, do=dev(tr(do)), dht=dev(dht),
                                        offsets=doffs, indices=idx, head_first=head_first, chunk_size=64)
    grads = _grads_ref(q, k, v, g, h0, do, dht, offsets=offs)
    for name, r, x, tol in zip(("dq", "dk", "dv", "dg", "dh0"), grads, (dq, dk, dv, dg, dh0), (8e-3, 8e-3, 8e-3, 1e-2, 5e-3)):
        assert_close(name, r, tr(x) if (head_first and name != "dh0") else x, tol)


def test_chunk_gla_internal_entries_strong_gates_fp16(device):
    """The internal forward and backward stay exact where the single-reference-point scores leave their
    range (fp16: a chunk-cumulative log-gate beyond 8): o and the gradients come from the guarded launches."""
    from fla_amd.ops.gla.chunk import chunk_gla_bwd, chunk_gla_fwd
    from oracle.recurrent import naive_recurrent_gla
    B, T, H, D = 2, 130, 2, 64
    q, k, v, g, h0 = gla_inputs(B, T, H, D, D, seed=36, dtype=torch.float16, normalizer=1.0, h0_std=1.0)
    gen = torch.Generator().manual_seed(11)
    do = torch.randn(B, T, H, D, generator=gen).half()
    dht = torch.randn(B, H, D, D, generator=gen) * 0.1
    dev = lambda x: x.to(device)
    print("chunk_gla_fwd / bwd, fp16, strong gates", flush=True)
    gc, A, h, ht, o = chunk_gla_fwd(dev(q), dev(k), dev(v), dev(g), None, D ** -0.5, dev(h0), True, head_first=False)
    ro, rht = naive_recurrent_gla(q, k, v, g, initial_state=h0, output_final_state=True)
    assert_close("o", ro, o, TOL_O)
    assert_close("ht", rht, ht, TOL_HT)
    dq, dk, dv, dg, dh0 = chunk_gla_bwd(dev(q), dev(k), dev(v), dev(g), gc, D ** -0.5, dev(h0), h, A, dev(do), dev(dht),
                                        head_first=False)
    grads = _grads_ref(q, k, v, g, h0, do, dht)
    for name, r, x, tol in zip(("dq", "dk", "dv", "dg", "dh0"), grads, (dq, dk, dv, dg, dh0), (1e-2, 1e-2, 1e-2, 2e-2, 5e-3)):
        assert_close(name, r, x, tol)


def test_chunk_backward_of_an_empty_batch(device):
    """No chunk at all (a packed batch whose sequences are all empty): the gradient of the initial
    states is the gradient of the final states, and nothing else is touched."""
    from fla_amd.ops.gated_delta_rule import chunk_gated_delta_rule
    from fla_amd.ops.gla import chunk_gla
    H, D, N = 2, 64, 2
    offs = torch.zeros(N + 1, dtype=torch.int64, device=device)
    z = lambda *sh: torch.zeros(*sh, device=device, dtype=torch.bfloat16).requires_grad_()
    dht = torch.randn(N, H, D, D, device=device)
    print("backward of an empty packed batch", flush=True)
    for name in ("gla", "gdr"):
        h0 = torch.randn(N, H, D, D, device=device).requires_grad_()
        if name == "gla":
            o, ht = chunk_gla(z(1, 0, H, D), z(1, 0, H, D), z(1, 0, H, D), torch.zeros(1, 0, H, D, device=device),
                              initial_state=h0, output_final_state=True, offsets=offs, head_first=False)
        else:
            o, ht = chunk_gated_delta_rule(z(1, 0, H, D), z(1, 0, H, D), z(1, 0, H, D),
                                           torch.zeros(1, 0, H, device=device), torch.zeros(1, 0, H, device=device),
                                           initial_state=h0, output_final_state=True, offsets=offs, head_first=False)
        assert torch.equal(ht, h0.detach())
        (ht * dht).sum().backward()
        assert torch.equal(h0.grad, dht), name


# The reference's own ladder (tests/ops/test_gla.py:90-146): head dims 300 and 100 (key and value
# slabs of 128 after padding), both layouts, gate_logit_normalizer 1 / 0.05 / 20.
@pytest.mark.parametrize("D,T,normalizer,head_first", [
    (300, 130, 1.0, False),
    (300, 178, 0.05, True),
    (300, 300, 20.0, False),
    (100, 146, 0.05, False),
    (100, 2048, 20.0, True),
])
def test_chunk_gla_reference_ladder(device, D, T, normalizer, head_first):
    from fla_amd.ops.gla import chunk_gla
    from helpers import gla_inputs
    from oracle.recurrent import naive_recurrent_gla
    B, H = 2, 2
    q, k, v, g, h0 = gla_inputs(B, T, H, D, D, seed=81 + T, normalizer=normalizer, h0_std=1.0)
    gen = torch.Generator().manual_seed(11)
    do = torch.randn(B, T, H, D, generator=gen).bfloat16()
    dht = torch.randn(B, H, D, D, generator=gen) * 0.1
    print(f"chunk_gla ladder D={D} T={T} normalizer={normalizer} head_first={head_first}", flush=True)
    tr = (lambda x: x.transpose(1, 2).contiguous()) if head_first else (lambda x: x)
    leaves = [tr(x.to(device)).detach().requires_grad_() for x in (q, k, v, g)]
    h0l = h0.to(device).requires_grad_()
    o, ht = chunk_gla(*leaves, initial_state=h0l, output_final_state=True, head_first=head_first)
    ((o.float() * tr(do.to(device)).float()).sum() + (ht * dht.to(device)).sum()).backward()
    refs = [x.float().requires_grad_() for x in (q, k, v, g)]
    rh0 = h0.clone().requires_grad_()
    ro, rht = naive_recurrent_gla(*refs, initial_state=rh0, output_final_state=True)
    ((ro * do.float()).sum() + (rht * dht).sum()).backward()
    assert_close("o", ro, tr(o), 1e-2)
    assert_close("ht", rht, ht, 5e-3)
    for name, a, b in zip(("dq", "dk", "dv", "dg"), refs, leaves):
        assert_close(name, a.grad, tr(b.grad), 1e-2)
    assert_close("dh0", rh0.grad, h0l.grad, 1e-2)


@pytest.mark.parametrize("varlen", [False, True])
def test_chunk_gla_keep_vs_recompute(device, varlen, monkeypatch):
    """The backward from the states the fused forward kept and the reference-style backward that
    recomputes them agree to the rounding of their 16-bit operands (the kept path reads states and
    gated queries rounded once in the forward and carries dH / scale; the recomputing path rounds
    scale * q * e^G itself), well inside the oracle's tolerances, which both meet."""
    import fla_amd.ops.gla.chunk as mod
    gen = torch.Generator().manual_seed(13)
    T, N, H, D = 400, 3, 2, 128
    offs = random_offsets(T, N, gen, min_len=1) if varlen else None
    q, k, v, g, h0 = gla_inputs(1 if varlen else 2, T, H, D, D, seed=64, N=N if varlen else None, h0_std=1.0)
    do = torch.randn(q.shape[0], T, H, D, generator=gen).bfloat16()
    dht = torch.randn(h0.shape, generator=gen) * 0.1
    print(f"chunk_gla keep vs recompute varlen={varlen}", flush=True)
    assert mod.KEEP_STATES_FOR_BACKWARD
    kept = _grads_dev(device, q, k, v, g, h0, do, dht, offsets=offs)
    monkeypatch.setattr(mod, "KEEP_STATES_FOR_BACKWARD", False)
    rec = _grads_dev(device, q, k, v, g, h0, do, dht, offsets=offs)
    ref = _grads_ref(q, k, v, g, h0, do, dht, offsets=None if offs is None else offs.tolist())
    # (dv of the kept path is formed inside the reverse state scan from the kept k^ and score tiles and the 16-bit
    # dH of that scan; the recomputing path re-forms all three in another kernel: two more independent roundings)
    for name, a, b, r, tol, tol2 in zip(("dq", "dk", "dv", "dg", "dh0"), kept, rec, ref, (8e-3, 8e-3, 8e-3, 1e-2, 5e-3),
                                        (4e-3, 4e-3, 6e-3, 4e-3, 4e-3)):
        assert_close(f"{name} kept vs recomputed", b, a, tol2)
        assert_close(f"{name} recomputed vs oracle", r, b, tol)
        assert_close(f"{name} kept vs oracle", r, a, tol)


@pytest.mark.parametrize("varlen", [False, True])
def test_chunk_gla_gradients_are_reproducible(device, varlen):
    """Same inputs twice: every gradient identical bit for bit."""
    gen = torch.Generator().manual_seed(14)
    T, N, H, D = 700, 4, 3, 128
    offs = random_offsets(T, N, gen, min_len=1) if varlen else None
    q, k, v, g, h0 = gla_inputs(1 if varlen else 2, T, H, D, D, seed=65, N=N if varlen else None, h0_std=1.0)
    do = torch.randn(q.shape[0], T, H, D, generator=gen).bfloat16()
    dht = torch.randn(h0.shape, generator=gen) * 0.1
    print(f"chunk_gla reproducibility varlen={varlen}", flush=True)
    first = _grads_dev(device, q, k, v, g, h0, do, dht, offsets=offs)
    for _ in range(3):
        again = _grads_dev(device, q, k, v, g, h0, do, dht, offsets=offs)
        for name, a, b in zip(("dq", "dk", "dv", "dg", "dh0"), first, again):
            assert torch.equal(a, b), name


def test_chunk_gla_slab_width_independence_training(device):
    """A forward that keeps the states runs on 32-column slabs while B*H*V/64 <= 128 (B=4 x H=16 here) and on
    64-column slabs for the same batch stacked twice; every value column is computed the same way either way, so
    the gradients (which the backward forms from the kept states) of both copies agree bit for bit with those of
    the batch alone.  Sequence 0, heads 0-1 are also checked against autograd through the recurrence."""
    B, T, H, D = 4, 512, 16, 128
    gen = torch.Generator().manual_seed(73)
    q, k, v, g, h0 = gla_inputs(B, T, H, D, D, seed=73)
    do = torch.randn(B, T, H, D, generator=gen).bfloat16()
    dht = torch.randn(h0.shape, generator=gen) * 0.1
    print("chunk_gla slab-width independence (training) B=4 vs B=8", flush=True)
    twice = lambda x: torch.cat([x, x], 0)
    g4 = _grads_dev(device, q, k, v, g, h0, do, dht)
    g8 = _grads_dev(device, twice(q), twice(k), twice(v), twice(g), twice(h0), twice(do), twice(dht))
    for i, (a, b) in enumerate(zip(g4, g8)):
        assert torch.equal(b[:B], a) and torch.equal(b[B:], a), i
    gr = _grads_ref(q[:1, :, :2], k[:1, :, :2], v[:1, :, :2], g[:1, :, :2], h0[:1, :2], do[:1, :, :2], dht[:1, :2])
    for i, (r, a) in enumerate(zip(gr, g4)):
        x = a[:1, :2] if a.dim() == 4 and a.shape[1] == H else a[:1, :, :2]
        assert_close(f"gradient {i} of sequence 0, heads 0-1", r, x, 2e-2)


@pytest.mark.parametrize("B,H,varlen", [(2, 2, False), (1, 3, True), (3, 48, False)])
def test_chunk_gla_kept_gated_queries_and_decays(device, B, H, varlen):
    """What a states-keeping forward leaves beside the states: q e^{G} (G the log-gates summed from the chunk's
    first token), rounded once to the inputs' type, for every real token, and e^{G} of every chunk's last token
    in fp32.  Both are elementwise, so they are checked against torch's cumulative sum directly; (3, 48) is a
    launch on 64-column slabs, the others on 32-column slabs."""
    from fla_amd.ops.gla.chunk import chunk_gla_fwd_fused
    gen = torch.Generator().manual_seed(15)
    T, N, D, BT = 333, 4, 128, 64   # (the forward also leaves k^ and the score tiles: checked chunk by chunk below)
    offs = random_offsets(T, N, gen, min_len=1) if varlen else None
    q, k, v, g, h0 = gla_inputs(B, T, H, D, D, seed=66, N=N if varlen else None, normalizer=4.0)
    print(f"chunk_gla kept outputs B={B} H={H} varlen={varlen}", flush=True)
    kept = []
    chunk_gla_fwd_fused(*(x.to(device) for x in (q, k, v, g)), D ** -0.5, h0.to(device), True,
                        None if offs is None else offs.to(device), states_out=kept)
    _, qg, decay, kh, scores = kept
    kh, scores = kh.reshape(-1, H, D, BT).cpu(), scores.reshape(-1, H, BT, BT).cpu()
    bounds = offs.tolist() if varlen else [0, T]
    want_decay = []
    ci = 0
    for b in range(B):
        for s, e in zip(bounds[:-1], bounds[1:]):
            for c0 in range(s, e, BT):
                c1 = min(c0 + BT, e)
                G = g[b, c0:c1].float().cumsum(0)
                want = (q[b, c0:c1].float() * G.exp()).to(q.dtype)
                got = qg[b, c0:c1].cpu()
                # e^{G} on the device is a fast exponential: a unit in the last place of the 16-bit result
                assert_close(f"gated queries of rows {c0}..{c1} of batch {b}", want.float(), got.float(), 3e-3)
                assert (want.float() - got.float()).abs().max() <= 2.0 ** -7 * want.float().abs().max()
                want_decay.append(G[-1].exp())
                # k^ = k e^{G_last - G}, key-major, zero past the end of a short chunk; and the unscaled causal
                # scores of the rounded gated operands
                L = c1 - c0
                kf = k[b, c0:c1].float()
                want_kh = torch.zeros(H, D, BT)
                want_kh[:, :, :L] = (kf * (G[-1:] - G).exp()).to(q.dtype).float().permute(1, 2, 0)
                assert_close(f"k^ of chunk {ci}", want_kh, kh[ci].float(), 3e-3)
                assert torch.equal(kh[ci][:, :, L:].float(), torch.zeros(H, D, BT - L))
                qt = want.float().permute(1, 0, 2)                                   # [H, L, K]
                kt = (kf * (-G).exp()).to(q.dtype).float().permute(1, 0, 2)
                want_p = torch.zeros(H, BT, BT)
                want_p[:, :L, :L] = (qt @ kt.transpose(1, 2)).tril()
                assert_close(f"scores of chunk {ci}", want_p, scores[ci].float(), 5e-3)
                assert torch.equal(scores[ci].float().triu(1), torch.zeros(H, BT, BT))
                ci += 1
    want_decay = torch.stack(want_decay)
    got_decay = decay.reshape(-1, H, D)[:want_decay.shape[0]].cpu()
    torch.testing.assert_close(got_decay, want_decay, rtol=2e-5, atol=1e-30)


@pytest.mark.parametrize("logit_dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("K,V,T,normalizer,clamp_min,varlen", [
    (128, 128, 300, 16.0, None, False),
    (128, 128, 257, 16.0, -0.02, True),
    (64, 128, 130, 1.0, None, False),
    (128, 64, 200, 0.05, None, True),      # strong gates: the flagged chunks go through the exact launch
    (64, 64, 1, 16.0, None, False),
])
def test_chunk_gla_from_gate_logits(device, logit_dtype, K, V, T, normalizer, clamp_min, varlen):
    """The opt-in form that takes the gate projection's output: the fused launch applies
    logsigmoid(x) / normalizer (+ clamp) itself (fla/layers/gla.py:214-217).  Against the recurrence on the
    oracle's gates, and against the two-step form (gate launch, then the operator) of the same library."""
    from fla_amd.modules import gla_gate_fwd
    from fla_amd.ops.gla import chunk_gla
    from oracle.modules import gla_gate
    from oracle.recurrent import naive_recurrent_gla
    gen = torch.Generator().manual_seed(T + K)
    B, H = (1, 3) if varlen else (2, 3)
    q, k, v, _, _ = gla_inputs(B, T, H, K, V, seed=T + V)
    x = (torch.randn(B, T, H, K, generator=gen) * 2).to(logit_dtype)
    offs = random_offsets(T, 3, gen) if varlen else None
    h0 = torch.randn(3 if varlen else B, H, K, V, generator=gen) * 0.1
    print(f"chunk_gla gate logits {logit_dtype} K={K} V={V} T={T} normalizer={normalizer} clamp={clamp_min} "
          f"varlen={varlen}", flush=True)
    dev = lambda t: None if t is None else t.to(device)
    o, ht = chunk_gla(dev(q), dev(k), dev(v), dev(x), initial_state=dev(h0), output_final_state=True,
                      offsets=dev(offs), head_first=False, gate_logit_normalizer=normalizer,
                      gate_clamp_min=clamp_min)
    g = gla_gate(x, normalizer, clamp_min)
    ro, rht = naive_recurrent_gla(q, k, v, g, initial_state=h0, output_final_state=True,
                                  offsets=None if offs is None else offs.tolist())
    assert o.dtype == torch.bfloat16
    assert_close("o", ro, o, TOL_O)
    assert_close("ht", rht, ht, TOL_HT)
    g_dev = gla_gate_fwd(dev(x), normalizer, clamp_min)
    o2, ht2 = chunk_gla(dev(q), dev(k), dev(v), g_dev, initial_state=dev(h0), output_final_state=True,
                        offsets=dev(offs), head_first=False)
    assert_close("o vs two-step", o2, o, 2e-3)
    assert_close("ht vs two-step", ht2, ht, 1e-4)


def test_chunk_gla_from_gate_logits_backward(device):
    """With gradients the logits form runs the gate launch and its backward either side of the operator:
    d(logits) against autograd through the oracle's gate and recurrence."""
    from fla_amd.ops.gla import chunk_gla
    from oracle.modules import gla_gate
    from oracle.recurrent import naive_recurrent_gla
    gen = torch.Generator().manual_seed(5)
    B, T, H, K, V = 2, 130, 2, 64, 64
    q, k, v, _, h0 = gla_inputs(B, T, H, K, V, seed=9)
    x = (torch.randn(B, T, H, K, generator=gen) * 2).bfloat16()
    do = torch.randn(B, T, H, V, generator=gen).bfloat16()
    print("chunk_gla gate logits backward", flush=True)
    leaves = [t.to(device).requires_grad_() for t in (q, k, v, x)]
    o, _ = chunk_gla(*leaves, initial_state=h0.to(device), head_first=False, gate_logit_normalizer=16.0,
                     gate_clamp_min=-0.05)
    o.backward(do.to(device))
    ref = [t.float().requires_grad_() for t in (q, k, v, x)]
    ro, _ = naive_recurrent_gla(ref[0], ref[1], ref[2], gla_gate(ref[3], 16.0, -0.05), initial_state=h0)
    ro.backward(do.float())
    assert_close("o", ro, o, TOL_O)
    for name, a, b in zip(("dq", "dk", "dv", "dx"), ref, leaves):
        assert b.grad.dtype == b.dtype
        assert_close(name, a.grad, b.grad, 1.5e-2)


def test_kept_forward_rejects_value_dims_its_row_split_does_not_cover(device):
    """fla_chunk_gla_fwd_fused_kept shares the rows of the kept tiles out over the value slabs of a head: value
    dims that do not divide them evenly (V = 192) are refused, as are the score tiles beyond V = 128."""
    from fla_amd import _backend as be
    B, T, H, K = 1, 64, 1, 128
    for V, with_scores, want in ((192, False, -2), (256, True, -2), (256, False, 0), (128, True, 0)):
        q, k = (torch.randn(B, T, H, K, device=device).bfloat16() for _ in range(2))
        v = torch.randn(B, T, H, V, device=device).bfloat16()
        g = -torch.rand(B, T, H, K, device=device)
        o, hT, qg = torch.empty_like(v), q.new_empty(B, 1, H, K, V), torch.empty_like(q)
        decay = q.new_empty(B, 1, H, K, dtype=torch.float32)
        kh = q.new_empty(B, 1, H, K, 64) if with_scores else None
        sc = q.new_empty(B, 1, H, 64, 64) if with_scores else None
        print(f"kept forward V={V} scores={with_scores}", flush=True)
        rc = be.lib().fla_chunk_gla_fwd_fused_kept(
            be.ptr(q), be.ptr(k), be.ptr(v), be.ptr(g), None, be.ptr(o), None, None, None, be.ptr(hT), be.ptr(qg),
            be.ptr(decay), be.ptr(kh), be.ptr(sc), None, None, None, None, 0, be.dt(q), be.dt(g), B, T, H, K, V, B,
            K ** -0.5, be.stream_of(q))
        torch.cuda.synchronize()
        assert rc == want, (V, with_scores, rc)


@pytest.mark.parametrize("T,bt", [(7, 16), (16, 16), (20, 32), (32, 32)])
def test_chunk_gla_internal_entries_short_sequences(device, T, bt):
    """chunk_gla_fwd / chunk_gla_bwd for T <= 32, where the reference's chunk length is 16 or 32
    (fla/ops/gla/chunk.py:1350): the score tile comes back with that many columns, everything else as for one
    chunk of 64."""
    from fla_amd.ops.gla.chunk import chunk_gla_bwd, chunk_gla_fwd
    from oracle.chunked import chunked_gla
    B, H, K, V = 2, 2, 64, 128
    q, k, v, g, h0 = gla_inputs(B, T, H, K, V, seed=T, h0_std=1.0)
    gen = torch.Generator().manual_seed(T)
    do = torch.randn(B, T, H, V, generator=gen).bfloat16()
    dht = torch.randn(B, H, K, V, generator=gen) * 0.1
    dev = lambda x: x.to(device)
    print(f"chunk_gla_fwd / bwd T={T}", flush=True)
    gc, A, h, ht, o = chunk_gla_fwd(dev(q), dev(k), dev(v), dev(g), None, K ** -0.5, dev(h0), True, head_first=False)
    ref = chunked_gla(q, k, v, g, initial_state=h0)
    assert tuple(A.shape) == (B, T, H, bt) and tuple(h.shape) == (B, 1, H, K, V)
    assert_close("o", ref['o'], o, TOL_O)
    assert_close("ht", ref['ht'], ht, TOL_HT)
    assert_close("A", ref['A'][..., :bt], A, 1e-2)
    assert_close("g_cumsum", ref['g_cumsum'], gc, 1e-5)
    dq, dk, dv, dg, dh0 = chunk_gla_bwd(dev(q), dev(k), dev(v), dev(g), gc, K ** -0.5, dev(h0), h, A, dev(do), dev(dht),
                                        head_first=False)
    grads = _grads_ref(q, k, v, g, h0, do, dht)
    for name, r, x, tol in zip(("dq", "dk", "dv", "dg", "dh0"), grads, (dq, dk, dv, dg, dh0), (8e-3, 8e-3, 8e-3, 1e-2, 5e-3)):
        assert_close(name, r, x, tol)
