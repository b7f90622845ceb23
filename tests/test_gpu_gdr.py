"""GPU: chunk_gated_delta_rule forward against the fp32 naive recurrence and, kernel
by kernel, against the fp32 chunked oracle."""
import pytest
import torch

from helpers import assert_close, gdr_inputs, random_offsets

pytestmark = pytest.mark.gpu

TOL_O, TOL_HT = 1e-2, 5e-3


def _run(device, q, k, v, g, beta, h0, offsets=None, head_first=False, scale=None):
    from fla_amd.ops.gated_delta_rule import chunk_gated_delta_rule
    dev = lambda x: None if x is None else x.to(device)
    if head_first:
        q, k, v = (x.transpose(1, 2).contiguous() for x in (q, k, v))
        g, beta = g.transpose(1, 2).contiguous(), beta.transpose(1, 2).contiguous()
    o, ht = chunk_gated_delta_rule(dev(q), dev(k), dev(v), dev(g), dev(beta), scale=scale, initial_state=dev(h0),
                                   output_final_state=True, offsets=dev(offsets), head_first=head_first)
    torch.cuda.synchronize()
    if head_first:
        o = o.transpose(1, 2)
    return o, ht


def test_gdr_kernel_by_kernel(device):
    """Aw, Au, w, u, per-chunk h, v_new, o and ht against the fp32 chunked oracle."""
    from fla_amd.ops.common.chunk_delta_h import chunk_gated_delta_rule_fwd_h
    from fla_amd.ops.common.chunk_o import chunk_fwd_o
    from fla_amd.ops.gated_delta_rule.wy_fast import fwd_prepare_wy_repr
    from fla_amd.ops.utils import chunk_local_cumsum
    from oracle.chunked import chunked_gated_delta_rule
    q, k, v, g, beta, h0 = gdr_inputs(2, 200, 2, 128, 128, seed=21)
    ref = chunked_gated_delta_rule(q, k, v, g, beta, initial_state=h0)
    dev = lambda x: x.to(device)
    print("gdr kernel by kernel", flush=True)
    gc = chunk_local_cumsum(dev(g), 64, head_first=False)
    torch.testing.assert_close(gc.cpu(), ref['g_cumsum'], rtol=1e-5, atol=1e-5)
    w, u, Aw, Au = fwd_prepare_wy_repr(dev(k), dev(v), dev(beta), gc, head_first=False)
    torch.cuda.synchronize()
    assert_close("Aw", ref['Aw'], Aw, 5e-3)
    assert_close("Au", ref['Au'], Au, 5e-3)
    assert_close("w", ref['w'], w, 8e-3)
    assert_close("u", ref['u'], u, 8e-3)
    h, v_new, ht = chunk_gated_delta_rule_fwd_h(dev(k), w, u, gc, dev(h0), True, head_first=False)
    torch.cuda.synchronize()
    assert_close("h", ref['h'], h, 8e-3)
    assert_close("v_new", ref['v_new'], v_new, 1e-2)
    assert_close("ht", ref['ht'], ht, TOL_HT)
    hf, v_new2, _ = chunk_gated_delta_rule_fwd_h(dev(k), w, u, gc, dev(h0), False, head_first=False,
                                                 fragment_layout=True)
    assert torch.equal(v_new, v_new2)
    o = chunk_fwd_o(dev(q), dev(k), v_new2, hf, gc, 128 ** -0.5, head_first=False, fragment_layout=True)
    torch.cuda.synchronize()
    assert_close("o", ref['o'], o, TOL_O)
    # the reference's calling form: row-major states, re-ordered on the way in
    o_rm = chunk_fwd_o(dev(q), dev(k), v_new2, h, gc, 128 ** -0.5, head_first=False)
    torch.cuda.synchronize()
    assert torch.equal(o, o_rm)


def _dense_tiles(ref, beta, B, T, H, offsets=None):
    """Oracle Tu = Au diag(beta) and Aqk per chunk as dense [chunks, H, 64, 64] (zero outside the chunk's rows)."""
    spans = [(b, 0, T) for b in range(B)] if offsets is None else [(0, a, e) for a, e in zip(offsets[:-1], offsets[1:])]
    tu, aqk = [], []
    for b, bos, eos in spans:
        for c0 in range(bos, eos, 64):
            L = min(64, eos - c0)
            t_, a_ = torch.zeros(H, 64, 64), torch.zeros(H, 64, 64)
            t_[:, :L, :L] = ref['Au'][b, c0:c0 + L].permute(1, 0, 2)[:, :, :L] * beta[b, c0:c0 + L].t()[:, None, :]
            a_[:, :L, :L] = ref['Aqk'][b, c0:c0 + L].permute(1, 0, 2)[:, :, :L]
            tu.append(t_)
            aqk.append(a_)
    return torch.stack(tu), torch.stack(aqk)


@pytest.mark.parametrize("B,T,H,K,V", [(2, 200, 2, 128, 128), (2, 64, 2, 64, 64), (1, 1, 1, 128, 64), (2, 300, 3, 64, 128)])
def test_gdr_two_launch_forward_pieces(device, B, T, H, K, V):
    """The operator's own decomposition: fla_gdr_fwd_prep (gate prefix sums and Tu = Au diag(beta) as a packed
    triangular tile) against the fp32 chunked oracle, then the scan on it against the naive recurrence."""
    from fla_amd.ops.common.chunk_delta_h import chunk_gated_delta_rule_fwd_scan
    from fla_amd.ops.gated_delta_rule.wy_fast import fwd_prepare_scan_operands, unpack_triangular_tiles
    from oracle.chunked import chunked_gated_delta_rule
    from oracle.recurrent import naive_recurrent_gated_delta_rule
    q, k, v, g, beta, h0 = gdr_inputs(B, T, H, K, V, seed=21)
    ref = chunked_gated_delta_rule(q, k, v, g, beta, initial_state=h0)
    dev = lambda x: x.to(device)
    print(f"gdr prep + scan B={B} T={T} H={H} K={K} V={V}", flush=True)
    AT, gc = fwd_prepare_scan_operands(dev(k), dev(beta), dev(g))
    torch.cuda.synchronize()
    torch.testing.assert_close(gc.cpu(), ref['g_cumsum'], rtol=1e-5, atol=1e-5)
    dense = unpack_triangular_tiles(AT).float().cpu()
    tu_ref, aqk_ref = _dense_tiles(ref, beta, B, T, H)
    assert_close("Tu", tu_ref, dense, 5e-3)
    assert torch.equal(dense.triu(1), torch.zeros_like(dense))          # nothing above the diagonal
    # the same tiles from gates that are already cumulative
    AT2, gc2 = fwd_prepare_scan_operands(dev(k), dev(beta), gc, g_is_cumsum=True)
    assert gc2 is gc and torch.equal(AT, AT2)
    # the variant a differentiated forward runs: the same tiles, plus w = Aw (beta k) and Aw for the backward
    AT3, gc3, w, Aw = fwd_prepare_scan_operands(dev(k), dev(beta), dev(g), keep_w=True)
    torch.cuda.synchronize()
    assert torch.equal(AT, AT3) and torch.equal(gc, gc3)
    assert_close("Aw", ref['Aw'], Aw, 5e-3)
    assert_close("w", ref['w'], w, 8e-3)
    o, ht = chunk_gated_delta_rule_fwd_scan(dev(q), dev(k), dev(v), AT, gc, K ** -0.5, dev(h0), True)
    torch.cuda.synchronize()
    ro, rht = naive_recurrent_gated_delta_rule(q, k, v, g, beta, initial_state=h0, output_final_state=True)
    assert_close("o", ro, o, TOL_O)
    assert_close("ht", rht, ht, TOL_HT)
    # the scan of a differentiated forward: same outputs, plus v_new, the states and the score tiles it formed
    o2, ht2, v_new, hT, Aqk = chunk_gated_delta_rule_fwd_scan(dev(q), dev(k), dev(v), AT, gc, K ** -0.5, dev(h0), True,
                                                              keep=True)
    torch.cuda.synchronize()
    assert torch.equal(o, o2) and torch.equal(ht, ht2)
    assert_close("v_new", ref['v_new'], v_new, 8e-3)
    dense_p = unpack_triangular_tiles(Aqk).float().cpu()
    assert_close("Aqk", aqk_ref, dense_p, 5e-3)
    assert torch.equal(dense_p.triu(1), torch.zeros_like(dense_p))


def test_gdr_two_launch_forward_pieces_packed(device):
    from fla_amd.ops.common.chunk_delta_h import chunk_gated_delta_rule_fwd_scan
    from fla_amd.ops.gated_delta_rule.wy_fast import fwd_prepare_scan_operands, unpack_triangular_tiles
    from fla_amd.utils import VarlenPlan
    from oracle.chunked import chunked_gated_delta_rule
    from oracle.recurrent import naive_recurrent_gated_delta_rule
    T, N, H = 500, 4, 2
    offs = random_offsets(T, N, torch.Generator().manual_seed(5), min_len=1)
    q, k, v, g, beta, h0 = gdr_inputs(1, T, H, 128, 128, seed=31, N=N)
    ref = chunked_gated_delta_rule(q, k, v, g, beta, initial_state=h0, offsets=offs.tolist())
    dev = lambda x: x.to(device)
    plan = VarlenPlan(dev(offs), 64)
    print(f"gdr prep + scan packed {offs.tolist()}", flush=True)
    AT, gc = fwd_prepare_scan_operands(dev(k), dev(beta), dev(g), offsets=plan.offsets, indices=plan.indices)
    torch.cuda.synchronize()
    dense = unpack_triangular_tiles(AT).float().cpu()
    tu_ref, aqk_ref = _dense_tiles(ref, beta, 1, T, H, offs.tolist())
    assert_close("Tu", tu_ref, dense, 5e-3)
    AT3, _, w, Aw = fwd_prepare_scan_operands(dev(k), dev(beta), dev(g), offsets=plan.offsets,
                                              indices=plan.indices, keep_w=True)
    torch.cuda.synchronize()
    assert torch.equal(AT, AT3)
    assert_close("Aw", ref['Aw'], Aw, 5e-3)
    assert_close("w", ref['w'], w, 8e-3)
    o, ht = chunk_gated_delta_rule_fwd_scan(dev(q), dev(k), dev(v), AT, gc, 128 ** -0.5, dev(h0), True,
                                            offsets=plan.offsets, chunk_offsets=plan.chunk_offsets,
                                            seq_order=plan.seq_order)
    torch.cuda.synchronize()
    ro, rht = naive_recurrent_gated_delta_rule(q, k, v, g, beta, initial_state=h0, output_final_state=True,
                                               offsets=offs.tolist())
    assert_close("o", ro, o, TOL_O)
    assert_close("ht", rht, ht, TOL_HT)
    o2, ht2, _, _, Aqk = chunk_gated_delta_rule_fwd_scan(dev(q), dev(k), dev(v), AT, gc, 128 ** -0.5, dev(h0), True,
                                                         offsets=plan.offsets, chunk_offsets=plan.chunk_offsets,
                                                         seq_order=plan.seq_order, keep=True)
    torch.cuda.synchronize()
    assert torch.equal(o, o2) and torch.equal(ht, ht2)
    assert_close("Aqk", aqk_ref, unpack_triangular_tiles(Aqk).float().cpu(), 5e-3)


@pytest.mark.parametrize("K", [64, 128])
@pytest.mark.parametrize("B,H", [(2, 2), (3, 48)])
def test_gdr_scan_forms_the_gated_scores(device, K, B, H):
    """The scan forms Aqk = scale tril(q k^T * Gamma) itself, one chunk ahead of its use.  With Tu the identity, a
    zero initial state and v zero except in one chunk, where its rows are unit vectors, the state entering that
    chunk is zero and the output rows of the chunk are Aqk: checked against the fp32 chunked oracle's scores for
    the first chunk (formed before the loop), inner chunks and a short last chunk; (3, 48) runs 64-column slabs
    of a 128-column value (four waves share the blocks), (2, 2) 32-column slabs of a 64-column one (two waves)."""
    from fla_amd.ops.common.chunk_delta_h import chunk_gated_delta_rule_fwd_scan
    from oracle.chunked import chunked_gated_delta_rule
    T, V = 64 * 4 + 37, 64 if H == 2 else 128
    q, k, v, g, beta, _ = gdr_inputs(B, T, H, K, V, seed=23)
    ref = chunked_gated_delta_rule(q[:1, :, :2], k[:1, :, :2], v[:1, :, :2], g[:1, :, :2], beta[:1, :, :2])
    _, aqk_ref = _dense_tiles(ref, beta[:1, :, :2], 1, T, 2)
    chunks = -(-T // 64)
    eye_tile = torch.zeros(10, 16, 16)
    for i in range(4):
        eye_tile[i * (i + 1) // 2 + i] = torch.eye(16)
    AT = eye_tile.expand(B * chunks, H, 10, 16, 16).contiguous().to(device).bfloat16()
    gc = g.view(B, T, H).clone()
    for c0 in range(0, T, 64):
        gc[:, c0:c0 + 64] = g[:, c0:c0 + 64].cumsum(1)
    dev = lambda x: x.to(device)
    for c in (0, 1, chunks - 2, chunks - 1):
        L = min(64, T - 64 * c)
        print(f"gdr scan scores K={K} B={B} H={H} chunk {c}", flush=True)
        vv = torch.zeros(B, T, H, V)
        vv[:, 64 * c:64 * c + L, :, :L] = torch.eye(L)[None, :, None, :]
        o, ht = chunk_gated_delta_rule_fwd_scan(dev(q), dev(k), dev(vv.bfloat16()), AT, dev(gc), K ** -0.5, None, True)
        torch.cuda.synchronize()
        got = o[0, 64 * c:64 * c + L, :2, :L].float().cpu().permute(1, 0, 2)     # [head, row, column]
        assert_close(f"Aqk of chunk {c}", aqk_ref[c, :, :L, :L], got, 5e-3)
        assert torch.equal(got.triu(1), torch.zeros_like(got))
        assert torch.equal(o[:, :64 * c].float().cpu(), torch.zeros(B, 64 * c, H, V))   # nothing before the chunk


@pytest.mark.parametrize("varlen", [False, True])
def test_gdr_unfused_pipeline(device, varlen):
    """The reference's two-step form (state scan, then output stage) stays available."""
    from fla_amd.ops.gated_delta_rule.chunk import chunk_gated_delta_rule_fwd
    from oracle.recurrent import naive_recurrent_gated_delta_rule
    T, N = 500, 3
    offs = random_offsets(T, N, torch.Generator().manual_seed(5), min_len=1) if varlen else None
    q, k, v, g, beta, h0 = gdr_inputs(1 if varlen else 2, T, 2, 128, 128, seed=31, N=N if varlen else None)
    dev = lambda x: None if x is None else x.to(device)
    print(f"gdr unfused varlen={varlen}", flush=True)
    _, o, _, _, ht = chunk_gated_delta_rule_fwd(dev(q), dev(k), dev(v), dev(g), dev(beta), 128 ** -0.5, dev(h0), True,
                                                offsets=dev(offs), head_first=False, fused=False)
    torch.cuda.synchronize()
    ro, rht = naive_recurrent_gated_delta_rule(q, k, v, g, beta, initial_state=h0, output_final_state=True,
                                               offsets=None if offs is None else offs.tolist())
    assert_close("o", ro, o, TOL_O)
    assert_close("ht", rht, ht, TOL_HT)


# reference ladder: tests/ops/test_gated_delta.py:220-294 (T in {7,63,286,300,1000}, scale in {1, 0.1})
@pytest.mark.parametrize("T", [1, 7, 63, 64, 65, 286, 1000])
@pytest.mark.parametrize("K,V", [(128, 128), (64, 64), (64, 128), (128, 64)])
def test_chunk_gdr_shapes(device, T, K, V):
    from oracle.recurrent import naive_recurrent_gated_delta_rule
    q, k, v, g, beta, h0 = gdr_inputs(2, T, 2, K, V, seed=T + K)
    print(f"chunk_gdr T={T} K={K} V={V}", flush=True)
    o, ht = _run(device, q, k, v, g, beta, h0)
    ro, rht = naive_recurrent_gated_delta_rule(q, k, v, g, beta, initial_state=h0, output_final_state=True)
    assert o.dtype == q.dtype and ht.dtype == torch.float32
    assert_close("o", ro, o, TOL_O)
    assert_close("ht", rht, ht, TOL_HT)


@pytest.mark.parametrize("scale", [1.0, 0.1])
@pytest.mark.parametrize("normalizer", [0.1, 1.0, 10.0])
def test_chunk_gdr_gates_and_scale(device, scale, normalizer):
    """Strong and weak decays: the scalar gate is applied in fp32 with exponents <= 0."""
    from oracle.recurrent import naive_recurrent_gated_delta_rule
    q, k, v, g, beta, h0 = gdr_inputs(2, 300, 2, 128, 128, seed=22, h0_std=1.0, normalizer=normalizer)
    print(f"chunk_gdr scale={scale} normalizer={normalizer}", flush=True)
    o, ht = _run(device, q, k, v, g, beta, h0, scale=scale)
    ro, rht = naive_recurrent_gated_delta_rule(q, k, v, g, beta, scale=scale, initial_state=h0,
                                               output_final_state=True)
    assert_close("o", ro, o, TOL_O)
    assert_close("ht", rht, ht, TOL_HT)


def test_chunk_gdr_head_first_odd_dims_no_h0(device):
    from oracle.recurrent import naive_recurrent_gated_delta_rule
    q, k, v, g, beta, _ = gdr_inputs(2, 150, 3, 100, 100, seed=23, h0=False)
    print("chunk_gdr head-first D=100", flush=True)
    o, ht = _run(device, q, k, v, g, beta, None, head_first=True)
    ro, rht = naive_recurrent_gated_delta_rule(q, k, v, g, beta, output_final_state=True)
    assert_close("o", ro, o, TOL_O)
    assert_close("ht", rht, ht, TOL_HT)


# tests/ops/test_gated_delta.py:297-375
@pytest.mark.parametrize("T,N", [(64, 2), (300, 4), (1000, 5), (2048, 4)])
@pytest.mark.parametrize("H", [2, 16])
def test_chunk_gdr_varlen(device, T, N, H):
    from oracle.recurrent import naive_recurrent_gated_delta_rule
    gen = torch.Generator().manual_seed(T + H)
    offs = random_offsets(T, N, gen, min_len=1)
    q, k, v, g, beta, h0 = gdr_inputs(1, T, H, 128, 128, seed=24, N=N, h0_std=1.0)
    print(f"chunk_gdr varlen T={T} H={H} offs={offs.tolist()}", flush=True)
    o, ht = _run(device, q, k, v, g, beta, h0, offsets=offs)
    ro, rht = naive_recurrent_gated_delta_rule(q, k, v, g, beta, initial_state=h0, output_final_state=True,
                                               offsets=offs.tolist())
    assert_close("o", ro, o, TOL_O)
    assert_close("ht", rht, ht, TOL_HT)


# ---------------------------------------------------------------- backward
def _grads_ref(q, k, v, g, beta, h0, do, dht, offsets=None, scale=None):
    from oracle.recurrent import naive_recurrent_gated_delta_rule
    leaves = [x.detach().float().requires_grad_() for x in (q, k, v, g, beta)]
    h0l = None if h0 is None else h0.detach().float().requires_grad_()
    o, ht = naive_recurrent_gated_delta_rule(*leaves, scale=scale, initial_state=h0l, output_final_state=True,
                                             offsets=offsets)
    ((o * do.float()).sum() + (ht * dht.float()).sum()).backward()
    return [x.grad for x in leaves] + [None if h0l is None else h0l.grad]


def _grads_dev(device, q, k, v, g, beta, h0, do, dht, offsets=None, scale=None, head_first=False):
    from fla_amd.ops.gated_delta_rule import chunk_gated_delta_rule
    dev = lambda x: None if x is None else x.to(device)
    tr = (lambda x: x.transpose(1, 2).contiguous()) if head_first else (lambda x: x)
    leaves = [tr(dev(x)).detach().requires_grad_() for x in (q, k, v, g, beta)]
    h0l = None if h0 is None else dev(h0).detach().requires_grad_()
    o, ht = chunk_gated_delta_rule(*leaves, scale=scale, initial_state=h0l, output_final_state=True,
                                   offsets=dev(offsets), head_first=head_first)
    ((o.float() * tr(dev(do)).float()).sum() + (ht * dev(dht)).sum()).backward()
    torch.cuda.synchronize()
    return [tr(x.grad) for x in leaves] + [None if h0l is None else h0l.grad]


NAMES = ("dq", "dk", "dv", "dg", "dbeta", "dh0")
# reference tolerances (tests/ops/test_gated_delta.py:220-294): dq,dk,dv,dh0 0.008; dbeta, dg 0.02
TOLS = (8e-3, 8e-3, 8e-3, 2e-2, 2e-2, 8e-3)


@pytest.mark.parametrize("T", [64, 130, 300])
@pytest.mark.parametrize("K,V", [(128, 128), (64, 64), (64, 128), (128, 64)])
def test_chunk_gdr_backward(device, T, K, V):
    B, H = 2, 2
    q, k, v, g, beta, h0 = gdr_inputs(B, T, H, K, V, seed=51 + T, h0_std=1.0)
    gen = torch.Generator().manual_seed(7)
    do = torch.randn(B, T, H, V, generator=gen).bfloat16()
    dht = torch.randn(B, H, K, V, generator=gen) * 0.1
    print(f"chunk_gdr backward T={T} K={K} V={V}", flush=True)
    got = _grads_dev(device, q, k, v, g, beta, h0, do, dht)
    ref = _grads_ref(q, k, v, g, beta, h0, do, dht)
    for name, r, x, tol in zip(NAMES, ref, got, TOLS):
        assert_close(name, r, x, tol)


def test_chunk_gdr_backward_varlen_and_headfirst(device):
    gen = torch.Generator().manual_seed(8)
    T, N, H, D = 500, 4, 2, 128
    offs = random_offsets(T, N, gen, min_len=1)
    q, k, v, g, beta, h0 = gdr_inputs(1, T, H, D, D, seed=61, N=N, h0_std=1.0)
    do = torch.randn(1, T, H, D, generator=gen).bfloat16()
    dht = torch.randn(N, H, D, D, generator=gen) * 0.1
    print(f"chunk_gdr backward varlen offs={offs.tolist()}", flush=True)
    got = _grads_dev(device, q, k, v, g, beta, h0, do, dht, offsets=offs, scale=0.1)
    ref = _grads_ref(q, k, v, g, beta, h0, do, dht, offsets=offs.tolist(), scale=0.1)
    for name, r, x, tol in zip(NAMES, ref, got, TOLS):
        assert_close(name, r, x, tol)
    q, k, v, g, beta, _ = gdr_inputs(2, 150, 2, 100, 100, seed=62, h0=False)
    do = torch.randn(2, 150, 2, 100, generator=gen).bfloat16()
    dht = torch.randn(2, 2, 100, 100, generator=gen) * 0.1
    got = _grads_dev(device, q, k, v, g, beta, None, do, dht, head_first=True)
    ref = _grads_ref(q, k, v, g, beta, None, do, dht)
    for name, r, x, tol in zip(NAMES[:5], ref, got, TOLS):
        assert_close(name, r, x, tol)


# The reference's own ladder (tests/ops/test_gated_delta.py:220-294): head dims 50, 100, 200 (not
# multiples of 64, 200 needing 256 key channels), both layouts, strong and weak decays.
@pytest.mark.parametrize("D,T,scale,normalizer,head_first", [
    (50, 63, 1.0, 1.0, False),
    (100, 286, 0.1, 0.05, True),
    (200, 7, 1.0, 1.0, True),
    (200, 300, 0.1, 20.0, False),
    (200, 1000, 1.0, 0.05, False),
])
def test_chunk_gdr_reference_ladder(device, D, T, scale, normalizer, head_first):
    B, H = 2, 2
    q, k, v, g, beta, h0 = gdr_inputs(B, T, H, D, D, seed=71 + T, h0_std=1.0, normalizer=normalizer)
    gen = torch.Generator().manual_seed(9)
    do = torch.randn(B, T, H, D, generator=gen).bfloat16()
    dht = torch.randn(B, H, D, D, generator=gen) * 0.1
    print(f"chunk_gdr ladder D={D} T={T} scale={scale} normalizer={normalizer} head_first={head_first}", flush=True)
    o, ht = _run(device, q, k, v, g, beta, h0, scale=scale, head_first=head_first)
    from oracle.recurrent import naive_recurrent_gated_delta_rule
    ro, rht = naive_recurrent_gated_delta_rule(q, k, v, g, beta, scale=scale, initial_state=h0,
                                               output_final_state=True)
    assert_close("o", ro, o, TOL_O)
    assert_close("ht", rht, ht, TOL_HT)
    got = _grads_dev(device, q, k, v, g, beta, h0, do, dht, scale=scale, head_first=head_first)
    ref = _grads_ref(q, k, v, g, beta, h0, do, dht, scale=scale)
    for name, r, x, tol in zip(NAMES, ref, got, TOLS):
        assert_close(name, r, x, tol)


@pytest.mark.parametrize("varlen", [False, True])
def test_chunk_gdr_keep_vs_recompute(device, varlen, monkeypatch):
    """The backward from what the forward kept (w, Aw and the v_new / states the scan wrote) and the
    reference-style backward that recomputes them (WY launch + state scan on w, u) run the same backward
    kernels on operands that differ by one 16-bit rounding (v_new = Tu (v - e^g (k h)) against u - e^g (w h)):
    the two sets of gradients carry independent rounding errors and stay within the operator's tolerances of each
    other; the forward within tolerance."""
    import fla_amd.ops.gated_delta_rule.chunk as mod
    from oracle.recurrent import naive_recurrent_gated_delta_rule
    gen = torch.Generator().manual_seed(12)
    T, N, H, D = 400, 3, 2, 128
    offs = random_offsets(T, N, gen, min_len=1) if varlen else None
    q, k, v, g, beta, h0 = gdr_inputs(1 if varlen else 2, T, H, D, D, seed=63, N=N if varlen else None, h0_std=1.0)
    do = torch.randn(q.shape[0], T, H, D, generator=gen).bfloat16()
    dht = torch.randn(h0.shape, generator=gen) * 0.1
    print(f"chunk_gdr keep vs recompute varlen={varlen}", flush=True)
    assert mod.KEEP_STATES_FOR_BACKWARD
    kept = _grads_dev(device, q, k, v, g, beta, h0, do, dht, offsets=offs)
    o_keep, ht_keep = _run(device, *[x.requires_grad_() for x in (q.clone(), k.clone(), v.clone())], g, beta, h0,
                           offsets=offs)
    monkeypatch.setattr(mod, "KEEP_STATES_FOR_BACKWARD", False)
    rec = _grads_dev(device, q, k, v, g, beta, h0, do, dht, offsets=offs)
    for name, a, b, tol in zip(NAMES, kept, rec, TOLS):
        assert_close(name + " kept vs recomputed", b.float().cpu(), a, tol)
    ro, rht = naive_recurrent_gated_delta_rule(q, k, v, g, beta, initial_state=h0, output_final_state=True,
                                               offsets=None if offs is None else offs.tolist())
    assert_close("o (two launches, states kept)", ro, o_keep, TOL_O)
    assert_close("ht (two launches, states kept)", rht, ht_keep, TOL_HT)


@pytest.mark.parametrize("varlen", [False, True])
def test_chunk_gdr_gradients_are_reproducible(device, varlen):
    """Same inputs twice: every gradient identical bit for bit (no atomics anywhere in the backward)."""
    gen = torch.Generator().manual_seed(13)
    T, N, H, D = 700, 4, 3, 128
    offs = random_offsets(T, N, gen, min_len=1) if varlen else None
    q, k, v, g, beta, h0 = gdr_inputs(1 if varlen else 2, T, H, D, D, seed=64, N=N if varlen else None, h0_std=1.0)
    do = torch.randn(q.shape[0], T, H, D, generator=gen).bfloat16()
    dht = torch.randn(h0.shape, generator=gen) * 0.1
    print(f"chunk_gdr reproducibility varlen={varlen}", flush=True)
    first = _grads_dev(device, q, k, v, g, beta, h0, do, dht, offsets=offs)
    for _ in range(3):
        again = _grads_dev(device, q, k, v, g, beta, h0, do, dht, offsets=offs)
        for name, a, b in zip(NAMES, first, again):
            assert torch.equal(a, b), name


def test_chunk_gdr_slab_width_independence(device):
    """B=4 x H=16 puts the scan on 32-column slabs (128 workgroups of 64 columns would leave half the CUs idle),
    the same batch stacked twice on 64-column slabs; the delta rule is independent per value column, so outputs
    and final states of the first four sequences agree bit for bit.  Also against the recurrence on one pair."""
    from oracle.recurrent import naive_recurrent_gated_delta_rule
    B, T, H, D = 4, 1024, 16, 128
    q, k, v, g, beta, h0 = gdr_inputs(B, T, H, D, D, seed=71)
    print("chunk_gdr slab-width independence B=4 vs B=8", flush=True)
    o4, ht4 = _run(device, q, k, v, g, beta, h0)
    twice = lambda x: torch.cat([x, x], 0)
    o8, ht8 = _run(device, twice(q), twice(k), twice(v), twice(g), twice(beta), twice(h0))
    assert torch.equal(o8[:B], o4) and torch.equal(o8[B:], o4)
    assert torch.equal(ht8[:B], ht4) and torch.equal(ht8[B:], ht4)
    b, h = 3, 11
    sl = lambda x: x[b:b + 1, :, h:h + 1]
    ro, rht = naive_recurrent_gated_delta_rule(sl(q), sl(k), sl(v), sl(g), sl(beta), initial_state=h0[b:b + 1, h:h + 1],
                                               output_final_state=True)
    assert_close("o[3,11]", ro, o4[b:b + 1, :, h:h + 1], TOL_O)
    assert_close("ht[3,11]", rht, ht4[b:b + 1, h:h + 1], TOL_HT)


def test_chunk_gdr_slab_width_independence_backward(device):
    """The same for a forward that keeps its intermediates and the backward that reads them: gradients of the
    batch stacked twice (64-column slabs) equal those of the batch alone (32-column slabs) bit for bit, except the
    gradients shared by nothing (all of them are per sequence)."""
    B, T, H, D = 4, 512, 16, 128
    gen = torch.Generator().manual_seed(72)
    q, k, v, g, beta, h0 = gdr_inputs(B, T, H, D, D, seed=72)
    do = torch.randn(B, T, H, D, generator=gen).bfloat16()
    dht = torch.randn(h0.shape, generator=gen) * 0.1
    print("chunk_gdr slab-width independence (backward) B=4 vs B=8", flush=True)
    twice = lambda x: torch.cat([x, x], 0)
    g4 = _grads_dev(device, q, k, v, g, beta, h0, do, dht)
    g8 = _grads_dev(device, twice(q), twice(k), twice(v), twice(g), twice(beta), twice(h0), twice(do), twice(dht))
    for name, a, b in zip(NAMES, g4, g8):
        assert torch.equal(b[:B], a) and torch.equal(b[B:], a), name


@pytest.mark.parametrize("K,V,T,varlen", [(128, 128, 300, False), (128, 128, 1000, True), (64, 128, 130, False),
                                          (64, 64, 65, True), (128, 64, 1, False)])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_chunk_gdr_qk_l2norm_in_kernel(device, dtype, K, V, T, varlen):
    """The opt-in form on un-normalised q and k: the two forward launches l2-normalise the rows themselves
    (fla/layers/gated_deltanet.py:234-235).  Against the recurrence on the oracle's l2norm (rounded to the
    storage type, as the stand-alone launch leaves it), and against that two-step form of the same library."""
    from fla_amd.modules import l2norm_fwd
    from fla_amd.ops.gated_delta_rule import chunk_gated_delta_rule
    from oracle.modules import l2norm
    from oracle.recurrent import naive_recurrent_gated_delta_rule
    gen = torch.Generator().manual_seed(T + K + V)
    B, H, N = (1, 3, 3) if varlen else (2, 3, 2)
    q = (torch.randn(B, T, H, K, generator=gen) * 1.7).to(dtype)
    k = (torch.randn(B, T, H, K, generator=gen) * 0.6).to(dtype)
    _, _, v, g, beta, h0 = gdr_inputs(B, T, H, K, V, seed=T, dtype=dtype, N=N)
    offs = random_offsets(T, N, gen) if varlen else None
    print(f"chunk_gdr in-kernel l2norm {dtype} K={K} V={V} T={T} varlen={varlen}", flush=True)
    dev = lambda t: None if t is None else t.to(device)
    o, ht = chunk_gated_delta_rule(dev(q), dev(k), dev(v), dev(g), dev(beta), initial_state=dev(h0),
                                   output_final_state=True, offsets=dev(offs), head_first=False,
                                   use_qk_l2norm_in_kernel=True)
    qn, kn = l2norm(q).to(dtype), l2norm(k).to(dtype)
    ro, rht = naive_recurrent_gated_delta_rule(qn, kn, v, g, beta, initial_state=h0, output_final_state=True,
                                               offsets=None if offs is None else offs.tolist())
    assert_close("o", ro, o, TOL_O)
    assert_close("ht", rht, ht, TOL_HT)
    o2, ht2 = chunk_gated_delta_rule(l2norm_fwd(dev(q)), l2norm_fwd(dev(k)), dev(v), dev(g), dev(beta),
                                     initial_state=dev(h0), output_final_state=True, offsets=dev(offs),
                                     head_first=False)
    assert_close("o vs two-step", o2, o, 6e-3)
    assert_close("ht vs two-step", ht2, ht, 6e-3)


def test_chunk_gdr_qk_l2norm_backward(device):
    """With gradients the l2norm form runs the stand-alone l2 norm and its backward either side of the operator:
    gradients of the raw q and k against autograd through the oracle's l2norm and recurrence."""
    from fla_amd.ops.gated_delta_rule import chunk_gated_delta_rule
    from oracle.modules import l2norm
    from oracle.recurrent import naive_recurrent_gated_delta_rule
    gen = torch.Generator().manual_seed(3)
    B, T, H, K, V = 2, 130, 2, 64, 64
    q = (torch.randn(B, T, H, K, generator=gen) * 1.7).bfloat16()
    k = (torch.randn(B, T, H, K, generator=gen) * 0.6).bfloat16()
    _, _, v, g, beta, h0 = gdr_inputs(B, T, H, K, V, seed=4)
    do = torch.randn(B, T, H, V, generator=gen).bfloat16()
    print("chunk_gdr l2norm backward", flush=True)
    leaves = [t.to(device).requires_grad_() for t in (q, k, v, g, beta)]
    o, _ = chunk_gated_delta_rule(*leaves, initial_state=h0.to(device), head_first=False, use_qk_l2norm_in_kernel=True)
    o.backward(do.to(device))
    ref = [t.float().requires_grad_() for t in (q, k, v, g, beta)]
    ro, _ = naive_recurrent_gated_delta_rule(l2norm(ref[0]), l2norm(ref[1]), ref[2], ref[3], ref[4], initial_state=h0)
    ro.backward(do.float())
    assert_close("o", ro, o, TOL_O)
    for name, a, b in zip(("dq", "dk", "dv", "dg", "dbeta"), ref, leaves):
        assert_close(name, a.grad, b.grad, 2e-2)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("K,V,T,varlen,gated,h0", [
    (128, 128, 300, False, True, True), (128, 128, 1000, True, True, True), (64, 128, 130, False, True, False),
    (128, 64, 65, True, True, True), (64, 64, 1, False, True, True), (128, 128, 63, False, False, True),
    (128, 128, 257, True, False, False), (128, 256, 200, False, True, True)])
def test_chunk_gdr_onepass_forward(device, monkeypatch, dtype, K, V, T, varlen, gated, h0):
    """The one-launch forward (the WY blocks formed inside the scan, block forward substitution instead of the
    64x64 inverse), forced at these small shapes: against the fp32 recurrence, and against the two-launch form."""
    import fla_amd.ops.gated_delta_rule.chunk as mod
    from oracle.recurrent import naive_recurrent_gated_delta_rule
    gen = torch.Generator().manual_seed(T + K + V)
    B, H, N = (1, 3, 4) if varlen else (2, 3, 2)
    q, k, v, g, beta, s0 = gdr_inputs(B, T, H, K, V, seed=T + 1, dtype=dtype, N=N)
    if not gated:
        g = None
    if not h0:
        s0 = None
    offs = random_offsets(T, N, gen) if varlen else None
    print(f"chunk_gdr one-pass {dtype} K={K} V={V} T={T} varlen={varlen} gated={gated} h0={h0}", flush=True)
    dev = lambda t: None if t is None else t.to(device)
    args = (dev(q), dev(k), dev(v), dev(g), dev(beta))
    kw = dict(initial_state=dev(s0), output_final_state=True, offsets=dev(offs), head_first=False)
    monkeypatch.setattr(mod, "_ONEPASS_MIN_WORKGROUPS", 1)
    monkeypatch.setattr(mod, "ONEPASS_FORWARD", True)
    calls = []
    real = mod.chunk_gated_delta_rule_fwd_onepass
    monkeypatch.setattr(mod, "chunk_gated_delta_rule_fwd_onepass", lambda *a, **k2: (calls.append(1), real(*a, **k2))[1])
    o, ht = mod.chunk_gated_delta_rule(*args, **kw)
    assert calls, "the one-launch form was not taken"
    monkeypatch.setattr(mod, "ONEPASS_FORWARD", False)
    o2, ht2 = mod.chunk_gated_delta_rule(*args, **kw)
    ro, rht = naive_recurrent_gated_delta_rule(q, k, v, g, beta, initial_state=s0, output_final_state=True,
                                               offsets=None if offs is None else offs.tolist())
    assert_close("o", ro, o, TOL_O)
    assert_close("ht", rht, ht, TOL_HT)
    assert_close("o vs two-launch", o2, o, 6e-3)
    assert_close("ht vs two-launch", ht2, ht, 6e-3)
