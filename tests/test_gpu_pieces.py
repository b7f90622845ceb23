"""GPU: the chunk-parallel GLA stages under the reference's internal signatures
(``chunk_gla_fwd_o_gk``, ``chunk_gla_bwd_dA``, ``chunk_gla_bwd_dv`` of ``fla/ops/gla/chunk.py``,
called that way by RWKV6) against the fp32 oracle, with the scores ``A`` and the row-major
per-chunk states supplied by the caller.

Tolerances (rel-L2): 1e-2 on o and dv (bf16 operands of two matrix products), 5e-3 on dA (one
product, fp32 output)."""
import pytest
import torch
import torch.nn.functional as F

from helpers import assert_close, gla_inputs, random_offsets

pytestmark = pytest.mark.gpu

TOL_O, TOL_DA = 1e-2, 5e-3


def _case(B, T, H, K, V, varlen, seed, dtype=torch.bfloat16):
    from oracle import chunked
    N = 4
    offs = random_offsets(T, N, torch.Generator().manual_seed(seed), min_len=1) if varlen else None
    q, k, v, g, _ = gla_inputs(1 if varlen else B, T, H, K, V, seed=seed, dtype=dtype, h0=False)
    ol = None if offs is None else offs.tolist()
    r = chunked.chunked_gla(q, k, v, g, offsets=ol)
    gen = torch.Generator().manual_seed(seed + 1)
    do = torch.randn(v.shape, generator=gen).to(dtype)
    dh = torch.randn(r["h"].shape, generator=gen) * 0.1
    return dict(q=q, k=k, v=v, g=g, G=r["g_cumsum"].float(), A=r["A"].float(), h=r["h"].float(), o=r["o"], do=do, dh=dh,
                offs=offs, ol=ol, scale=K ** -0.5)


def _plan(offs, device):
    if offs is None:
        return None, None
    from fla_amd.utils import VarlenPlan
    plan = VarlenPlan(offs.to(device), 64)
    return plan.offsets, plan.indices


SHAPES = [
    # B, T, H, K, V
    (2, 256, 3, 128, 128),
    (2, 200, 2, 64, 64),
    (1, 300, 2, 128, 64),
    (2, 130, 2, 256, 256),
    (2, 150, 2, 100, 50),   # neither a power of two nor a multiple of 64: padded by the wrapper
    (2, 40, 2, 64, 64),     # shorter than a chunk: the reference shrinks BT to 64 here as well
    (1, 20, 2, 32, 32),     # BT = 32
]


@pytest.mark.parametrize("B,T,H,K,V", SHAPES)
@pytest.mark.parametrize("varlen", [False, True])
@pytest.mark.parametrize("state_dtype", ["fp32", "same"])
def test_chunk_gla_fwd_o_gk_reference_operands(device, B, T, H, K, V, varlen, state_dtype):
    from fla_amd.ops.gla.chunk import chunk_gla_fwd_o_gk
    if varlen and T < 64:
        pytest.skip("packed case covered at the longer shapes")
    c = _case(B, T, H, K, V, varlen, seed=T + K)
    print(f"o_gk B={B} T={T} H={H} K={K} V={V} varlen={varlen} states={state_dtype}", flush=True)
    offsets, indices = _plan(c["offs"], device)
    bt = min(64, max(16, 1 << (T - 1).bit_length()))
    A, h = c["A"][..., :bt], c["h"]
    if state_dtype == "same":
        A, h = A.to(c["q"].dtype), h.to(c["q"].dtype)
    o = chunk_gla_fwd_o_gk(c["q"].to(device), c["v"].to(device), c["G"].to(device), A.to(device), h.to(device),
                           c["scale"], offsets=offsets, indices=indices, head_first=False, chunk_size=64)
    torch.cuda.synchronize()
    assert o.dtype == c["v"].dtype
    assert_close("o", c["o"], o, TOL_O)


@pytest.mark.parametrize("B,T,H,K,V", SHAPES)
@pytest.mark.parametrize("varlen", [False, True])
def test_chunk_gla_bwd_dA_and_dv_reference_operands(device, B, T, H, K, V, varlen):
    from fla_amd.ops.gla.chunk import chunk_gla_bwd_dA, chunk_gla_bwd_dv
    from oracle import chunked
    if varlen and T < 64:
        pytest.skip("packed case covered at the longer shapes")
    c = _case(B, T, H, K, V, varlen, seed=T + V + 1)
    print(f"dA/dv B={B} T={T} H={H} K={K} V={V} varlen={varlen}", flush=True)
    offsets, indices = _plan(c["offs"], device)
    bt = min(64, max(16, 1 << (T - 1).bit_length()))
    dA = chunk_gla_bwd_dA(c["v"].to(device), c["do"].to(device), c["scale"], offsets=offsets, indices=indices,
                          head_first=False, chunk_size=64)
    dv = chunk_gla_bwd_dv(c["k"].to(device), c["G"].to(device), c["A"][..., :bt].to(device), c["do"].to(device),
                          c["dh"].to(device), offsets=offsets, indices=indices, head_first=False, chunk_size=64)
    torch.cuda.synchronize()
    assert dA.dtype == torch.float32 and dA.shape[-1] == bt and dv.dtype == c["do"].dtype
    ref_dA = chunked.gla_bwd_dA(c["v"], c["do"], c["scale"], offsets=c["ol"])[..., :bt]
    ref_dv = chunked.gla_bwd_dv(c["k"], c["G"], c["A"], c["do"], c["dh"], offsets=c["ol"])
    assert_close("dA", ref_dA, dA, TOL_DA)
    # nothing above the diagonal, bit for bit
    pos = torch.arange(T) % 64 if c["offs"] is None else torch.cat(
        [torch.arange(int(e - s)) % 64 for s, e in zip(c["offs"][:-1], c["offs"][1:])])
    upper = torch.arange(bt)[None, :] > pos[:, None]
    assert (dA.cpu()[:, upper.nonzero()[:, 0], :, upper.nonzero()[:, 1]] == 0).all()
    assert_close("dv", ref_dv, dv, TOL_O)


def test_gla_stages_head_first_and_fp16(device):
    """head_first=True (the reference's default for these functions) and fp16 operands."""
    from fla_amd.ops.gla.chunk import chunk_gla_bwd_dA, chunk_gla_bwd_dv, chunk_gla_fwd_o_gk
    from oracle import chunked
    B, T, H, K, V = 2, 192, 3, 64, 128
    c = _case(B, T, H, K, V, False, seed=5, dtype=torch.float16)
    hf = lambda x: x.transpose(1, 2).contiguous().to(device)
    o = chunk_gla_fwd_o_gk(hf(c["q"]), hf(c["v"]), hf(c["G"]), hf(c["A"]), hf(c["h"]), c["scale"])
    dA = chunk_gla_bwd_dA(hf(c["v"]), hf(c["do"]), c["scale"])
    dv = chunk_gla_bwd_dv(hf(c["k"]), hf(c["G"]), hf(c["A"]), hf(c["do"]), hf(c["dh"]))
    torch.cuda.synchronize()
    assert o.shape == (B, H, T, V) and dA.shape == (B, H, T, 64) and dv.shape == (B, H, T, V)
    assert_close("o", c["o"], o.transpose(1, 2), TOL_O)
    assert_close("dA", chunked.gla_bwd_dA(c["v"], c["do"], c["scale"]), dA.transpose(1, 2), TOL_DA)
    assert_close("dv", chunked.gla_bwd_dv(c["k"], c["G"], c["A"], c["do"], c["dh"]), dv.transpose(1, 2), TOL_O)


def test_gla_stages_compose_with_the_operator(device):
    """The output stage fed with row-major states from this library's own chunk_fwd_h (and the oracle's
    scores) reproduces chunk_gla's output."""
    from fla_amd.ops.common.chunk_h import chunk_fwd_h
    from fla_amd.ops.gla import chunk_gla
    from fla_amd.ops.gla.chunk import chunk_gla_fwd_o_gk
    from fla_amd.ops.utils.cumsum import chunk_local_cumsum
    from oracle import chunked
    B, T, H, K, V = 2, 512, 4, 128, 128
    q, k, v, g, _ = gla_inputs(B, T, H, K, V, seed=9, h0=False)
    q, k, v, g = (x.to(device) for x in (q, k, v, g))
    o_ref, _ = chunk_gla(q, k, v, g, head_first=False)
    G = chunk_local_cumsum(g, 64, head_first=False)
    h, _ = chunk_fwd_h(k, v, None, G, None, None, False, head_first=False, chunk_size=64, states_in_fp32=True)
    A = chunked.chunked_gla(q.cpu(), k.cpu(), v.cpu(), g.cpu())["A"].to(device)
    o = chunk_gla_fwd_o_gk(q, v, G, A, h, K ** -0.5, head_first=False)
    torch.cuda.synchronize()
    assert_close("o vs chunk_gla", o_ref.float(), o, TOL_O)


def test_gla_stage_argument_errors(device):
    from fla_amd.ops.gla.chunk import chunk_gla_bwd_dA, chunk_gla_fwd_o_gk
    c = _case(1, 64, 1, 64, 64, False, seed=1)
    d = lambda x: x.to(device)
    with pytest.raises(NotImplementedError):
        chunk_gla_bwd_dA(d(c["v"]), d(c["do"]), 1.0, head_first=False, chunk_size=32)
    with pytest.raises(NotImplementedError):
        chunk_gla_fwd_o_gk(d(c["q"]).float(), d(c["v"]), d(c["G"]), d(c["A"]), d(c["h"]), 1.0, head_first=False)


# chunk_bwd_dh with the reference's arguments (fla/ops/common/chunk_h.py:338-410): row-major dh, 5e-3 on dh / dh0
# (bf16 q~ and do operands, fp32 accumulation over the whole sequence)
@pytest.mark.parametrize("B,T,H,K,V", [(2, 256, 3, 128, 128), (2, 200, 2, 64, 128), (1, 1000, 2, 128, 64),
                                       (2, 130, 2, 256, 256), (2, 150, 2, 100, 50), (2, 40, 2, 64, 64)])
@pytest.mark.parametrize("varlen", [False, True])
@pytest.mark.parametrize("gates", ["gk", "g", "none"])
def test_chunk_bwd_dh_reference_operands(device, B, T, H, K, V, varlen, gates):
    from fla_amd.ops.common.chunk_h import chunk_bwd_dh
    from oracle import chunked, cumsum
    if varlen and T < 64:
        pytest.skip("packed case covered at the longer shapes")
    N = 4 if varlen else B
    gen = torch.Generator().manual_seed(T + K + V)
    offs = random_offsets(T, N, gen, min_len=1) if varlen else None
    Bq = 1 if varlen else B
    ol = None if offs is None else offs.tolist()
    q = torch.randn(Bq, T, H, K, generator=gen).bfloat16()
    k = torch.randn(Bq, T, H, K, generator=gen).bfloat16()
    v = torch.randn(Bq, T, H, V, generator=gen).bfloat16()
    do = torch.randn(Bq, T, H, V, generator=gen).bfloat16()
    dht = torch.randn(N, H, K, V, generator=gen) * 0.1
    h0 = torch.zeros(N, H, K, V)
    gk = cumsum.chunk_local_cumsum(F.logsigmoid(torch.randn(Bq, T, H, K, generator=gen)) / 16, 64, offsets=ol) \
        if gates == "gk" else None
    g = cumsum.chunk_local_cumsum(F.logsigmoid(torch.randn(Bq, T, H, generator=gen)), 64, offsets=ol) \
        if gates == "g" else None
    print(f"chunk_bwd_dh B={B} T={T} H={H} K={K} V={V} varlen={varlen} gates={gates}", flush=True)
    d = lambda x: None if x is None else x.to(device)
    indices = None
    if varlen:
        from fla_amd.utils import VarlenPlan
        indices = VarlenPlan(offs.to(device), 64).indices
    scale = K ** -0.5
    for fp32 in (True, False):
        dh, dh0 = chunk_bwd_dh(d(q), d(k), d(v), d(g), d(gk), None, d(do), d(h0), d(dht), scale, offsets=d(offs),
                               indices=indices, head_first=False, chunk_size=64, states_in_fp32=fp32)
        torch.cuda.synchronize()
        ref_dh, ref_dh0 = chunked.chunk_bwd_dh(q, g, gk, do, dht, scale, offsets=ol)
        assert dh.dtype == (torch.float32 if fp32 else torch.bfloat16) and dh0.dtype == torch.float32
        assert_close("dh", ref_dh, dh, 5e-3)
        assert_close("dh0", ref_dh0, dh0, 5e-3)
    # without h0 no dh0 comes back, as in the reference; without dht the scan starts from zero
    dh, none = chunk_bwd_dh(d(q), d(k), d(v), d(g), d(gk), None, d(do), None, None, scale, offsets=d(offs),
                            indices=indices, head_first=False, states_in_fp32=True)
    torch.cuda.synchronize()
    assert none is None
    assert_close("dh (no dht)", chunked.chunk_bwd_dh(q, g, gk, do, None, scale, offsets=ol)[0], dh, 5e-3)


@pytest.mark.parametrize("varlen", [False, True])
def test_chunk_fwd_h_per_head_gates_row_major(device, varlen):
    """chunk_fwd_h(g=...) as chunk_simple_gla's pipeline calls it (fla/ops/simple_gla/chunk.py:33-46):
    per-head chunk-cumulative gates, row-major fp32 states; 5e-3 on the states."""
    from fla_amd.ops.common.chunk_h import chunk_fwd_h
    from oracle import chunked, cumsum
    B, T, H, K, V, N = (1 if varlen else 2), 300, 3, 128, 64, 3
    gen = torch.Generator().manual_seed(17)
    offs = random_offsets(T, N, gen, min_len=1) if varlen else None
    ol = None if offs is None else offs.tolist()
    k = torch.randn(B, T, H, K, generator=gen).bfloat16()
    v = torch.randn(B, T, H, V, generator=gen).bfloat16()
    g = F.logsigmoid(torch.randn(B, T, H, generator=gen))
    h0 = torch.randn(N if varlen else B, H, K, V, generator=gen) * 0.1
    r = chunked.chunked_gla(k, k, v, g[..., None].expand(B, T, H, K), initial_state=h0, offsets=ol)
    G = cumsum.chunk_local_cumsum(g, 64, offsets=ol)
    d = lambda x: None if x is None else x.to(device)
    indices = None
    if varlen:
        from fla_amd.utils import VarlenPlan
        indices = VarlenPlan(offs.to(device), 64).indices
    h, ht = chunk_fwd_h(d(k), d(v), d(G), None, None, d(h0), True, offsets=d(offs), indices=indices,
                        head_first=False, chunk_size=64, states_in_fp32=True)
    torch.cuda.synchronize()
    assert_close("h", r["h"], h, 5e-3)
    assert_close("ht", r["ht"], ht, 5e-3)


@pytest.mark.parametrize("K,V", [(128, 128), (64, 128), (128, 64)])
def test_states_to_fragments_matches_the_scan_kernels_own_layouts(device, K, V):
    """Row-major states re-ordered by fla_states_to_fragments are bit-identical to what the state scan
    writes directly in fragment order (both orientations), from fp32 and from 16-bit sources."""
    from fla_amd.ops.common.chunk_h import chunk_fwd_h
    from fla_amd.ops.common.chunk_o import states_to_fragments
    from fla_amd.ops.utils.cumsum import chunk_local_cumsum
    B, T, H = 2, 300, 3
    q, k, v, g, h0 = gla_inputs(B, T, H, K, V, seed=K + V)
    k, v, g, h0 = (x.to(device) for x in (k, v, g, h0))
    G = chunk_local_cumsum(g, 64, head_first=False)
    kw = dict(head_first=False, chunk_size=64)
    h_rm, _ = chunk_fwd_h(k, v, None, G, None, h0, False, **kw)
    h_f32, _ = chunk_fwd_h(k, v, None, G, None, h0, False, states_in_fp32=True, **kw)
    h_fr, _ = chunk_fwd_h(k, v, None, G, None, h0, False, fragment_layout=True, **kw)
    h_frt, _ = chunk_fwd_h(k, v, None, G, None, h0, False, fragment_layout=True, transposed_fragments=True, **kw)
    torch.cuda.synchronize()
    assert torch.equal(states_to_fragments(h_rm, k.dtype), h_fr)
    assert torch.equal(states_to_fragments(h_rm, k.dtype, transposed=True), h_frt)
    assert torch.equal(states_to_fragments(h_f32, k.dtype), h_fr)
    assert torch.equal(states_to_fragments(h_f32, k.dtype, transposed=True), h_frt)


@pytest.mark.parametrize("B,T,H,K,V", [(2, 256, 3, 128, 128), (2, 200, 2, 64, 128), (2, 130, 2, 256, 64),
                                       (2, 150, 2, 100, 50), (1, 300, 2, 128, 256), (2, 40, 2, 64, 64)])
@pytest.mark.parametrize("varlen", [False, True])
@pytest.mark.parametrize("gated", [True, False])
def test_chunk_bwd_dv_local_reference_operands(device, B, T, H, K, V, varlen, gated):
    """chunk_bwd_dv_local with the reference's arguments (fla/ops/common/chunk_o.py:551-599); 1e-2 on dv
    (the scores are rounded to bf16 before the second product, as in the reference)."""
    from fla_amd.ops.common.chunk_o import chunk_bwd_dv_local
    from oracle import chunked, cumsum
    if varlen and T < 64:
        pytest.skip("packed case covered at the longer shapes")
    gen = torch.Generator().manual_seed(T + K + V + 3)
    offs = random_offsets(T, 4, gen, min_len=1) if varlen else None
    ol = None if offs is None else offs.tolist()
    Bq = 1 if varlen else B
    q = torch.randn(Bq, T, H, K, generator=gen).bfloat16()
    k = torch.randn(Bq, T, H, K, generator=gen).bfloat16()
    do = torch.randn(Bq, T, H, V, generator=gen).bfloat16()
    g = cumsum.chunk_local_cumsum(F.logsigmoid(torch.randn(Bq, T, H, generator=gen)), 64, offsets=ol) if gated else None
    print(f"dv_local B={B} T={T} H={H} K={K} V={V} varlen={varlen} gated={gated}", flush=True)
    d = lambda x: None if x is None else x.to(device)
    dv = chunk_bwd_dv_local(d(q), d(k), d(g), d(do), None, K ** -0.5, offsets=d(offs), head_first=False)
    torch.cuda.synchronize()
    assert dv.shape == do.shape and dv.dtype == do.dtype
    assert_close("dv_local", chunked.chunk_bwd_dv_local(q, k, g, do, K ** -0.5, offsets=ol), dv, 1e-2)


# ---- the argument forms GSA and RWKV6 use beside the GLA stages (fla/ops/gsa/chunk.py:664-675, 794-820;
# fla/ops/rwkv6/chunk.py:1134-1147): decay on the value axis, head-first layout, grouped query heads
@pytest.mark.parametrize("head_first", [False, True])
@pytest.mark.parametrize("B,T,H,K,V,varlen", [(2, 200, 3, 64, 128, False), (1, 300, 2, 128, 64, True),
                                              (2, 130, 2, 100, 50, False), (2, 20, 2, 64, 64, False)])
def test_chunk_fwd_h_value_gates(device, head_first, B, T, H, K, V, varlen):
    """chunk_fwd_h(gv=...) as GSA calls it: row-major states and final state against the oracle's state scan with
    per-value gates (5e-3, bf16 operands); head-first operands give the same states, transposed."""
    from fla_amd.ops.common.chunk_h import chunk_fwd_h
    from oracle import chunked, cumsum
    if varlen and head_first:
        pytest.skip("packed batches are seq-first")
    gen = torch.Generator().manual_seed(T + K + V)
    N = 3 if varlen else B
    offs = random_offsets(T, N, gen, min_len=1) if varlen else None
    ol = None if offs is None else offs.tolist()
    k = torch.randn(B, T, H, K, generator=gen).bfloat16()
    v = torch.randn(B, T, H, V, generator=gen).bfloat16()
    gv = cumsum.chunk_local_cumsum(F.logsigmoid(torch.randn(B, T, H, V, generator=gen)) / 4, 64, offsets=ol)
    h0 = torch.randn(N, H, K, V, generator=gen) * 0.1
    print(f"chunk_fwd_h gv head_first={head_first} B={B} T={T} H={H} K={K} V={V} varlen={varlen}", flush=True)
    d = lambda x: None if x is None else x.to(device)
    hf = lambda x: x.transpose(1, 2).contiguous() if head_first else x
    indices = None
    if varlen:
        from fla_amd.utils import VarlenPlan
        indices = VarlenPlan(offs.to(device), 64).indices
    for fp32 in (True, False):
        h, ht = chunk_fwd_h(d(hf(k)), d(hf(v)), None, None, d(hf(gv)), d(h0), True, offsets=d(offs), indices=indices,
                            head_first=head_first, chunk_size=64, states_in_fp32=fp32)
        torch.cuda.synchronize()
        ref_h, ref_ht = chunked.chunk_fwd_h(k, v, None, None, gv, h0, offsets=ol)
        if head_first:
            h = h.transpose(1, 2)
        assert h.dtype == (torch.float32 if fp32 else torch.bfloat16) and ht.dtype == torch.float32
        assert_close("h", ref_h, h, 5e-3)
        assert_close("ht", ref_ht, ht, 5e-3)


@pytest.mark.parametrize("head_first", [False, True])
@pytest.mark.parametrize("gates", ["gv", "gk", "g"])
@pytest.mark.parametrize("NG", [1, 2])
def test_chunk_bwd_dh_value_gates_grouped_heads_and_head_first(device, head_first, gates, NG):
    """chunk_bwd_dh with decay on the value axis, with HQ = NG * H query heads (a query head decays with its
    group's gates; dh0 sums over the group) and in head-first layout, against the oracle's reverse scan."""
    from fla_amd.ops.common.chunk_h import chunk_bwd_dh
    from oracle import chunked, cumsum
    B, T, H, K, V = 2, 200, 2, 64, 128
    HQ = NG * H
    gen = torch.Generator().manual_seed(7 + NG)
    q = torch.randn(B, T, HQ, K, generator=gen).bfloat16()
    do = torch.randn(B, T, HQ, V, generator=gen).bfloat16()
    k = torch.randn(B, T, H, K, generator=gen).bfloat16()
    v = torch.randn(B, T, H, V, generator=gen).bfloat16()
    raw = {"gv": F.logsigmoid(torch.randn(B, T, H, V, generator=gen)) / 4,
           "gk": F.logsigmoid(torch.randn(B, T, H, K, generator=gen)) / 4,
           "g": F.logsigmoid(torch.randn(B, T, H, generator=gen))}
    gates_c = {n: (cumsum.chunk_local_cumsum(x, 64) if n == gates else None) for n, x in raw.items()}
    dht = torch.randn(B, HQ, K, V, generator=gen) * 0.1
    h0 = torch.zeros(B, H, K, V)
    scale = K ** -0.5
    print(f"chunk_bwd_dh gates={gates} NG={NG} head_first={head_first}", flush=True)
    d = lambda x: None if x is None else x.to(device)
    hf = lambda x: None if x is None else (x.transpose(1, 2).contiguous() if head_first else x)
    dh, dh0 = chunk_bwd_dh(d(hf(q)), d(hf(k)), d(hf(v)), d(hf(gates_c["g"])), d(hf(gates_c["gk"])),
                           d(hf(gates_c["gv"])), d(hf(do)), d(h0), d(dht), scale, head_first=head_first,
                           chunk_size=64, states_in_fp32=True)
    torch.cuda.synchronize()
    rep = lambda x: None if x is None else x.repeat_interleave(NG, dim=2)
    ref_dh, ref_dh0 = chunked.chunk_bwd_dh(q, rep(gates_c["g"]), rep(gates_c["gk"]), do, dht, scale,
                                           gv=rep(gates_c["gv"]))
    if head_first:
        dh = dh.transpose(1, 2)
    assert tuple(dh.shape) == (B, -(-T // 64), HQ, K, V) and tuple(dh0.shape) == (B, H, K, V)
    assert_close("dh", ref_dh, dh, 5e-3)
    assert_close("dh0", ref_dh0.reshape(B, H, NG, K, V).sum(2), dh0, 5e-3)
