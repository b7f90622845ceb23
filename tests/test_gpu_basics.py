"""GPU: MFMA fragment self-test, chunk_local_cumsum and chunk bookkeeping on device."""
import ctypes

import pytest
import torch

from helpers import assert_close, random_offsets

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("mode", [0, 1, 2])
def test_mfma_fragment_layout(device, mode):
    from fla_amd import _backend as be
    torch.manual_seed(0)
    M, N, Kd = 64, 96, 128
    A = torch.randn(M, Kd, device=device).bfloat16()
    B = torch.randn(N, Kd, device=device).bfloat16()
    C = torch.full((M, N), float('nan'), device=device)
    print(f"selftest mode={mode}", flush=True)
    be.check(be.lib().fla_selftest_mfma(be.ptr(A), be.ptr(B), be.ptr(C), M, N, Kd, mode, be.stream_of(A)), "selftest")
    torch.cuda.synchronize()
    ref = A.float() @ B.float().t()
    assert_close(f"mfma mode {mode}", ref, C, 1e-5)


@pytest.mark.parametrize("nt,share", [(1, 1), (3, 2), (4, 4)])
def test_stream_tiles_probe_reads_every_word_once(device, nt, share):
    """The feed-rate probe bench.py times: each workgroup must have read exactly the rows of its (sequence, head) in
    every tensor - its XOR over them is compared with numpy's."""
    import numpy as np
    from fla_amd import _backend as be
    B, T, H = 2, 192, 3
    gen = torch.Generator().manual_seed(5)
    x = torch.randint(-2**31, 2**31 - 1, (nt, B, T, H, 64), dtype=torch.int32, generator=gen)
    xd = x.to(device)
    sink = torch.zeros(B * H * share, dtype=torch.int32, device=device)
    print(f"stream tiles nt={nt} share={share}", flush=True)
    be.check(be.lib().fla_selftest_stream_tiles(be.ptr(xd), B * T * H * 256, nt, be.ptr(sink), B, T, H, share,
                                                be.stream_of(xd)), "stream_tiles")
    torch.cuda.synchronize()
    ref = np.bitwise_xor.reduce(x.numpy().view(np.uint32).transpose(1, 3, 0, 2, 4).reshape(B * H, -1), axis=1)
    got = sink.cpu().numpy().view(np.uint32).reshape(B * H, share)
    for s_ in range(share):
        assert (got[:, s_] == ref).all()


@pytest.mark.parametrize("shape", [(2, 300, 4, 64), (1, 150, 3, 100), (2, 1024, 2, 0), (3, 77, 5, 0), (1, 64, 2, 6)])
@pytest.mark.parametrize("chunk", [32, 64])
@pytest.mark.parametrize("reverse", [False, True])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_cumsum_fixed(device, shape, chunk, reverse, dtype):
    from fla_amd.ops.utils import chunk_local_cumsum
    from oracle.cumsum import chunk_local_cumsum as ref_cumsum
    B, T, H, S = shape
    gen = torch.Generator().manual_seed(1)
    g = torch.randn((B, T, H, S) if S else (B, T, H), generator=gen).to(dtype)
    print(f"cumsum {shape} chunk={chunk} reverse={reverse} {dtype}", flush=True)
    out = chunk_local_cumsum(g.to(device), chunk, reverse=reverse, head_first=False)
    assert out.dtype == torch.float32
    ref = ref_cumsum(g, chunk, reverse=reverse)
    torch.testing.assert_close(out.cpu(), ref, rtol=1e-5, atol=1e-5)
    # head-first entry point
    out_hf = chunk_local_cumsum(g.transpose(1, 2).contiguous().to(device), chunk, reverse=reverse, head_first=True)
    torch.testing.assert_close(out_hf.transpose(1, 2).cpu(), ref, rtol=1e-5, atol=1e-5)


@pytest.mark.parametrize("T,N", [(64, 2), (300, 4), (1000, 7), (2048, 4)])
@pytest.mark.parametrize("S", [0, 100])
@pytest.mark.parametrize("reverse", [False, True])
def test_cumsum_varlen(device, T, N, S, reverse):
    from fla_amd.ops.utils import chunk_local_cumsum
    from oracle.cumsum import chunk_local_cumsum as ref_cumsum
    gen = torch.Generator().manual_seed(2)
    offs = random_offsets(T, N, gen, min_len=1)
    g = torch.randn((1, T, 3, S) if S else (1, T, 3), generator=gen)
    print(f"cumsum varlen T={T} N={N} S={S} offs={offs.tolist()}", flush=True)
    out = chunk_local_cumsum(g.to(device), 64, reverse=reverse, offsets=offs.to(device), head_first=False)
    ref = ref_cumsum(g, 64, reverse=reverse, offsets=offs.tolist())
    torch.testing.assert_close(out.cpu(), ref, rtol=1e-5, atol=1e-5)


@pytest.mark.parametrize("shape", [(2, 1, 3), (2, 300, 3), (1, 5000, 2, 64), (2, 130, 4, 20), (1, 70, 3, 1)])
@pytest.mark.parametrize("reverse", [False, True])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_global_cumsum(device, shape, reverse, dtype):
    """Whole-sequence cumulative sum against torch.cumsum in fp64 (fp32 accumulation on the device:
    1e-5 relative for fp32 output; one rounding for bf16 output)."""
    from fla_amd.ops.utils import chunk_global_cumsum
    gen = torch.Generator().manual_seed(len(shape) + shape[1])
    s = torch.randn(*shape, generator=gen).to(dtype)
    print(f"global cumsum {shape} reverse={reverse} {dtype}", flush=True)
    out = chunk_global_cumsum(s.to(device), reverse=reverse, head_first=False)
    x = s.double()
    ref = x.flip(1).cumsum(1).flip(1) if reverse else x.cumsum(1)
    assert out.dtype == dtype and out.shape == s.shape
    assert_close("cumsum", ref, out, 1e-5 if dtype == torch.float32 else 4e-3)
    out32 = chunk_global_cumsum(s.transpose(1, 2).contiguous().to(device), dtype=torch.float32, reverse=reverse,
                                head_first=True)
    assert out32.dtype == torch.float32
    assert_close("cumsum head-first fp32", ref.transpose(1, 2), out32, 1e-5)


@pytest.mark.parametrize("reverse", [False, True])
def test_global_cumsum_varlen(device, reverse):
    from fla_amd.ops.utils import chunk_global_cumsum
    gen = torch.Generator().manual_seed(17)
    T, N = 700, 5
    offs = random_offsets(T, N, gen, min_len=1)
    s = torch.randn(1, T, 3, 8, generator=gen)
    print(f"global cumsum varlen offs={offs.tolist()} reverse={reverse}", flush=True)
    out = chunk_global_cumsum(s.to(device), reverse=reverse, offsets=offs.to(device), head_first=False)
    ref = torch.empty_like(s, dtype=torch.float64)
    for a, b in zip(offs[:-1].tolist(), offs[1:].tolist()):
        x = s[:, a:b].double()
        ref[:, a:b] = x.flip(1).cumsum(1).flip(1) if reverse else x.cumsum(1)
    assert_close("cumsum", ref, out, 1e-5)


@pytest.mark.parametrize("reverse", [False, True])
@pytest.mark.parametrize("varlen", [False, True])
def test_local_cumsum_inverse(device, varlen, reverse):
    """Differences of consecutive rows inside every chunk: undoes chunk_local_cumsum (to fp32 rounding) and is
    exact on integers."""
    from fla_amd.ops.utils.cumsum import chunk_local_cumsum, chunk_local_cumsum_inverse
    gen = torch.Generator().manual_seed(23)
    T = 333
    offs = torch.tensor([0, 5, 5, 200, 333], device=device) if varlen else None
    x = torch.randint(-8, 9, (1 if varlen else 2, T, 3, 8), generator=gen).float().to(device)
    print(f"local cumsum inverse varlen={varlen} reverse={reverse}", flush=True)
    G = chunk_local_cumsum(x, 64, reverse=reverse, offsets=offs, head_first=False)
    back = chunk_local_cumsum_inverse(G, 64, reverse=reverse, offsets=offs, head_first=False)
    assert torch.equal(back, x)
    y = torch.randn(2, T, 3, generator=gen).to(device)
    Gy = chunk_local_cumsum(y, 64, reverse=reverse, head_first=False)
    assert_close("round trip", y, chunk_local_cumsum_inverse(Gy, 64, reverse=reverse, head_first=False), 1e-5)
    Gh = chunk_local_cumsum(y.transpose(1, 2).contiguous(), 64, reverse=reverse, head_first=True)
    assert torch.equal(chunk_local_cumsum_inverse(Gh, 64, reverse=reverse, head_first=True).transpose(1, 2),
                       chunk_local_cumsum_inverse(Gy, 64, reverse=reverse, head_first=False))


def _config2_offsets():
    """The packed workload's boundaries: 12 lengths drawn uniformly in [256, 6000], rescaled to sum to 32768."""
    gen = torch.Generator().manual_seed(0)
    lens = torch.randint(256, 6001, (12,), generator=gen).double()
    lens = (lens / lens.sum() * 32768).round().long()
    lens[-1] += 32768 - lens.sum()
    return torch.cat([torch.zeros(1, dtype=torch.long), lens.cumsum(0)])


@pytest.mark.parametrize("bt", [16, 64])
def test_varlen_plan_device_tables_bit_exact(device, bt):
    """The chunk tables a packed launch reads on the device (indices, chunk_offsets, seq_order) against the
    oracle's, bit for bit, together with the reference-held known answer."""
    import json
    import os
    import numpy as np
    from fla_amd.utils import VarlenPlan
    from oracle import bookkeeping
    with open(os.path.join(os.path.dirname(__file__), "golden", "chunk_indices_known_answer.json")) as f:
        ka = json.load(f)
    cases = [_config2_offsets().tolist(), ka["offsets"], [0, 0], [0, 1], [0, 63, 64, 65, 1000], [0, 5, 5, 5, 700]]
    for offs in cases:
        print(f"varlen plan bt={bt} offsets={offs}", flush=True)
        plan = VarlenPlan(torch.tensor(offs, dtype=torch.int64, device=device), bt)
        assert plan.indices.is_cuda and plan.chunk_offsets.is_cuda and plan.seq_order.is_cuda
        assert plan.indices.dtype == torch.int64 and plan.chunk_offsets.dtype == torch.int64
        ref_idx = bookkeeping.prepare_chunk_indices(offs, bt)
        assert np.array_equal(plan.indices.cpu().numpy().reshape(-1, 2), ref_idx)
        assert np.array_equal(plan.chunk_offsets.cpu().numpy(), bookkeeping.prepare_chunk_offsets(offs, bt))
        assert plan.NT == ref_idx.shape[0] and plan.N == len(offs) - 1
        lens = np.diff(np.asarray(offs))
        order = plan.seq_order.cpu().numpy()
        assert sorted(order.tolist()) == list(range(len(lens)))            # a permutation of the sequence ids,
        assert (np.diff(lens[order]) <= 0).all()                           # longest first
    plan = VarlenPlan(torch.tensor(ka["offsets"], dtype=torch.int64, device=device), ka["chunk_size"])
    assert plan.indices.cpu().tolist() == ka["indices"]
