"""GPU: the allocation-free whole-sequence cumulative sum (``fla_chunk_global_cumsum_static``, scratch in a
static device array) against ``fla_chunk_global_cumsum`` (scratch in a caller workspace), both called
through the C ABI on the same inputs.  Same kernels, so the results must be bit-identical; two calls in a
row share the static array, the second on a smaller input."""
import ctypes

import pytest
import torch

pytestmark = pytest.mark.gpu

CAP = 4 * 1024 * 1024   # FLA_STATIC_SCRATCH_FLOATS


def _both(be, s, out_dtype, chunk_size, reverse, offsets=None, indices=None):
    lib = be.lib()
    B, T, H = s.shape[:3]
    S = s.shape[3] if s.dim() == 4 else 1
    NT = 0 if indices is None else indices.shape[0]
    tail = (be.dt(s), be._DTYPES[out_dtype], B, T, H, S, chunk_size, int(reverse), be.ptr(offsets), be.ptr(indices), NT,
            be.stream_of(s))
    ref = torch.full(s.shape, float("nan"), dtype=out_dtype, device=s.device)
    ws = torch.empty(s.shape, dtype=torch.float32, device=s.device)
    be.check(lib.fla_chunk_global_cumsum(be.ptr(s), be.ptr(ws), be.ptr(ref), *tail), "fla_chunk_global_cumsum")
    out = torch.full(s.shape, float("nan"), dtype=out_dtype, device=s.device)
    be.check(lib.fla_chunk_global_cumsum_static(be.ptr(s), be.ptr(out), *tail), "fla_chunk_global_cumsum_static")
    torch.cuda.synchronize()
    return ref, out


@pytest.mark.parametrize("reverse", [False, True])
def test_static_scratch_matches_workspace_entry(device, reverse):
    from fla_amd import _backend as be
    gen = torch.Generator().manual_seed(3)
    # first call: a large input (3/4 of the scratch array); second call: a smaller one on the same array
    for shape, dtype in (((2, 6144, 4, 64), torch.float32), ((1, 300, 3, 20), torch.bfloat16), ((2, 1, 5), torch.float32)):
        s = torch.randn(*shape, generator=gen).to(dtype).to(device)
        print(f"static-scratch cumsum {shape} {dtype} reverse={reverse}", flush=True)
        ref, out = _both(be, s, dtype, 128, reverse)
        assert torch.isfinite(out.float()).all()
        assert torch.equal(ref, out)
        x = s.double()
        exact = x.flip(1).cumsum(1).flip(1) if reverse else x.cumsum(1)
        err = ((exact - out.double()).norm() / exact.norm()).item()
        assert err < (1e-5 if dtype == torch.float32 else 4e-3), err


def test_static_scratch_packed_batch(device):
    from fla_amd import _backend as be
    from fla_amd.utils import VarlenPlan
    gen = torch.Generator().manual_seed(4)
    offs = torch.tensor([0, 5, 5, 400, 1000], dtype=torch.int64, device=device)
    plan = VarlenPlan(offs, 64)
    s = torch.randn(1, 1000, 3, 8, generator=gen).to(device)
    print("static-scratch cumsum, packed batch", flush=True)
    ref, out = _both(be, s, torch.float32, 64, False, plan.offsets, plan.indices)
    assert torch.equal(ref, out)


def test_static_scratch_rejects_oversize(device):
    from fla_amd import _backend as be
    lib = be.lib()
    s = torch.zeros(16, device=device)
    p = be.ptr(s)
    st = be.stream_of(s)
    # one element more than the array holds: refused before anything is launched
    assert lib.fla_chunk_global_cumsum_static(p, p, 0, 0, 1, CAP // 64 + 1, 8, 8, 64, 0, None, None, 0, st) == -4
    assert lib.fla_chunk_global_cumsum_static(p, p, 0, 0, 1 << 40, 1 << 40, 1 << 40, 1, 64, 0, None, None, 0, st) == -4
    with pytest.raises(RuntimeError, match="static scratch"):
        be.check(-4, "fla_chunk_global_cumsum_static")
    torch.cuda.synchronize()
