"""CPU: the C-ABI library loads, exports every symbol include/fla_hip.h declares,
the ctypes signature table covers them all, and the host-side integer
bookkeeping is bit-exact against the oracle.  No device compute."""
import ctypes
import os
import re

import numpy as np
import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared():
    text = open(os.path.join(ROOT, "include", "fla_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(fla_[A-Za-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    from fla_amd import _backend as be
    names = _declared()
    assert len(names) >= 10
    handle = ctypes.CDLL(be.lib_path())
    for n in names:
        assert hasattr(handle, n), f"{n} declared in fla_hip.h but not exported"
    assert sorted(be.SIGNATURES) == names, "ctypes signature table out of sync with fla_hip.h"
    assert be.lib().fla_abi_version() == be.ABI_VERSION


def test_error_strings():
    from fla_amd import _backend as be
    lib = be.lib()
    assert lib.fla_error_string(0) == b"success"
    for code in (-1, -2, -3):
        assert b"fla_hip" in lib.fla_error_string(code)
    with pytest.raises(RuntimeError, match="code -2"):
        be.check(-2, "unit test")


def test_argument_validation_without_device():
    """Invalid arguments are rejected before anything is launched."""
    from fla_amd import _backend as be
    lib = be.lib()
    assert lib.fla_chunk_local_cumsum(None, None, 0, 1, 1, 1, 1, 64, 0, None, None, 0, None) == -1
    buf = torch.zeros(64)
    p = ctypes.c_void_p(buf.data_ptr())
    assert lib.fla_chunk_local_cumsum(p, p, 0, 1, 1, 1, 1, 48, 0, None, None, 0, None) == -1     # not a power of two
    assert lib.fla_chunk_local_cumsum(p, p, 7, 1, 0, 1, 1, 64, 0, None, None, 0, None) == -2     # unknown dtype
    assert lib.fla_chunk_gla_fwd_h(p, p, p, 0, None, p, None, None, None, 1, 0, 1, 1, 1, 64, 1, 100, 64, 1, None) == -2
    assert lib.fla_selftest_mfma(p, p, p, 33, 32, 32, 0, None) == -2
    assert lib.fla_selftest_stream_tiles(p, 1 << 20, 3, p, 1, 100, 1, 1, None) == -2   # T not a multiple of 64
    assert lib.fla_selftest_stream_tiles(p, 1 << 10, 3, p, 1, 64, 1, 1, None) == -1     # tensors overlap
    # the allocation-free cumsum refuses what its static scratch array (4 Mi floats) cannot hold
    assert lib.fla_chunk_global_cumsum_static(p, p, 0, 0, 1, 4 * 1024 * 1024 // 64 + 1, 8, 8, 64, 0, None, None, 0, None) == -4
    assert lib.fla_chunk_global_cumsum_static(None, p, 0, 0, 1, 1, 1, 1, 64, 0, None, None, 0, None) == -1
    # the states-keeping GLA forward that also leaves gated queries and chunk decays: all three outputs or none,
    # at most 256 value columns; its backward divides by the scale
    z = (None,) * 4
    fwd = lambda hT, qg, dec, V: lib.fla_chunk_gla_fwd_fused_kept(p, p, p, p, None, p, None, None, None, hT, qg, dec, None, None, *z,
                                                                  0, 0, 2, 1, 64, 1, 64, V, 1, 1.0, None)
    assert fwd(p, p, None, 64) == -1 and fwd(None, p, p, 64) == -1 and fwd(p, None, None, 64) == -1
    assert fwd(p, p, p, 320) == -2
    bwd = lambda qg, dec, scale: lib.fla_chunk_gla_bwd_kept(p, p, p, p, p, None, p, qg, dec, None, None, p, p, p, p, p, None, None,
                                                            None, None, None, 0, 0, 2, 1, 64, 1, 64, 64, 1, scale, None)
    assert bwd(p, None, 1.0) == -1 and bwd(p, p, 0.0) == -1
    # the per-head-gate backward needs the kept gated queries and a gate-gradient buffer
    sgb = lambda qg, dg: lib.fla_chunk_simple_gla_bwd(p, p, p, p, p, None, p, qg, p, None, None, p, p, p, p, dg, None, None, None, None,
                                                      None, 0, 2, 1, 64, 1, 64, 64, 1, 1.0, None)
    assert sgb(None, p) == -1 and sgb(p, None) == -1
    # the delta rule's chunk-parallel launch: w and Aw together or not at all, K in {64, 128}
    prep = lambda w, Aw, K: lib.fla_gdr_fwd_prep(p, p, None, 0, None, p, w, Aw, None, None, 0, 0, 1, 64, 1, K, None)
    assert prep(p, None, 64) == -1 and prep(None, p, 64) == -1
    assert lib.fla_gdr_fwd_prep(None, p, None, 0, None, p, None, None, None, None, 0, 0, 1, 64, 1, 64, None) == -1
    # its scan: v_new and the states together or not at all, the score tiles only with them
    scan = lambda vn, hT, aqk: lib.fla_chunk_gated_delta_rule_fwd_scan(p, p, p, p, None, None, p, None, vn, hT, aqk, None, None,
                                                                       None, 0, 1, 64, 1, 64, 64, 1, 1.0, None)
    assert scan(p, None, None) == -1 and scan(None, None, p) == -1


@pytest.mark.parametrize("bt", [16, 64])
def test_bookkeeping_bit_exact(bt):
    from fla_amd.utils import prepare_chunk_indices, prepare_chunk_offsets
    from oracle import bookkeeping
    rng = np.random.default_rng(0)
    cases = [[0, 100, 356], [0, 0], [0, 1], [0, 64, 128], [0, 63, 64, 65, 1000]]
    for _ in range(40):
        lens = rng.integers(0, 700, size=rng.integers(1, 12))
        cases.append(np.concatenate([[0], np.cumsum(lens)]).tolist())
    for offs in cases:
        idx = prepare_chunk_indices(torch.tensor(offs), bt)
        co = prepare_chunk_offsets(torch.tensor(offs), bt)
        assert idx.dtype == torch.int64 and co.dtype == torch.int64
        assert np.array_equal(idx.numpy().reshape(-1, 2), bookkeeping.prepare_chunk_indices(offs, bt))
        assert np.array_equal(co.numpy(), bookkeeping.prepare_chunk_offsets(offs, bt))
    import json
    import os
    with open(os.path.join(os.path.dirname(__file__), "golden", "chunk_indices_known_answer.json")) as f:
        ka = json.load(f)   # the reference's stored known answer (fla/ops/gla/chunk.py:1352-1355)
    assert prepare_chunk_indices(torch.tensor(ka["offsets"]), ka["chunk_size"]).tolist() == ka["indices"]


def test_boundary_error_conventions():
    """ValueError / RuntimeError / AssertionError behaviour of the reference entry
    points (fla/ops/gla/chunk.py:1483-1491; gated_delta_rule/fused_recurrent.py:292-301)."""
    from fla_amd.ops.gated_delta_rule import fused_recurrent_gated_delta_rule
    from fla_amd.ops.gla import chunk_gla, fused_recurrent_gla
    q = torch.zeros(2, 8, 2, 64)
    offs = torch.tensor([0, 4, 8])
    for fn, extra in ((chunk_gla, (q,)), (fused_recurrent_gla, (q,)), (fused_recurrent_gated_delta_rule, (q[..., 0], q[..., 0]))):
        with pytest.raises(ValueError, match="batch size"):
            fn(q, q, q, *extra, offsets=offs, head_first=False)
        with pytest.raises(RuntimeError, match="head-first"):
            fn(q[:1], q[:1], q[:1], *[e[:1] for e in extra], offsets=offs, head_first=True)
        with pytest.raises(ValueError, match="initial states"):
            fn(q[:1], q[:1], q[:1], *[e[:1] for e in extra], offsets=offs, head_first=False,
               initial_state=torch.zeros(3, 2, 64, 64))
        with pytest.raises(ValueError, match="either"):
            fn(q[:1], q[:1], q[:1], *[e[:1] for e in extra], offsets=offs, cu_seqlens=offs, head_first=False)
        # CPU tensors never reach a kernel and never fall back
        with pytest.raises(RuntimeError, match="no CPU fallback"):
            fn(q, q, q, *extra, head_first=False)
    with pytest.raises(AssertionError, match="positive"):
        fused_recurrent_gated_delta_rule(q, q, q, q[..., 0], q[..., 0], scale=-1.0, head_first=False)
