"""Boundary helpers mirroring ``fla/utils.py``: ``contiguous`` and the autocast
shims (``fla/utils.py:10-21,88-93``), plus the host-side chunk bookkeeping.

The reference caches bookkeeping results keyed on ``data_ptr``
(``fla/utils.py:24-63``), which goes stale when a buffer is reused; here the
``offsets`` values themselves form the key.
"""
import ctypes
import functools
import weakref
from typing import Optional, Tuple

import torch

from . import _backend as be


def contiguous(fn):
    """Make every tensor argument after the first (``ctx``) contiguous."""
    @functools.wraps(fn)
    def wrapper(ctx, *args, **kwargs):
        return fn(ctx,
                  *(a.contiguous() if isinstance(a, torch.Tensor) else a for a in args),
                  **{k: (v.contiguous() if isinstance(v, torch.Tensor) else v) for k, v in kwargs.items()})
    return wrapper


autocast_custom_fwd = functools.partial(torch.amp.custom_fwd, device_type="cuda")
autocast_custom_bwd = functools.partial(torch.amp.custom_bwd, device_type="cuda")


# Host copies of device-resident offsets, keyed by tensor identity: a model passes the same
# cu_seqlens tensor to every layer, and reading it back costs a device synchronisation.
# An entry is valid only for the very same, unmodified tensor object.
_HOST_OFFSETS_CACHE = {}


def _host_offsets(offsets) -> Tuple[int, ...]:
    if not isinstance(offsets, torch.Tensor):
        return tuple(int(x) for x in offsets)
    key = id(offsets)
    hit = _HOST_OFFSETS_CACHE.get(key)
    if hit is not None:
        ref, version, host = hit
        if ref() is offsets and version == offsets._version:
            return host
    host = tuple(int(x) for x in offsets.detach().cpu().tolist())
    if len(_HOST_OFFSETS_CACHE) > 256:
        _HOST_OFFSETS_CACHE.clear()
    _HOST_OFFSETS_CACHE[key] = (weakref.ref(offsets), offsets._version, host)
    return host


@functools.lru_cache(maxsize=64)
def _chunk_tables(offs: Tuple[int, ...], chunk_size: int):
    n = len(offs) - 1
    arr = (ctypes.c_int64 * (n + 1))(*offs)
    nt = be.lib().fla_count_chunks(arr, n, chunk_size)
    if nt < 0:
        raise ValueError("offsets must be non-decreasing int64 positions")
    indices = torch.empty(nt, 2, dtype=torch.int64)
    chunk_offsets = torch.empty(n + 1, dtype=torch.int64)
    be.check(be.lib().fla_prepare_chunk_indices(arr, n, chunk_size,
                                                ctypes.c_void_p(indices.data_ptr()),
                                                ctypes.c_void_p(chunk_offsets.data_ptr())),
             "fla_prepare_chunk_indices")
    return indices, chunk_offsets


def prepare_chunk_indices(offsets, chunk_size: int, device=None) -> torch.Tensor:
    """int64 ``[NT, 2]`` rows (sequence, chunk in sequence); the reference's
    ``prepare_varlen_inputs`` (``fla/ops/gla/chunk.py:1323-1330``)."""
    idx, _ = _chunk_tables(_host_offsets(offsets), int(chunk_size))
    if device is None and isinstance(offsets, torch.Tensor):
        device = offsets.device
    return idx.to(device) if device is not None else idx.clone()


def prepare_chunk_offsets(offsets, chunk_size: int, device=None) -> torch.Tensor:
    """int64 ``[N+1]`` exclusive prefix sum of per-sequence chunk counts
    (``fla/ops/common/chunk_h.py:274-279``)."""
    _, co = _chunk_tables(_host_offsets(offsets), int(chunk_size))
    if device is None and isinstance(offsets, torch.Tensor):
        device = offsets.device
    return co.to(device) if device is not None else co.clone()


class VarlenPlan:
    """Everything the kernels need to address a packed batch.  Plans are cached per offsets
    tensor (same object, unmodified), so the layers of a model that share one ``cu_seqlens``
    build the device tables once."""

    _cache = {}

    def __new__(cls, offsets: torch.Tensor, chunk_size: int):
        key = (id(offsets), int(chunk_size))
        hit = cls._cache.get(key)
        if hit is not None:
            ref, version, plan = hit
            if ref() is offsets and version == offsets._version:
                return plan
        plan = super().__new__(cls)
        plan._build(offsets, chunk_size)
        if len(cls._cache) > 256:
            cls._cache.clear()
        cls._cache[key] = (weakref.ref(offsets), offsets._version, plan)
        return plan

    def _build(self, offsets: torch.Tensor, chunk_size: int):
        host = _host_offsets(offsets)
        idx, co = _chunk_tables(host, int(chunk_size))
        dev = offsets.device
        self.offsets = offsets.to(torch.int64).contiguous()
        self.indices = idx.to(dev, non_blocking=True)
        self.chunk_offsets = co.to(dev, non_blocking=True)
        self.N = len(host) - 1
        self.NT = idx.shape[0]
        # sequence ids, longest first: the order in which the serial scan kernels start sequences
        lens = [host[i + 1] - host[i] for i in range(self.N)]
        order = sorted(range(self.N), key=lambda i: -lens[i])
        self.seq_order = torch.tensor(order, dtype=torch.int64).to(dev, non_blocking=True)


def resolve_offsets(offsets: Optional[torch.Tensor], cu_seqlens: Optional[torch.Tensor]):
    """``cu_seqlens`` is accepted as a synonym of ``offsets``."""
    if offsets is not None and cu_seqlens is not None:
        raise ValueError("pass either `offsets` or `cu_seqlens`, not both")
    return offsets if offsets is not None else cu_seqlens


def check_varlen_args(q, offsets, head_first, initial_state):
    """Error behaviour of the reference entry points
    (``fla/ops/gla/chunk.py:1483-1491`` and the identical blocks elsewhere)."""
    if offsets is not None:
        if q.shape[0] != 1:
            raise ValueError(f"The batch size is expected to be 1 rather than {q.shape[0]} when using `offsets`."
                             f"Please flatten variable-length inputs before processing.")
        if head_first:
            raise RuntimeError("Sequences with variable lengths are not supported for head-first mode")
        if initial_state is not None and initial_state.shape[0] != len(offsets) - 1:
            raise ValueError(f"The number of initial states is expected to be equal to the number of input sequences, "
                             f"i.e., {len(offsets) - 1} rather than {initial_state.shape[0]}.")


def empty_batch_result(q, v, offsets, initial_state, output_final_state):
    """What a chunk operator returns for a batch without a single token (zero-size tensors have no
    device address to hand to a kernel): an empty output and the initial states as final states,
    through ``clone`` so that the gradient of the final states reaches the initial ones."""
    o = torch.empty_like(v)
    ht = None
    if output_final_state:
        if initial_state is not None:
            ht = initial_state.float().clone()
        else:
            N = q.shape[0] if offsets is None else len(offsets) - 1
            H = q.shape[2] if q.dim() == 4 else 1
            ht = q.new_zeros(N, H, q.shape[-1], v.shape[-1], dtype=torch.float32)
    return o, ht
