"""Integer chunk bookkeeping for variable-length (packed) batches.

Restates, with numpy int64 arithmetic, what the reference derives on the host:

* ``prepare_chunk_indices`` - ``prepare_varlen_inputs``
  (``fla/ops/gla/chunk.py:1323-1330``; same construction inline at
  ``fla/ops/gated_delta_rule/chunk.py:204-207``): one row ``(sequence id,
  chunk id inside that sequence)`` per chunk, sequences in order.
* ``prepare_chunk_offsets`` - the exclusive prefix sum of per-sequence chunk
  counts used to address per-chunk states (``fla/ops/common/chunk_h.py:274-279``,
  ``fla/ops/common/chunk_delta_h.py:240-245``).

Test infrastructure only.
"""
import numpy as np


def _lengths(offsets) -> np.ndarray:
    offs = np.asarray(offsets, dtype=np.int64)
    if offs.ndim != 1 or offs.size < 2:
        raise ValueError("offsets must be a 1-d array with at least two entries")
    lens = offs[1:] - offs[:-1]
    if (lens < 0).any():
        raise ValueError("offsets must be non-decreasing")
    return lens


def prepare_chunk_indices(offsets, chunk_size: int) -> np.ndarray:
    """int64 ``[NT, 2]``: for every chunk its (sequence, chunk-in-sequence)."""
    lens = _lengths(offsets)
    rows = []
    for n, length in enumerate(lens.tolist()):
        for c in range(-(-length // chunk_size)):
            rows.append((n, c))
    return np.asarray(rows, dtype=np.int64).reshape(-1, 2)


def prepare_chunk_offsets(offsets, chunk_size: int) -> np.ndarray:
    """int64 ``[N+1]``: exclusive cumsum of ``ceil(T_n / chunk_size)``."""
    lens = _lengths(offsets)
    counts = -(-lens // chunk_size)
    out = np.zeros(lens.size + 1, dtype=np.int64)
    np.cumsum(counts, out=out[1:])
    return out


def gla_chunk_size(T: int) -> int:
    """``min(64, max(16, next_pow2(T)))`` (``fla/ops/gla/chunk.py:1350``)."""
    p = 1
    while p < T:
        p *= 2
    return min(64, max(16, p))
