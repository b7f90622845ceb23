"""CPU oracle for the chunked linear-attention hot path.

TEST INFRASTRUCTURE ONLY.  Nothing in the shipped package imports this
directory: only ``tests/``, ``__graft_entry__.smoke()`` and the
``cpu_baseline`` leg of ``bench.py`` do, and there only as the checker or the
timed CPU baseline, never as a product code path.

Every function is a from-scratch fp32 (or fp64) restatement of the mathematics
of the reference operator it cites; none of it executes reference code.

Pinning status (what independent fact fixes each function; the checks live in
``tests/test_oracle_pins.py``):

* ``bookkeeping.prepare_chunk_indices`` / ``prepare_chunk_offsets`` - integer,
  bit exact; pinned by the known answer the reference holds in a comment
  (``fla/ops/gla/chunk.py:1352-1355``) and by a brute-force enumeration.
* ``cumsum.chunk_local_cumsum`` - pinned by ``torch.cumsum`` applied chunk by
  chunk (how the reference tests it, ``tests/ops/test_cumsum.py:24-36``).
* ``recurrent.naive_recurrent_gla`` - pinned by the K=V=1 scalar closed form,
  the ``gk = 0`` reduction to causal linear attention ``tril(q k^T) v``, a
  brute-force O(T^2) evaluation, and segment chaining.
* ``recurrent.naive_recurrent_gated_delta_rule`` - pinned by ``beta = 0``
  (pure decay), ``g = 0, beta = 1`` with orthonormal keys (exact overwrite),
  the T=1 closed form, and an independent dense "materialise every transition
  matrix" evaluation.
* ``chunked.chunked_gla`` / ``chunked.chunked_gated_delta_rule`` - the chunked algorithms are pinned
  against the two naive recurrences above plus ``torch.linalg.solve_triangular`` for the WY inverse.
* ``chunked.gla_fwd_o_gk`` - pinned by the recurrence: fed with ``chunked_gla``'s scores and states
  (and garbage above the diagonal of the scores) it must reproduce the recurrence's output.
* ``chunked.gla_bwd_dA`` / ``gla_bwd_dv`` / ``chunk_bwd_dv_local`` / ``chunk_bwd_dh`` - pinned by
  ``torch.autograd`` through the fp64 chunk step (the one ``chunked_gla`` is built from), with a zero
  tap on every per-chunk state for ``dh``.
* gradients - ``torch.autograd`` through the fp64 recurrences, with
  ``torch.autograd.gradcheck`` on tiny shapes.
"""
