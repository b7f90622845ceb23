"""``chunk_fwd_h`` for per-key log-gates (``fla/ops/common/chunk_h.py:282-335``),
served by ``fla_chunk_gla_fwd_h``."""
from typing import Optional, Tuple

import torch

from ... import _backend as be
from ...utils import prepare_chunk_offsets

BT = 64


def chunk_fwd_h(
    k: torch.Tensor,
    v: torch.Tensor,
    g: Optional[torch.Tensor],
    gk: Optional[torch.Tensor],
    gv: Optional[torch.Tensor],
    h0: Optional[torch.Tensor],
    output_final_state: bool,
    offsets: Optional[torch.Tensor] = None,
    indices: Optional[torch.Tensor] = None,
    head_first: bool = True,
    chunk_size: int = 64,
    states_in_fp32: bool = False,
    *,
    gates_are_cumsum: bool = True,
    fragment_layout: bool = False,
    transposed_fragments: bool = False,
    chunk_offsets: Optional[torch.Tensor] = None,
    store_states: bool = True,
) -> Tuple[Optional[torch.Tensor], Optional[torch.Tensor]]:
    """Per-chunk states ``h`` ``[B,NT,H,K,V]`` (the state entering each chunk)
    and the final state.  ``gk`` is the chunk-local cumsum of the log-gates, as
    in the reference, unless ``gates_are_cumsum=False`` (raw gates; the prefix
    sum is formed in the kernel).  ``fragment_layout=True`` stores ``h`` in the
    MFMA-fragment order only ``fla_chunk_gla_fwd_o`` understands."""
    if g is not None or gv is not None:
        raise NotImplementedError("fla_amd chunk_fwd_h: only per-key gates (gk) are covered")
    if gk is None:
        raise NotImplementedError("fla_amd chunk_fwd_h: gk is required")
    if head_first:
        raise NotImplementedError("fla_amd chunk_fwd_h: seq-first layout only (transpose at the operator boundary)")
    if chunk_size != BT:
        raise NotImplementedError("fla_amd chunk_fwd_h: chunk size is fixed to 64")
    be.require_gpu(k, v, gk)
    B, T, H, K = k.shape
    V = v.shape[-1]
    if offsets is None:
        N, NT = B, -(-T // BT)
    else:
        if chunk_offsets is None:
            chunk_offsets = prepare_chunk_offsets(offsets, BT, device=k.device)
        N = len(offsets) - 1
        NT = int(indices.shape[0]) if indices is not None else int(prepare_chunk_offsets(offsets, BT)[-1])
        offsets = offsets.to(torch.int64).contiguous()
    h_dtype = torch.float32 if states_in_fp32 else k.dtype
    if fragment_layout and states_in_fp32:
        raise ValueError("fragment-layout states are 16-bit")
    h = k.new_empty(B, NT, H, K, V, dtype=h_dtype) if store_states else None
    ht = k.new_empty(N, H, K, V, dtype=torch.float32) if output_final_state else None
    if h0 is not None:
        h0 = (h0 if h0.dtype == torch.float32 else h0.float()).contiguous()
    if gates_are_cumsum and gk.dtype != torch.float32:
        gk = gk.float()
    be.check(be.lib().fla_chunk_gla_fwd_h(
        be.ptr(k), be.ptr(v), be.ptr(gk), int(gates_are_cumsum), be.ptr(h0), be.ptr(h), be.ptr(ht),
        be.ptr(offsets), be.ptr(chunk_offsets), be.dt(k), be.dt(gk), be._DTYPES[h_dtype],
        (be.FLA_H_FRAGMENT_T if transposed_fragments else be.FLA_H_FRAGMENT) if fragment_layout
        else be.FLA_H_ROW_MAJOR,
        B, T, H, K, V, N, be.stream_of(k)), "fla_chunk_gla_fwd_h")
    return h, ht
