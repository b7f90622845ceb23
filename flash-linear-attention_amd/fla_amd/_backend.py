"""ctypes binding of libfla_hip.so (the C ABI declared in include/fla_hip.h).

The shared object is built in-tree by ``flash-linear-attention_amd/build.py``.
There is no fallback: if the library is missing, or an entry point returns a
non-zero code, a RuntimeError is raised.
"""
import ctypes
import os
from ctypes import c_char_p, c_float, c_int, c_int64, c_void_p
from typing import Optional

import torch

_LIB_PATH = os.path.join(os.path.dirname(os.path.abspath(__file__)), "lib", "libfla_hip.so")
_lib = None

FLA_F32, FLA_BF16, FLA_F16 = 0, 1, 2
FLA_H_ROW_MAJOR, FLA_H_FRAGMENT, FLA_H_FRAGMENT_T = 0, 1, 2
ABI_VERSION = 14

_DTYPES = {torch.float32: FLA_F32, torch.bfloat16: FLA_BF16, torch.float16: FLA_F16}

P, I64, I, F = c_void_p, c_int64, c_int, c_float

# name -> (restype, argtypes); mirrors include/fla_hip.h declaration by declaration
SIGNATURES = {
    "fla_abi_version": (c_int, []),
    "fla_error_string": (c_char_p, [c_int]),
    "fla_count_chunks": (c_int64, [P, I64, I64]),
    "fla_prepare_chunk_indices": (c_int, [P, I64, I64, P, P]),
    "fla_chunk_local_cumsum": (c_int, [P, P, I, I64, I64, I64, I64, I64, I, P, P, I64, P]),
    "fla_chunk_local_cumsum_inverse": (c_int, [P, P, I64, I64, I64, I64, I64, I, P, P, I64, P]),
    "fla_chunk_global_cumsum": (c_int, [P, P, P, I, I, I64, I64, I64, I64, I64, I, P, P, I64, P]),
    "fla_chunk_global_cumsum_static": (c_int, [P, P, I, I, I64, I64, I64, I64, I64, I, P, P, I64, P]),
    "fla_fused_recurrent_fwd": (c_int, [P, P, P, P, P, P, P, P, P, P, I, I, I,
                                        I64, I64, I64, I64, I64, I64, F, I, P]),
    "fla_fused_recurrent_bwd": (c_int, [P] * 14 + [I, I, I64, I64, I64, I64, I64, I64, F, I, P]),
    "fla_fused_recurrent_gated_delta_rule_fwd": (c_int, [P, P, P, P, P, P, P, P, P, I, I, I, I,
                                                         I64, I64, I64, I64, I64, I64, F, P]),
    "fla_fused_recurrent_gated_delta_rule_fwd_l2norm": (c_int, [P, P, P, P, P, P, P, P, P, I, I, I, I,
                                                                I64, I64, I64, I64, I64, I64, F, F, P]),
    "fla_chunk_gla_fwd_h": (c_int, [P, P, P, I, P, P, P, P, P, I, I, I, I,
                                    I64, I64, I64, I64, I64, I64, P]),
    "fla_chunk_gla_fwd_o": (c_int, [P, P, P, P, I, P, P, P, P, P, I64, I, I,
                                    I64, I64, I64, I64, I64, F, P]),
    "fla_chunk_gla_fwd_fused": (c_int, [P] * 13 + [I64, I, I, I64, I64, I64, I64, I64, I64, F, P]),
    "fla_chunk_gla_fwd_fused_first_launch": (c_int, [P] * 13 + [I64, I, I, I64, I64, I64, I64, I64, I64, F, P]),
    "fla_chunk_gla_fwd_fused_logits": (c_int, [P] * 13 + [I64, I, I, I64, I64, I64, I64, I64, I64, F, F, I, F, P]),
    "fla_chunk_gla_fwd_fused_states": (c_int, [P] * 14 + [I64, I, I, I64, I64, I64, I64, I64, I64, F, P]),
    "fla_chunk_gla_fwd_fused_kept": (c_int, [P] * 18 + [I64, I, I, I64, I64, I64, I64, I64, I64, F, P]),
    "fla_chunk_simple_gla_fwd_fused": (c_int, [P] * 18 + [I64, I, I64, I64, I64, I64, I64, I64, F, P]),
    "fla_gdr_fwd_wy": (c_int, [P, P, P, P, P, P, P, P, P, P, I64, I, I64, I64, I64, I64, I64, P]),
    "fla_chunk_gated_delta_rule_fwd_h": (c_int, [P, P, P, P, P, P, P, P, P, P, I, I, I,
                                                 I64, I64, I64, I64, I64, I64, P]),
    "fla_chunk_gated_delta_rule_fwd_h_both": (c_int, [P] * 11 + [I, I64, I64, I64, I64, I64, I64, P]),
    "fla_gdr_fwd_prep": (c_int, [P, P, P, I, P, P, P, P, P, P, I64, I, I64, I64, I64, I64, P]),
    "fla_chunk_gated_delta_rule_fwd_scan": (c_int, [P] * 14 + [I, I64, I64, I64, I64, I64, I64, F, P]),
    "fla_chunk_simple_gla_fwd_scan": (c_int, [P] * 10 + [I, I64, I64, I64, I64, I64, I64, F, P]),
    "fla_gdr_fwd_prep_l2norm": (c_int, [P, P, P, I, P, P, P, P, P, I64, I, I64, I64, I64, I64, F, P]),
    "fla_chunk_gated_delta_rule_fwd_scan_l2norm": (c_int, [P] * 12 + [I, I64, I64, I64, I64, I64, I64, F, F, P]),
    "fla_chunk_gated_delta_rule_fwd_onepass": (c_int, [P] * 11 + [I, I64, I64, I64, I64, I64, I64, F, I, F, P]),
    "fla_chunk_fwd_o": (c_int, [P, P, P, P, P, P, P, P, I64, I, I64, I64, I64, I64, I64, F, P]),
    "fla_chunk_gla_bwd": (c_int, [P] * 17 + [I64, I, I, I64, I64, I64, I64, I64, I64, F, P]),
    "fla_chunk_gla_bwd_kept": (c_int, [P] * 21 + [I64, I, I, I64, I64, I64, I64, I64, I64, F, P]),
    "fla_chunk_simple_gla_bwd": (c_int, [P] * 21 + [I64, I, I64, I64, I64, I64, I64, I64, F, P]),
    "fla_chunk_gla_fwd_o_gk": (c_int, [P] * 8 + [I64, I, I, I, I64, I64, I64, I64, I64, F, P]),
    "fla_chunk_gla_bwd_dA": (c_int, [P] * 5 + [I64, I, I64, I64, I64, I64, F, P]),
    "fla_chunk_gla_bwd_dv": (c_int, [P] * 8 + [I64, I, I, I, I64, I64, I64, I64, I64, P]),
    "fla_chunk_bwd_dh": (c_int, [P] * 9 + [I, I, I64, I64, I64, I64, I64, I64, F, P]),
    "fla_states_to_fragments": (c_int, [P, P, I, I, I, I64, I64, I64, P]),
    "fla_chunk_bwd_dv_local": (c_int, [P] * 7 + [I64, I, I64, I64, I64, I64, I64, F, P]),
    "fla_chunk_gated_delta_rule_bwd": (c_int, [P] * 27 + [I64, I, I64, I64, I64, I64, I64, I64, F, P]),
    "fla_chunk_gated_delta_rule_bwd_dhu": (c_int, [P] * 12 + [I, I64, I64, I64, I64, I64, I64, F, P]),
    "fla_chunk_bwd_dqkwg": (c_int, [P] * 15 + [I64, I, I64, I64, I64, I64, I64, F, P]),
    "fla_bwd_prepare_wy_repr": (c_int, [P] * 14 + [I64, I, I64, I64, I64, I64, I64, P]),
    "fla_fwd_recompute_w_u": (c_int, [P] * 9 + [I64, I, I64, I64, I64, I64, I64, P]),
    "fla_fragments_to_states": (c_int, [P, P, I, I, I, I64, I64, I64, P]),
    "fla_l2norm_fwd": (c_int, [P, P, I64, I64, F, I, I, P]),
    "fla_l2norm_bwd": (c_int, [P, P, P, I64, I64, F, I, I, P]),
    "fla_norm_swish_gate_workgroups": (c_int, [I64, I64]),
    "fla_norm_swish_gate_fwd": (c_int, [P, P, P, P, P, P, P, I64, I64, F, I, I, P]),
    "fla_norm_swish_gate_bwd": (c_int, [P] * 11 + [I64, I64, F, I, I, P]),
    "fla_norm_swish_gate_residual_fwd": (c_int, [P, P, P, P, P, I, P, P, I, P, P, I64, I64, F, I, I, P]),
    "fla_norm_swish_gate_residual_bwd": (c_int, [P, P, I] + [P] * 11 + [I64, I64, F, I, I, P]),
    "fla_causal_conv1d_fwd": (c_int, [P, P, P, P, I64, I64, I64, I64, I, I, P]),
    "fla_causal_conv1d_bwd_partials": (c_int, [I64, I64]),
    "fla_causal_conv1d_bwd": (c_int, [P] * 7 + [I64, I64, I64, I64, I, I, P]),
    "fla_causal_conv1d_update": (c_int, [P] * 5 + [I64, I64, I64, I, I, P]),
    "fla_gate_logsigmoid_fwd": (c_int, [P, P, I64, F, I, F, I, I, P]),
    "fla_gate_logsigmoid_bwd": (c_int, [P, P, P, I64, F, I, F, I, I, P]),
    "fla_gdn_gate_workgroups": (c_int, [I64, I64]),
    "fla_gdn_gate_fwd": (c_int, [P, P, P, P, P, P, I64, I64, I, I, P]),
    "fla_gdn_gate_bwd": (c_int, [P] * 9 + [I64, I64, I, I, P]),
    "fla_selftest_mfma": (c_int, [P, P, P, I64, I64, I64, I, P]),
    "fla_selftest_stream_tiles": (c_int, [P, I64, I, P, I64, I64, I64, I, P]),
}


def lib_path() -> str:
    return _LIB_PATH


def lib():
    """The loaded shared object; raises if it has not been built."""
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            raise RuntimeError(
                f"fla_amd: HIP extension not built ({_LIB_PATH} is missing). "
                "Run `python flash-linear-attention_amd/build.py` (needs hipcc); there is no CPU fallback.")
        handle = ctypes.CDLL(_LIB_PATH)
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(handle, name)  # AttributeError if the symbol is missing
            fn.restype = res
            fn.argtypes = args
        if handle.fla_abi_version() != ABI_VERSION:
            raise RuntimeError("fla_amd: libfla_hip.so ABI version mismatch; rebuild it")
        _lib = handle
    return _lib


def check(code: int, what: str) -> None:
    if code != 0:
        msg = lib().fla_error_string(int(code)).decode()
        raise RuntimeError(f"{what} failed with code {code}: {msg}")


def dt(t: torch.Tensor) -> int:
    try:
        return _DTYPES[t.dtype]
    except KeyError:
        raise TypeError(f"fla_amd: unsupported dtype {t.dtype}") from None


def ptr(t: Optional[torch.Tensor]):
    """Device (or host) address of a contiguous tensor, or NULL."""
    if t is None:
        return None
    assert t.is_contiguous(), "fla_amd: tensors crossing the C ABI must be contiguous"
    return c_void_p(t.data_ptr())


def stream_of(t: torch.Tensor):
    """HIP stream handle the kernels are enqueued on: torch's current stream."""
    return c_void_p(torch.cuda.current_stream(t.device).cuda_stream)


def require_gpu(*tensors: torch.Tensor) -> None:
    for t in tensors:
        if t is not None and not t.is_cuda:
            raise RuntimeError("fla_amd: the HIP kernels need tensors on a GPU device; there is no CPU fallback")
