"""ctypes binding of libnatsl.so (the C ABI declared in include/natsl.h).

There is no CPU fallback: if the library has not been built the import of any operator fails
with an explicit error.
"""
from __future__ import annotations

import ctypes
import os
from ctypes import c_char_p, c_float, c_int, c_int64, c_longlong, c_size_t, c_void_p

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "csrc", "libnatsl.so")

F32, BF16 = 0, 1
DECAY_NON_LINEAR, QK_L2NORM, INTRA_CHUNK, QUERY_ONLY = 1, 2, 4, 8

_lib = None

_SIGNATURES = {
    "natsl_version": (c_int, []),
    "natsl_last_error": (c_char_p, []),
    "natsl_mean_pool": (c_int, [c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int, c_void_p, c_int, c_int, c_void_p]),
    "natsl_hard_select": (c_int, [c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int, c_void_p, c_int, c_int, c_void_p]),
    "natsl_route": (c_int, [c_void_p, c_int, c_int, c_int, c_int, c_int, c_int, c_void_p, c_void_p, c_void_p, c_void_p,
                            c_void_p, c_void_p, c_void_p, c_int, c_int, c_void_p]),
    "natsl_softmax_sparse_fwd": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_void_p, c_void_p,
                                         c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_float, c_int, c_int,
                                         c_void_p, c_int, c_int, c_void_p]),
    "natsl_softmax_sparse_fwd_per_tile": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_void_p, c_void_p,
                                         c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_float, c_int, c_int,
                                         c_void_p, c_int, c_int, c_void_p]),
    "natsl_softmax_fwd_variant": (c_int, [c_int, c_int, c_int, c_int, c_int, c_int]),
    "natsl_softmax_bwd_workspace_bytes": (c_size_t, [c_int, c_int, c_int]),
    "natsl_softmax_sparse_bwd": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,
                                         c_void_p, c_void_p, c_int, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int, c_int,
                                         c_int, c_int, c_int, c_float, c_int, c_int, c_void_p, c_size_t, c_void_p, c_int, c_int, c_int,
                                         c_void_p]),
    "natsl_linear_workspace_bytes": (c_size_t, [c_int64, c_int]),
    "natsl_gdn_chunk_fwd": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,
                                    c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_float, c_int, c_void_p,
                                    c_size_t, c_int, c_void_p, c_int, c_int, c_void_p]),
    "natsl_mamba_chunk_fwd": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,
                                      c_void_p, c_void_p, c_int,
                                      c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_float, c_int, c_void_p, c_size_t,
                                      c_int, c_void_p, c_int, c_int, c_void_p]),
    "natsl_linear_chunk_bwd": (c_int, [c_int] + [c_void_p] * 9 + [c_int] + [c_void_p] * 12 + [c_int] * 8 + [c_float, c_int, c_int, c_void_p, c_int, c_int, c_void_p]),
    "natsl_norm_gate_bwd_workspace_bytes": (c_size_t, [c_int64, c_int]),
    "natsl_norm_gate_bwd": (c_int, [c_void_p] * 14 + [c_size_t, c_int64, c_int, c_int, c_float, c_int, c_void_p]),
    "natsl_row_norm_bwd_workspace_bytes": (c_size_t, [c_int64, c_int]),
    "natsl_row_norm_bwd": (c_int, [c_void_p] * 6 + [c_size_t, c_int64, c_int, c_float, c_int, c_int, c_int, c_void_p]),
    "natsl_short_conv_fwd": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int, c_int,
                                     c_int, c_int, c_void_p]),
    "natsl_short_conv_bwd_workspace_bytes": (c_size_t, [c_int, c_int, c_int, c_int]),
    "natsl_short_conv_bwd": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_size_t,
                                     c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_void_p]),
    "natsl_row_norm_fwd": (c_int, [c_void_p, c_void_p, c_void_p, c_int64, c_int, c_float, c_int, c_int, c_int, c_void_p]),
    "natsl_norm_gate_fwd": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int64, c_int, c_int,
                                    c_float, c_int, c_void_p]),
    "natsl_gdn_recurrent_fwd": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,
                                        c_void_p, c_void_p, c_int, c_void_p, c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_int,
                                        c_float, c_int, c_int, c_void_p]),
    "natsl_mamba_recurrent_fwd": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,
                                          c_void_p, c_int, c_void_p, c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_int,
                                          c_float, c_int, c_int, c_void_p]),
    "natsl_attn_masked_workspace_bytes": (c_size_t, [c_int, c_int, c_int, c_int, c_int]),
    "natsl_attn_masked_fwd": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int, c_int,
                                      c_int, c_int, c_float, c_int, c_void_p, c_size_t, c_int64, c_int64, c_void_p]),
    "natsl_attn_masked_static_scratch_bytes": (c_size_t, []),
    "natsl_attn_masked_fwd_static": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int, c_int,
                                             c_int, c_int, c_float, c_int, c_void_p]),
    "natsl_kv_compact": (c_int, [c_void_p, c_void_p, c_longlong, c_int, c_void_p, c_void_p, c_longlong, c_void_p, c_int, c_void_p,
                                 c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_void_p]),
}


class NatslError(RuntimeError):
    pass


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise NatslError(
                f"{LIB_PATH} is missing: build it with `python -m neuralattentionsearchlinear_amd._build` "
                "(there is no CPU fallback for the NAtS-L hot path)")
        L = ctypes.CDLL(LIB_PATH)
        for name, (res, args) in _SIGNATURES.items():
            if hasattr(L, name):
                fn = getattr(L, name)
                fn.restype, fn.argtypes = res, args
        _lib = L
    return _lib


def exported_symbols():
    return list(_SIGNATURES)


def check(rc: int, what: str):
    if rc == 0:
        return
    msg = lib().natsl_last_error().decode()
    if rc == -2:
        raise NotImplementedError(f"{what}: {msg}")
    if rc == -1:
        raise ValueError(f"{what}: {msg}")
    raise NatslError(f"{what} failed ({rc}): {msg}")


def dtype_code(t: torch.dtype) -> int:
    if t == torch.bfloat16:
        return BF16
    if t == torch.float32:
        return F32
    raise NotImplementedError(f"dtype {t} is not supported by the HIP path (bf16 or fp32)")


def ptr(t):
    return None if t is None else c_void_p(t.data_ptr())


def stream_ptr(device=None):
    return c_void_p(torch.cuda.current_stream(device).cuda_stream)
