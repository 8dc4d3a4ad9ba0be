"""Softmax branch entry (host-side mirror of parallel_attn_nats_fwd, src/nats/ops/attns/attns.py:1421-1531)."""
from __future__ import annotations

from typing import Optional

import torch

from . import _capi
from .nats_util import PackedSeqs, _seq_args


def parallel_attn_nats_fwd(
        q: torch.Tensor, k: torch.Tensor, v: torch.Tensor,
        nats_block_types: torch.Tensor, nats_block_indices: torch.Tensor,
        g_cumsum: Optional[torch.Tensor], scale: float, NAtS_block_size: int,
        offset_attn: int = 0, compute_incomplete_chunk_scores: bool = False,
        chunk_size: int = 128, sliding_window_size: Optional[int] = None,
        cu_seqlens=None, cu_seqlens_nats=None, is_causal: bool = True, store_msk: bool = False,
        n_nats_blocks: Optional[torch.Tensor] = None, seqs: Optional[PackedSeqs] = None):
    """q [B,T,HQ,K], k [B,T,H,K], v [B,T,H,V] bf16 -> (o [B,T,HQ,V], lse fp32 [B,T,HQ] in log2 units, None).

    `chunk_size` (the reference's Triton query tile) has no effect on the result and is ignored.
    n_nats_blocks int32 [B,HN,2] is required (the reference recomputes it inside its index helper).
    """
    if g_cumsum is not None:
        raise NotImplementedError("use_g_for_attn is disabled in every reference layer and is not built")
    if sliding_window_size is not None:
        raise NotImplementedError("attn_sw_size is not used by the reference layers and is not built")
    if not is_causal or store_msk or offset_attn != 0:
        raise NotImplementedError("only the causal forward without mask dump is built")
    if n_nats_blocks is None:
        raise ValueError("n_nats_blocks is required")
    q, k, v = q.contiguous(), k.contiguous(), v.contiguous()
    ty = nats_block_types.contiguous()
    B, T, HQ, K = q.shape
    H, V = k.shape[2], v.shape[-1]
    TN, HN = ty.shape[1], ty.shape[2]
    o = torch.empty(B, T, HQ, V, dtype=v.dtype, device=q.device)
    lse = torch.empty(B, T, HQ, dtype=torch.float32, device=q.device)
    sp, ns, tot = _seq_args(seqs, seqs.total_qtiles if seqs is not None else 0)
    rc = _capi.lib().natsl_softmax_sparse_fwd(
        _capi.ptr(q), _capi.ptr(k), _capi.ptr(v), _capi.ptr(o), _capi.ptr(lse), _capi.ptr(ty), _capi.dtype_code(ty.dtype),
        _capi.ptr(nats_block_indices), _capi.ptr(n_nats_blocks), B, T, HQ, H, HN, K, V, TN, NAtS_block_size, float(scale),
        int(bool(compute_incomplete_chunk_scores)), _capi.dtype_code(q.dtype), sp, ns, tot, _capi.stream_ptr(q.device))
    _capi.check(rc, "natsl_softmax_sparse_fwd")
    return o, lse, None
