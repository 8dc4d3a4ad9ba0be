"""Softmax branch entry (host-side mirror of parallel_attn_nats_fwd, src/nats/ops/attns/attns.py:1421-1531)."""
from __future__ import annotations

from typing import Optional

import torch

from . import _capi
from .nats_util import PackedSeqs, _seq_args, pack_sequences


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


def parallel_attn_nats_bwd(
        q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, o: torch.Tensor,
        nats_block_types: torch.Tensor, nats_block_indices: torch.Tensor, n_nats_blocks: torch.Tensor,
        g_cumsum: Optional[torch.Tensor], lse: torch.Tensor, do: torch.Tensor, scale: float = None,
        NAtS_block_size: int = 64, OFFSET_ATTN: int = 0, compute_incomplete_chunk_scores: bool = False,
        compute_dnats_for_invalid_blocks_attn: bool = False, sliding_window_size: Optional[int] = None,
        cu_seqlens=None, cu_seqlens_nats=None, is_causal: bool = True, chunk_indices_attn_nats=None,
        seqs: Optional[PackedSeqs] = None):
    """Backward of the softmax branch (host-side mirror of parallel_attn_nats_bwd, src/nats/ops/attns/attns.py:1562-1759)
    -> (dq [B,T,HQ,K], dk [B,T,H,K], dv [B,T,H,V], None, dnats [B,TNAtS,HNAtS]).

    dnats holds, per block typed attention, the summed score gradient of later blocks' queries on its keys (the
    straight-through gradient of the selector, attns.py:946-961); the other blocks get 0, or, with
    compute_dnats_for_invalid_blocks_attn, what their keys would contribute if they were visible (probabilities against
    the queries' lse, clamped to 1: attns.py:1318-1325).  Packed sequences: cu_seqlens (and cu_seqlens_nats), or the table
    `seqs` built from them; n_nats_blocks is then [n_seqs,HN,2].  g_cumsum and sliding windows are not built."""
    if g_cumsum is not None or sliding_window_size is not None or not is_causal or OFFSET_ATTN != 0:
        raise NotImplementedError("only the causal backward without g_cumsum / sliding window is built")
    if seqs is None and cu_seqlens is not None:
        seqs = pack_sequences(cu_seqlens, cu_seqlens_nats, NAtS_block_size, q.device)
    if seqs is not None and q.shape[0] != 1:
        raise ValueError("batch size must be 1 when cu_seqlens are provided")
    if scale is None:
        scale = k.shape[-1] ** -0.5
    q, k, v, o, do = (t.contiguous() for t in (q, k, v, o, do))
    if not (q.dtype == k.dtype == v.dtype == o.dtype == do.dtype):
        raise ValueError("q, k, v, o, do must share a dtype")
    ty = nats_block_types.contiguous()
    B, T, HQ, K = q.shape
    H, V = k.shape[2], v.shape[-1]
    TN, HN = ty.shape[1], ty.shape[2]
    dq, dk, dv = torch.empty_like(q), torch.empty_like(k), torch.empty_like(v)
    dnats = torch.zeros(B, TN, HQ, dtype=torch.float32, device=q.device)
    L = _capi.lib()
    sp, ns, tot = _seq_args(seqs, seqs.total_qtiles if seqs is not None else 0)
    ws_bytes = L.natsl_softmax_bwd_workspace_bytes(B, T, HQ)
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device=q.device)
    rc = L.natsl_softmax_sparse_bwd(
        _capi.ptr(q), _capi.ptr(k), _capi.ptr(v), _capi.ptr(o), _capi.ptr(lse.contiguous()), _capi.ptr(do), _capi.ptr(dq),
        _capi.ptr(dk), _capi.ptr(dv), _capi.ptr(dnats), _capi.ptr(ty), _capi.dtype_code(ty.dtype), _capi.ptr(nats_block_indices),
        _capi.ptr(n_nats_blocks), B, T, HQ, H, HN, K, V, TN, NAtS_block_size, float(scale),
        int(bool(compute_incomplete_chunk_scores)) | (2 if compute_dnats_for_invalid_blocks_attn else 0), _capi.dtype_code(q.dtype),
        _capi.ptr(ws), ws_bytes, sp, ns, tot, seqs.total_chunks if seqs is not None else 0, _capi.stream_ptr(q.device))
    _capi.check(rc, "natsl_softmax_sparse_bwd")
    dnats = dnats.view(B, TN, HN, HQ // HN).sum(-1)          # over the query heads of a selector head (attns.py:1755)
    return dq, dk, dv, None, dnats


class AttentionNAtSFunction(torch.autograd.Function):
    """The softmax branch with its backward (src/nats/ops/attns/attns.py:1762-1831)."""

    @staticmethod
    def forward(ctx, q, k, v, g, nats_block_types, nats_block_indices, n_nats_blocks, scale, cu_seqlens, cu_seqlens_nats,
                NAtS_block_size, sliding_window_size=None, offset_attn=0, compute_incomplete_chunk_scores=True,
                compute_dnats_for_invalid_blocks_attn=False, is_causal=True, store_msk=False):
        if g is not None:
            raise NotImplementedError("use_g_for_attn is disabled in every reference layer and is not built")
        seqs = pack_sequences(cu_seqlens, cu_seqlens_nats, NAtS_block_size, q.device)
        q, k, v = q.contiguous(), k.contiguous(), v.contiguous()
        o, lse, _ = parallel_attn_nats_fwd(q, k, v, nats_block_types, nats_block_indices, None, scale, NAtS_block_size,
                                           offset_attn=offset_attn, compute_incomplete_chunk_scores=compute_incomplete_chunk_scores,
                                           sliding_window_size=sliding_window_size, is_causal=is_causal, store_msk=store_msk,
                                           n_nats_blocks=n_nats_blocks, seqs=seqs)
        ctx.seqs = seqs
        ctx.save_for_backward(q, k, v, nats_block_types, nats_block_indices, n_nats_blocks, o, lse)
        ctx.scale, ctx.block, ctx.same_block = scale, NAtS_block_size, compute_incomplete_chunk_scores
        ctx.dnats_invalid = compute_dnats_for_invalid_blocks_attn
        ctx.mark_non_differentiable(lse)
        return o, lse

    @staticmethod
    def backward(ctx, do, _dlse):
        q, k, v, ty, idx, nblk, o, lse = ctx.saved_tensors
        dq, dk, dv, _, dnats = parallel_attn_nats_bwd(
            q, k, v, o, ty, idx, nblk, None, lse, do.contiguous(), scale=ctx.scale, NAtS_block_size=ctx.block,
            compute_incomplete_chunk_scores=ctx.same_block, compute_dnats_for_invalid_blocks_attn=ctx.dnats_invalid,
            seqs=ctx.seqs)
        d_types = torch.nn.functional.pad(dnats.unsqueeze(-1), (0, ty.shape[-1] - 1)).to(ty.dtype)   # attns.py:1825-1829
        return (dq, dk, dv, None, d_types) + (None,) * 12


def parallel_nats_attn(q, k, v, g, nats_block_types, nats_block_indices, n_nats_blocks, scale, cu_seqlens=None,
                       cu_seqlens_nats=None, NAtS_block_size: int = 64, sliding_window_size=None, offset_attn: int = 0,
                       compute_incomplete_chunk_scores: bool = False, compute_dnats_for_invalid_blocks_attn: bool = False,
                       head_first: bool = False, is_causal: bool = True, store_msk: bool = False):
    """The differentiable softmax branch (src/nats/ops/attns/attns.py:1834-1929) -> (o [B,T,HQ,V], None)."""
    if head_first:
        raise DeprecationWarning("head_first is deprecated and will be removed in a future version. "
                                 "Please use head_first=False for now instead.")
    if scale is None:
        scale = k.shape[-1] ** -0.5
    if cu_seqlens is not None:
        assert q.shape[0] == 1, "batch size must be 1 when cu_seqlens are provided"
    o, _ = AttentionNAtSFunction.apply(q, k, v, g, nats_block_types, nats_block_indices, n_nats_blocks, scale, cu_seqlens,
                                       cu_seqlens_nats, NAtS_block_size, sliding_window_size, offset_attn,
                                       compute_incomplete_chunk_scores, compute_dnats_for_invalid_blocks_attn, is_causal,
                                       store_msk)
    return o, None
