"""Selector and routing on the GPU (host-side mirror of src/nats/ops/nats_util.py and of the
selector statements in src/nats/layers/natsl_attn_gdn.py:47-61,412-420,553-555).

Every function enqueues HIP kernels on the current stream and returns device tensors; none of
them synchronises with the host except `prepare_nats_block_indices`, whose result length is
data dependent (exactly as in the reference).
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Optional

import torch

from . import _capi

CHUNK_SIZE = 64
SOFTMAX_QUERY_TILE = 256


@dataclass
class PackedSeqs:
    """Device table describing packed sequences (cu_seqlens of the reference)."""
    table: torch.Tensor          # int32 [N, 8] rows of natsl_seq_row
    n_seqs: int
    total_chunks: int
    total_qtiles: int
    total_blocks: int
    cu_seqlens: list
    cu_seqlens_nats: list


def pack_sequences(cu_seqlens, cu_seqlens_nats, block: int, device) -> Optional[PackedSeqs]:
    """Build the per-sequence table (one host read of cu_seqlens; the reference's varlen helpers
    do the same at fla prepare_chunk_indices)."""
    if cu_seqlens is None:
        return None
    cu = [int(x) for x in (cu_seqlens.tolist() if torch.is_tensor(cu_seqlens) else cu_seqlens)]
    if cu_seqlens_nats is None:
        cn = [0]
        for a, b in zip(cu[:-1], cu[1:]):
            cn.append(cn[-1] + -(-(b - a) // block))
    else:
        cn = [int(x) for x in (cu_seqlens_nats.tolist() if torch.is_tensor(cu_seqlens_nats) else cu_seqlens_nats)]
    rows, coff, qoff = [], 0, 0
    for i, (a, b) in enumerate(zip(cu[:-1], cu[1:])):
        if b <= a:
            raise ValueError("cu_seqlens must be strictly increasing")
        if cn[i + 1] - cn[i] != -(-(b - a) // block):
            raise ValueError("cu_seqlens_nats does not match cu_seqlens and nats_block_size")
        rows.append([a, b, cn[i], coff, qoff, 0, 0, 0])
        coff += -(-(b - a) // CHUNK_SIZE)
        qoff += -(-(b - a) // SOFTMAX_QUERY_TILE)
    table = torch.tensor(rows, dtype=torch.int32).to(device)
    return PackedSeqs(table, len(rows), coff, qoff, cn[-1], cu, cn)


def _seq_args(seqs: Optional[PackedSeqs], total: int = 0):
    if seqs is None:
        return None, 0, 0
    return _capi.ptr(seqs.table), seqs.n_seqs, total


def _mean_pooling_fwd(x: torch.Tensor, chunk_size: int, seqs: Optional[PackedSeqs]) -> torch.Tensor:
    B, T, H, D = x.shape
    x = x.contiguous()
    nb = seqs.total_blocks if seqs is not None else -(-T // chunk_size)
    out = torch.empty(B, nb, H, D, dtype=x.dtype, device=x.device)
    sp, ns, tot = _seq_args(seqs, nb)
    rc = _capi.lib().natsl_mean_pool(_capi.ptr(x), _capi.ptr(out), B, T, H * D, chunk_size, _capi.dtype_code(x.dtype), sp, ns,
                                     tot, _capi.stream_ptr(x.device))
    _capi.check(rc, "natsl_mean_pool")
    return out


class _MeanPooling(torch.autograd.Function):
    """Block means with their backward: every token of a block receives the block's gradient over the block's length
    (the reference's pooling backward, src/nats/ops/utils/pooling.py:60-100)."""

    @staticmethod
    def forward(ctx, x, chunk_size):
        ctx.chunk, ctx.T = chunk_size, x.shape[1]
        return _mean_pooling_fwd(x, chunk_size, None)

    @staticmethod
    def backward(ctx, dy):
        T, n = ctx.T, ctx.chunk
        nb = dy.shape[1]
        lens = torch.full((nb,), float(n), device=dy.device, dtype=torch.float32)
        lens[-1] = float(T - (nb - 1) * n)
        dx = (dy.float() / lens.view(1, nb, 1, 1)).to(dy.dtype).repeat_interleave(n, dim=1)[:, :T]
        return dx, None


def mean_pooling(x: torch.Tensor, chunk_size: int, cu_seqlens=None, seqs: Optional[PackedSeqs] = None) -> torch.Tensor:
    """x [B,T,H,D] (or [B,T,D]) -> block means [B,ceil(T/chunk),H,D]; replaces fla's mean_pooling
    as used at src/nats/layers/natsl_attn_gdn.py:412-417 (kernel src/nats/ops/utils/pooling.py:26-57)."""
    squeeze = x.dim() == 3
    if squeeze:
        x = x.unsqueeze(-2)
    if cu_seqlens is not None and seqs is None:
        seqs = pack_sequences(cu_seqlens, None, chunk_size, x.device)
    if torch.is_grad_enabled() and x.requires_grad:
        if seqs is not None:
            raise NotImplementedError("the pooling backward is not built for packed sequences")
        out = _MeanPooling.apply(x, chunk_size)
    else:
        out = _mean_pooling_fwd(x, chunk_size, seqs)
    return out.squeeze(-2) if squeeze else out


def hard_select(logits: torch.Tensor, force_last_block: bool = False, seqs: Optional[PackedSeqs] = None):
    """logits [B,TN,HN,2] -> (types [B,TN,HN,2] with values exactly {0,1}, n_nats_blocks int32 [B,HN,2]).

    Forward value of hard_softmax (src/nats/layers/natsl_attn_gdn.py:47-61); with
    force_last_block it also applies `types[:, -1] = 1` and counts the blocks (:553-554)."""
    if logits.shape[-1] != 2:
        raise NotImplementedError("the selector is built for n_ops == 2")
    logits = logits.contiguous()
    B, TN, HN, _ = logits.shape
    types = torch.empty_like(logits)
    n = seqs.n_seqs if seqs is not None else B
    nblk = torch.empty(n, HN, 2, dtype=torch.int32, device=logits.device)
    sp, ns, tot = _seq_args(seqs)
    rc = _capi.lib().natsl_hard_select(_capi.ptr(logits), _capi.ptr(types), _capi.ptr(nblk), B, TN, HN,
                                       _capi.dtype_code(logits.dtype), int(force_last_block), sp, ns, tot,
                                       _capi.stream_ptr(logits.device))
    _capi.check(rc, "natsl_hard_select")
    if torch.is_grad_enabled() and logits.requires_grad:
        # straight-through estimator of the reference (hard value, gradient of the softmax:
        # `y_hard - y_soft.detach() + y_soft`, src/nats/layers/natsl_attn_gdn.py:47-61); the added term is exactly zero
        y_soft = logits.softmax(-1)
        types = types + (y_soft - y_soft.detach())
    return types, nblk


def route(nats_block_types: torch.Tensor, T: int, nats_block_size: int, seqs: Optional[PackedSeqs] = None,
          tables: bool = False) -> dict:
    """nats_block_indices and n_nats_blocks (always) plus, with tables=True, the reference's other
    routing tensors (src/nats/ops/nats_util.py) -- those are not needed by the HIP kernels and exist
    for parity checks."""
    ty = nats_block_types.contiguous()
    B, TN, HN, n_ops = ty.shape
    if n_ops != 2:
        raise NotImplementedError("routing is built for n_ops == 2")
    dev = ty.device
    n = seqs.n_seqs if seqs is not None else B
    idx = torch.empty(B, TN, HN, 2, dtype=torch.int32, device=dev)
    nblk = torch.empty(n, HN, 2, dtype=torch.int32, device=dev)
    out = dict(nats_block_indices=idx, n_nats_blocks=nblk)
    off = ci = sh = ni = None
    if tables:
        off = torch.empty(n * HN + 1, dtype=torch.int64, device=dev)
        ci = torch.empty(n * HN * TN * (nats_block_size // CHUNK_SIZE), 2, dtype=torch.int32, device=dev)
        if seqs is None:
            sh = torch.empty(B, -(-T // CHUNK_SIZE), HN, dtype=torch.int64, device=dev)
            ni = torch.empty(B, -(-T // 128), HN, dtype=torch.int64, device=dev)
    sp, ns, tot = _seq_args(seqs)
    rc = _capi.lib().natsl_route(_capi.ptr(ty), _capi.dtype_code(ty.dtype), B, TN, HN, T, nats_block_size, _capi.ptr(idx),
                                 _capi.ptr(nblk), _capi.ptr(off), _capi.ptr(ci), _capi.ptr(sh), _capi.ptr(ni), sp, ns, tot,
                                 _capi.stream_ptr(dev))
    _capi.check(rc, "natsl_route")
    if tables:
        out.update(linear_chunk_offsets=off, chunk_indices_linear_buffer=ci, starting_h_idx=sh, attn_n_iters=ni)
    return out


def prepare_nats_block_indices(n_nats_blocks: torch.Tensor, nats_block_size: int, chunk_size: int) -> torch.Tensor:
    """Same result as src/nats/ops/nats_util.py:6-32 for n_nats_blocks [..] of ONE op: rows
    (flat_bh, j), j < cdiv(n*block, chunk).  Data-dependent length => one host read."""
    n = (n_nats_blocks.flatten().to(torch.int64) * nats_block_size + chunk_size - 1) // chunk_size
    bh = torch.repeat_interleave(torch.arange(n.numel(), device=n.device), n)
    start = torch.cumsum(n, 0) - n
    j = torch.arange(bh.numel(), device=n.device) - start[bh]
    return torch.stack([bh, j], 1).to(n_nats_blocks.dtype)


def prepare_nats_chunk_offsets(n_nats_blocks: torch.Tensor, nats_block_types: torch.Tensor, nats_block_size: int,
                               chunk_size: int, op_idx: int) -> torch.Tensor:
    """src/nats/ops/nats_util.py:35-64."""
    n = (n_nats_blocks[..., op_idx].flatten().to(torch.int64) * nats_block_size + chunk_size - 1) // chunk_size
    return torch.nn.functional.pad(n, (1, 0)).cumsum(0)
