"""Oracle for the chunk selector and the routing tables (integer / bit-exact part).

TEST INFRASTRUCTURE ONLY -- see oracle/__init__.py.

Pins (what makes a wrong sign / index / transposition fail):
  * hard_select: torch library semantics of softmax-then-first-max on CPU; the
    bf16 tie trap (argmax over the ROUNDED softmax) is covered by an exhaustive
    sweep over near-tie bf16 pairs in tests/test_oracle_routing.py.
  * routing tables: each table is restated twice -- once in the reference's
    vectorised form (sort / compare-and-sum) and once as a plain Python integer
    loop written from the table's meaning -- and the two are compared on random
    masks; the hand-derived known-answer case (attention column [1,0,1,1],
    linear column [0,1,0,1]) and the reference docstring example
    (src/nats/ops/nats_util.py:134, linear blocks [2,5] of 8) are fixed vectors.
"""
from __future__ import annotations

import numpy as np
import torch

OFFSET_ATTN = 0     # src/nats/ops/mixed_ops/mixed_attn_gdn.py:107
OFFSET_LINEAR = 1   # src/nats/ops/mixed_ops/mixed_attn_gdn.py:108
CHUNK = 64          # src/nats/ops/mixed_ops/mixed_attn_gdn.py:16
ATTN_QUERY_TILE = 128  # src/nats/ops/attns/attns.py:1432


def mean_pool(hidden: torch.Tensor, block: int) -> torch.Tensor:
    """Block mean of hidden [B,T,D] -> [B,ceil(T/block),D]; divisor min(block, T-c*block).

    Restates mean_pooling_fwd_kernel, src/nats/ops/utils/pooling.py:26-57 (fp32
    accumulate, round to the input dtype on store).
    """
    B, T, D = hidden.shape
    nb = -(-T // block)
    out = torch.empty(B, nb, D, dtype=hidden.dtype)
    x = hidden.float()
    for c in range(nb):
        lo, hi = c * block, min(T, (c + 1) * block)
        out[:, c] = (x[:, lo:hi].sum(1) / float(hi - lo)).to(hidden.dtype)
    return out


def hard_select(logits: torch.Tensor) -> torch.Tensor:
    """Forward value of hard_softmax, src/nats/layers/natsl_attn_gdn.py:47-61.

    softmax in the logits dtype, first-max index, one-hot, then the
    straight-through expression y_hard - y_soft + y_soft evaluated literally in
    that dtype.
    """
    y_soft = logits.softmax(-1)
    index = y_soft.max(-1, keepdim=True)[1]
    y_hard = torch.zeros_like(logits).scatter_(-1, index, 1.0)
    return y_hard - y_soft + y_soft


def force_last_block(types: torch.Tensor) -> torch.Tensor:
    """nats_op_types[:, -1] = 1, src/nats/layers/natsl_attn_gdn.py:553,582."""
    out = types.clone()
    out[:, -1] = 1
    return out


def block_indices(types: torch.Tensor) -> torch.Tensor:
    """nats_block_indices, src/nats/ops/mixed_ops/mixed_attn_gdn.py:88-97.

    types [B,TN,HN,n_ops] -> int32 same shape: ascending ids of blocks whose
    rounded type is 1, padded with the sentinel TN.
    """
    t = torch.round(types.float())
    TN = t.shape[1]
    ar = torch.arange(TN, dtype=torch.int32).view(1, -1, 1, 1)
    idx = torch.where(t == 1.0, ar, torch.tensor(TN, dtype=torch.int32))
    return idx.sort(1)[0].to(torch.int32)


def block_indices_loop(types: torch.Tensor) -> torch.Tensor:
    """Same table from its meaning, by integer loops (independent restatement)."""
    t = np.rint(types.float().numpy())
    B, TN, HN, NO = t.shape
    out = np.full((B, TN, HN, NO), TN, dtype=np.int32)
    for b in range(B):
        for h in range(HN):
            for o in range(NO):
                j = 0
                for c in range(TN):
                    if t[b, c, h, o] == 1.0:
                        out[b, j, h, o] = c
                        j += 1
    return torch.from_numpy(out)


def n_blocks(types: torch.Tensor) -> torch.Tensor:
    """n_nats_blocks = types.int().sum(1), src/nats/layers/natsl_attn_gdn.py:554."""
    return types.int().sum(1).to(torch.int32)


def _cdiv(a, b):
    return -(-a // b)


def chunk_indices_linear(n_lin: torch.Tensor, block: int, chunk: int = CHUNK) -> torch.Tensor:
    """prepare_nats_block_indices, src/nats/ops/nats_util.py:6-32.

    n_lin [B,HN] -> [sum n_chunks, 2] rows (flat_bh, j), j < cdiv(n_lin*block, chunk).
    """
    rows = []
    for bh, n in enumerate(n_lin.flatten().tolist()):
        for j in range(_cdiv(int(n) * block, chunk)):
            rows.append((bh, j))
    if not rows:
        return torch.zeros(0, 2, dtype=torch.int32)
    return torch.tensor(rows, dtype=torch.int32)


def linear_chunk_offsets(n_lin: torch.Tensor, block: int, chunk: int = CHUNK) -> torch.Tensor:
    """prepare_nats_chunk_offsets, src/nats/ops/nats_util.py:35-64: exclusive
    prefix sum of the per-(b,hn) linear chunk counts, length B*HN+1, int64."""
    n = [_cdiv(int(x) * block, chunk) for x in n_lin.flatten().tolist()]
    return torch.tensor(np.concatenate([[0], np.cumsum(n)]), dtype=torch.int64)


def starting_h_idx(idx: torch.Tensor, T: int, block: int, chunk: int = CHUNK) -> torch.Tensor:
    """compute_starting_idx_for_chunks, src/nats/ops/nats_util.py:124-162
    (op column = linear): for every chunk c the number of linear blocks whose
    first token is < c*chunk.  idx [B,TN,HN,n_ops] -> int64 [B,cdiv(T,chunk),HN]."""
    lin = idx[..., OFFSET_LINEAR].long()                      # [B,TN,HN]
    m_start = torch.arange(_cdiv(T, chunk)) * chunk
    return (lin.unsqueeze(1) * block < m_start.view(1, -1, 1, 1)).sum(2)


def starting_h_idx_loop(types: torch.Tensor, T: int, block: int, chunk: int = CHUNK) -> torch.Tensor:
    t = np.rint(types.float().numpy())
    B, TN, HN, _ = t.shape
    NT = _cdiv(T, chunk)
    out = np.zeros((B, NT, HN), dtype=np.int64)
    for b in range(B):
        for h in range(HN):
            for c in range(NT):
                out[b, c, h] = sum(1 for j in range(TN) if t[b, j, h, OFFSET_LINEAR] == 1.0 and j * block < c * chunk)
    return torch.from_numpy(out)


def attn_n_iters(idx: torch.Tensor, T: int, block: int, tile: int = ATTN_QUERY_TILE) -> torch.Tensor:
    """compute_attn_n_iters_per_block (no sliding window, tile > block),
    src/nats/ops/nats_util.py:67-121: number of attention blocks that end at or
    before the first row of each query tile.  -> int64 [B,cdiv(T,tile),HN]."""
    att = idx[..., OFFSET_ATTN].long()
    m_start = torch.arange(_cdiv(T, tile)) * tile
    return ((att.unsqueeze(1) + 1) * block <= m_start.view(1, -1, 1, 1)).sum(2)


def attn_n_iters_loop(types: torch.Tensor, T: int, block: int, tile: int = ATTN_QUERY_TILE) -> torch.Tensor:
    t = np.rint(types.float().numpy())
    B, TN, HN, _ = t.shape
    NQ = _cdiv(T, tile)
    out = np.zeros((B, NQ, HN), dtype=np.int64)
    for b in range(B):
        for h in range(HN):
            for i in range(NQ):
                out[b, i, h] = sum(1 for j in range(TN) if t[b, j, h, OFFSET_ATTN] == 1.0 and (j + 1) * block <= i * tile)
    return torch.from_numpy(out)


def attn_fraction(types: torch.Tensor) -> torch.Tensor:
    """attn_fraction metric, src/nats/layers/natsl_attn_gdn.py:555."""
    nb = n_blocks(types)
    return (nb.float()[..., OFFSET_ATTN] / types.shape[1]).mean(0)


def route(types: torch.Tensor, T: int, block: int) -> dict:
    """All routing tensors the mixed op derives from `types` (already forced)."""
    idx = block_indices(types)
    nb = n_blocks(torch.round(types.float()))
    n_lin = nb[..., OFFSET_LINEAR]
    return dict(
        nats_block_indices=idx,
        n_nats_blocks=nb,
        chunk_indices_linear=chunk_indices_linear(n_lin, block),
        linear_chunk_offsets=linear_chunk_offsets(n_lin, block),
        starting_h_idx=starting_h_idx(idx, T, block),
        attn_n_iters=attn_n_iters(idx, T, block),
    )
