"""Oracle for the softmax branch (sparse-KV causal attention over selected chunks).

TEST INFRASTRUCTURE ONLY -- see oracle/__init__.py.

Restates parallel_nats_attn_fwd_kernel, src/nats/ops/attns/attns.py:62-353, as a
dense masked softmax.  The visibility mask is the closed form of the kernel's
two phases (whole attention blocks before the query tile :173-217, the tile's
own keys with causal / same-block rules :271-340); the same recipe is built in
torch by the reference's debug script at :2041-2062.

Pins: all-attention types => plain causal attention and all-linear types =>
block-diagonal causal attention, both checked against
torch.nn.functional.scaled_dot_product_attention (a library routine) in
tests/test_oracle_branches.py; a brute-force per-row Python loop checks the mask.
"""
from __future__ import annotations

import math

import torch

LOG2E = 1.4426950408889634


def visibility_mask(attn_types: torch.Tensor, T: int, block: int, same_block_visible: bool = True) -> torch.Tensor:
    """attn_types [NB] in {0,1} for ONE (batch, selector head) -> bool [T,T] (rows = queries).

    same_block_visible=True  (modes 'all' / 'attn', COMPUTE_INCOMPLETE_CHUNK_SCORES):
        M(t,s) = s<=t and (blk(s)==blk(t) or a[blk(s)]==1)
    same_block_visible=False (modes 'gated_delta_net' / 'mamba'):
        M(t,s) = a[blk(s)]==1 and t >= (blk(s)+1)*block          (attns.py:318-320)
    """
    t = torch.arange(T)
    blk = t // block
    a = attn_types.reshape(-1)[blk].bool()                       # per key
    if same_block_visible:
        causal = t.view(-1, 1) >= t.view(1, -1)
        same = blk.view(-1, 1) == blk.view(1, -1)
        return causal & (same | a.view(1, -1))
    return a.view(1, -1) & (t.view(-1, 1) >= ((blk + 1) * block).view(1, -1))


def softmax_branch(q, k, v, types, scale, block, same_block_visible=True, dtype=torch.float32):
    """q [B,T,HQ,K], k [B,T,HKV,K], v [B,T,HKV,V], types [B,NB,HN,n_ops] -> (o [B,T,HQ,V], lse [B,T,HQ]).

    lse is in log2 units, m + log2(sum) with scores scaled by scale*log2(e)
    (attns.py:158-159,346-353); rows that see no key give o = 0, lse = 0
    (attns.py:343-350).  GQA: kv head = hq // (HQ//HKV); selector head =
    hq // (HQ//HN) (attns.py:99-101).
    """
    B, T, HQ, K = q.shape
    HKV, V = k.shape[2], v.shape[-1]
    HN = types.shape[2]
    G, GN = HQ // HKV, HQ // HN
    o = torch.zeros(B, T, HQ, V, dtype=dtype)
    lse = torch.zeros(B, T, HQ, dtype=dtype)
    a = torch.round(types[..., 0].float())
    for b in range(B):
        masks = [visibility_mask(a[b, :, hn], T, block, same_block_visible) for hn in range(HN)]
        for hq in range(HQ):
            m = masks[hq // GN]
            s = (q[b, :, hq].to(dtype) @ k[b, :, hq // G].to(dtype).T) * (scale * LOG2E)
            s = s.masked_fill(~m, float('-inf'))
            mx = s.max(-1, keepdim=True)[0]
            valid = torch.isfinite(mx)
            mx = torch.where(valid, mx, torch.zeros_like(mx))
            p = torch.exp2(s - mx)
            den = p.sum(-1, keepdim=True)
            den_safe = torch.where(valid, den, torch.ones_like(den))
            o[b, :, hq] = torch.where(valid, (p @ v[b, :, hq // G].to(dtype)) / den_safe, torch.zeros(1, dtype=dtype))
            lse[b, :, hq] = torch.where(valid, mx + torch.log2(den_safe), torch.zeros_like(mx)).squeeze(-1)
    return o, lse


def softmax_branch_sdpa(q, k, v, types, scale, block, same_block_visible=True):
    """Same result through F.scaled_dot_product_attention with an explicit mask
    (used for the CPU baseline timing and as a library cross-check)."""
    B, T, HQ, K = q.shape
    HKV = k.shape[2]
    HN = types.shape[2]
    G, GN = HQ // HKV, HQ // HN
    a = torch.round(types[..., 0].float())
    mask = torch.stack([
        torch.stack([visibility_mask(a[b, :, hq // GN], T, block, same_block_visible) for hq in range(HQ)])
        for b in range(B)])
    kk = k.repeat_interleave(G, 2) if G > 1 else k
    vv = v.repeat_interleave(G, 2) if G > 1 else v
    o = torch.nn.functional.scaled_dot_product_attention(
        q.transpose(1, 2), kk.transpose(1, 2), vv.transpose(1, 2), attn_mask=mask, scale=scale)
    o = o.transpose(1, 2)
    empty = ~mask.any(-1)                                        # [B,HQ,T]
    if empty.any():
        o = torch.where(empty.transpose(1, 2).unsqueeze(-1), torch.zeros((), dtype=o.dtype), o)
    return o


def flops(types: torch.Tensor, T: int, block: int, K: int, V: int, heads_per_selector: int) -> float:
    """Algorithmic FLOPs 2(K+V) * sum_t n_keys(t) for the visibility rule 'all'."""
    a = torch.round(types[..., 0].float())                       # [B,NB,HN]
    B, NB, HN = a.shape
    prior = torch.cumsum(a, 1) - a                               # attention blocks before each block
    tot = 0.0
    for c in range(NB):
        n = min(block, T - c * block)
        tot += float((n * (n + 1) / 2 + n * block * prior[:, c]).sum())
    return 2.0 * (K + V) * tot * heads_per_selector


def softmax_branch_bwd(q, k, v, types, do, scale, block, same_block_visible=True, dtype=torch.float64, with_magnitude=False,
                       dnats_invalid=False, clamp_invalid=True):
    """Gradients of the softmax branch in closed form (parallel_attn_nats_bwd, src/nats/ops/attns/attns.py:1562-1759;
    kernels :383-708 for dq, :719-983 for dk, dv and dnats):
        P = softmax(masked scores), delta = rowsum(dO * O) (:357-372), dP = dO V^T, dS = P * (dP - delta)
        dq = scale dS K (:704), dk = scale dS^T Q (:966, summed over the query heads of a kv head :1746),
        dv = P^T dO (:1747)
        dnats[b, j, hn] = sum of dS over (keys of block j) x (queries of LATER blocks), summed over the query heads of
        selector head hn, for blocks typed attention (:946-961, :1755); 0 for the other blocks (the default
        compute_dnats_for_invalid_blocks_attn=False).  It is the gradient with respect to a bias added to the
        (natural-log scale) scores of a block's keys as later blocks see them.
        dnats_invalid (compute_dnats_for_invalid_blocks_attn=True, :1318-1325): a block that is NOT typed attention gets
        sum min(exp(s - lse), 1) (dP - delta) over the same (keys) x (later queries) instead of 0: the score gradient its
        keys would have if they were visible, with the probabilities taken against the lse of what the query does see and
        clamped to 1.  (A query that sees nothing has lse = 0 here, as the forward kernel reports it; the reference leaves
        that case undefined.)  For a block that is typed attention the expression equals dS, which is how it is pinned.
    -> (dq [B,T,HQ,K], dk [B,T,HKV,K], dv [B,T,HKV,V], dnats [B,NB,HN]); with_magnitude adds the same sums over |dS|
    (the scale rounding errors of dnats are measured against: the signed sums cancel, down to exactly 0 when a query
    sees a single earlier block and nothing else).

    What pins it: torch.autograd through the same dense masked softmax with that bias as a zero tensor
    (tests/test_oracle_branches.py)."""
    B, T, HQ, K = q.shape
    HKV, V = k.shape[2], v.shape[-1]
    NB, HN = types.shape[1], types.shape[2]
    G, GN = HQ // HKV, HQ // HN
    dq = torch.zeros(B, T, HQ, K, dtype=dtype)
    dk = torch.zeros(B, T, HKV, K, dtype=dtype)
    dv = torch.zeros(B, T, HKV, V, dtype=dtype)
    dnats = torch.zeros(B, NB, HN, dtype=dtype)
    dnats_mag = torch.zeros(B, NB, HN, dtype=dtype)
    a = torch.round(types[..., 0].float())
    blk = torch.arange(T) // block
    later = blk.view(-1, 1) > blk.view(1, -1)                                  # [query, key]: the key's block is an earlier one
    for b in range(B):
        for hq in range(HQ):
            hn, hk = hq // GN, hq // G
            m = visibility_mask(a[b, :, hn], T, block, same_block_visible)
            qq, kk, vv, dd = (x.to(dtype) for x in (q[b, :, hq], k[b, :, hk], v[b, :, hk], do[b, :, hq]))
            s = (qq @ kk.T) * scale
            s = s.masked_fill(~m, float('-inf'))
            valid = m.any(-1, keepdim=True)
            p = torch.where(valid, torch.softmax(torch.where(valid, s, torch.zeros_like(s)), -1), torch.zeros_like(s))
            p = p * m
            o = p @ vv
            delta = (dd * o).sum(-1, keepdim=True)
            ds = p * (dd @ vv.T - delta)
            dq[b, :, hq] = scale * ds @ kk
            dk[b, :, hk] += scale * ds.T @ qq
            dv[b, :, hk] += p.T @ dd
            inter = ds * later                                                  # [query, key]
            per_block = torch.zeros(NB, dtype=dtype).index_add_(0, blk, inter.sum(0))
            dnats[b, :, hn] += per_block * a[b, :, hn].to(dtype)
            if dnats_invalid:
                s_all = (qq @ kk.T) * scale
                lse = torch.where(valid, torch.logsumexp(torch.where(valid, s, torch.zeros_like(s)), -1, keepdim=True), torch.zeros_like(delta))
                p1 = torch.exp(s_all - lse)
                if clamp_invalid:   # (False only in the test that pins the unclamped expression as an exact derivative)
                    p1 = p1.clamp(max=1.0)
                inter1 = p1 * (dd @ vv.T - delta) * later
                per_block1 = torch.zeros(NB, dtype=dtype).index_add_(0, blk, inter1.sum(0))
                dnats[b, :, hn] += per_block1 * (1 - a[b, :, hn].to(dtype))
                dnats_mag[b, :, hn] += torch.zeros(NB, dtype=dtype).index_add_(0, blk, inter1.abs().sum(0)) * (1 - a[b, :, hn].to(dtype))
            dnats_mag[b, :, hn] += torch.zeros(NB, dtype=dtype).index_add_(0, blk, inter.abs().sum(0)) * a[b, :, hn].to(dtype)
    if with_magnitude:
        return dq, dk, dv, dnats, dnats_mag
    return dq, dk, dv, dnats
