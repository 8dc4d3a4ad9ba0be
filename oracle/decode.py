"""CPU restatement of the decode-time operators (test infrastructure only, see oracle/__init__.py).

gdn_recurrent   follows src/nats/ops/gated_delta_rule/fused_recurrent.py:28-358 on the path the reference's
                decode takes (UPDATE_HS_FOR_EACH_ITER, one selector block, src/nats/ops/mixed_ops/
                mixed_attn_gdn.py:485-503), line by line.
recurrent_query_only  the decode output of the 'attn' mode (no state update on the incomplete block).
attn_masked     dense softmax attention under an explicit mask, the scaled_dot_product_attention call at
                src/nats/ops/mixed_ops/mixed_attn_gdn.py:475-481 with repeat_masks
                (src/nats/ops/attns/attn_utils.py:3-16).

What pins gdn_recurrent: feeding a whole sequence through it block by block, a few tokens per call, with the
caller keeping (state, block-start state, sum of g in the block) as the reference's cache does
(src/nats/models/utils.py:625-657), must reproduce linear_branch.gdn_token_recurrence on the whole sequence
(tests/test_oracle_decode.py) -- a different code path for the same recurrence, pinned in turn by the
chunked form and its own checks.
"""
import torch


def mamba_recurrent(q, k, v, g, g_cumsum, lin_types, n_in_block, h0, h_block_start, scale, block=64,
                    decay_non_linear=True, dtype=torch.float64):
    """The SSD form of gdn_recurrent (src/nats/ops/mamba/fused_recurrent.py:150-178 and the same block-end rule):
    S <- e^g S + k v^T, no beta, no normalisation."""
    return gdn_recurrent(q, k, v, g, g_cumsum, None, lin_types, n_in_block, h0, h_block_start, scale, block,
                         decay_non_linear, l2norm_qk=False, dtype=dtype, delta=False)


def gdn_recurrent(q, k, v, g, g_cumsum, beta, lin_types, n_in_block, h0, h_block_start, scale, block=64,
                  decay_non_linear=True, l2norm_qk=True, dtype=torch.float64, delta=True):
    """q,k [N,T,H,K]; v [N,T,H,V]; g,beta [N,T,H]; g_cumsum [N,H] or None; lin_types [N,1,HN] in {0,1};
    n_in_block int; h0, h_block_start [N,H,K,V] or None -> (o [N,T,H,V], ht, h_block_start')."""
    N, T, H, K = q.shape
    V = v.shape[-1]
    q, k, v, g = (x.to(dtype) for x in (q, k, v, g))
    beta = beta.to(dtype) if delta else None
    S = torch.zeros(N, H, K, V, dtype=dtype) if h0 is None else h0.to(dtype).clone()          # :129-133
    if h_block_start is None:                                                                    # wrapper :398-402
        Scur = S.clone()
    else:
        Scur = h_block_start.to(dtype).clone()
    gcum = torch.zeros(N, H, dtype=dtype) if g_cumsum is None else g_cumsum.to(dtype).clone()   # :117-121
    o = torch.zeros(N, T, H, V, dtype=dtype)
    n_tok = min(T, block - n_in_block)                                                           # :144
    for t in range(n_tok):
        qt, kt = q[:, t], k[:, t]
        if l2norm_qk:                                                                            # :165-169
            qt = qt / torch.sqrt((qt * qt).sum(-1, keepdim=True) + 1e-6)
            kt = kt / torch.sqrt((kt * kt).sum(-1, keepdim=True) + 1e-6)
        qt = qt * scale                                                                          # :171
        S = S * torch.exp(g[:, t])[..., None, None]                                              # :181-182
        if decay_non_linear:
            gcum = gcum + g[:, t]                                                                # :183-184
        dv = beta[:, t][..., None] * (v[:, t] - torch.einsum('nhkv,nhk->nhv', S, kt)) if delta else v[:, t]   # :195 / mamba :177
        S = S + torch.einsum('nhk,nhv->nhkv', kt, dv)                                            # :196
        o[:, t] = torch.einsum('nhkv,nhk->nhv', S, qt)                                           # :199-201
    if n_in_block + T >= block:                                                                  # wrapper :405, kernel :343-352
        HN = lin_types.shape[2]
        is_delta = torch.round(lin_types[:, 0].to(dtype)).bool().repeat_interleave(H // HN, dim=1)   # [N,H]
        f = torch.exp(gcum) if decay_non_linear else torch.ones_like(gcum)
        S = torch.where(is_delta[..., None, None], S, Scur * f[..., None, None])
        Scur = S.clone()
    return o, S, Scur


def recurrent_query_only(q, g, g_cumsum, h_block_start, scale, l2norm_qk=True, dtype=torch.float64):
    """The decode output of the mode in which the linear operator skips the incomplete block (ops_for_incomplete_chunks =
    'attn'): the kernel's loop without UPDATE_HS_FOR_EACH_ITER (src/nats/ops/gated_delta_rule/fused_recurrent.py:156-201) --
    per token the state only decays, b_h *= exp(g), and o = b_h^T (scale q^) -- started from the state that entered the
    block times e^(g_cumsum), which is what the reference's call with g + g_cumsum gives for a one-token step
    (src/nats/ops/mixed_ops/mixed_attn_gdn.py:510-527).  q [N,T,H,K]; g [N,T,H]; g_cumsum [N,H] or None;
    h_block_start [N,H,K,V] -> o [N,T,H,V].
    Pinned in tests/test_oracle_decode.py: fed token by token with the cache's bookkeeping, and the state advanced by
    gdn_recurrent over a block's tokens once the block is complete, it reproduces the chunked forward without its
    intra-chunk term (linear_branch.gdn_chunked / mamba_chunked, intra=False) for a selector block of one chunk."""
    q, g = q.to(dtype), g.to(dtype)
    N, T, H, K = q.shape
    S = h_block_start.to(dtype).clone()
    if g_cumsum is not None:
        S = S * torch.exp(g_cumsum.to(dtype))[..., None, None]
    o = torch.zeros(N, T, H, S.shape[-1], dtype=dtype)
    for t in range(T):
        qt = q[:, t]
        if l2norm_qk:
            qt = qt / torch.sqrt((qt * qt).sum(-1, keepdim=True) + 1e-6)
        S = S * torch.exp(g[:, t])[..., None, None]
        o[:, t] = torch.einsum('nhkv,nhk->nhv', S, qt * scale)
    return o


def attn_masked(q, k, v, mask, scale, dtype=torch.float64):
    """q [B,TQ,HQ,K]; k [B,TK,HKV,K]; v [B,TK,HKV,V]; mask bool [B,HM,TQ,TK] -> o [B,TQ,HQ,V]; a query that sees
    no key gives 0."""
    B, TQ, HQ, K = q.shape
    HKV, HM = k.shape[2], mask.shape[1]
    q, k, v = (x.to(dtype) for x in (q, k, v))
    k = k.repeat_interleave(HQ // HKV, dim=2)
    v = v.repeat_interleave(HQ // HKV, dim=2)
    m = mask.bool().repeat_interleave(HQ // HM, dim=1)                       # attn_utils.py:3-16
    s = torch.einsum('bqhk,bthk->bhqt', q, k) * scale
    s = s.masked_fill(~m, float('-inf'))
    p = torch.softmax(s, -1).nan_to_num(0.0)
    return torch.einsum('bhqt,bthv->bqhv', p, v)
