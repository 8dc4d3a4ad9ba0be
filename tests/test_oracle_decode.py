"""Pins oracle/decode.py (CPU): the recurrent restatement, driven the way the reference's cache drives it,
must reproduce the whole-sequence token recurrence; the masked attention must agree with torch's
scaled_dot_product_attention wherever a query sees at least one key."""
import pytest
import torch
import torch.nn.functional as F

from oracle import decode as D, linear_branch as LB
from tests._util import make_gates, make_qkv, make_types


@pytest.mark.parametrize("decay", [True, False])
@pytest.mark.parametrize("step", [1, 7, 64])
def test_recurrent_calls_reproduce_token_recurrence(step, decay):
    N, T, H, K, V, block, HN = 2, 200, 2, 16, 8, 64, 1
    q, k, v = make_qkv(N, T, H, K, V, 3, torch.float32)
    g, beta = make_gates(N, T, H, 4, torch.float32)
    ty = make_types(N, -(-T // block), HN, 0.5, 5, force_last=False)
    scale = K ** -0.5
    o_ref, S_ref = LB.gdn_token_recurrence(q, k, v, g, beta, ty[..., 1], scale, None, block=block, decay_non_linear=decay)
    # the last block is incomplete (200 = 3*64 + 8): the token recurrence rolls back only at block ends
    S, Scur, gcum, n_in = None, None, None, 0
    outs = []
    t = 0
    while t < T:
        n = min(step, block - n_in, T - t)
        blk = (t // block)
        o, S, Scur_new = D.gdn_recurrent(q[:, t:t + n], k[:, t:t + n], v[:, t:t + n], g[:, t:t + n], gcum, beta[:, t:t + n],
                                         ty[:, blk:blk + 1, :, 1], n_in, S, Scur, scale, block, decay)
        outs.append(o)
        # what the cache does between calls (src/nats/models/utils.py:625-657)
        if n_in + n >= block:
            n_in, gcum, Scur = 0, None, Scur_new
        else:
            n_in += n
            gs = g[:, t:t + n].double().sum(1)
            gcum = gs if gcum is None else gcum + gs
            Scur = Scur_new
        t += n
    o = torch.cat(outs, 1)
    assert float((o - o_ref).abs().max()) < 1e-9
    assert float((S - S_ref).abs().max()) < 1e-9


def test_masked_attention_matches_sdpa():
    B, TQ, TK, HQ, HKV, HM, K, V = 2, 3, 50, 4, 2, 2, 16, 8
    g = torch.Generator().manual_seed(0)
    q = torch.randn(B, TQ, HQ, K, generator=g)
    k = torch.randn(B, TK, HKV, K, generator=g)
    v = torch.randn(B, TK, HKV, V, generator=g)
    mask = torch.rand(B, HM, TQ, TK, generator=g) < 0.4
    mask[..., 0] = True                                   # every query sees something
    o = D.attn_masked(q, k, v, mask, K ** -0.5, torch.float32)
    m = mask.repeat_interleave(HQ // HM, dim=1)
    kk, vv = k.repeat_interleave(HQ // HKV, 2), v.repeat_interleave(HQ // HKV, 2)
    ref = F.scaled_dot_product_attention(q.transpose(1, 2), kk.transpose(1, 2), vv.transpose(1, 2), attn_mask=m,
                                         scale=K ** -0.5).transpose(1, 2)
    assert float((o - ref).abs().max()) < 1e-5
    mask[0, 0, 1] = False                                  # a query that sees nothing gives 0
    o = D.attn_masked(q, k, v, mask, K ** -0.5, torch.float32)
    assert float(o[0, 1, :2].abs().max()) == 0.0


def test_mamba_recurrent_calls_reproduce_token_recurrence():
    N, T, H, K, V, block = 1, 150, 2, 16, 8, 64
    q, k, v = make_qkv(N, T, H, K, V, 8, torch.float32)
    g, _ = make_gates(N, T, H, 9, torch.float32)
    ty = make_types(N, 3, H, 0.5, 10, force_last=False)
    ref_ty = ty.clone(); ref_ty[:, -1] = 1           # the trailing incomplete block is never rolled back
    o_ref, S_ref = LB.mamba_token_recurrence(q, k, v, g, ref_ty[..., 1], 1.0, None, block, True)
    S, Scur, gcum, n_in, outs, t = None, None, None, 0, [], 0
    while t < T:
        n = min(5, block - n_in, T - t)
        o, S, Scur = D.mamba_recurrent(q[:, t:t + n], k[:, t:t + n], v[:, t:t + n], g[:, t:t + n], gcum, ty[:, t // block:t // block + 1, :, 1],
                                       n_in, S, Scur, 1.0, block, True)
        outs.append(o)
        if n_in + n >= block:
            n_in, gcum = 0, None
        else:
            n_in += n
            gs = g[:, t:t + n].double().sum(1)
            gcum = gs if gcum is None else gcum + gs
        t += n
    assert float((torch.cat(outs, 1) - o_ref).abs().max()) < 1e-9 and float((S - S_ref).abs().max()) < 1e-9


@pytest.mark.parametrize("kind", ['gdn', 'mamba'])
def test_attn_mode_decode_reproduces_the_chunked_forward_without_intra_chunk_term(kind):
    """ops_for_incomplete_chunks = 'attn', selector block = one chunk: every token reads the decayed state that entered its
    block (recurrent_query_only); when a block is complete the state advances over its tokens (gdn_recurrent /
    mamba_recurrent, outputs discarded).  Token by token this must give the chunked forward with intra=False."""
    N, T, H, K, V, block, HN = 2, 200, 2, 16, 8, 64, 1
    q, k, v = make_qkv(N, T, H, K, V, 13, torch.float32)
    g, beta = make_gates(N, T, H, 14, torch.float32)
    ty = make_types(N, -(-T // block), HN, 0.5, 15, force_last=False)
    delta = kind == 'gdn'
    scale = K ** -0.5 if delta else 1.0
    if delta:
        o_ref, _ = LB.gdn_chunked(q, k, v, g, beta, ty[..., 1], scale, None, block, True, True, torch.float64, False)
    else:
        o_ref, _ = LB.mamba_chunked(q, k, v, g, ty[..., 1], scale, None, block, True, torch.float64, False)
    S = torch.zeros(N, H, K, V, dtype=torch.float64)
    gcum, outs = None, []
    for t in range(T):
        n_in = t % block
        outs.append(D.recurrent_query_only(q[:, t:t + 1], g[:, t:t + 1], gcum, S, scale, l2norm_qk=delta))
        gs = g[:, t].double()
        gcum = gs if gcum is None else gcum + gs
        if n_in == block - 1:
            b0 = t + 1 - block
            blk = ty[:, t // block:t // block + 1, :, 1]
            if delta:
                _, S, _ = D.gdn_recurrent(k[:, b0:t + 1], k[:, b0:t + 1], v[:, b0:t + 1], g[:, b0:t + 1], None, beta[:, b0:t + 1], blk, 0, S,
                                          S, scale, block, True)
            else:
                _, S, _ = D.mamba_recurrent(k[:, b0:t + 1], k[:, b0:t + 1], v[:, b0:t + 1], g[:, b0:t + 1], None, blk, 0, S, S, scale, block, True)
            gcum = None
    o = torch.cat(outs, 1)
    assert float((o - o_ref).abs().max()) < 1e-9
