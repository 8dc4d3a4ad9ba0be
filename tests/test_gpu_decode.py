"""GPU parity of the decode-time operators against oracle/decode.py (tolerance for outputs and states:
max-abs 2e-2, rel-L2 5e-3), and the prefill -> decode hand-off against the whole-sequence token recurrence."""
import pytest
import torch

from oracle import decode as D, linear_branch as LB
from tests._util import assert_close, make_gates, make_qkv, make_types

pytestmark = pytest.mark.gpu
DEV = 'cuda:0'


def _dev(*ts):
    return [None if t is None else t.to(DEV) for t in ts]


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("decay", [True, False])
@pytest.mark.parametrize("K,V,T,n_in", [(128, 128, 1, 0), (128, 128, 1, 63), (128, 128, 5, 10), (64, 64, 64, 0),
                                        (128, 64, 7, 57), (64, 128, 9, 60)])       # the last: only 4 of 9 tokens fit
def test_recurrent_against_oracle(K, V, T, n_in, decay, dtype):
    from neuralattentionsearchlinear_amd.mixed_attn_gdn import fused_recurrent_gated_delta_rule_nats_fwd
    N, H, HN, block = 3, 4, 2, 64
    q, k, v = make_qkv(N, T, H, K, V, 11, dtype)
    g, beta = make_gates(N, T, H, 12, dtype)
    gen = torch.Generator().manual_seed(13)
    h0 = torch.randn(N, H, K, V, generator=gen) * 0.3
    hcur = torch.randn(N, H, K, V, generator=gen) * 0.3
    gcum = -torch.rand(N, H, generator=gen) * 3
    ty = make_types(N, 1, HN, 0.5, 14, dtype, force_last=False)
    scale = K ** -0.5
    o_ref, S_ref, cur_ref = D.gdn_recurrent(q.float(), k.float(), v.float(), g, gcum, beta.float(), ty[..., 1].float(), n_in, h0, hcur,
                                            scale, block, decay)
    qd, kd, vd, gd, bd, tyd, h0d, gcd = _dev(q, k, v, g, beta, ty, h0, gcum)
    hcurd = hcur.to(DEV).clone()
    o, S, cur = fused_recurrent_gated_delta_rule_nats_fwd(qd, kd, vd, gd, gcd, bd, tyd, n_in, block, scale, h0d, hcurd,
                                                          decay_for_non_gdn_blocks=decay)
    torch.cuda.synchronize()
    assert cur.data_ptr() == hcurd.data_ptr()          # updated in place, as the reference's kernel does
    n_tok = min(T, block - n_in)
    assert_close(o[:, :n_tok].float(), o_ref[:, :n_tok], "o")
    assert_close(S, S_ref, "final_state")
    assert_close(cur, cur_ref, "block_start_state")
    if n_in + T < block:
        assert torch.equal(cur.cpu(), hcur), "the block is not complete: its start state must be untouched"


def test_recurrent_defaults_and_per_sequence_counts():
    from neuralattentionsearchlinear_amd.mixed_attn_gdn import fused_recurrent_gated_delta_rule_nats_fwd
    N, T, H, K, V, block = 2, 3, 2, 64, 64, 64
    q, k, v = make_qkv(N, T, H, K, V, 1)
    g, beta = make_gates(N, T, H, 2)
    ty = make_types(N, 1, H, 0.5, 3, torch.bfloat16, force_last=False)
    n_in = torch.tensor([5, 5], dtype=torch.int32)
    o_ref, S_ref, cur_ref = D.gdn_recurrent(q.float(), k.float(), v.float(), g, None, beta.float(), ty[..., 1].float(), 5, None, None,
                                            K ** -0.5, block, True)
    o, S, cur = fused_recurrent_gated_delta_rule_nats_fwd(*_dev(q, k, v, g), None, beta.to(DEV), ty.to(DEV), n_in.to(DEV), block,
                                                          K ** -0.5, None, None, decay_for_non_gdn_blocks=True)
    assert_close(o.float(), o_ref, "o"); assert_close(S, S_ref, "final_state"); assert_close(cur, cur_ref, "block_start_state")
    with pytest.raises(AssertionError):
        fused_recurrent_gated_delta_rule_nats_fwd(*_dev(q, k, v, g), None, beta.to(DEV), torch.cat([ty, ty], 1).to(DEV), 0, block,
                                                  K ** -0.5, None, None)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("K,V", [(128, 128), (64, 64), (64, 128), (128, 64)])
@pytest.mark.parametrize("TQ,TK,HM", [(1, 700, 2), (3, 64, 1), (2, 130, 4), (1, 3000, 2)])   # the last: keys split over workgroups
def test_masked_attention_against_oracle(K, V, TQ, TK, HM, dtype):
    from neuralattentionsearchlinear_amd.mixed_attn_gdn import masked_attention
    B, HQ, HKV = 2, 4, 2
    gen = torch.Generator().manual_seed(5)
    q = torch.randn(B, TQ, HQ, K, generator=gen).to(dtype)
    k = torch.randn(B, TK, HKV, K, generator=gen).to(dtype)
    v = torch.randn(B, TK, HKV, V, generator=gen).to(dtype)
    mask = torch.rand(B, HM, TQ, TK, generator=gen) < 0.3
    mask[0, 0, 0] = False                                  # a query that sees nothing
    mask[1, :, :, 64:128] = False                          # a whole chunk of hidden keys
    ref = D.attn_masked(q.float(), k.float(), v.float(), mask, K ** -0.5)
    o = masked_attention(*_dev(q, k, v, mask), K ** -0.5)
    assert o.dtype == dtype
    assert_close(o.float(), ref, "o_attn")
    assert float(o[0, 0, :HQ // HM].abs().max()) == 0.0


def test_masked_attention_reads_a_cache_buffer_in_place():
    """Keys / values that are the front part of a larger cache buffer [B, capacity, H, D] are read where they are (batch
    stride = capacity * H * D): same result as on a dense copy, bit for bit, and the buffer's tail is never touched."""
    from neuralattentionsearchlinear_amd.mixed_attn_gdn import masked_attention
    B, HQ, HKV, HM, K, V, TQ, TK, cap = 3, 8, 4, 2, 64, 128, 2, 777, 1024
    gen = torch.Generator().manual_seed(9)
    q = torch.randn(B, TQ, HQ, K, generator=gen).bfloat16().to(DEV)
    kbuf = torch.randn(B, cap, HKV, K, generator=gen).bfloat16().to(DEV)
    vbuf = torch.randn(B, cap, HKV, V, generator=gen).bfloat16().to(DEV)
    kbuf[:, TK:], vbuf[:, TK:] = float('nan'), float('nan')       # reading past TK would poison the result
    mask = (torch.rand(B, HM, TQ, TK, generator=gen) < 0.4).to(DEV)
    kv, vv = kbuf[:, :TK], vbuf[:, :TK]
    assert not kv.is_contiguous()
    a = masked_attention(q, kv, vv, mask, K ** -0.5)
    b = masked_attention(q, kv.contiguous(), vv.contiguous(), mask, K ** -0.5)
    torch.cuda.synchronize()
    assert bool(torch.isfinite(a.float()).all()) and torch.equal(a, b)


@pytest.mark.parametrize("decay", [True, False])
def test_prefill_then_decode_matches_whole_sequence(decay):
    """Prefill 3 blocks + 10 tokens with the chunked operator, then decode token by token through the end of
    that block, across the block boundary (where the block's TRUE type decides about the roll-back) and 20
    tokens into the next block, keeping (state, block-start state, sum of g in the block) as the reference's
    cache does (src/nats/models/utils.py:625-657).  Every decoded output and the final state must match the
    token recurrence over the whole sequence."""
    from neuralattentionsearchlinear_amd.mixed_attn_gdn import (nats_mixed_attn_gdn_chunk_inference,
                                                                nats_mixed_attn_gdn_recurrent)
    B, H, K, V, block = 2, 4, 128, 128, 64
    T0, T = 3 * block + 10, 4 * block + 20
    q, k, v = make_qkv(B, T, H, K, V, 41)
    g, beta = make_gates(B, T, H, 42)
    true_ty = make_types(B, 5, H, 0.5, 43, torch.bfloat16, force_last=False)
    scale = K ** -0.5
    # whole-sequence reference: blocks 0..3 complete with their true types; block 4 is incomplete, so no roll-back
    # applies to it (the token recurrence treats the end of the sequence as a block end: type it linear)
    ref_ty = true_ty.clone(); ref_ty[:, -1] = 1
    o_ref, S_ref = LB.gdn_token_recurrence(q, k, v, g, beta, ref_ty[..., 1], scale, None, block, decay, dtype=torch.float64)
    qd, kd, vd, gd, bd = _dev(q, k, v, g, beta)
    forced = true_ty[:, :4].clone(); forced[:, -1] = 1
    with torch.no_grad():
        o0, _, S, S_start = nats_mixed_attn_gdn_chunk_inference(
            qd[:, :T0], kd[:, :T0], vd[:, :T0], qd[:, :T0], kd[:, :T0], vd[:, :T0], None, gd[:, :T0], bd[:, :T0], forced.to(DEV), None, None,
            nats_block_size=block, ops_for_incomplete_chunks='all', output_final_state_gated_delta=True, decay_for_non_gdn_blocks=decay)
    assert_close(o0.float(), o_ref[:, :T0], "prefill o_gdn")
    n_in = T0 % block
    gcum = gd[:, T0 - n_in:T0].sum(1)                                      # [B,H]
    outs = []
    for t in range(T0, T):
        blk = t // block
        sl = lambda x: x[:, t:t + 1].contiguous()
        # the attention inputs are irrelevant here: one visible key
        msk = torch.ones(B, 1, 1, 1, dtype=torch.bool, device=DEV)
        o, _, S, S_start = nats_mixed_attn_gdn_recurrent(
            sl(qd), sl(kd), sl(vd), sl(qd), sl(kd), sl(vd), msk, S, S_start, sl(gd), gcum, sl(bd), true_ty[:, blk:blk + 1].to(DEV),
            n_tokens_in_current_block=n_in, nats_block_size=block, ops_for_incomplete_chunks='all',
            decay_for_non_gdn_blocks=decay)
        outs.append(o)
        if n_in + 1 >= block:
            n_in, gcum = 0, torch.zeros_like(gcum)
        else:
            n_in += 1
            gcum = gcum + gd[:, t]
    o_dec = torch.cat(outs, 1)
    assert_close(o_dec.float(), o_ref[:, T0:], "decoded o_gdn")
    assert_close(S, S_ref, "final_state")


@pytest.mark.parametrize("decay", [True, False])
@pytest.mark.parametrize("K,V,T,n_in,block", [(128, 64, 1, 255, 256), (128, 64, 3, 10, 256), (64, 128, 6, 60, 64)])
def test_mamba_recurrent_against_oracle(K, V, T, n_in, block, decay):
    from neuralattentionsearchlinear_amd.mixed_attn_mamba import nats_mixed_attn_mamba_recurrent
    N, H = 2, 4
    q, k, v = make_qkv(N, T, H, K, V, 61)
    # unit-norm C and B rows keep the outputs O(1), where the absolute tolerance is meaningful in bf16
    q = torch.nn.functional.normalize(q.float(), dim=-1).bfloat16(); k = torch.nn.functional.normalize(k.float(), dim=-1).bfloat16()
    g, _ = make_gates(N, T, H, 62)
    gen = torch.Generator().manual_seed(63)
    h0 = torch.randn(N, H, K, V, generator=gen) * 0.3
    hcur = torch.randn(N, H, K, V, generator=gen) * 0.3
    gcum = -torch.rand(N, H, generator=gen) * 3
    ty = make_types(N, 1, H, 0.5, 64, torch.bfloat16, force_last=False)
    o_ref, S_ref, cur_ref = D.mamba_recurrent(q.float(), k.float(), v.float(), g, gcum, ty[..., 1].float(), n_in, h0, hcur, 1.0, block, decay)
    TK = 40
    ka, va = make_qkv(N, TK, H, K, V, 65)[1:]
    mask = torch.rand(N, H, T, TK, generator=gen) < 0.5
    mask[..., 0] = True
    a_ref = D.attn_masked(q.float(), ka.float(), va.float(), mask, K ** -0.5)
    o, o_attn, S, cur = nats_mixed_attn_mamba_recurrent(*_dev(q, ka, va, q, k, v, mask, h0, hcur, g, gcum, ty), n_tokens_in_current_block=n_in,
                                                        scale_lattn=1.0, nats_block_size=block, decay_for_non_mamba_blocks=decay)
    n_tok = min(T, block - n_in)
    assert_close(o[:, :n_tok].float(), o_ref[:, :n_tok], "o_mamba"); assert_close(o_attn.float(), a_ref, "o_attn")
    assert_close(S, S_ref, "final_state"); assert_close(cur, cur_ref, "block_start_state")


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("kind,K,V,T,n_in", [('gdn', 128, 128, 1, 0), ('gdn', 128, 256, 1, 63), ('gdn', 64, 64, 5, 10), ('gdn', 192, 128, 3, 7),
                                             ('mamba', 128, 64, 1, 33), ('mamba', 64, 128, 4, 60)])
def test_query_only_outputs_against_oracle(kind, K, V, T, n_in, dtype):
    """NATSL_QUERY_ONLY (the decode output of ops_for_incomplete_chunks = 'attn'): the decayed block-start state read by the
    new queries; nothing is written back."""
    from neuralattentionsearchlinear_amd.mixed_attn_gdn import fused_recurrent_gated_delta_rule_nats_fwd
    from neuralattentionsearchlinear_amd.mixed_attn_mamba import fused_recurrent_mamba_nats_fwd
    N, H, HN, block = 3, 4, 2, 64
    q, _, _ = make_qkv(N, T, H, K, V, 21, dtype)
    g, _ = make_gates(N, T, H, 22, dtype)
    gen = torch.Generator().manual_seed(23)
    hcur = torch.randn(N, H, K, V, generator=gen) * 0.3
    gcum = -torch.rand(N, H, generator=gen) * 3
    ty = make_types(N, 1, HN, 0.5, 24, dtype, force_last=False)
    scale = K ** -0.5
    delta = kind == 'gdn'
    o_ref = D.recurrent_query_only(q.float(), g, gcum, hcur, scale, l2norm_qk=delta)
    qd, gd, tyd, gcd = _dev(q, g, ty, gcum)
    hcurd = hcur.to(DEV).clone()
    if delta:
        o, S, cur = fused_recurrent_gated_delta_rule_nats_fwd(qd, None, None, gd, gcd, None, tyd, n_in, block, scale, None, hcurd, query_only=True)
    else:
        o, S, cur = fused_recurrent_mamba_nats_fwd(qd, None, None, gd, gcd, tyd, n_in, block, scale, None, hcurd, query_only=True)
    torch.cuda.synchronize()
    n_tok = min(T, block - n_in)
    assert_close(o[:, :n_tok].float(), o_ref[:, :n_tok], "o")
    assert S is None and torch.equal(cur.cpu(), hcur), "query-only must not write a state"
