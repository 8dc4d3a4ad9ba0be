"""Pins the oracle's softmax / GDN / Mamba branches against each other, against library
routines and against special cases the mathematics fixes (CPU only)."""
import math

import pytest
import torch
import torch.nn.functional as F

from oracle import linear_branch as lb
from oracle import mixed, norm_gate, routing
from oracle import softmax_branch as sb


def _inputs(B, T, H, K, V, seed=0, HN=None, block=64, p_attn=0.4):
    g = torch.Generator().manual_seed(seed)
    HN = HN or H
    q = torch.randn(B, T, H, K, generator=g, dtype=torch.float64)
    k = torch.randn(B, T, H, K, generator=g, dtype=torch.float64)
    v = torch.randn(B, T, H, V, generator=g, dtype=torch.float64)
    beta = torch.sigmoid(torch.randn(B, T, H, generator=g, dtype=torch.float64))
    gl = -F.softplus(torch.randn(B, T, H, generator=g, dtype=torch.float64))
    NB = -(-T // block)
    lin = (torch.rand(B, NB, HN, generator=g) > p_attn).double()
    types = torch.stack([1 - lin, lin], -1)
    types = routing.force_last_block(types)
    return q, k, v, gl, beta, types


def _close(a, b, tol=1e-9):
    assert (a - b).abs().max().item() < tol, (a - b).abs().max().item()


@pytest.mark.parametrize("decay", [True, False])
@pytest.mark.parametrize("block,T", [(64, 256), (64, 200), (128, 384), (256, 512)])
def test_gdn_chunked_equals_token_recurrence(decay, block, T):
    q, k, v, g, beta, types = _inputs(2, T, 4, 16, 24, seed=3, HN=2, block=block)
    h0 = torch.randn(2, 4, 16, 24, dtype=torch.float64, generator=torch.Generator().manual_seed(9))
    o1, s1 = lb.gdn_token_recurrence(q, k, v, g, beta, types[..., 1], 0.25, h0, block, decay)
    o2, s2 = lb.gdn_chunked(q, k, v, g, beta, types[..., 1], 0.25, h0, block, decay, dtype=torch.float64)
    _close(o1, o2)
    _close(s1, s2)


@pytest.mark.parametrize("decay", [True, False])
def test_gdn_reference_pipeline_equals_token_recurrence(decay):
    q, k, v, g, beta, types = _inputs(2, 512, 4, 16, 8, seed=5, HN=2, p_attn=0.6)
    h0 = torch.randn(2, 4, 16, 8, dtype=torch.float64, generator=torch.Generator().manual_seed(2))
    o1, s1 = lb.gdn_token_recurrence(q, k, v, g, beta, types[..., 1], 0.3, h0, 64, decay)
    o2, s2 = lb.gdn_chunked_reference(q, k, v, g, beta, types[..., 1], 0.3, h0, decay)
    _close(o1, o2)
    _close(s1, s2)


def test_gdn_all_linear_is_textbook_gated_delta_rule():
    q, k, v, g, beta, types = _inputs(1, 128, 2, 8, 8, seed=7)
    types = torch.zeros_like(types); types[..., 1] = 1
    o, S = lb.gdn_chunked(q, k, v, g, beta, types[..., 1], 1.0, None, 64, True, dtype=torch.float64)
    # textbook: S_t = S_{t-1} e^{g_t} (I - beta_t k_t k_t^T) + beta_t k_t v_t^T  (state as [K,V]: S <- e^g (I - beta k k^T) S + beta k v^T)
    qn, kn = lb.l2norm(q), lb.l2norm(k)
    for h in range(2):
        St = torch.zeros(8, 8, dtype=torch.float64)
        for t in range(128):
            kt, vt, bt = kn[0, t, h], v[0, t, h], beta[0, t, h]
            St = math.exp(g[0, t, h]) * (torch.eye(8, dtype=torch.float64) - bt * torch.outer(kt, kt)) @ St + bt * torch.outer(kt, vt)
            _close(o[0, t, h], St.T @ qn[0, t, h])
        _close(S[0, h], St)


def test_gdn_g0_beta1_is_plain_delta_rule():
    q, k, v, g, beta, types = _inputs(1, 64, 1, 8, 4, seed=11)
    types = torch.zeros_like(types); types[..., 1] = 1
    o, S = lb.gdn_chunked(q, k, v, torch.zeros_like(g), torch.ones_like(beta), types[..., 1], 1.0, None, 64, True,
                          dtype=torch.float64)
    kn = lb.l2norm(k)
    St = torch.zeros(8, 4, dtype=torch.float64)
    for t in range(64):
        kt = kn[0, t, 0]
        St = St + torch.outer(kt, v[0, t, 0] - St.T @ kt)
    _close(S[0, 0], St)


def test_gdn_masked_inputs_identity():
    """Final state with non-linear chunks == stock gated delta rule on inputs whose k, v, beta are
    zeroed on the non-linear chunks (decay still applied there)."""
    q, k, v, g, beta, types = _inputs(2, 384, 2, 8, 8, seed=13)
    lin_tok = types[..., 1].repeat_interleave(64, 1)                    # [B,T,HN]
    all_lin = torch.ones_like(types[..., 1])
    _, S_mixed = lb.gdn_token_recurrence(q, k, v, g, beta, types[..., 1], 1.0, None, 64, True)
    _, S_stock = lb.gdn_token_recurrence(q, lb.l2norm(k) * lin_tok[..., None], v * lin_tok[..., None], g, beta * lin_tok,
                                         all_lin, 1.0, None, 64, True, l2norm_qk=False)
    _close(S_mixed, S_stock)


def test_gdn_split_and_chain():
    q, k, v, g, beta, types = _inputs(1, 512, 2, 8, 8, seed=17)
    types[:, 3] = torch.tensor([0., 1.])                                 # block before the split is linear
    o_full, S_full = lb.gdn_chunked(q, k, v, g, beta, types[..., 1], 0.5, None, 64, True, dtype=torch.float64)
    cut = 256
    o_a, S_a = lb.gdn_chunked(q[:, :cut], k[:, :cut], v[:, :cut], g[:, :cut], beta[:, :cut], types[:, :4, :, 1], 0.5, None,
                              64, True, dtype=torch.float64)
    o_b, S_b = lb.gdn_chunked(q[:, cut:], k[:, cut:], v[:, cut:], g[:, cut:], beta[:, cut:], types[:, 4:, :, 1], 0.5, S_a,
                              64, True, dtype=torch.float64)
    _close(torch.cat([o_a, o_b], 1), o_full)
    _close(S_b, S_full)


def test_all_attention_state_is_decayed_initial_state():
    q, k, v, g, beta, types = _inputs(1, 256, 2, 8, 8, seed=19)
    types = torch.zeros_like(types); types[..., 0] = 1
    types = routing.force_last_block(types)
    h0 = torch.randn(1, 2, 8, 8, dtype=torch.float64, generator=torch.Generator().manual_seed(1))
    for decay in (True, False):
        # state entering the last block: run only the first three blocks
        _, S3 = lb.gdn_chunked(q[:, :192], k[:, :192], v[:, :192], g[:, :192], beta[:, :192], types[:, :3, :, 1], 1.0, h0,
                               64, decay, dtype=torch.float64)
        expect = h0 * torch.exp(g[:, :192].sum(1))[..., None, None] if decay else h0
        _close(S3, expect)


@pytest.mark.parametrize("decay", [True, False])
@pytest.mark.parametrize("block,T", [(64, 256), (64, 150), (256, 768)])
def test_mamba_chunked_equals_token_recurrence(decay, block, T):
    q, k, v, g, _, types = _inputs(2, T, 4, 16, 8, seed=23, HN=2, block=block)
    h0 = torch.randn(2, 4, 16, 8, dtype=torch.float64, generator=torch.Generator().manual_seed(4))
    o1, s1 = lb.mamba_token_recurrence(q, k, v, g, types[..., 1], 1.0, h0, block, decay)
    o2, s2 = lb.mamba_chunked(q, k, v, g, types[..., 1], 1.0, h0, block, decay, dtype=torch.float64)
    _close(o1, o2)
    _close(s1, s2)


def test_mamba_all_linear_is_decayed_linear_attention():
    q, k, v, g, _, types = _inputs(1, 128, 1, 8, 4, seed=29)
    types = torch.zeros_like(types); types[..., 1] = 1
    o, _ = lb.mamba_chunked(q, k, v, g, types[..., 1], 1.0, None, 64, True, dtype=torch.float64)
    G = g[0, :, 0].cumsum(0)
    W = torch.tril(torch.exp(G[:, None] - G[None, :]) * (q[0, :, 0] @ k[0, :, 0].T))
    _close(o[0, :, 0], W @ v[0, :, 0])


def test_softmax_mask_brute_force():
    a = torch.tensor([1., 0., 1., 0., 0.])
    T, block = 5 * 8, 8
    m = sb.visibility_mask(a, T, block, True)
    m2 = sb.visibility_mask(a, T, block, False)
    for t in range(T):
        for s in range(T):
            same = (s // block) == (t // block)
            assert bool(m[t, s]) == (s <= t and (same or a[s // block] == 1))
            assert bool(m2[t, s]) == (a[s // block] == 1 and t >= (s // block + 1) * block)


def test_softmax_special_cases_match_sdpa():
    g = torch.Generator().manual_seed(31)
    B, T, HQ, HKV, K, V = 2, 192, 4, 2, 16, 8
    q = torch.randn(B, T, HQ, K, generator=g); k = torch.randn(B, T, HKV, K, generator=g); v = torch.randn(B, T, HKV, V, generator=g)
    kk, vv = k.repeat_interleave(2, 2), v.repeat_interleave(2, 2)
    scale = K ** -0.5
    # all attention -> plain causal
    types = torch.zeros(B, 3, 2, 2); types[..., 0] = 1
    o, lse = sb.softmax_branch(q, k, v, types, scale, 64)
    ref = F.scaled_dot_product_attention(q.transpose(1, 2), kk.transpose(1, 2), vv.transpose(1, 2), is_causal=True, scale=scale).transpose(1, 2)
    _close(o, ref, 1e-5)
    s = torch.einsum('bthk,bshk->bhts', q, kk) * scale
    s = s.masked_fill(~torch.tril(torch.ones(T, T, dtype=torch.bool)), float('-inf'))
    _close(lse, (torch.logsumexp(s, -1) / math.log(2)).transpose(1, 2), 1e-4)
    # all linear -> block-diagonal causal
    types = torch.zeros(B, 3, 2, 2); types[..., 1] = 1
    o, _ = sb.softmax_branch(q, k, v, types, scale, 64)
    for c in range(3):
        sl = slice(64 * c, 64 * c + 64)
        ref = F.scaled_dot_product_attention(q[:, sl].transpose(1, 2), kk[:, sl].transpose(1, 2), vv[:, sl].transpose(1, 2), is_causal=True, scale=scale).transpose(1, 2)
        _close(o[:, sl], ref, 1e-5)
    # random types: explicit-mask SDPA path agrees, in both visibility modes
    types = (torch.rand(B, 3, 2, 2, generator=g) < 0.5).float()
    for mode in (True, False):
        o, lse = sb.softmax_branch(q, k, v, types, scale, 64, mode)
        _close(o, sb.softmax_branch_sdpa(q, k, v, types, scale, 64, mode), 1e-5)
    # rows with no visible key give exactly 0 / 0
    types = torch.zeros(B, 3, 2, 2)
    o, lse = sb.softmax_branch(q, k, v, types, scale, 64, False)
    assert float(o.abs().max()) == 0.0 and float(lse.abs().max()) == 0.0


def test_softmax_flops_formula():
    types = torch.zeros(1, 4, 1, 2); types[0, [0, 2], 0, 0] = 1
    T, block, K, V = 256, 64, 8, 8
    m = sb.visibility_mask(types[0, :, 0, 0], T, block, True)
    assert sb.flops(types, T, block, K, V, 1) == 2.0 * (K + V) * float(m.sum())


def test_mixed_varlen_is_per_sequence():
    q, k, v, g, beta, _ = _inputs(1, 320, 2, 8, 8, seed=37)
    cu = [0, 128, 320]
    types = (torch.rand(1, 5, 2, 2, generator=torch.Generator().manual_seed(3)) < 0.5).double()
    types[:, 1] = 1; types[:, 4] = 1
    o_lin, o_attn, S, _ = mixed.mixed_attn_gdn(q, k, v, q, k, v, None, g, beta, types, cu_seqlens=cu,
                                               ops_for_incomplete_chunks='all', output_final_state=True,
                                               decay_for_non_gdn_blocks=True, dtype=torch.float64)
    a, b, Sa, _ = mixed.mixed_attn_gdn(q[:, :128], k[:, :128], v[:, :128], q[:, :128], k[:, :128], v[:, :128], None,
                                       g[:, :128], beta[:, :128], types[:, :2], ops_for_incomplete_chunks='all',
                                       output_final_state=True, decay_for_non_gdn_blocks=True, dtype=torch.float64)
    _close(o_lin[:, :128], a); _close(o_attn[:, :128], b); _close(S[0:1], Sa)
    assert S.shape == (2, 2, 8, 8)


def test_norm_gate_closed_form():
    g = torch.Generator().manual_seed(41)
    x1, x2, gate = (torch.randn(2, 5, 3, 16, generator=g) for _ in range(3))
    xw = torch.softmax(torch.randn(2, 5, 3, 2, generator=g), -1)
    w1, w2 = torch.randn(16, generator=g), torch.randn(16, generator=g)
    y = norm_gate.two_input_rmsnorm_gated(x1, x2, gate, xw, w1, w2, eps=1e-5)
    ref = (F.rms_norm(x1, (16,), w1, 1e-5) * xw[..., :1] + F.rms_norm(x2, (16,), w2, 1e-5) * xw[..., 1:]) * F.silu(gate)
    _close(y, ref, 1e-5)


@pytest.mark.parametrize("same_block", [True, False])
def test_softmax_backward_closed_form_equals_autograd(same_block):
    """oracle/softmax_branch.softmax_branch_bwd against torch.autograd through a dense masked softmax in which every
    block's keys carry a bias (a zero tensor) as LATER blocks see them: d/d(bias) is what the reference calls dnats."""
    from oracle import softmax_branch as sb
    from tests._util import make_types
    torch.manual_seed(3)
    B, T, HQ, HKV, HN, K, V, block = 2, 200, 4, 2, 2, 16, 8, 64
    NB = -(-T // block)
    q = torch.randn(B, T, HQ, K, dtype=torch.float64, requires_grad=True)
    k = torch.randn(B, T, HKV, K, dtype=torch.float64, requires_grad=True)
    v = torch.randn(B, T, HKV, V, dtype=torch.float64, requires_grad=True)
    do = torch.randn(B, T, HQ, V, dtype=torch.float64)
    ty = make_types(B, NB, HN, 0.5, 4, force_last=False)
    bias = torch.zeros(B, NB, HQ, dtype=torch.float64, requires_grad=True)
    scale = K ** -0.5
    blk = torch.arange(T) // block
    later = (blk.view(-1, 1) > blk.view(1, -1)).double()
    loss = 0
    for b in range(B):
        for hq in range(HQ):
            m = sb.visibility_mask(torch.round(ty[b, :, hq // (HQ // HN), 0]), T, block, same_block)
            s = (q[b, :, hq] @ k[b, :, hq // (HQ // HKV)].T) * scale + bias[b, blk, hq].view(1, -1) * later
            s = s.masked_fill(~m, -1e300)
            p = torch.softmax(s, -1) * m
            loss = loss + ((p @ v[b, :, hq // (HQ // HKV)]) * do[b, :, hq]).sum()
    gq, gk, gv, gb = torch.autograd.grad(loss, (q, k, v, bias))
    dq, dk, dv, dnats = sb.softmax_branch_bwd(q.detach(), k.detach(), v.detach(), ty, do, scale, block, same_block)
    a = torch.round(ty[..., 0]).double()
    want_dnats = (gb.view(B, NB, HN, HQ // HN).sum(-1)) * a                     # attention-typed blocks only
    for got, want, name in ((dq, gq, 'dq'), (dk, gk, 'dk'), (dv, gv, 'dv'), (dnats, want_dnats, 'dnats')):
        assert float((got - want).abs().max()) < 1e-9, name


@pytest.mark.parametrize("same_block", [True, False])
def test_softmax_backward_dnats_of_blocks_that_are_not_attention(same_block):
    """compute_dnats_for_invalid_blocks_attn: a block that is not typed attention gets sum min(exp(s - lse), 1) (dP - delta)
    over its keys and the later queries.  Without the clamp that is an exact derivative: give the block's keys the weight
    eps * exp(s) in the softmax of later queries, and differentiate the loss with respect to eps at eps = 0 (autograd
    below, against the oracle with its clamp switched off); the clamped expression is checked against plain loops (a
    query at the start of its block sees few keys, so earlier keys do exceed its lse)."""
    from oracle import softmax_branch as sb
    from tests._util import make_types
    torch.manual_seed(5)
    B, T, HQ, HKV, HN, K, V, block = 1, 200, 4, 2, 2, 16, 8, 64
    NB = -(-T // block)
    ty = make_types(B, NB, HN, 0.4, 6, force_last=False)
    a = torch.round(ty[..., 0]).double()
    blk = torch.arange(T) // block
    later = (blk.view(-1, 1) > blk.view(1, -1)).double()
    for big in (False, True):
        q = torch.randn(B, T, HQ, K, dtype=torch.float64) * (6.0 if big else 0.3)
        k = torch.randn(B, T, HKV, K, dtype=torch.float64)
        v = torch.randn(B, T, HKV, V, dtype=torch.float64)
        do = torch.randn(B, T, HQ, V, dtype=torch.float64)
        scale = K ** -0.5
        *_, dn0 = sb.softmax_branch_bwd(q, k, v, ty, do, scale, block, same_block)
        *_, dn1 = sb.softmax_branch_bwd(q, k, v, ty, do, scale, block, same_block, dnats_invalid=True)
        assert torch.equal(dn1 * a, dn0 * a), "attention-typed blocks keep their dnats"
        if not big:
            eps = torch.zeros(B, NB, HQ, dtype=torch.float64, requires_grad=True)
            loss = 0
            for hq in range(HQ):
                hn, hk = hq // (HQ // HN), hq // (HQ // HKV)
                m = sb.visibility_mask(a[0, :, hn], T, block, same_block).double()
                e = torch.exp((q[0, :, hq] @ k[0, :, hk].T) * scale)
                w = e * m + e * later * ((1 - a[0, :, hn]) * eps[0, :, hq])[blk].view(1, -1)
                z = w.sum(-1, keepdim=True)
                seen = m.sum(-1, keepdim=True) > 0
                p = torch.where(seen, w / torch.where(seen, z, torch.ones_like(z)), torch.zeros_like(w))
                loss = loss + ((p @ v[0, :, hk]) * do[0, :, hq]).sum()
            want = torch.autograd.grad(loss, eps)[0].view(B, NB, HN, HQ // HN).sum(-1) * (1 - a)
            *_, dn_free = sb.softmax_branch_bwd(q, k, v, ty, do, scale, block, same_block, dnats_invalid=True, clamp_invalid=False)
            got = dn_free * (1 - a)
            if same_block:   # (a query that sees nothing has no normaliser: the oracle then uses lse = 0, the gate form 0)
                assert float((got - want).abs().max()) < 1e-9
            else:
                rows_seen = torch.stack([sb.visibility_mask(a[0, :, hn], T, block, same_block).any(-1) for hn in range(HN)])
                assert not bool(rows_seen.all()), "the case is meant to hold queries that see nothing"
        else:
            want = torch.zeros(B, NB, HN, dtype=torch.float64)
            clamped = 0
            for hq in range(HQ):
                hn, hk = hq // (HQ // HN), hq // (HQ // HKV)
                m = sb.visibility_mask(a[0, :, hn], T, block, same_block)
                s = (q[0, :, hq] @ k[0, :, hk].T) * scale
                for t in range(T):
                    vis = m[t]
                    lse = torch.logsumexp(s[t][vis], 0) if bool(vis.any()) else torch.zeros((), dtype=torch.float64)
                    pv = torch.exp(s[t][vis] - lse) if bool(vis.any()) else torch.zeros(0, dtype=torch.float64)
                    o_t = pv @ v[0, vis, hk] if bool(vis.any()) else torch.zeros(V, dtype=torch.float64)
                    delta = (do[0, t, hq] * o_t).sum()
                    for j in range(int(blk[t])):
                        if a[0, j, hn] == 0:
                            ks = slice(j * block, min((j + 1) * block, T))
                            p1 = torch.exp(s[t, ks] - lse)
                            clamped += int((p1 > 1).sum())
                            want[0, j, hn] += (p1.clamp(max=1.0) * (v[0, ks, hk] @ do[0, t, hq] - delta)).sum()
            assert clamped > 0, "the case is meant to need the clamp"
            assert float((dn1 * (1 - a) - want).abs().max()) < 1e-8 * float(want.abs().max())


# --------------------------------------------------------------------------------------------
# gradients of the linear branches (the oracle of the mixed operators' backward)
# --------------------------------------------------------------------------------------------
def test_linear_branch_gradients_match_finite_differences_and_the_token_recurrence():
    """linear_branch_bwd is autograd through the chunked form; pinned by (i) autograd through the token-by-token
    recurrence (a different computation of the same function) and (ii) central differences of the gates: the selector
    gradient of a block typed linear is d loss / d (gate on its update), that of a block not typed linear
    d loss / d (zero gate on the update it would have made)."""
    import torch.nn.functional as F
    from oracle import linear_branch as LB
    g_ = torch.Generator().manual_seed(3)
    B, T, H, K, V, block = 1, 256, 2, 16, 8, 64
    q, k, v = (torch.randn(B, T, H, d, generator=g_, dtype=torch.float64) for d in (K, K, V))
    beta = torch.sigmoid(torch.randn(B, T, H, generator=g_, dtype=torch.float64))
    g = -F.softplus(torch.randn(B, T, H, generator=g_, dtype=torch.float64))
    lin = torch.tensor([1., 0., 0., 1.]).view(1, 4, 1).expand(1, 4, 2).contiguous()
    do = torch.randn(B, T, H, V, generator=g_, dtype=torch.float64)
    dht = torch.randn(B, H, K, V, generator=g_, dtype=torch.float64)
    r = LB.linear_branch_bwd('gdn', q, k, v, g, beta, lin, 0.3, do, dht, None, block, True, True, True, True)
    # (i) the same gradients through the token recurrence
    leaves = [t.clone().requires_grad_(True) for t in (q, k, v, g, beta)]
    o, S = LB.gdn_token_recurrence(*leaves, lin, 0.3, None, block, True, True, torch.float64)
    ((o * do).sum() + (S * dht).sum()).backward()
    for name, t in zip(('dq', 'dk', 'dv', 'dg', 'dbeta'), leaves):
        assert torch.allclose(r[name], t.grad, rtol=1e-7, atol=1e-9), name
    # (ii) gates by central differences
    NT = T // 64

    def loss(gate_on, gate_off):
        o, S = LB.gdn_chunked(q, k, v, g, beta, lin, 0.3, None, block, True, True, torch.float64, True, gate_on, gate_off)
        return float((o * do).sum() + (S * dht).sum())
    eps = 1e-5
    for c in range(NT):
        for h in range(H):
            on, off = torch.ones(B, NT, H, dtype=torch.float64), torch.zeros(B, NT, H, dtype=torch.float64)
            which = on if lin[0, c, h] == 1 else off
            which[0, c, h] += eps
            up = loss(on, off)
            which[0, c, h] -= 2 * eps
            fd = (up - loss(on, off)) / (2 * eps)
            assert abs(fd - float(r['dnats'][0, c, h])) <= 1e-6 * max(1.0, abs(fd)), (c, h, fd, float(r['dnats'][0, c, h]))
    # without the gradient of the other blocks they get exactly zero
    r0 = LB.linear_branch_bwd('gdn', q, k, v, g, beta, lin, 0.3, do, dht, None, block, True, True, True, False)
    assert float(r0['dnats'][0, 1:3].abs().max()) == 0.0 and torch.equal(r0['dnats'][0, [0, 3]], r['dnats'][0, [0, 3]])
    # Mamba: against its token recurrence
    rm = LB.linear_branch_bwd('mamba', q, k, v, g, None, lin, 1.0, do, dht, None, block, True)
    leaves = [t.clone().requires_grad_(True) for t in (q, k, v, g)]
    o, S = LB.mamba_token_recurrence(*leaves, lin, 1.0, None, block, True, torch.float64)
    ((o * do).sum() + (S * dht).sum()).backward()
    for name, t in zip(('dq', 'dk', 'dv', 'dg'), leaves):
        assert torch.allclose(rm[name], t.grad, rtol=1e-7, atol=1e-9), name
