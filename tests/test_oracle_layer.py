"""Pins for oracle/layer.py (CPU only).  The reference ships no fixture for its layers, so the layer oracle is pinned
by properties that a wiring mistake breaks, and by reduction to pieces that are pinned elsewhere:

  * which branch meets which mix-weight column and which norm weight (the x1/x2-versus-op-index trap:
    src/nats/layers/natsl_attn_gdn.py:652-661, src/nats/modules/fused_norm_gate.py:83-87);
  * identity projections and convolutions reduce the layer to oracle.mixed + torch.nn.functional.rms_norm;
  * attn_with_short_conv decides whether the attention view is cut after or before the convolution (:425-491);
  * the short convolution is causal with the taps in the order of torch's conv1d (explicit loop);
  * strict causality: the outputs for a prefix do not depend on what follows, block types included -- the property the
    reference's own check (prefill, then token-by-token decode == one full forward, :669-712) rests on;
  * the rounding switch `act_dtype` only rounds (bf16 run close to the fp32 run).
"""
import pytest
import torch
import torch.nn.functional as F

from oracle import layer as OL
from oracle import mixed as OM
from oracle import routing as R


def _weights(cfg, hidden_size, seed=0, kind='gdn'):
    g = torch.Generator().manual_seed(seed)
    H, Dk = cfg['num_heads'], cfg['head_dim']
    Dv = int(Dk * cfg['expand_v'])
    HA = cfg['num_attn_heads']
    kd, vd = H * Dk, H * Dv
    rn = lambda *s: torch.randn(*s, generator=g)
    w = {
        'q_proj.weight': rn(kd, hidden_size) / hidden_size ** 0.5, 'k_proj.weight': rn(kd, hidden_size) / hidden_size ** 0.5,
        'v_proj.weight': rn(vd, hidden_size) / hidden_size ** 0.5, 'g_proj.weight': rn(vd, hidden_size) / hidden_size ** 0.5,
        'a_proj.weight': rn(H, hidden_size) / hidden_size ** 0.5, 'b_proj.weight': rn(H, hidden_size) / hidden_size ** 0.5,
        'nats_layer.weight': rn(2 * cfg['num_nats_head'], hidden_size), 'nats_out_weights_layer.weight': rn(2 * HA, kd) / kd ** 0.5,
        'o_proj.weight': rn(hidden_size, vd) / vd ** 0.5, 'A_log': torch.log(torch.rand(H, generator=g) * 15 + 1),
        'dt_bias': rn(H) * 0.1, 'q_conv1d.weight': rn(kd, 1, 4) * 0.5, 'k_conv1d.weight': rn(kd, 1, 4) * 0.5,
        'v_conv1d.weight': rn(vd, 1, 4) * 0.5, 'o_norm.weight1': 1 + 0.1 * rn(vd // HA), 'o_norm.weight2': 1 + 0.1 * rn(vd // HA),
        'q_norm.weight': 1 + 0.1 * rn(kd // HA), 'k_norm.weight': 1 + 0.1 * rn(kd // HA),
    }
    return w


GDN = dict(head_dim=32, num_heads=2, num_attn_heads=4, expand_v=2, nats_block_size=64, num_nats_head=2, attn_qk_norm=True,
           attn_with_short_conv=True, decay_for_non_gdn_blocks=True, ops_for_incomplete_chunks='all', norm_eps=1e-5)
MAMBA = dict(head_dim=32, num_heads=4, num_attn_heads=4, expand_v=0.5, nats_block_size=64, num_nats_head=4,
             decay_for_non_mamba_blocks=True, ops_for_incomplete_chunks='all', norm_eps=1e-5)
CASES = [('gdn', GDN, OL.gdn_layer), ('mamba', MAMBA, OL.mamba_layer)]


def _flip(types, col):
    """Another valid selection that differs in column `col` only (the last block stays forced)."""
    t = types.clone()
    t[:, :-1, :, col] = 1 - t[:, :-1, :, col]
    return t


@pytest.mark.parametrize("kind,cfg,fn", CASES)
def test_branch_meets_its_own_mix_column_and_norm_weight(kind, cfg, fn):
    """weight2 = 0 silences the softmax branch: the output must then ignore the attention column of the types and follow
    the linear column; weight1 = 0 the other way round.  Swapping x1/x2, the weights or the mix columns breaks this."""
    D = 48
    w = _weights(cfg, D, 1, kind)
    x = torch.randn(2, 200, D, generator=torch.Generator().manual_seed(2))
    types = R.force_last_block(R.hard_select(torch.randn(2, 4, cfg['num_nats_head'], 2, generator=torch.Generator().manual_seed(3))))
    for silent, dead_col, live_col in (('o_norm.weight2', 0, 1), ('o_norm.weight1', 1, 0)):
        ws = dict(w)
        ws[silent] = torch.zeros_like(w[silent])
        base, _ = fn(ws, cfg, x, types=types)
        same, _ = fn(ws, cfg, x, types=_flip(types, dead_col))
        moved, _ = fn(ws, cfg, x, types=_flip(types, live_col))
        assert torch.equal(base, same), f"{silent}=0: output still depends on op {dead_col}"
        assert float((base - moved).abs().max()) > 1e-3, f"{silent}=0: output does not follow op {live_col}"
    # mix column 0 belongs to the linear branch (x1), column 1 to the softmax branch (x2): one-hot mix weights
    HA, Da = cfg['num_attn_heads'], w['o_norm.weight1'].numel()
    g = torch.Generator().manual_seed(4)
    o_lin, o_attn, o_other, gate = (torch.randn(2, 10, HA, Da, generator=g) for _ in range(4))
    onehot = lambda c: F.one_hot(torch.full((2, 10, HA), c), 2).float()
    tail = lambda a, b, xw: OL._tail(w, cfg, a, b, gate, xw, lambda t: t, False, None)[0]
    assert torch.equal(tail(o_lin, o_attn, onehot(0)), tail(o_lin, o_other, onehot(0)))
    assert torch.equal(tail(o_lin, o_attn, onehot(1)), tail(o_other, o_attn, onehot(1)))
    assert not torch.equal(tail(o_lin, o_attn, onehot(0)), tail(o_other, o_attn, onehot(0)))


def test_gdn_layer_reduces_to_the_mixed_operator_with_identity_projections():
    """q/k/v projections = identity blocks, convolutions = a unit tap at lag 0: the layer must equal
    o_proj(norm_gate(mixed_attn_gdn(silu(x) views))) assembled here from oracle.mixed, F.rms_norm and plain torch."""
    cfg = dict(GDN, expand_v=1, attn_qk_norm=False)
    H, Dk, HA = cfg['num_heads'], cfg['head_dim'], cfg['num_attn_heads']
    D = H * Dk
    w = _weights(cfg, D, 4)
    eye = torch.eye(D)
    for n in ('q', 'k', 'v'):
        w[n + '_proj.weight'] = eye.clone()
        tap = torch.zeros(D, 1, 4)
        tap[:, 0, 3] = 1.0                                   # last tap = lag 0
        w[n + '_conv1d.weight'] = tap
    gq, gk, gv = 0.5 + torch.rand(D), 0.5 + torch.rand(D), 0.5 + torch.rand(D)
    w['q_proj.weight'], w['k_proj.weight'], w['v_proj.weight'] = torch.diag(gq), torch.diag(gk), torch.diag(gv)
    x = torch.randn(1, 192, D, generator=torch.Generator().manual_seed(5))
    types = R.force_last_block(R.hard_select(torch.randn(1, 3, 2, 2, generator=torch.Generator().manual_seed(6))))
    out, _ = OL.gdn_layer(w, cfg, x, types=types)
    q, k, v = F.silu(x * gq), F.silu(x * gk), F.silu(x * gv)
    beta = torch.sigmoid(x @ w['b_proj.weight'].T)
    g = -w['A_log'].exp() * F.softplus(x @ w['a_proj.weight'].T + w['dt_bias'])
    hv = lambda t, h: t.unflatten(-1, (h, -1))
    o_lin, o_attn, _, _ = OM.mixed_attn_gdn(hv(q, HA), hv(k, HA), hv(v, HA), hv(q, H), hv(k, H), hv(v, H), None, g, beta, types,
                                            ops_for_incomplete_chunks='all', decay_for_non_gdn_blocks=True)
    xw = (q @ w['nats_out_weights_layer.weight'].T).unflatten(-1, (HA, 2)).softmax(-1)
    Da = D // HA
    n1 = F.rms_norm(o_lin.reshape(o_attn.shape), (Da,), w['o_norm.weight1'], 1e-5)
    n2 = F.rms_norm(o_attn, (Da,), w['o_norm.weight2'], 1e-5)
    gate = (x @ w['g_proj.weight'].T).reshape(o_attn.shape)
    y = (n1 * xw[..., 0:1] + n2 * xw[..., 1:2]) * F.silu(gate)
    ref = y.flatten(-2) @ w['o_proj.weight'].T
    assert torch.allclose(out, ref, rtol=1e-4, atol=1e-5), float((out - ref).abs().max())


def test_mamba_layer_reduces_to_the_mixed_operator_with_identity_projections():
    """The same for the Mamba2 layer: q = l2norm(silu(C)), k = l2norm(silu(B)), v = silu(x) * dt for the SSD branch, the bare
    projections (un-scaled v) for the attention view, g = -exp(A_log) dt, scale 1."""
    cfg = dict(MAMBA, expand_v=1)
    H, Dk, HA = cfg['num_heads'], cfg['head_dim'], cfg['num_attn_heads']
    D = H * Dk
    w = _weights(cfg, D, 7, 'mamba')
    for n in ('q', 'k', 'v'):
        w[n + '_proj.weight'] = torch.eye(D)
        tap = torch.zeros(D, 1, 4)
        tap[:, 0, 3] = 1.0
        w[n + '_conv1d.weight'] = tap
    x = torch.randn(1, 192, D, generator=torch.Generator().manual_seed(8))
    types = R.force_last_block(R.hard_select(torch.randn(1, 3, H, 2, generator=torch.Generator().manual_seed(9))))
    out, _ = OL.mamba_layer(w, cfg, x, types=types)
    hv = lambda t, h: t.unflatten(-1, (h, -1))
    s = F.silu(x)
    l2 = lambda t: t * torch.rsqrt((t * t).sum(-1, keepdim=True) + 1e-5)
    dt = F.softplus(x @ w['a_proj.weight'].T + w['dt_bias'])
    g = -w['A_log'].exp() * dt
    o_lin, o_attn, _, _ = OM.mixed_attn_mamba(hv(x, HA), hv(x, HA), hv(x, HA), l2(hv(s, H)), l2(hv(s, H)), hv(s, H) * dt.unsqueeze(-1),
                                              None, g, types, scale_lattn=1, ops_for_incomplete_chunks='all',
                                              decay_for_non_mamba_blocks=True)
    xw = (s @ w['nats_out_weights_layer.weight'].T).unflatten(-1, (HA, 2)).softmax(-1)
    Da = D // HA
    n1 = F.rms_norm(o_lin.reshape(o_attn.shape), (Da,), w['o_norm.weight1'], 1e-5)
    n2 = F.rms_norm(o_attn, (Da,), w['o_norm.weight2'], 1e-5)
    gate = (x @ w['g_proj.weight'].T).reshape(o_attn.shape)
    ref = ((n1 * xw[..., 0:1] + n2 * xw[..., 1:2]) * F.silu(gate)).flatten(-2) @ w['o_proj.weight'].T
    assert torch.allclose(out, ref, rtol=1e-4, atol=1e-5), float((out - ref).abs().max())


def test_attention_view_is_cut_after_or_before_the_convolution():
    """With the linear branch silenced (weight1 = 0) and constant mix weights, the output sees the convolution weights
    only through the attention view: it must move with them when attn_with_short_conv is on and must not when it is off."""
    D = 48
    x = torch.randn(1, 130, D, generator=torch.Generator().manual_seed(11))
    types = R.force_last_block(R.hard_select(torch.randn(1, 3, 2, 2, generator=torch.Generator().manual_seed(12))))
    for with_conv in (True, False):
        cfg = dict(GDN, attn_with_short_conv=with_conv)
        w = _weights(cfg, D, 10)
        w['o_norm.weight1'] = torch.zeros_like(w['o_norm.weight1'])
        w['nats_out_weights_layer.weight'] = torch.zeros_like(w['nats_out_weights_layer.weight'])
        a, _ = OL.gdn_layer(w, cfg, x, types=types)
        w2 = dict(w)
        for n in ('q', 'k', 'v'):
            w2[n + '_conv1d.weight'] = w[n + '_conv1d.weight'] * 1.5 + 0.1
        b, _ = OL.gdn_layer(w2, cfg, x, types=types)
        if with_conv:
            assert float((a - b).abs().max()) > 1e-3
        else:
            assert torch.equal(a, b)


def test_short_convolution_is_causal_with_conv1d_tap_order():
    g = torch.Generator().manual_seed(13)
    x, w = torch.randn(2, 9, 5, generator=g), torch.randn(5, 1, 4, generator=g)
    y = OL._conv(x, w, act=False)
    ref = torch.zeros_like(x)
    for t in range(9):
        for j in range(4):
            s = t - 3 + j
            if s >= 0:
                ref[:, t] += w[:, 0, j] * x[:, s]
    assert torch.allclose(y, ref, atol=1e-6)
    assert torch.allclose(OL._conv(x, w), F.silu(ref), atol=1e-6)


@pytest.mark.parametrize("kind,cfg,fn", CASES)
@pytest.mark.parametrize("mode", ['all', 'lin_only'])
def test_layer_is_strictly_causal(kind, cfg, fn, mode):
    """The output at token t depends on tokens <= t only, selector included: a block's type is decided from its own
    tokens and matters only to LATER blocks (as attention keys / through the roll-back at its end), and forcing the
    last block to both ops changes no output.  This is what lets the reference decode token by token after a prefill
    and reproduce the full forward (natsl_attn_gdn.py:669-712).  Checked with the selector live (types=None)."""
    D = 40
    if mode == 'lin_only':
        cfg = dict(cfg, ops_for_incomplete_chunks='gated_delta_net' if kind == 'gdn' else 'mamba')
    w = _weights(cfg, D, 14, kind)
    x = torch.randn(2, 300, D, generator=torch.Generator().manual_seed(15))
    full, ty_full = fn(w, cfg, x)
    for t1 in (300 - 44, 192, 100):
        part, ty_part = fn(w, cfg, x[:, :t1])
        assert torch.allclose(full[:, :t1], part, rtol=1e-4, atol=1e-5), f"prefix of {t1} tokens differs: {float((full[:, :t1] - part).abs().max()):.2e}"
        nb = t1 // 64                                        # complete blocks of the prefix keep their types
        assert torch.equal(ty_full[:, :nb][:, :max(nb - (t1 % 64 == 0), 0)], ty_part[:, :max(nb - (t1 % 64 == 0), 0)])
    x2 = x.clone()
    x2[:, 200:] += 1.0
    moved, _ = fn(w, cfg, x2)
    assert torch.allclose(full[:, :200], moved[:, :200], rtol=1e-4, atol=1e-5) and float((full[:, 200:] - moved[:, 200:]).abs().max()) > 1e-3


@pytest.mark.parametrize("kind,cfg,fn", CASES)
def test_act_dtype_only_rounds(kind, cfg, fn):
    D = 64
    w = {k: v.bfloat16().float() for k, v in _weights(cfg, D, 16, kind).items()}
    x = torch.randn(1, 160, D, generator=torch.Generator().manual_seed(17)).bfloat16()
    types = R.force_last_block(R.hard_select(torch.randn(1, 3, cfg['num_nats_head'], 2, generator=torch.Generator().manual_seed(18))))
    a, _ = fn(w, cfg, x, types=types)
    b, _ = fn(w, cfg, x, types=types, act_dtype=torch.bfloat16)
    assert torch.equal(b, b.bfloat16().float())
    rel = float((a - b).norm() / a.norm())
    assert 0 < rel < 2e-2, rel
