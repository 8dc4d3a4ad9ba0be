"""Oracle for the two hybrid layers' forward (training mode, no cache).

TEST INFRASTRUCTURE ONLY -- see oracle/__init__.py.

Restates NeuralAttentionSearchLinearAttnGDN.forward (src/nats/layers/natsl_attn_gdn.py:368-666) and
NeuralAttentionSearchLinearAttnMamba.forward (src/nats/layers/natsl_attn_mamba2.py:311-599) on a plain
dict of fp32 weights, using the oracle's own branches.  The selector decision can be injected
(`types`): a GEMM computed in bf16 on another device may round a near-tie logit pair differently, and
the mask is compared bit-exactly on its own.  Parity unpinned by reference fixtures (there are none);
each piece it calls is pinned in tests/test_oracle_*.py.
"""
import torch
import torch.nn.functional as F

from . import mixed, norm_gate, routing
from .linear_branch import l2norm


def _conv(x, w, act=True):
    """fla ShortConvolution: depthwise causal conv over time (weight [D,1,W]) then SiLU."""
    D, W = w.shape[0], w.shape[-1]
    y = F.conv1d(x.transpose(1, 2), w, None, padding=W - 1, groups=D)[..., :x.shape[1]].transpose(1, 2)
    return F.silu(y) if act else y


def _rms(x, w, eps):
    return x * torch.rsqrt(x.pow(2).mean(-1, keepdim=True) + eps) * w


def gdn_layer(w, cfg, hidden, types=None):
    """w: state dict (fp32 tensors); cfg: dict with head_dim, num_heads, num_attn_heads, expand_v, nats_block_size,
    num_nats_head, attn_qk_norm, attn_with_short_conv, decay_for_non_gdn_blocks, ops_for_incomplete_chunks, norm_eps."""
    x = hidden.float()
    B, T, _ = x.shape
    H, Dk = cfg['num_heads'], cfg['head_dim']
    Dv = int(Dk * cfg['expand_v'])
    HA = cfg['num_attn_heads']
    blk = cfg['nats_block_size']
    if types is None:
        pooled = routing.mean_pool(hidden, blk).float()
        logits = (pooled @ w['nats_layer.weight'].T).to(hidden.dtype).unflatten(-1, (cfg['num_nats_head'], 2))
        types = routing.force_last_block(routing.hard_select(logits))
    lin = lambda name, t: t @ w[name + '.weight'].T
    if cfg.get('attn_with_short_conv', True):
        q, k, v = (_conv(lin(n + '_proj', x), w[n + '_conv1d.weight']) for n in ('q', 'k', 'v'))
        q_attn, k_attn, v_attn = q, k, v
    else:
        q_attn, k_attn, v_attn = lin('q_proj', x), lin('k_proj', x), lin('v_proj', x)
        q, k, v = (_conv(t, w[n + '_conv1d.weight']) for n, t in (('q', q_attn), ('k', k_attn), ('v', v_attn)))
    o_weights = lin('nats_out_weights_layer', q).unflatten(-1, (HA, 2)).softmax(-1)
    q, k = q.unflatten(-1, (H, Dk)), k.unflatten(-1, (H, Dk))
    v = v.unflatten(-1, (H, Dv))
    q_attn, k_attn = (t.unflatten(-1, (HA, -1)) for t in (q_attn, k_attn))
    v_attn = v_attn.unflatten(-1, (HA, -1))
    if cfg.get('attn_qk_norm', True):
        q_attn, k_attn = _rms(q_attn, w['q_norm.weight'], cfg['norm_eps']), _rms(k_attn, w['k_norm.weight'], cfg['norm_eps'])
    beta = torch.sigmoid(lin('b_proj', x))
    g = -torch.exp(w['A_log']) * F.softplus(lin('a_proj', x) + w['dt_bias'])
    o_lin, o_attn, _, _ = mixed.mixed_attn_gdn(q_attn, k_attn, v_attn, q, k, v, None, g, beta, types,
                                               nats_block_size=blk, ops_for_incomplete_chunks=cfg['ops_for_incomplete_chunks'],
                                               decay_for_non_gdn_blocks=cfg['decay_for_non_gdn_blocks'])
    gate = lin('g_proj', x).unflatten(-1, (H, Dv))
    y = norm_gate.two_input_rmsnorm_gated(o_lin.reshape(o_attn.shape), o_attn, gate.reshape(o_attn.shape), o_weights,
                                          w['o_norm.weight1'], w['o_norm.weight2'], cfg['norm_eps'])
    return lin('o_proj', y.flatten(-2)), types


def mamba_layer(w, cfg, hidden, types=None):
    x = hidden.float()
    H, Dk = cfg['num_heads'], cfg['head_dim']
    Dv = int(Dk * cfg['expand_v'])
    HA = cfg['num_attn_heads']
    blk = cfg['nats_block_size']
    if types is None:
        pooled = routing.mean_pool(hidden, blk).float()
        logits = (pooled @ w['nats_layer.weight'].T).to(hidden.dtype).unflatten(-1, (cfg['num_nats_head'], 2))
        types = routing.force_last_block(routing.hard_select(logits))
    lin = lambda name, t: t @ w[name + '.weight'].T
    q_attn, k_attn, v_attn = lin('q_proj', x), lin('k_proj', x), lin('v_proj', x)      # attn_with_short_conv=False (default)
    q, k, v = (_conv(t, w[n + '_conv1d.weight']) for n, t in (('q', q_attn), ('k', k_attn), ('v', v_attn)))
    o_weights = lin('nats_out_weights_layer', q).unflatten(-1, (HA, 2)).softmax(-1)
    q, k = q.unflatten(-1, (H, Dk)), k.unflatten(-1, (H, Dk))
    v = v.unflatten(-1, (H, Dv))
    q_attn, k_attn = (t.unflatten(-1, (HA, -1)) for t in (q_attn, k_attn))
    v_attn = v_attn.unflatten(-1, (HA, -1))
    q, k = l2norm(q, cfg['norm_eps']), l2norm(k, cfg['norm_eps'])
    dt = F.softplus(lin('a_proj', x) + w['dt_bias'])
    v = v * dt.unsqueeze(-1)
    g = -torch.exp(w['A_log']) * dt
    o_lin, o_attn, _, _ = mixed.mixed_attn_mamba(q_attn, k_attn, v_attn, q, k, v, None, g, types, scale_lattn=1,
                                                 nats_block_size=blk, ops_for_incomplete_chunks=cfg['ops_for_incomplete_chunks'],
                                                 decay_for_non_mamba_blocks=cfg['decay_for_non_mamba_blocks'])
    gate = lin('g_proj', x).unflatten(-1, (H, Dv))
    y = norm_gate.two_input_rmsnorm_gated(o_lin.reshape(o_attn.shape), o_attn, gate.reshape(o_attn.shape), o_weights,
                                          w['o_norm.weight1'], w['o_norm.weight2'], cfg['norm_eps'])
    return lin('o_proj', y.flatten(-2)), types
