"""Oracle for the two hybrid layers' forward (training mode, no cache).

TEST INFRASTRUCTURE ONLY -- see oracle/__init__.py.

Restates NeuralAttentionSearchLinearAttnGDN.forward (src/nats/layers/natsl_attn_gdn.py:368-666) and
NeuralAttentionSearchLinearAttnMamba.forward (src/nats/layers/natsl_attn_mamba2.py:311-599) on a plain
dict of fp32 weights, using the oracle's own branches.  The selector decision can be injected
(`types`): a GEMM computed in bf16 on another device may round a near-tie logit pair differently, and
the mask is compared bit-exactly on its own.

`act_dtype` restates the reference layer run as a bf16 module: every torch module or elementwise op of the
reference's forward (Linear, ShortConvolution, RMSNorm, sigmoid, softmax of the mix weights) returns a tensor
in the model dtype, so with act_dtype=torch.bfloat16 the oracle rounds at exactly those points and evaluates
the operators themselves (mixed op, norm-gate) in fp32 on the rounded tensors.  `g` stays fp32 as in the
reference (natsl_attn_gdn.py:530 computes it in float).  round_at='ops' restates an fp32 module whose operators
(mixed op, norm-gate) compute on bf16 copies of their inputs and return bf16-rounded outputs: only the operators'
inputs and outputs are rounded.

There is no reference fixture for the layers; what pins this file is tests/test_oracle_layer.py: invariances
that a wiring mistake breaks (which branch meets which mix-weight column and norm weight, which tensors the
attention view is cut from, causal convolution, strict causality of the whole layer = the reference's own
prefill-then-decode check at natsl_attn_gdn.py:669-712) and the reduction to oracle.mixed + F.rms_norm when
the projections are identities.
"""
import torch
import torch.nn.functional as F

from . import mixed, norm_gate, routing
from .linear_branch import l2norm


def _conv(x, w, act=True):
    """fla ShortConvolution: depthwise causal conv over time (weight [D,1,W]) then SiLU:
    y_t = sum_j w[j] x[t-(W-1)+j]."""
    D, W = w.shape[0], w.shape[-1]
    y = F.conv1d(x.transpose(1, 2), w, None, padding=W - 1, groups=D)[..., :x.shape[1]].transpose(1, 2)
    return F.silu(y) if act else y


def _rounders(act_dtype, round_at):
    """(rounding at module outputs, rounding at operator inputs/outputs)."""
    ident = lambda t: t
    if act_dtype is None:
        return ident, ident
    rnd = lambda t: t.to(act_dtype).float()
    assert round_at in ('modules', 'ops')
    return (rnd, rnd) if round_at == 'modules' else (ident, rnd)


def _rms(x, w, eps):
    return x * torch.rsqrt(x.pow(2).mean(-1, keepdim=True) + eps) * w


def _select(w, cfg, hidden, rnd):
    """Selector (natsl_attn_gdn.py:411-420, :553): block means -> nats_layer -> hard selection, last block forced."""
    pooled = routing.mean_pool(hidden, cfg['nats_block_size']).float()
    logits = (pooled @ w['nats_layer.weight'].T).to(hidden.dtype).unflatten(-1, (cfg['num_nats_head'], 2))
    return routing.force_last_block(routing.hard_select(logits))


def _tail(w, cfg, o_lin, o_attn, gate, o_weights, rnd, return_parts, types, rop=None):
    """Output norm-gate and projection (natsl_attn_gdn.py:650-664): x1 = linear branch meets weight1 and mix column
    0, x2 = softmax branch meets weight2 and mix column 1."""
    rop = rop or rnd
    gate, o_weights = rop(gate), rop(o_weights)
    y = rop(norm_gate.two_input_rmsnorm_gated(o_lin.reshape(o_attn.shape), o_attn, gate.reshape(o_attn.shape), o_weights,
                                              w['o_norm.weight1'], w['o_norm.weight2'], cfg['norm_eps']))
    out = rnd(y.flatten(-2) @ w['o_proj.weight'].T)
    if return_parts:
        return out, types, dict(o_lin=o_lin, o_attn=o_attn, gate=gate, o_weights=o_weights, y=y)
    return out, types


def gdn_layer(w, cfg, hidden, types=None, act_dtype=None, return_parts=False, round_at='modules'):
    """w: state dict (fp32 tensors); cfg: dict with head_dim, num_heads, num_attn_heads, expand_v, nats_block_size,
    num_nats_head, attn_qk_norm, attn_with_short_conv, decay_for_non_gdn_blocks, ops_for_incomplete_chunks, norm_eps.
    Returns (output [B,T,hidden], types) and, with return_parts, a dict of the tensors that enter the tail."""
    rnd, rop = _rounders(act_dtype, round_at)
    x = hidden.float()
    H, Dk = cfg['num_heads'], cfg['head_dim']
    Dv = int(Dk * cfg['expand_v'])
    HA = cfg['num_attn_heads']
    blk = cfg['nats_block_size']
    if types is None:
        types = _select(w, cfg, hidden, rnd)
    lin = lambda name, t: rnd(t @ w[name + '.weight'].T)
    conv = lambda n, t: rnd(_conv(t, w[n + '_conv1d.weight']))
    if cfg.get('attn_with_short_conv', True):
        # natsl_attn_gdn.py:425-449: the attention view is cut from the convolved tensors
        q, k, v = (conv(n, lin(n + '_proj', x)) for n in ('q', 'k', 'v'))
        q_attn, k_attn, v_attn = q, k, v
    else:
        # natsl_attn_gdn.py:450-472: the attention view is the bare projection
        q_attn, k_attn, v_attn = lin('q_proj', x), lin('k_proj', x), lin('v_proj', x)
        q, k, v = conv('q', q_attn), conv('k', k_attn), conv('v', v_attn)
    o_weights = rnd(rnd(q @ w['nats_out_weights_layer.weight'].T).unflatten(-1, (HA, 2)).softmax(-1))   # :491
    q, k = q.unflatten(-1, (H, Dk)), k.unflatten(-1, (H, Dk))
    v = v.unflatten(-1, (H, Dv))
    q_attn, k_attn = (t.unflatten(-1, (HA, -1)) for t in (q_attn, k_attn))
    v_attn = v_attn.unflatten(-1, (HA, -1))
    if cfg.get('attn_qk_norm', True):
        q_attn = rnd(_rms(q_attn, w['q_norm.weight'], cfg['norm_eps']))
        k_attn = rnd(_rms(k_attn, w['k_norm.weight'], cfg['norm_eps']))
    beta = rnd(torch.sigmoid(lin('b_proj', x)))
    g = -torch.exp(w['A_log']) * F.softplus(lin('a_proj', x) + w['dt_bias'])           # fp32 in the reference (:530)
    q_attn, k_attn, v_attn, q, k, v, beta = (rop(t) for t in (q_attn, k_attn, v_attn, q, k, v, beta))
    o_lin, o_attn, _, _ = mixed.mixed_attn_gdn(q_attn, k_attn, v_attn, q, k, v, None, g, beta, types,
                                               nats_block_size=blk, ops_for_incomplete_chunks=cfg['ops_for_incomplete_chunks'],
                                               decay_for_non_gdn_blocks=cfg['decay_for_non_gdn_blocks'])
    o_lin, o_attn = rop(o_lin), rop(o_attn)
    gate = lin('g_proj', x).unflatten(-1, (H, Dv))
    return _tail(w, cfg, o_lin, o_attn, gate, o_weights, rnd, return_parts, types, rop)


def mamba_layer(w, cfg, hidden, types=None, act_dtype=None, return_parts=False, round_at='modules'):
    """NeuralAttentionSearchLinearAttnMamba.forward (natsl_attn_mamba2.py:311-599) with attn_with_short_conv=False
    (its default): q = C, k = B (L2-normalised, :469-470), v = x*dt (:473), g = A*dt (:474), scale_lattn = 1 (:505);
    the attention view takes the un-scaled v (:391-393)."""
    rnd, rop = _rounders(act_dtype, round_at)
    x = hidden.float()
    H, Dk = cfg['num_heads'], cfg['head_dim']
    Dv = int(Dk * cfg['expand_v'])
    HA = cfg['num_attn_heads']
    blk = cfg['nats_block_size']
    if types is None:
        types = _select(w, cfg, hidden, rnd)
    lin = lambda name, t: rnd(t @ w[name + '.weight'].T)
    conv = lambda n, t: rnd(_conv(t, w[n + '_conv1d.weight']))
    q_attn, k_attn, v_attn = lin('q_proj', x), lin('k_proj', x), lin('v_proj', x)
    q, k, v = conv('q', q_attn), conv('k', k_attn), conv('v', v_attn)
    o_weights = rnd(rnd(q @ w['nats_out_weights_layer.weight'].T).unflatten(-1, (HA, 2)).softmax(-1))
    q, k = q.unflatten(-1, (H, Dk)), k.unflatten(-1, (H, Dk))
    v = v.unflatten(-1, (H, Dv))
    q_attn, k_attn = (t.unflatten(-1, (HA, -1)) for t in (q_attn, k_attn))
    v_attn = v_attn.unflatten(-1, (HA, -1))
    if cfg.get('attn_qk_norm', False):                                                 # :447-448 (off by default)
        q_attn = rnd(_rms(q_attn, w['q_norm.weight'], cfg['norm_eps']))
        k_attn = rnd(_rms(k_attn, w['k_norm.weight'], cfg['norm_eps']))
    q, k = rnd(l2norm(q, cfg['norm_eps'])), rnd(l2norm(k, cfg['norm_eps']))
    dt = F.softplus(lin('a_proj', x) + w['dt_bias'])
    v = rnd(v * dt.unsqueeze(-1))
    g = -torch.exp(w['A_log']) * dt
    q_attn, k_attn, v_attn, q, k, v = (rop(t) for t in (q_attn, k_attn, v_attn, q, k, v))
    o_lin, o_attn, _, _ = mixed.mixed_attn_mamba(q_attn, k_attn, v_attn, q, k, v, None, g, types, scale_lattn=1,
                                                 nats_block_size=blk, ops_for_incomplete_chunks=cfg['ops_for_incomplete_chunks'],
                                                 decay_for_non_mamba_blocks=cfg['decay_for_non_mamba_blocks'])
    o_lin, o_attn = rop(o_lin), rop(o_attn)
    gate = lin('g_proj', x).unflatten(-1, (H, Dv))
    return _tail(w, cfg, o_lin, o_attn, gate, o_weights, rnd, return_parts, types, rop)
