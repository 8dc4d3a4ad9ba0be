"""Oracle for the mixed operators (softmax branch + linear branch behind one call).

TEST INFRASTRUCTURE ONLY -- see oracle/__init__.py.

Mirrors NAtSMixedAttentionGDN.forward (src/nats/ops/mixed_ops/mixed_attn_gdn.py:47-191)
and NAtSMixedAttentionMamba.forward (src/nats/ops/mixed_ops/mixed_attn_mamba.py:51-192).
Variable-length input (cu_seqlens) is defined as independent evaluation of each
packed sequence: the reference's layers never exercise that path.  Parity
unpinned by any reference fixture for cu_seqlens and for block sizes above 64
(the reference indexes its state array inconsistently there); both are pinned
instead by the token-level recurrence with roll-back at block ends.
"""
from __future__ import annotations

import torch

from . import linear_branch as lb
from . import softmax_branch as sb

# ops_for_incomplete_chunks -> (softmax branch sees its own block, linear branch adds the intra-chunk term)
# src/nats/ops/mixed_ops/mixed_attn_gdn.py:35-42, src/nats/ops/mixed_ops/mixed_attn_mamba.py:39-46
MODES = {
    'all': (True, True),
    'attn': (True, False),
    'gated_delta_net': (False, True),
    'mamba': (False, True),
}


def _sequences(T, cu_seqlens, cu_seqlens_nats, block):
    if cu_seqlens is None:
        return None
    cu = [int(x) for x in cu_seqlens]
    if cu_seqlens_nats is None:
        cn = [0]
        for i in range(len(cu) - 1):
            cn.append(cn[-1] + -(-(cu[i + 1] - cu[i]) // block))
    else:
        cn = [int(x) for x in cu_seqlens_nats]
    return list(zip(cu[:-1], cu[1:], cn[:-1], cn[1:]))


def mixed_attn_gdn(q_attn, k_attn, v_attn, q_lattn, k_lattn, v_lattn, initial_state, g, beta, nats_block_types,
                   scale_attn=None, scale_lattn=None, cu_seqlens=None, cu_seqlens_nats=None, nats_block_size=64,
                   ops_for_incomplete_chunks='gated_delta_net', output_final_state=False,
                   decay_for_non_gdn_blocks=False, lattn_use_qk_l2norm_in_kernel=True, dtype=torch.float32,
                   token_level=False):
    """-> (o_lin [B,T,H,V], o_attn [B,T,HQ,Va], final_state [N,H,K,V] or None, lse [B,T,HQ])."""
    scale_attn = k_attn.shape[-1] ** -0.5 if scale_attn is None else scale_attn
    scale_lattn = k_lattn.shape[-1] ** -0.5 if scale_lattn is None else scale_lattn
    attn_same_block, lin_intra = MODES[ops_for_incomplete_chunks]
    types = torch.round(nats_block_types.float())

    def one(sl_t, sl_n, h0):
        ty = types[:, sl_n]
        o_attn, lse = sb.softmax_branch(q_attn[:, sl_t], k_attn[:, sl_t], v_attn[:, sl_t], ty, scale_attn,
                                        nats_block_size, attn_same_block, dtype)
        if token_level:
            assert lin_intra
            o_lin, S = lb.gdn_token_recurrence(q_lattn[:, sl_t], k_lattn[:, sl_t], v_lattn[:, sl_t], g[:, sl_t],
                                               beta[:, sl_t], ty[..., 1], scale_lattn, h0, nats_block_size,
                                               decay_for_non_gdn_blocks, lattn_use_qk_l2norm_in_kernel, dtype)
        else:
            o_lin, S = lb.gdn_chunked(q_lattn[:, sl_t], k_lattn[:, sl_t], v_lattn[:, sl_t], g[:, sl_t], beta[:, sl_t],
                                      ty[..., 1], scale_lattn, h0, nats_block_size, decay_for_non_gdn_blocks,
                                      lattn_use_qk_l2norm_in_kernel, dtype, lin_intra)
        return o_lin, o_attn, S, lse

    return _run(one, q_lattn.shape[1], initial_state, cu_seqlens, cu_seqlens_nats, nats_block_size, output_final_state)


def mixed_attn_mamba(q_attn, k_attn, v_attn, q_lattn, k_lattn, v_lattn, initial_state, g, nats_block_types,
                     scale_attn=None, scale_lattn=None, cu_seqlens=None, cu_seqlens_nats=None, nats_block_size=64,
                     ops_for_incomplete_chunks='all', output_final_state=False, decay_for_non_mamba_blocks=False,
                     dtype=torch.float32, token_level=False):
    scale_attn = k_attn.shape[-1] ** -0.5 if scale_attn is None else scale_attn
    scale_lattn = 1.0 if scale_lattn is None else scale_lattn      # src/nats/ops/mixed_ops/mixed_attn_mamba.py:316-317
    attn_same_block, lin_intra = MODES[ops_for_incomplete_chunks]
    types = torch.round(nats_block_types.float())

    def one(sl_t, sl_n, h0):
        ty = types[:, sl_n]
        o_attn, lse = sb.softmax_branch(q_attn[:, sl_t], k_attn[:, sl_t], v_attn[:, sl_t], ty, scale_attn,
                                        nats_block_size, attn_same_block, dtype)
        if token_level:
            assert lin_intra
            o_lin, S = lb.mamba_token_recurrence(q_lattn[:, sl_t], k_lattn[:, sl_t], v_lattn[:, sl_t], g[:, sl_t],
                                                 ty[..., 1], scale_lattn, h0, nats_block_size,
                                                 decay_for_non_mamba_blocks, dtype)
        else:
            o_lin, S = lb.mamba_chunked(q_lattn[:, sl_t], k_lattn[:, sl_t], v_lattn[:, sl_t], g[:, sl_t], ty[..., 1],
                                        scale_lattn, h0, nats_block_size, decay_for_non_mamba_blocks, dtype, lin_intra)
        return o_lin, o_attn, S, lse

    return _run(one, q_lattn.shape[1], initial_state, cu_seqlens, cu_seqlens_nats, nats_block_size, output_final_state)


def _run(one, T, initial_state, cu_seqlens, cu_seqlens_nats, block, output_final_state):
    seqs = _sequences(T, cu_seqlens, cu_seqlens_nats, block)
    if seqs is None:
        o_lin, o_attn, S, lse = one(slice(None), slice(None), initial_state)
        return o_lin, o_attn, (S if output_final_state else None), lse
    outs = []
    for n, (bos, eos, bn, en) in enumerate(seqs):
        h0 = None if initial_state is None else initial_state[n:n + 1]
        outs.append(one(slice(bos, eos), slice(bn, en), h0))
    o_lin = torch.cat([x[0] for x in outs], 1)
    o_attn = torch.cat([x[1] for x in outs], 1)
    S = torch.cat([x[2] for x in outs], 0)
    lse = torch.cat([x[3] for x in outs], 1)
    return o_lin, o_attn, (S if output_final_state else None), lse
