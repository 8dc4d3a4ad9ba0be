"""nats_mixed_attn_gdn: softmax branch + Gated DeltaNet branch behind the reference's operator API
(src/nats/ops/mixed_ops/mixed_attn_gdn.py:286-325), forward only."""
from __future__ import annotations

from dataclasses import dataclass

import torch

from ._mixed_common import mixed_forward

CHUNK_SIZE = 64


@dataclass
class RunIncompleteBlock:
    attn: bool = False
    gated_delta_net: bool = False


# src/nats/ops/mixed_ops/mixed_attn_gdn.py:35-42
all_incomplete_ops = {
    'all': RunIncompleteBlock(attn=True, gated_delta_net=True),
    'attn': RunIncompleteBlock(attn=True, gated_delta_net=False),
    'gated_delta_net': RunIncompleteBlock(attn=False, gated_delta_net=True),
}


def nats_mixed_attn_gdn(
        q_attn: torch.Tensor, k_attn: torch.Tensor, v_attn: torch.Tensor,
        q_lattn: torch.Tensor, k_lattn: torch.Tensor, v_lattn: torch.Tensor,
        initial_state_gated_delta: torch.Tensor,
        g: torch.Tensor,
        beta: torch.Tensor,
        nats_block_types: torch.Tensor,
        n_nats_blocks: torch.Tensor,
        scale_attn=None, scale_lattn=None,
        cu_seqlens=None, cu_seqlens_nats=None,
        nats_block_size: int = 64,
        attn_sw_size: int | None = None,
        ops_for_incomplete_chunks: str = 'gated_delta_net',
        output_final_state_gated_delta: bool = False,
        compute_dnats_for_invalid_blocks_attn: bool = False,
        compute_dnats_for_invalid_blocks_linear_att: bool = True,
        decay_for_non_gdn_blocks: bool = False,
        incomplete_block_start_with_ht: bool = True,
        use_g_for_attn: bool = False,
        lattn_use_qk_l2norm_in_kernel: bool = True,
):
    """-> (o_gated_delta_net [B,T,H,V], o_attn [B,T,HQ,Va], final_state fp32 [N,H,K,V] or None).

    n_nats_blocks and the two compute_dnats_* flags (backward-only) are accepted for signature
    compatibility; the block counts are recomputed on the device from nats_block_types.
    """
    strategy = all_incomplete_ops[ops_for_incomplete_chunks]
    if scale_attn is None:
        scale_attn = k_attn.shape[-1] ** -0.5
    if scale_lattn is None:
        scale_lattn = k_lattn.shape[-1] ** -0.5
    return mixed_forward(
        'gdn', q_attn, k_attn, v_attn, q_lattn, k_lattn, v_lattn, initial_state_gated_delta, g, beta, nats_block_types,
        scale_attn, scale_lattn, cu_seqlens, cu_seqlens_nats, nats_block_size, attn_sw_size,
        attn_same_block=strategy.attn, lin_intra=strategy.gated_delta_net,
        output_final_state=output_final_state_gated_delta, decay_non_linear=decay_for_non_gdn_blocks,
        incomplete_block_start_with_ht=incomplete_block_start_with_ht, use_g_for_attn=use_g_for_attn,
        qk_l2norm=lattn_use_qk_l2norm_in_kernel)


def nats_mixed_attn_gdn_chunk_inference(
        q_attn: torch.Tensor, k_attn: torch.Tensor, v_attn: torch.Tensor,
        q_lattn: torch.Tensor, k_lattn: torch.Tensor, v_lattn: torch.Tensor,
        initial_state_gated_delta_chunk_start: torch.Tensor,
        g: torch.Tensor,
        beta: torch.Tensor,
        nats_block_types: torch.Tensor,
        op_type_last_chunk: torch.Tensor | None,
        n_nats_blocks: torch.Tensor,
        n_tokens_in_current_block: int = 0,
        scale_attn=None, scale_lattn=None,
        cu_seqlens=None, cu_seqlens_nats=None,
        nats_block_size: int = 64,
        attn_sw_size: int | None = None,
        ops_for_incomplete_chunks: str = 'gated_delta_net',
        output_final_state_gated_delta: bool = False,
        decay_for_non_gdn_blocks: bool = False,
        incomplete_block_start_with_ht: bool = True,
        use_g_for_attn: bool = False,
        lattn_use_qk_l2norm_in_kernel: bool = True,
):
    """Prefill variant (src/nats/ops/mixed_ops/mixed_attn_gdn.py:328-440):
    -> (o_gated_delta_net, o_attn, final_state, state at the start of the current block)."""
    strategy = all_incomplete_ops[ops_for_incomplete_chunks]
    if scale_attn is None:
        scale_attn = k_attn.shape[-1] ** -0.5
    if scale_lattn is None:
        scale_lattn = k_lattn.shape[-1] ** -0.5
    return mixed_forward(
        'gdn', q_attn, k_attn, v_attn, q_lattn, k_lattn, v_lattn, initial_state_gated_delta_chunk_start, g, beta,
        nats_block_types, scale_attn, scale_lattn, cu_seqlens, cu_seqlens_nats, nats_block_size, attn_sw_size,
        attn_same_block=strategy.attn, lin_intra=strategy.gated_delta_net,
        output_final_state=output_final_state_gated_delta, decay_non_linear=decay_for_non_gdn_blocks,
        incomplete_block_start_with_ht=incomplete_block_start_with_ht, use_g_for_attn=use_g_for_attn,
        qk_l2norm=lattn_use_qk_l2norm_in_kernel, inference=True, op_type_last_chunk=op_type_last_chunk,
        n_tokens_in_current_block=n_tokens_in_current_block)
