"""nats_mixed_attn_mamba: softmax branch + Mamba2-style SSD branch behind the reference's operator
API (src/nats/ops/mixed_ops/mixed_attn_mamba.py:295-332), forward only."""
from __future__ import annotations

from dataclasses import dataclass

import torch

from ._mixed_common import mixed_forward

CHUNK_SIZE = 64


@dataclass
class RunIncompleteBlock:
    attn: bool = False
    mamba: bool = False


# src/nats/ops/mixed_ops/mixed_attn_mamba.py:39-46
all_incomplete_ops = {
    'all': RunIncompleteBlock(attn=True, mamba=True),
    'attn': RunIncompleteBlock(attn=True, mamba=False),
    'mamba': RunIncompleteBlock(attn=False, mamba=True),
}


def nats_mixed_attn_mamba(
        q_attn: torch.Tensor, k_attn: torch.Tensor, v_attn: torch.Tensor,
        q_lattn: torch.Tensor, k_lattn: torch.Tensor, v_lattn: torch.Tensor,
        initial_state_mamba: torch.Tensor,
        g: torch.Tensor,
        nats_block_types: torch.Tensor,
        n_nats_blocks: torch.Tensor,
        scale_attn=None, scale_lattn=None,
        cu_seqlens=None, cu_seqlens_nats=None,
        nats_block_size: int = 64,
        attn_sw_size: int | None = None,
        ops_for_incomplete_chunks: str = 'all',
        output_final_state_mamba: bool = False,
        compute_dnats_for_invalid_blocks_attn: bool = False,
        compute_dnats_for_invalid_blocks_linear_att: bool = True,
        decay_for_non_mamba_blocks: bool = False,
        incomplete_block_start_with_ht: bool = True,
        use_g_for_attn: bool = False,
):
    """q_lattn = C, k_lattn = B, v_lattn = X*dt, g = A*dt -> (o_mamba, o_attn, final_state or None)."""
    strategy = all_incomplete_ops[ops_for_incomplete_chunks]
    if scale_attn is None:
        scale_attn = k_attn.shape[-1] ** -0.5
    if scale_lattn is None:
        scale_lattn = 1
    return mixed_forward(
        'mamba', q_attn, k_attn, v_attn, q_lattn, k_lattn, v_lattn, initial_state_mamba, g, None, nats_block_types,
        scale_attn, scale_lattn, cu_seqlens, cu_seqlens_nats, nats_block_size, attn_sw_size,
        attn_same_block=strategy.attn, lin_intra=strategy.mamba,
        output_final_state=output_final_state_mamba, decay_non_linear=decay_for_non_mamba_blocks,
        incomplete_block_start_with_ht=incomplete_block_start_with_ht, use_g_for_attn=use_g_for_attn,
        qk_l2norm=False)


def nats_mixed_attn_mamba_chunk_inference(
        q_attn: torch.Tensor, k_attn: torch.Tensor, v_attn: torch.Tensor,
        q_lattn: torch.Tensor, k_lattn: torch.Tensor, v_lattn: torch.Tensor,
        initial_state_mamba_start: torch.Tensor,
        g: torch.Tensor,
        nats_block_types: torch.Tensor,
        op_type_last_chunk: torch.Tensor | None,
        n_nats_blocks: torch.Tensor,
        n_tokens_in_current_block: int = 0,
        scale_attn=None, scale_lattn=None,
        cu_seqlens=None, cu_seqlens_nats=None,
        nats_block_size: int = 64,
        ops_for_incomplete_chunks: str = 'all',
        output_final_state_mamba: bool = True,
        decay_for_non_mamba_blocks: bool = True,
        incomplete_block_start_with_ht: bool = True,
        use_g_for_attn: bool = False,
):
    """Prefill variant (src/nats/ops/mixed_ops/mixed_attn_mamba.py:363-457):
    -> (o_mamba, o_attn, final_state, state at the start of the current block).
    As in the reference, scale_lattn defaults to K**-0.5 HERE (and to 1 in nats_mixed_attn_mamba)."""
    strategy = all_incomplete_ops[ops_for_incomplete_chunks]
    if scale_attn is None:
        scale_attn = k_attn.shape[-1] ** -0.5
    if scale_lattn is None:
        scale_lattn = k_lattn.shape[-1] ** -0.5
    return mixed_forward(
        'mamba', q_attn, k_attn, v_attn, q_lattn, k_lattn, v_lattn, initial_state_mamba_start, g, None, nats_block_types,
        scale_attn, scale_lattn, cu_seqlens, cu_seqlens_nats, nats_block_size, None,
        attn_same_block=strategy.attn, lin_intra=strategy.mamba,
        output_final_state=output_final_state_mamba, decay_non_linear=decay_for_non_mamba_blocks,
        incomplete_block_start_with_ht=incomplete_block_start_with_ht, use_g_for_attn=use_g_for_attn,
        qk_l2norm=False, inference=True, op_type_last_chunk=op_type_last_chunk,
        n_tokens_in_current_block=n_tokens_in_current_block)
