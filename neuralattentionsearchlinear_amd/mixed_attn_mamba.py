"""nats_mixed_attn_mamba: softmax branch + Mamba2-style SSD branch behind the reference's operator
API (src/nats/ops/mixed_ops/mixed_attn_mamba.py:295-332)."""
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
        qk_l2norm=False,
        dnats_invalid_attn=compute_dnats_for_invalid_blocks_attn,
        dnats_invalid_linear=compute_dnats_for_invalid_blocks_linear_att)


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
        attn_prefix_valid: torch.Tensor | None = None,
):
    """Prefill variant (src/nats/ops/mixed_ops/mixed_attn_mamba.py:363-457):
    -> (o_mamba, o_attn, final_state, state at the start of the current block).
    As in the reference, scale_lattn defaults to K**-0.5 HERE (and to 1 in nats_mixed_attn_mamba).
    attn_prefix_valid (not in the reference): k_attn / v_attn start with that many more whole blocks of cached keys, visible
    per selector head where the flag is set; see _mixed_common._mixed_forward_impl."""
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
        n_tokens_in_current_block=n_tokens_in_current_block, attn_prefix_valid=attn_prefix_valid)


def fused_recurrent_mamba_nats_fwd(q, k, v, g, g_cumsum, nats_block_types, n_tokens_in_current_block, nats_block_size, scale,
                                   initial_state, initial_state_in_current_block, output_final_state=True,
                                   decay_for_non_mamba_blocks=False, query_only=False):
    """The SSD recurrence token by token on a cached state, for tokens that continue the current selector block
    (src/nats/ops/mamba/fused_recurrent.py with update_hs_for_each_iter=True).
    -> (o, final_state or None, initial_state_in_current_block), the last updated in place when the tokens
    complete the block.
    query_only: o_t = scale q_t^T (e^(g_cumsum + g_1..t) times initial_state_in_current_block); k, v are not read (may be
    None) and no state is written."""
    from . import _capi
    N, T, H, K = q.shape
    if query_only:
        if initial_state_in_current_block is None:
            raise ValueError("query_only needs the state that entered the block")
        k, v = q, q                               # placeholders: the kernel does not read them in this mode
    V = initial_state_in_current_block.shape[-1] if query_only else v.shape[-1]
    if nats_block_types.shape[1] != 1:
        raise AssertionError("the recurrent form only continues the current selector block: nats_block_types must hold one block")
    HN = nats_block_types.shape[2]
    dev = q.device
    q, k, v = (t.contiguous() for t in (q, k, v))
    if not (q.dtype == k.dtype == v.dtype):
        raise ValueError("q, k, v must share a dtype")
    g = g.to(torch.float32).contiguous()
    types = nats_block_types if nats_block_types.dtype in (torch.float32, torch.bfloat16) else nats_block_types.float()
    types = types.contiguous()
    if initial_state is not None:
        initial_state = initial_state.to(torch.float32).contiguous()
    if initial_state_in_current_block is None:
        initial_state_in_current_block = (initial_state.clone() if initial_state is not None
                                          else torch.zeros(N, H, K, V, dtype=torch.float32, device=dev))
    if initial_state_in_current_block.dtype != torch.float32 or not initial_state_in_current_block.is_contiguous():
        raise ValueError("initial_state_in_current_block must be a contiguous fp32 tensor (it is updated in place)")
    if g_cumsum is not None:
        g_cumsum = g_cumsum.to(torch.float32).reshape(N, H).contiguous()
    if torch.is_tensor(n_tokens_in_current_block):
        n_ptr, n_scalar = n_tokens_in_current_block.to(device=dev, dtype=torch.int32).contiguous(), 0
    else:
        n_ptr, n_scalar = None, int(n_tokens_in_current_block)
    o = torch.empty(N, T, H, V, dtype=q.dtype, device=dev)
    ht = torch.empty(N, H, K, V, dtype=torch.float32, device=dev) if output_final_state and not query_only else None
    flags = (_capi.DECAY_NON_LINEAR if decay_for_non_mamba_blocks else 0) | (_capi.QUERY_ONLY if query_only else 0)
    rc = _capi.lib().natsl_mamba_recurrent_fwd(
        _capi.ptr(q), _capi.ptr(k), _capi.ptr(v), _capi.ptr(g), _capi.ptr(g_cumsum), _capi.ptr(initial_state),
        _capi.ptr(initial_state_in_current_block), _capi.ptr(o), _capi.ptr(ht), _capi.ptr(types), _capi.dtype_code(types.dtype),
        _capi.ptr(n_ptr), n_scalar, N, T, H, HN, K, V, int(nats_block_size), float(scale), flags, _capi.dtype_code(q.dtype),
        _capi.stream_ptr(dev))
    _capi.check(rc, "natsl_mamba_recurrent_fwd")
    return o, ht, initial_state_in_current_block


def nats_mixed_attn_mamba_recurrent(
        q_attn: torch.Tensor, k_attn: torch.Tensor, v_attn: torch.Tensor,
        q_lattn: torch.Tensor, k_lattn: torch.Tensor, v_lattn: torch.Tensor,
        attn_msk: torch.Tensor,
        initial_state_mamba: torch.Tensor,
        initial_state_mamba_chunk_start: torch.Tensor,
        g: torch.Tensor,
        g_cumsum: torch.Tensor,
        nats_block_types: torch.Tensor,
        n_tokens_in_current_block: int = 0,
        scale_attn=None, scale_lattn=None,
        cu_seqlens=None, cu_seqlens_nats=None,
        nats_block_size: int = 64,
        ops_for_incomplete_chunks: str = 'all',
        output_final_state_mamba: bool = False,
        decay_for_non_mamba_blocks: bool = False,
        incomplete_block_start_with_ht: bool = True,
        use_g_for_attn: bool = False,
):
    """Decode step(s) of the Mamba hybrid layer (src/nats/ops/mixed_ops/mixed_attn_mamba.py:460-593).
    -> (o_mamba, o_attn, final_state, initial_state_in_current_block).  As in the reference, scale_lattn
    defaults to K**-0.5 here.  'all' / 'mamba': the linear operator also runs on the incomplete block.  'attn' (:516-591): the
    new tokens read the (decayed) state that entered the block, and the state advances when the block is complete, by the
    token recurrence over the block's cached k, v, g; built for nats_block_size = 64 and steps that stay inside the block."""
    from .mixed_attn_gdn import masked_attention
    if scale_attn is None:
        scale_attn = k_attn.shape[-1] ** -0.5
    if scale_lattn is None:
        scale_lattn = k_lattn.shape[-1] ** -0.5
    strategy = all_incomplete_ops[ops_for_incomplete_chunks]
    if not strategy.mamba:
        if nats_block_size != 64:
            raise NotImplementedError("ops_for_incomplete_chunks='attn' is built for decode with nats_block_size=64 only (with longer "
                                      "blocks the chunked forward of that mode reads the state at the start of each 64-token chunk)")
        if torch.is_tensor(n_tokens_in_current_block):
            raise NotImplementedError("ops_for_incomplete_chunks='attn': n_tokens_in_current_block must be an int")
        if int(n_tokens_in_current_block) + q_lattn.shape[1] > nats_block_size:
            raise NotImplementedError("ops_for_incomplete_chunks='attn': a decode step must stay inside the current selector block")
    if cu_seqlens is not None or cu_seqlens_nats is not None:
        raise NotImplementedError("packed sequences are not supported by the recurrent (decode) operator")
    if use_g_for_attn:
        raise NotImplementedError("use_g_for_attn is not built")
    if not q_lattn.is_cuda:
        from . import _capi
        raise _capi.NatslError("the NAtS-L mixed operator runs on the GPU only (no CPU fallback)")
    with torch.no_grad():
        o_attn = masked_attention(q_attn, k_attn, v_attn, attn_msk, scale_attn)
        if strategy.mamba:
            o_mamba, final_state, start = fused_recurrent_mamba_nats_fwd(
                q_lattn, k_lattn, v_lattn, g, g_cumsum, nats_block_types, n_tokens_in_current_block, nats_block_size, scale_lattn,
                initial_state_mamba, initial_state_mamba_chunk_start, output_final_state=True,
                decay_for_non_mamba_blocks=decay_for_non_mamba_blocks)
        else:
            T, n_in = q_lattn.shape[1], int(n_tokens_in_current_block)
            start = initial_state_mamba_chunk_start
            if start is None:
                N, _, H, K = q_lattn.shape
                start = (initial_state_mamba.to(torch.float32).clone() if initial_state_mamba is not None
                         else torch.zeros(N, H, K, v_lattn.shape[-1], dtype=torch.float32, device=q_lattn.device))
            o_mamba, _, _ = fused_recurrent_mamba_nats_fwd(q_lattn, None, None, g[:, -T:], g_cumsum, nats_block_types, n_in, nats_block_size,
                                                           scale_lattn, None, start, query_only=True)
            final_state = start
            if n_in + T == nats_block_size:
                # the block is complete: its tokens (handed over by the cache) advance the state, as in the other modes
                if k_lattn.shape[1] != nats_block_size or g.shape[1] != nats_block_size:
                    raise ValueError("ops_for_incomplete_chunks='attn': the step that completes a block needs k, v, g of the whole "
                                     f"block ({nats_block_size} tokens), got {k_lattn.shape[1]}")
                _, final_state, start = fused_recurrent_mamba_nats_fwd(
                    k_lattn, k_lattn, v_lattn, g, None, nats_block_types, 0, nats_block_size, scale_lattn, start.clone(), start,
                    output_final_state=True, decay_for_non_mamba_blocks=decay_for_non_mamba_blocks)
    return o_mamba, o_attn, final_state, start
