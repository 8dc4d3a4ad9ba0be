"""nats_mixed_attn_gdn: softmax branch + Gated DeltaNet branch behind the reference's operator API
(src/nats/ops/mixed_ops/mixed_attn_gdn.py:286-325)."""
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

    n_nats_blocks is accepted for signature compatibility (the block counts are recomputed on the device from
    nats_block_types); the two compute_dnats_* flags select the selector gradient of the backward.
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
        qk_l2norm=lattn_use_qk_l2norm_in_kernel,
        dnats_invalid_attn=compute_dnats_for_invalid_blocks_attn,
        dnats_invalid_linear=compute_dnats_for_invalid_blocks_linear_att)


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
        attn_prefix_valid: torch.Tensor | None = None,
):
    """Prefill variant (src/nats/ops/mixed_ops/mixed_attn_gdn.py:328-440):
    -> (o_gated_delta_net, o_attn, final_state, state at the start of the current block).
    attn_prefix_valid (not in the reference): k_attn / v_attn start with that many more whole blocks of cached keys, visible
    per selector head where the flag is set; see _mixed_common._mixed_forward_impl."""
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
        n_tokens_in_current_block=n_tokens_in_current_block, attn_prefix_valid=attn_prefix_valid)


def fused_recurrent_gated_delta_rule_nats_fwd(q, k, v, g, g_cumsum, beta, nats_block_types, n_tokens_in_current_block,
                                              nats_block_size, scale, initial_state, initial_state_in_current_block,
                                              output_final_state=True, use_qk_l2norm_in_kernel=True,
                                              decay_for_non_gdn_blocks=False, query_only=False):
    """The gated delta rule token by token on a cached state, for tokens that continue the current selector
    block (src/nats/ops/gated_delta_rule/fused_recurrent.py:360-470 with update_hs_for_each_iter=True).
    -> (o, final_state or None, initial_state_in_current_block); the last is updated in place when the
    tokens complete the block, as the reference's kernel does.
    query_only (the call without update_hs_for_each_iter, for one-token steps): o_t = scale q_t^T (e^(g_cumsum + g_1..t) times
    initial_state_in_current_block); k, v, beta are not read (may be None) and no state is written."""
    from . import _capi
    N, T, H, K = q.shape
    if query_only:
        if initial_state_in_current_block is None:
            raise ValueError("query_only needs the state that entered the block")
        k, v, beta = q, q, q                      # placeholders: the kernel does not read them in this mode
    V = initial_state_in_current_block.shape[-1] if query_only else v.shape[-1]
    if nats_block_types.shape[1] != 1:
        raise AssertionError("the recurrent form only continues the current selector block: nats_block_types must hold one block")  # :417-419
    HN = nats_block_types.shape[2]
    dev = q.device
    q, k, v, beta = (t.contiguous() for t in (q, k, v, beta))
    if not (q.dtype == k.dtype == v.dtype == beta.dtype):
        raise ValueError("q, k, v, beta must share a dtype")
    g = g.to(torch.float32).contiguous()
    types = nats_block_types if nats_block_types.dtype in (torch.float32, torch.bfloat16) else nats_block_types.float()
    types = types.contiguous()
    if initial_state is not None:
        initial_state = initial_state.to(torch.float32).contiguous()
    if initial_state_in_current_block is None:                                           # :398-402
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
    flags = (_capi.DECAY_NON_LINEAR if decay_for_non_gdn_blocks else 0) | (_capi.QK_L2NORM if use_qk_l2norm_in_kernel else 0) | \
            (_capi.QUERY_ONLY if query_only else 0)
    rc = _capi.lib().natsl_gdn_recurrent_fwd(
        _capi.ptr(q), _capi.ptr(k), _capi.ptr(v), _capi.ptr(g), _capi.ptr(g_cumsum), _capi.ptr(beta), _capi.ptr(initial_state),
        _capi.ptr(initial_state_in_current_block), _capi.ptr(o), _capi.ptr(ht), _capi.ptr(types), _capi.dtype_code(types.dtype),
        _capi.ptr(n_ptr), n_scalar, N, T, H, HN, K, V, int(nats_block_size), float(scale), flags, _capi.dtype_code(q.dtype),
        _capi.stream_ptr(dev))
    _capi.check(rc, "natsl_gdn_recurrent_fwd")
    return o, ht, initial_state_in_current_block


def masked_attention(q, k, v, attn_msk, scale):
    """Softmax attention of a few queries over cached keys under a boolean mask [B, HM, TQ, TK] (HM divides the
    number of query heads); replaces repeat_masks + scaled_dot_product_attention at
    src/nats/ops/mixed_ops/mixed_attn_gdn.py:475-481.  A query that sees no key gives 0."""
    from . import _capi
    B, TQ, HQ, K = q.shape
    TK, HKV, V = k.shape[1], k.shape[2], v.shape[-1]
    if attn_msk.dim() != 4 or attn_msk.shape[0] != B or attn_msk.shape[2] != TQ or attn_msk.shape[3] != TK:
        raise ValueError(f"attn_msk must be [B, heads, {TQ}, {TK}], got {tuple(attn_msk.shape)}")
    if TK == 0:
        return q.new_zeros(B, TQ, HQ, V)          # no cached key yet: every query sees nothing
    q = q.contiguous()

    def cache_view(t):
        # the front part [:, :TK] of a cache buffer [B, capacity, H, D] is read in place (only its batch stride differs
        # from a dense tensor's); anything else is made contiguous
        D = t.shape[-1]
        if t.stride(3) == 1 and t.stride(2) == D and t.stride(1) == HKV * D and t.stride(0) >= TK * HKV * D and t.stride(0) % 8 == 0:
            return t, t.stride(0)
        return t.contiguous(), 0
    (k, k_bs), (v, v_bs) = cache_view(k), cache_view(v)
    if not (q.dtype == k.dtype == v.dtype):
        raise ValueError("q, k, v must share a dtype")
    mask = attn_msk.to(torch.bool).contiguous().view(torch.uint8)
    o = torch.empty(B, TQ, HQ, V, dtype=q.dtype, device=q.device)
    L = _capi.lib()
    ws_bytes = L.natsl_attn_masked_workspace_bytes(B, TQ, TK, HQ, V)
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device=q.device) if ws_bytes else None
    rc = L.natsl_attn_masked_fwd(_capi.ptr(q), _capi.ptr(k), _capi.ptr(v), _capi.ptr(mask), _capi.ptr(o), B, TQ, TK, HQ,
                                 HKV, mask.shape[1], K, V, float(scale), _capi.dtype_code(q.dtype), _capi.ptr(ws), ws_bytes,
                                 k_bs, v_bs, _capi.stream_ptr(q.device))
    _capi.check(rc, "natsl_attn_masked_fwd")
    return o


def nats_mixed_attn_gdn_recurrent(
        q_attn: torch.Tensor, k_attn: torch.Tensor, v_attn: torch.Tensor,
        q_lattn: torch.Tensor, k_lattn: torch.Tensor, v_lattn: torch.Tensor,
        attn_msk: torch.Tensor,
        initial_state_gated_delta: torch.Tensor,
        initial_state_gated_delta_chunk_start: torch.Tensor,
        g: torch.Tensor,
        g_cumsum: torch.Tensor,
        beta: torch.Tensor,
        nats_block_types: torch.Tensor,
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
    """Decode step(s) of the hybrid layer (src/nats/ops/mixed_ops/mixed_attn_gdn.py:443-591): masked attention
    of the new queries over the cached keys/values, and the gated delta rule token by token on the cached
    state. -> (o_gated_delta_net, o_attn, final_state, initial_state_in_current_block).

    'all' / 'gated_delta_net': the linear operator also runs on the incomplete block.  'attn' (:504-589): the new tokens read
    the state that entered the block (decayed), and the state advances when the block is complete -- here by the same token
    recurrence over the block's cached k, v, beta, g that the cache hands over with the completing step (the reference does
    it in parallel form, :529-589: the same state).  Built for a selector block of one 64-token chunk, where it gives what
    the chunked forward of that mode gives, and for steps that stay inside the block (the layers split longer ones)."""
    if scale_attn is None:
        scale_attn = k_attn.shape[-1] ** -0.5
    if scale_lattn is None:
        scale_lattn = k_lattn.shape[-1] ** -0.5
    strategy = all_incomplete_ops[ops_for_incomplete_chunks]
    if not strategy.gated_delta_net:
        if nats_block_size != 64:
            raise NotImplementedError("ops_for_incomplete_chunks='attn' is built for decode with nats_block_size=64 only (with longer "
                                      "blocks the chunked forward of that mode reads the state at the start of each 64-token chunk)")
        if torch.is_tensor(n_tokens_in_current_block):
            raise NotImplementedError("ops_for_incomplete_chunks='attn': n_tokens_in_current_block must be an int")
        if int(n_tokens_in_current_block) + q_lattn.shape[1] > nats_block_size:
            raise NotImplementedError("ops_for_incomplete_chunks='attn': a decode step must stay inside the current selector block")
    if cu_seqlens is not None or cu_seqlens_nats is not None:
        raise NotImplementedError("packed sequences are not supported by the recurrent (decode) operator")
    if attn_sw_size is not None or use_g_for_attn:
        raise NotImplementedError("attn_sw_size / use_g_for_attn are not built")
    if not q_lattn.is_cuda:
        from . import _capi
        raise _capi.NatslError("the NAtS-L mixed operator runs on the GPU only (no CPU fallback)")
    with torch.no_grad():
        o_attn = masked_attention(q_attn, k_attn, v_attn, attn_msk, scale_attn)
        if strategy.gated_delta_net:
            o_gdn, final_state, start = fused_recurrent_gated_delta_rule_nats_fwd(
                q_lattn, k_lattn, v_lattn, g, g_cumsum, beta, nats_block_types, n_tokens_in_current_block, nats_block_size,
                scale_lattn, initial_state_gated_delta, initial_state_gated_delta_chunk_start, output_final_state=True,
                use_qk_l2norm_in_kernel=lattn_use_qk_l2norm_in_kernel, decay_for_non_gdn_blocks=decay_for_non_gdn_blocks)
        else:
            T, n_in = q_lattn.shape[1], int(n_tokens_in_current_block)
            start = initial_state_gated_delta_chunk_start
            if start is None:
                N, _, H, K = q_lattn.shape
                start = (initial_state_gated_delta.to(torch.float32).clone() if initial_state_gated_delta is not None
                         else torch.zeros(N, H, K, v_lattn.shape[-1], dtype=torch.float32, device=q_lattn.device))
            o_gdn, _, _ = fused_recurrent_gated_delta_rule_nats_fwd(
                q_lattn, None, None, g[:, -T:], g_cumsum, None, nats_block_types, n_in, nats_block_size, scale_lattn, None, start,
                use_qk_l2norm_in_kernel=lattn_use_qk_l2norm_in_kernel, query_only=True)
            final_state = start
            if n_in + T == nats_block_size:
                # the block is complete: its tokens (handed over by the cache) advance the state, as in the other modes
                if k_lattn.shape[1] != nats_block_size or g.shape[1] != nats_block_size or beta.shape[1] != nats_block_size:
                    raise ValueError("ops_for_incomplete_chunks='attn': the step that completes a block needs k, v, g, beta of the "
                                     f"whole block ({nats_block_size} tokens), got {k_lattn.shape[1]}")
                _, final_state, start = fused_recurrent_gated_delta_rule_nats_fwd(
                    k_lattn, k_lattn, v_lattn, g, None, beta, nats_block_types, 0, nats_block_size, scale_lattn, start.clone(), start,
                    output_final_state=True, use_qk_l2norm_in_kernel=lattn_use_qk_l2norm_in_kernel,
                    decay_for_non_gdn_blocks=decay_for_non_gdn_blocks)
    return o_gdn, o_attn, final_state, start
