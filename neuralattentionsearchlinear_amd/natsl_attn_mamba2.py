"""Mamba2-SSD / softmax hybrid token mixer with the forward signature, returns and parameter names of
the reference layer (src/nats/layers/natsl_attn_mamba2.py:100-599).  Same scope as the Gated-DeltaNet
layer: trainable with the same HIP backwards (natsl_softmax_sparse_bwd, natsl_linear_chunk_bwd in its Mamba form,
natsl_short_conv_bwd, natsl_row_norm_bwd, natsl_norm_gate_bwd; the pooling's backward and the projections are torch
operations); with a cache, chunked prefill (also of a second prompt on a filled cache: the kept blocks as a key prefix, the
linear branch from the state that entered the incomplete block) and decode steps of fewer than 64 tokens."""
from __future__ import annotations

import math
from typing import Optional

import torch
import torch.nn as nn
import torch.nn.functional as F

from . import nats_util
from .cache import NAtSLayerCache
from .mixed_attn_mamba import (nats_mixed_attn_mamba, nats_mixed_attn_mamba_chunk_inference,
                               nats_mixed_attn_mamba_recurrent)
from .modules import FusedMultiInputRMSNormGated, L2Norm, RMSNorm, ShortConvolution


class NeuralAttentionSearchLinearAttnMamba(nn.Module):
    def __init__(self, hidden_size: int = 2048, expand_v: float = 2, head_dim: int = 256, num_heads: int = 6,
                 num_attn_heads: int = 24, num_v_heads: int = None, n_ops: int = 2, num_nats_head: Optional[int] = None,
                 nats_block_size: int = 64, nats_block_agg_type: str = 'mean', nats_sample_strategy: str = 'argmax',
                 ops_for_incomplete_chunks: str = 'gated_delta_net', mode: str = 'chunk', use_gate: bool = True,
                 use_short_conv: bool = True, allow_neg_eigval: bool = False, conv_size: int = 4, conv_bias: bool = False,
                 conv_activation: Optional[str] = 'silu', outputs_are_wighted: bool = True, attn_qk_norm: bool = False,
                 attn_with_short_conv: bool = False, compute_dnats_for_invalid_blocks_attn: bool = False,
                 compute_dnats_for_invalid_blocks_linear_att: bool = False, decay_for_non_mamba_blocks: bool = True,
                 incomplete_block_start_with_ht: bool = True, attn_apply_pos_encoding: bool = False,
                 attn_rope_theta: Optional[float] = 10000., attn_max_position_embeddings: Optional[int] = None,
                 layer_idx: int = None, norm_eps: float = 1e-5, **kwargs):
        super().__init__()
        if n_ops != 2 or nats_block_agg_type != 'mean' or nats_sample_strategy != 'argmax':
            raise NotImplementedError("two ops, mean pooling and the hard selector are built")
        if attn_apply_pos_encoding:
            raise NotImplementedError("rotary position encoding for the attention view is not built")
        if not use_gate or not outputs_are_wighted:
            raise NotImplementedError("only use_gate=True with weighted outputs is built")
        if ops_for_incomplete_chunks == 'gated_delta_net':
            # the reference default names a mode its own Mamba operator does not know (KeyError at
            # src/nats/ops/mixed_ops/mixed_attn_mamba.py:73); the equivalent Mamba mode is meant
            ops_for_incomplete_chunks = 'mamba'
        assert mode in ['chunk', 'fused_recurrent'], f"Not supported mode `{mode}`."
        self.mode, self.hidden_size, self.expand_v = mode, hidden_size, expand_v
        self.use_gate, self.use_short_conv, self.conv_size, self.conv_bias = use_gate, use_short_conv, conv_size, conv_bias
        self.head_dim, self.num_heads = head_dim, num_heads
        self.num_v_heads = num_v_heads if num_v_heads is not None else num_heads
        self.n_ops = n_ops
        self.head_k_dim = head_dim
        self.head_v_dim = int(head_dim * expand_v)
        self.key_dim = int(num_heads * self.head_k_dim)
        self.value_dim = int(self.num_v_heads * self.head_v_dim)
        self.layer_idx = layer_idx
        self.attn_qk_norm, self.num_attn_heads = attn_qk_norm, num_attn_heads
        self.head_attn_k_dim = self.key_dim // num_attn_heads
        self.head_attn_v_dim = self.value_dim // num_attn_heads
        self.attn_with_short_conv = attn_with_short_conv
        self.incomplete_block_start_with_ht = incomplete_block_start_with_ht
        self.decay_for_non_mamba_blocks = decay_for_non_mamba_blocks
        self.nats_block_size = nats_block_size
        self.num_nats_head = num_heads if num_nats_head is None else num_nats_head
        self.ops_for_incomplete_chunks = ops_for_incomplete_chunks
        if attn_qk_norm:
            self.q_norm = RMSNorm(self.head_attn_k_dim, eps=norm_eps)
            self.k_norm = RMSNorm(self.head_attn_k_dim, eps=norm_eps)
        self.q_norm2 = L2Norm(eps=norm_eps)
        self.k_norm2 = L2Norm(eps=norm_eps)
        self.q_proj = nn.Linear(hidden_size, self.key_dim, bias=False)
        self.k_proj = nn.Linear(hidden_size, self.key_dim, bias=False)
        self.v_proj = nn.Linear(hidden_size, self.value_dim, bias=False)
        self.a_proj = nn.Linear(hidden_size, self.num_v_heads, bias=False)
        self.nats_layer = nn.Linear(hidden_size, n_ops * self.num_nats_head, bias=False)
        self.dt_bias = nn.Parameter(torch.ones(self.num_heads))
        self.A_log = nn.Parameter(torch.log(torch.arange(1, self.num_heads + 1).float()))
        self.nats_out_weights_layer = nn.Linear(self.key_dim, n_ops * num_attn_heads, bias=False)
        if use_short_conv:
            self.q_conv1d = ShortConvolution(self.key_dim, conv_size, conv_bias, conv_activation)
            self.k_conv1d = ShortConvolution(self.key_dim, conv_size, conv_bias, conv_activation)
            self.v_conv1d = ShortConvolution(self.value_dim, conv_size, conv_bias, conv_activation)
        self.g_proj = nn.Linear(hidden_size, self.value_dim, bias=False)
        self.o_norm = FusedMultiInputRMSNormGated(self.head_attn_v_dim, eps=norm_eps)
        self.o_proj = nn.Linear(self.value_dim, hidden_size, bias=False)
        self.attn_fraction = torch.zeros(1)

    def select_ops(self, hidden_states: torch.Tensor, cu_seqlens=None, force_last_block: bool = True):
        B, _, dim = hidden_states.shape
        pooled = nats_util.mean_pooling(hidden_states.unsqueeze(-2), self.nats_block_size, cu_seqlens=cu_seqlens)
        logits = self.nats_layer(pooled.view(B, pooled.shape[1], dim)).unflatten(-1, (self.num_nats_head, self.n_ops))
        types, n_blocks = nats_util.hard_select(logits, force_last_block=False)
        last = types[:, -1].clone()
        if force_last_block:
            n_blocks = n_blocks + (1 - last.to(torch.int32))
            types[:, -1] = 1
        return types, n_blocks, last

    def _layer_cache(self, cache_params) -> Optional[NAtSLayerCache]:
        """The layer's own cache in cache_params.nats_cache, created on first use (reference :332-343)."""
        if cache_params is None:
            return None
        if self.layer_idx not in cache_params.nats_cache:
            cache_params.add_natsl_layer_cache(self.layer_idx, 0, n_tokens_in_nats_block=0, n_attn_blocks=None,
                                               nats_block_size=self.nats_block_size,
                                               op_for_incomplete_chunk=self.ops_for_incomplete_chunks)
        return cache_params.nats_cache[self.layer_idx]

    def forward(self, hidden_states: torch.Tensor, attention_mask: Optional[torch.Tensor] = None, cache_params=None,
                use_cache: Optional[bool] = False, output_attentions: Optional[bool] = False, **kwargs):
        if attention_mask is not None:
            assert len(attention_mask.shape) == 2, "Expected attention_mask as a 0-1 matrix with shape [batch_size, seq_len]"
        B, q_len, _ = hidden_states.shape
        mode = 'fused_recurrent' if q_len < 64 else self.mode                  # reference :328
        if self.training:
            assert mode == 'chunk', "Only chunk mode is supported in training."
        cu_seqlens = kwargs.get('cu_seqlens', None)
        cache = self._layer_cache(cache_params)
        if cache is not None:
            use_cache = True
        if cache is None and mode != 'chunk':
            raise ValueError("fewer than 64 tokens are decoded on a cache: pass cache_params")
        # 64 or more new tokens on a cache that already holds tokens (a second prompt): the chunked operators run again, the
        # linear branch from the state that entered the incomplete block (its cached tokens in front of the new ones), the
        # softmax branch with the kept blocks as a key prefix
        continuing = cache is not None and mode == 'chunk' and cache.n_observed_tokens > 0
        if cache is not None and cu_seqlens is not None:
            raise NotImplementedError("packed sequences are not supported together with a cache")

        if cache is not None and mode != 'chunk' and q_len > 1:
            if cache._n_tokens_in_nats_block + q_len > self.nats_block_size:
                # the step crosses a selector-block boundary: the tokens that complete the block first, then the rest as the
                # start of the next block (src/nats/ops/mamba/fused_recurrent.py handles the two blocks in one call)
                first = self.nats_block_size - cache._n_tokens_in_nats_block
                kw = dict(cache_params=cache_params, use_cache=use_cache, output_attentions=output_attentions, **kwargs)
                return torch.cat([self.forward(hidden_states[:, :first], attention_mask, **kw),
                                  self.forward(hidden_states[:, first:], attention_mask, **kw)], 1)
        selector_input = cache.update_attn_types(input_hidden_states=hidden_states) if cache is not None else hidden_states
        if selector_input is not None:
            raw_types, _, _ = self.select_ops(selector_input, cu_seqlens, force_last_block=False)
        else:
            raw_types = torch.ones(B, 1, self.num_nats_head, self.n_ops, device=hidden_states.device, dtype=hidden_states.dtype)

        conv_states = cache.conv_state if cache is not None and cache.conv_state is not None else (None, None, None)
        new_conv_states = []

        def conv_or_act(x, conv, state):
            if self.use_short_conv:
                y, final = conv(x=x, cache=state, output_final_state=bool(use_cache), cu_seqlens=cu_seqlens)
                new_conv_states.append(final)
                return y
            return F.silu(x)

        if self.attn_with_short_conv:
            q = conv_or_act(self.q_proj(hidden_states), getattr(self, 'q_conv1d', None), conv_states[0])
            k = conv_or_act(self.k_proj(hidden_states), getattr(self, 'k_conv1d', None), conv_states[1])
            v = conv_or_act(self.v_proj(hidden_states), getattr(self, 'v_conv1d', None), conv_states[2])
            q_attn, k_attn, v_attn = q, k, v
        else:
            q_attn, k_attn, v_attn = self.q_proj(hidden_states), self.k_proj(hidden_states), self.v_proj(hidden_states)
            q = conv_or_act(q_attn, getattr(self, 'q_conv1d', None), conv_states[0])
            k = conv_or_act(k_attn, getattr(self, 'k_conv1d', None), conv_states[1])
            v = conv_or_act(v_attn, getattr(self, 'v_conv1d', None), conv_states[2])
        o_weights = self.nats_out_weights_layer(q).unflatten(-1, (self.num_attn_heads, self.n_ops)).softmax(-1)
        q, k = (x.unflatten(-1, (-1, self.head_k_dim)) for x in (q, k))
        v = v.unflatten(-1, (-1, self.head_v_dim))
        q_attn, k_attn = (x.unflatten(-1, (-1, self.head_attn_k_dim)) for x in (q_attn, k_attn))
        v_attn = v_attn.unflatten(-1, (-1, self.head_attn_v_dim))
        if self.num_v_heads > self.num_heads:
            q, k = (x.repeat_interleave(self.num_v_heads // self.num_heads, dim=-2) for x in (q, k))
        if self.attn_qk_norm:
            q_attn, k_attn = self.q_norm(q_attn), self.k_norm(k_attn)
        q, k = self.q_norm2(q), self.k_norm2(k)
        dt = F.softplus(self.a_proj(hidden_states).float() + self.dt_bias)
        v = (v * dt.unsqueeze(-1)).to(v.dtype)                 # the attention view keeps the un-scaled v (:391-393, :473)
        g = -self.A_log.float().exp() * dt

        state, state_block_start, g_cumsum = None, None, None
        k_new, v_new, g_new = k_attn, v_attn, g
        if cache is not None:
            k_attn, v_attn = cache.update_attn_cache((k_attn, v_attn), nats_block_types=raw_types)
            k, v, _, g = cache.update_lattn_cache((k, v), None, g, mode, self.ops_for_incomplete_chunks)
            state, state_block_start, g_cumsum = cache.recurrent_state, cache.recurrent_state_block_start, cache.g_cumsum
        n_cached, prefix_valid = 0, None
        if continuing:
            # keys: the kept blocks, the incomplete block's cached tokens, the new tokens -- the cache's buffer as it lies; the
            # linear inputs came back with the incomplete block's tokens in front; the queries of those tokens are not needed
            n_cached = cache._n_tokens_in_nats_block
            n_keys = cache.n_attn_tokens_max + q_len
            k_attn, v_attn = cache.attn_k[:, :n_keys], cache.attn_v[:, :n_keys]
            if cache.n_attn_blocks_max > 0:
                prefix_valid = cache.valid_attn_tokens[:, :cache.n_attn_blocks_max]
            if n_cached:
                front = lambda t: torch.cat([t.new_zeros(t.shape[0], n_cached, *t.shape[2:]), t], 1)
                q, q_attn = front(q), front(q_attn)
                state = state_block_start

        common = dict(q_attn=q_attn, k_attn=k_attn, v_attn=v_attn, q_lattn=q, k_lattn=k, v_lattn=v, g=g,
                      scale_attn=k_attn.shape[-1] ** -0.5, scale_lattn=1,
                      cu_seqlens=cu_seqlens, cu_seqlens_nats=None, nats_block_size=self.nats_block_size,
                      ops_for_incomplete_chunks=self.ops_for_incomplete_chunks, output_final_state_mamba=bool(use_cache),
                      incomplete_block_start_with_ht=self.incomplete_block_start_with_ht,
                      decay_for_non_mamba_blocks=self.decay_for_non_mamba_blocks, use_g_for_attn=False)
        if mode == 'chunk':
            types = raw_types.clone()
            last_type = types[:, -1].clone()
            types[:, -1] = 1
            n_nats_blocks = types.to(torch.int32).sum(1)
            self.attn_fraction = (n_nats_blocks.float()[..., 0] / types.shape[1]).mean(0).detach()
            if self.training:
                o_lin, o_attn, state = nats_mixed_attn_mamba(initial_state_mamba=state, nats_block_types=types,
                                                             n_nats_blocks=n_nats_blocks, **common)
                state_block_start = None
            else:
                o_lin, o_attn, state, state_block_start = nats_mixed_attn_mamba_chunk_inference(
                    initial_state_mamba_start=state if continuing else state_block_start, nats_block_types=types,
                    n_nats_blocks=n_nats_blocks, attn_prefix_valid=prefix_valid,
                    op_type_last_chunk=last_type if k.shape[1] % self.nats_block_size == 0 else None, **common)
                o_lin, o_attn = o_lin[:, n_cached:], o_attn[:, n_cached:]
        else:
            attn_msk = cache.generate_msk(n_data=q_len, nats_block_types=raw_types,
                                          compute_incomplete_chunk=self.ops_for_incomplete_chunks != 'mamba')
            o_lin, o_attn, state, state_block_start = nats_mixed_attn_mamba_recurrent(
                attn_msk=attn_msk, initial_state_mamba=state, initial_state_mamba_chunk_start=state_block_start,
                g_cumsum=g_cumsum, nats_block_types=raw_types, n_tokens_in_current_block=cache._n_tokens_in_nats_block, **common)
        self.last_recurrent_state, self.last_block_start_state = state, state_block_start

        if cache is not None:
            cache.update(recurrent_state=state, recurrent_state_block_start=state_block_start, attn_state=(k_new, v_new),
                         conv_state=tuple(new_conv_states) if self.use_short_conv else None, nats_block_types=raw_types,
                         l_attn_state=(k, v), g=g_new, n_new_tokens=q_len)

        gate = self.g_proj(hidden_states).unflatten(-1, (-1, self.head_v_dim))
        o = self.o_norm(o_lin.reshape(o_attn.shape), o_attn, gate.reshape(o_attn.shape), o_weights)
        return self.o_proj(o.flatten(-2))
