"""Per-layer cache of the hybrid layers for generation: compacted softmax K/V, the linear branch's states,
the incomplete block's linear inputs and hidden states, and the convolution states -- the attributes and
method names of the reference's NAtSLayerCache / NAtSCache (src/nats/models/utils.py:34-668, 671-850).

What the cache guarantees (the reference states the same in its own checks, src/nats/models/utils.py:855-1047):
  * for every (sequence, selector head) the attention-typed complete blocks seen so far sit back to back from
    block 0 of attn_k / attn_v, in order, for every kv head of that selector head's group;
  * the tokens of the current incomplete block sit at block index n_attn_blocks_max (the largest count), the
    same index for every head, zero padded;
  * valid_attn_tokens[b, i, hn] is true for i < n_attn_blocks[b, hn] and, while a block is incomplete, for
    i == n_attn_blocks_max; false elsewhere;
  * feeding a sequence in one piece, in two pieces or token by token gives the same cache.

The K/V movement is the HIP kernel natsl_kv_compact; the buffers grow geometrically and are never reallocated
per block.  The first (prefill) update gathers straight from the layer's K/V into a buffer sized for the kept
blocks, so the cache never holds the blocks the selector dropped.
"""
from __future__ import annotations

from typing import Any, Dict, List, Optional, Tuple

import torch

from . import _capi


def _cdiv(a: int, b: int) -> int:
    return -(-a // b)


class NAtSLayerCache:
    is_compileable = False

    def __init__(self, seen_tokens: int = 0, n_tokens_in_nats_block: int = 0, n_attn_blocks: Optional[torch.Tensor] = None,
                 nats_block_size: int = 64, attn_offset: int = 0, recurrent_offset: int = 1, n_ops: int = 2,
                 op_for_incomplete_chunk: str = 'attn'):
        self.nats_block_size = nats_block_size
        self.attn_offset, self.recurrent_offset, self.n_ops = attn_offset, recurrent_offset, n_ops
        self.op_for_incomplete_chunk = op_for_incomplete_chunk
        # the modes in which the softmax operator does not run on the incomplete block (the Mamba layer's name for it included)
        self._linear_only = op_for_incomplete_chunk in ('gated_delta_net', 'mamba')
        self.lazy_initialization(None)
        self.seen_tokens = seen_tokens
        self._n_tokens_in_nats_block = n_tokens_in_nats_block
        self.n_attn_blocks = n_attn_blocks

    # ------------------------------------------------------------------------------------------------
    def lazy_initialization(self, key_states: Optional[torch.Tensor] = None):
        """Back to the empty cache (src/nats/models/utils.py:151-176)."""
        self.seen_tokens = 0
        self.attn_k = self.attn_v = None                 # [B, capacity, HKV, K|V]; capacity is a multiple of the block
        self.l_attn_k = self.l_attn_v = None             # the incomplete block's linear-branch inputs [B, block, H, K|V]
        self.lattn_g = self.lattn_beta = None            # [B, block, H]
        self.recurrent_state = None                      # fp32 [B, H, K, V]
        self.recurrent_state_block_start = None
        self.block_type_state = None                     # hidden states of the incomplete block [B, block, D]
        self.block_type_state_logits = None
        self.conv_state = None
        self.ffn_state = None
        self._n_tokens_in_nats_block = 0
        self.n_attn_blocks = None                        # int64 [B, HN]: complete attention-typed blocks kept
        self.n_attn_blocks_max = 0
        self.n_attn_tokens_max = 0
        self.n_groups_nats = None
        self.valid_attn_tokens = None                    # bool [B, capacity/block, HN]
        self.g_cumsum = None                             # [B, 1, H]: sum of g over the incomplete block
        self.n_observed_tokens = 0
        self._pending_first = None                       # K/V of the first forward, kept until update() has the types

    # ------------------------------------------------------------------------------------------------
    def update_attn_types(self, input_hidden_states: torch.Tensor) -> Optional[torch.Tensor]:
        """Collect the hidden states of the incomplete block; once the new tokens complete at least one block,
        return [cached tokens of the block, new tokens] for the selector, else None
        (src/nats/models/utils.py:178-207)."""
        B, T, D = input_hidden_states.shape
        bs, n_in = self.nats_block_size, self._n_tokens_in_nats_block
        if self.block_type_state is None:
            self.block_type_state = torch.zeros(B, bs, D, dtype=input_hidden_states.dtype, device=input_hidden_states.device)
        total = n_in + T
        if total < bs:
            self.block_type_state[:, n_in:total] = input_hidden_states
            return None
        joined = torch.cat([self.block_type_state[:, :n_in], input_hidden_states], dim=1) if n_in else input_hidden_states
        self.block_type_state.zero_()
        rest = total % bs
        if rest:
            self.block_type_state[:, :rest] = joined[:, -rest:]
        return joined

    # ------------------------------------------------------------------------------------------------
    def generate_msk(self, n_data: int = 1, nats_block_types: Optional[torch.Tensor] = None,
                     compute_incomplete_chunk: bool = False):
        """Visibility of the cached keys for the new queries, bool [B, HN, n_data, keys]; call it after
        update_attn_cache and before update (src/nats/models/utils.py:209-287).  Keys are the kept blocks (per
        head: as many as that head has) followed by the tokens of the incomplete block, new ones included.

        n_data > 1 is supported while the new tokens stay inside the current block (the reference builds a mask
        without the kept blocks there, :246-256, which does not fit the keys it is used with).  In the mode whose softmax
        operator skips the incomplete block ('gated_delta_net' / 'mamba') the keys end at the last whole block and a new token
        sees the kept blocks only, as in the chunked forward of that mode.  (The reference's one-token rule, :237-243, shows the
        token that completes a block its own block, which its chunked forward never does; the chunked forward is followed.)"""
        bs, n_in, nmax = self.nats_block_size, self._n_tokens_in_nats_block, self.n_attn_blocks_max
        if n_data == 1:
            cols = self.n_attn_tokens_max + 1
            if self._linear_only:
                cols = cols // bs * bs
            msk = self.valid_attn_tokens[:, :nmax + 1].repeat_interleave(bs, 1)[:, :cols]
            if self._linear_only and cols > nmax * bs:
                msk = msk.clone()
                msk[:, nmax * bs:] = False          # the token that completes the block: its own block stays hidden
            return msk.transpose(1, 2).unsqueeze(-2).bool()
        if nats_block_types is None or nats_block_types.shape[1] != 1 or n_in + n_data > bs:
            raise NotImplementedError("a mask for several new tokens is built only while they stay inside the current block")
        if self.valid_attn_tokens is None:
            # an empty cache (a first input shorter than one block): no kept blocks yet, the keys are the new tokens
            dev, (B, _, HN, _) = nats_block_types.device, nats_block_types.shape
            past = torch.zeros(B, HN, n_data, 0, dtype=torch.bool, device=dev)
        else:
            dev = self.valid_attn_tokens.device
            B, _, HN = self.valid_attn_tokens.shape
            past = self.valid_attn_tokens[:, :nmax].repeat_interleave(bs, 1).transpose(1, 2)          # [B, HN, nmax*bs]
            past = past.unsqueeze(-2).expand(B, HN, n_data, nmax * bs)
        if self._linear_only:
            if self.valid_attn_tokens is None:
                return torch.zeros(B, HN, n_data, n_data, dtype=torch.bool, device=dev)     # (the keys are the new tokens themselves)
            if n_in + n_data < bs:
                return past
            return torch.cat([past, torch.zeros(B, HN, n_data, bs, dtype=torch.bool, device=dev)], dim=-1)
        cur = torch.ones(n_data, n_in + n_data, dtype=torch.bool, device=dev).tril_(n_in) if compute_incomplete_chunk \
            else torch.zeros(n_data, n_in + n_data, dtype=torch.bool, device=dev)
        return torch.cat([past, cur.view(1, 1, n_data, -1).expand(B, HN, -1, -1)], dim=-1)

    # ------------------------------------------------------------------------------------------------
    def _grow(self, need_tokens: int):
        bs = self.nats_block_size
        cap = self.attn_k.shape[1]
        if cap >= need_tokens:
            return
        new_cap = _cdiv(max(need_tokens, 2 * cap), bs) * bs
        for name in ('attn_k', 'attn_v'):
            old = getattr(self, name)
            buf = torch.zeros(old.shape[0], new_cap, *old.shape[2:], dtype=old.dtype, device=old.device)
            buf[:, :cap] = old
            setattr(self, name, buf)
        flags = torch.zeros(self.valid_attn_tokens.shape[0], new_cap // bs, self.valid_attn_tokens.shape[2], dtype=torch.bool,
                            device=self.valid_attn_tokens.device)
        flags[:, :self.valid_attn_tokens.shape[1]] = self.valid_attn_tokens
        self.valid_attn_tokens = flags

    def update_attn_cache(self, attn_state: Tuple[torch.Tensor, torch.Tensor], nats_block_types: torch.Tensor):
        """Append the new tokens' K/V behind the incomplete block and return the keys/values the attention of this
        forward runs on: kept blocks + incomplete block + new tokens (src/nats/models/utils.py:289-343).  On an
        empty cache nothing is copied yet: the new tensors are the keys, and update() gathers the kept blocks."""
        k_state, v_state = attn_state
        n_new, bs = k_state.shape[1], self.nats_block_size
        if self.attn_k is None:
            self._pending_first = (k_state, v_state)
            return k_state, v_state
        start = self.n_attn_tokens_max
        self._grow(start + n_new)
        self.attn_k[:, start:start + n_new] = k_state
        self.attn_v[:, start:start + n_new] = v_state
        first, last = self.n_attn_blocks_max, _cdiv(start + n_new, bs)
        self.valid_attn_tokens[:, first:last] = True
        end = start + n_new
        if self._linear_only:
            end = end // bs * bs
        return self.attn_k[:, :end], self.attn_v[:, :end]

    # ------------------------------------------------------------------------------------------------
    def update_lattn_cache(self, lattn_state: Tuple[torch.Tensor, torch.Tensor], lattn_beta: Optional[torch.Tensor],
                           lattn_g: Optional[torch.Tensor], mode: str, ops_for_incomplete_chunks: str):
        """Keep the incomplete block's linear-branch inputs (k, v, beta, g) and hand back what the linear operator
        of this forward runs on: the new tokens, preceded by the cached tokens of the block when a chunked
        forward (or the 'attn' mode) has to restart from the block's first token
        (src/nats/models/utils.py:345-457)."""
        k, v = lattn_state
        T, bs, n_in = k.shape[1], self.nats_block_size, self._n_tokens_in_nats_block
        fresh = self.l_attn_k is None
        if fresh:
            B, _, H, _ = k.shape
            self.l_attn_k = torch.zeros(B, bs, H, k.shape[3], dtype=k.dtype, device=k.device)
            self.l_attn_v = torch.zeros(B, bs, H, v.shape[3], dtype=k.dtype, device=k.device)
            if lattn_beta is not None:
                self.lattn_beta = torch.zeros(B, bs, H, dtype=lattn_beta.dtype, device=k.device)
            if lattn_g is not None:
                self.lattn_g = torch.zeros(B, bs, H, dtype=lattn_g.dtype, device=lattn_g.device)
            n_in = 0
        pairs = [(self.l_attn_k, k), (self.l_attn_v, v), (self.lattn_beta, lattn_beta), (self.lattn_g, lattn_g)]
        total = n_in + T
        if total < bs:
            for buf, new in pairs:
                if new is not None:
                    buf[:, n_in:total] = new
            return k, v, lattn_beta, lattn_g
        out = (k, v, lattn_beta, lattn_g)
        if not fresh and n_in and (mode == 'chunk' or ops_for_incomplete_chunks == 'attn'):
            out = tuple(None if new is None else torch.cat([buf[:, :n_in], new], dim=1) for buf, new in pairs)
        rest = total % bs
        if rest:
            for buf, new in pairs:
                if new is not None:
                    buf[:, :rest] = new[:, -rest:]
        return out

    # ------------------------------------------------------------------------------------------------
    def _compact(self, nats_block_types: torch.Tensor, attn_state, n_complete: int, tail_tokens: int):
        """Keep the attention-typed complete blocks of the region of new tokens; returns nothing, updates counts."""
        bs = self.nats_block_size
        types = nats_block_types
        if types.dtype not in (torch.float32, torch.bfloat16):
            types = types.float()
        types = types.contiguous()
        B, NB, HN, _ = types.shape
        new_blocks = (torch.round(types[:, :n_complete, :, self.attn_offset].float()) == 1).sum(1)                     # int64 [B, HN]
        before = self.n_attn_blocks
        after = new_blocks if before is None else before + new_blocks
        new_max = int(after.max()) if after.numel() else 0                                        # one host sync per completed block
        tail_dst = new_max if tail_tokens else -1
        if self.attn_k is None:
            src_k, src_v = (t.contiguous() for t in (self._pending_first if self._pending_first is not None else attn_state))
            self._pending_first = None
            cap = (new_max + 2) * bs
            self.attn_k = torch.zeros(B, cap, *src_k.shape[2:], dtype=src_k.dtype, device=src_k.device)
            self.attn_v = torch.zeros(B, cap, *src_v.shape[2:], dtype=src_v.dtype, device=src_v.device)
            self.valid_attn_tokens = torch.zeros(B, cap // bs, HN, dtype=torch.bool, device=src_k.device)
            src_block0 = 0
        else:
            src_k, src_v, src_block0 = self.attn_k, self.attn_v, self.n_attn_blocks_max
            self._grow((new_max + 1) * bs)
            src_k, src_v = self.attn_k, self.attn_v
        if src_k.dtype != src_v.dtype:
            raise ValueError("attention keys and values must share a dtype")
        HKV = src_k.shape[2]
        if before is not None:
            before = before.to(torch.int64).contiguous()
        rc = _capi.lib().natsl_kv_compact(
            _capi.ptr(src_k), _capi.ptr(src_v), src_k.shape[1], src_block0, _capi.ptr(self.attn_k), _capi.ptr(self.attn_v),
            self.attn_k.shape[1], _capi.ptr(types), _capi.dtype_code(types.dtype), _capi.ptr(before), B, HKV, HN,
            src_k.shape[3], src_v.shape[3], _capi.dtype_code(src_k.dtype), bs, NB, n_complete, tail_dst, tail_tokens,
            _capi.stream_ptr(src_k.device))
        _capi.check(rc, "natsl_kv_compact")
        self.n_attn_blocks = after
        self.n_attn_blocks_max = new_max
        idx = torch.arange(self.valid_attn_tokens.shape[1], device=after.device).view(1, -1, 1)
        self.valid_attn_tokens = idx < after.unsqueeze(1)
        if tail_tokens:
            self.valid_attn_tokens[:, new_max] = True

    def update(self, recurrent_state=None, recurrent_state_block_start=None, attn_state=None, conv_state=None,
               nats_block_types: Optional[torch.Tensor] = None, ffn_state=None, g: Optional[torch.Tensor] = None,
               n_new_tokens: int = 0, cache_kwargs: Optional[Dict[str, Any]] = None, l_attn_state=None):
        """Post-forward bookkeeping (src/nats/models/utils.py:459-668): store the states, and once the new tokens
        complete at least one block, keep the attention-typed blocks and drop the others.  `l_attn_state` is what
        the reference's layers pass (src/nats/layers/natsl_attn_gdn.py:637) and is not needed here."""
        bs = self.nats_block_size
        if attn_state is not None and not attn_state[0].is_cuda:
            raise _capi.NatslError("the NAtS cache runs on the GPU only (no CPU fallback)")
        if self.n_groups_nats is None and attn_state is not None:
            self.n_groups_nats = attn_state[0].shape[2] // nats_block_types.shape[2]
        if self.op_for_incomplete_chunk == 'attn' and recurrent_state_block_start is not None:
            recurrent_state = recurrent_state_block_start.clone()
        self.recurrent_state = recurrent_state
        self.recurrent_state_block_start = recurrent_state_block_start
        total = n_new_tokens + self._n_tokens_in_nats_block
        if total >= bs:
            NB = nats_block_types.shape[1]
            if NB != _cdiv(total, bs):
                raise ValueError(f"nats_block_types holds {NB} blocks, the cached and new tokens make {_cdiv(total, bs)}")
            rest = total % bs
            self._compact(nats_block_types, attn_state, NB - 1 if rest else NB, rest)
            self._n_tokens_in_nats_block = rest
            self.n_attn_tokens_max = self.n_attn_blocks_max * bs + rest
            if g is not None:
                self.g_cumsum = g[:, -rest:].sum(1, keepdim=True) if rest else torch.zeros(g.shape[0], 1, g.shape[2], dtype=g.dtype,
                                                                                           device=g.device)
        else:
            if self.attn_k is None:
                # fewer tokens than one block on an empty cache: they are the incomplete block
                k_state, v_state = self._pending_first if self._pending_first is not None else attn_state
                self._pending_first = None
                B, _, HKV, _ = k_state.shape
                HN = nats_block_types.shape[2]
                self.attn_k = torch.zeros(B, 2 * bs, HKV, k_state.shape[3], dtype=k_state.dtype, device=k_state.device)
                self.attn_v = torch.zeros(B, 2 * bs, HKV, v_state.shape[3], dtype=v_state.dtype, device=v_state.device)
                self.attn_k[:, :n_new_tokens] = k_state
                self.attn_v[:, :n_new_tokens] = v_state
                self.valid_attn_tokens = torch.zeros(B, 2, HN, dtype=torch.bool, device=k_state.device)
            if self.n_attn_blocks is None:
                self.n_attn_blocks = torch.zeros(self.attn_k.shape[0], nats_block_types.shape[2], dtype=torch.int64,
                                                 device=self.attn_k.device)
            self._n_tokens_in_nats_block = total
            self.n_attn_tokens_max += n_new_tokens
            if g is not None:
                s = g.sum(1, keepdim=True)
                self.g_cumsum = s if self.g_cumsum is None else self.g_cumsum + s
        if self._n_tokens_in_nats_block == 0:
            # the next block starts from the state the operator left as "start of the block"
            self.block_type_state_logits = None
            self.recurrent_state = self.recurrent_state_block_start
            self.recurrent_state_block_start = None
        elif self.valid_attn_tokens is not None:
            self.valid_attn_tokens[:, self.n_attn_blocks_max] = True
        if conv_state is not None:
            self.conv_state = conv_state
        if ffn_state is not None:
            self.ffn_state = ffn_state
        self.n_observed_tokens += n_new_tokens
        self.seen_tokens += n_new_tokens


class NAtSCache:
    """The per-model list of layer caches (src/nats/models/utils.py:671-850): the hybrid layers add and index their
    NAtSLayerCache themselves (add_natsl_layer_cache / []), as the reference's layers do."""

    def __init__(self, seen_tokens: int = 0, **kwargs):
        self.states: List[NAtSLayerCache] = []
        self._seen_tokens = seen_tokens

    def __getitem__(self, layer_idx: int) -> NAtSLayerCache:
        if layer_idx < len(self.states):
            return self.states[layer_idx]
        raise KeyError(f"Cache only has {len(self)} layers, attempted to access layer with index {layer_idx}")

    def __iter__(self):
        return iter(self.states)

    def __len__(self):
        return len(self.states)

    def add_natsl_layer_cache(self, seen_tokens: int = 0, n_tokens_in_nats_block: int = 0, n_attn_blocks=None,
                              nats_block_size: int = 64, attn_offset: int = 0, recurrent_offset: int = 1, n_ops: int = 2,
                              op_for_incomplete_chunk: str = 'all'):
        self.states.append(NAtSLayerCache(seen_tokens, n_tokens_in_nats_block, n_attn_blocks, nats_block_size, attn_offset,
                                          recurrent_offset, n_ops, op_for_incomplete_chunk))

    def get_seq_length(self, layer_idx: Optional[int] = 0) -> int:
        if len(self.states) <= layer_idx:
            return 0
        return self.states[layer_idx].n_observed_tokens

    def get_max_cache_shape(self) -> Optional[int]:
        return None

    def to_legacy_cache(self) -> Tuple:
        return tuple(self.states)

    @classmethod
    def from_legacy_cache(cls, past_key_values=None, seen_tokens: int = 0) -> 'NAtSCache':
        cache = cls(seen_tokens)
        if isinstance(past_key_values, (list, tuple)):
            cache.states.extend(past_key_values)
        return cache


class NAtSMamba2Cache:
    """The layer-cache holder the Mamba hybrid layer expects: a dict of NAtSLayerCache by layer index
    (src/nats/models/natsl_attn_mamba2/modeling_nats_mamba2.py:128,144-172)."""

    def __init__(self):
        self.nats_cache: Dict[int, NAtSLayerCache] = {}

    def add_natsl_layer_cache(self, layer_idx: int = 0, seen_tokens: int = 0, n_tokens_in_nats_block: int = 0, n_attn_blocks=None,
                              nats_block_size: int = 64, attn_offset: int = 0, recurrent_offset: int = 1, n_ops: int = 2,
                              op_for_incomplete_chunk: str = 'all'):
        self.nats_cache[layer_idx] = NAtSLayerCache(seen_tokens, n_tokens_in_nats_block, n_attn_blocks, nats_block_size,
                                                    attn_offset, recurrent_offset, n_ops, op_for_incomplete_chunk)

    def reset(self):
        self.nats_cache = {}
