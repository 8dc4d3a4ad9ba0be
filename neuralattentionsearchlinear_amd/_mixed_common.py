"""Shared host logic of the two mixed operators."""
from __future__ import annotations

from typing import Optional

import torch

from . import _capi
from .attns import parallel_attn_nats_fwd
from .nats_util import CHUNK_SIZE, PackedSeqs, _seq_args, pack_sequences, route

_attn_streams: dict = {}

# Optional timing hook: when set to a callable(name, stream) it is invoked right before and right
# after each branch is enqueued ("softmax:start", "softmax:end", "linear:start", "linear:end") so a
# caller can record events on the stream the kernels were launched on.
TIMING_HOOK = None

# Where the softmax branch is launched.  True: on a side stream next to the linear branch (as the
# reference's Mamba operator does); False: on the caller's stream, one branch after the other (as the
# reference's GDN operator does); None: decide per call - side by side only when the linear branch's scan
# cannot give every CU a workgroup even at its narrowest (one compute wave = 16 state columns per workgroup).
# Both kernels take most of a CU's LDS (127 KiB / 159 KiB), so they never share a CU: when each fills the
# machine alone, running them side by side gains nothing (measured) and only blurs timings.
CONCURRENT_BRANCHES = None

# What the differentiable operator keeps from its forward for the linear branch's backward.  Keeping means: the state entering
# every chunk (bf16, K*V per chunk and head), v_new (64*V bf16) and the prep kernel's workspace (17 KiB) stay in device memory
# until the backward, which then starts at its reverse scan - about 66 KiB per chunk and head at K = V = 128, 1.1 GB per call
# at B8 T8192 H16.  Not keeping means: only the inputs are saved and the backward runs the forward's two kernels once more, as
# the reference's backward does (src/nats/ops/gated_delta_rule/chunk.py:170-332 recomputes h); a model that fits in memory
# under the reference then fits here.  The gradients are the same bit for bit either way.
#   SAVE_CHUNK_STATES = None  (default) keep only when what would be kept is at most SAVE_CHUNK_STATES_MAX_BYTES per call
#                     = True  always keep        = False  never keep
SAVE_CHUNK_STATES = None
SAVE_CHUNK_STATES_MAX_BYTES = 64 << 20
_PREP_WORKSPACE_BYTES = 17 * 1024   # per chunk and head (csrc/natsl_linear.hip)
_SCAN_COLUMNS_PER_WG = 16   # state columns of the scan's narrowest workgroup (csrc/natsl_linear.hip)


def _run_side_by_side(dev, n_chains: int, V: int) -> bool:
    if CONCURRENT_BRANCHES is not None:
        return bool(CONCURRENT_BRANCHES)
    cus = torch.cuda.get_device_properties(dev).multi_processor_count
    return n_chains * (V // _SCAN_COLUMNS_PER_WG) < cus


def _keep_chunk_states(q, v, cu_seqlens) -> bool:
    """Whether the differentiable forward keeps the linear branch's chunk states (see SAVE_CHUNK_STATES)."""
    if SAVE_CHUNK_STATES is not None:
        return bool(SAVE_CHUNK_STATES)
    B, T, H, K = q.shape
    V = v.shape[-1]
    n_seq = B if cu_seqlens is None else len(cu_seqlens) - 1                     # (a host list here)
    chunks = -(-B * T // CHUNK_SIZE) + n_seq                       # upper bound on the chunks of all sequences
    return chunks * H * (2 * K * V + 2 * CHUNK_SIZE * V + _PREP_WORKSPACE_BYTES) <= SAVE_CHUNK_STATES_MAX_BYTES


def _mark(name, stream):
    if TIMING_HOOK is not None:
        TIMING_HOOK(name, stream)


def _get_attn_stream(device: torch.device) -> torch.cuda.Stream:
    """One cached side stream per device for the softmax branch (default priority), as the
    reference does at src/nats/ops/mixed_ops/mixed_attn_mamba.py:26-30,114-124."""
    idx = device.index if device.index is not None else torch.cuda.current_device()
    if idx not in _attn_streams:
        _attn_streams[idx] = torch.cuda.Stream(device=idx)
    return _attn_streams[idx]


def _wants_grad(*tensors) -> bool:
    return torch.is_grad_enabled() and any(t is not None and torch.is_tensor(t) and t.requires_grad for t in tensors)


def linear_chunk_fwd(kind: str, q, k, v, g, beta, h0, types, scale: float, block: int, flags: int,
                     output_final_state: bool, seqs: Optional[PackedSeqs], block_start_state: bool = False,
                     chunk_states: bool = False):
    """Launch the chunked linear branch ('gdn' or 'mamba'); returns (o, final_state or None), or with
    block_start_state (o, final_state, state entering the last block, sum of g over the last block), or with chunk_states
    (o, final_state, the state entering every chunk as bf16 [total_chunks, H, V, K], v_new [B, T, H, V] (for 'mamba': v),
    the workspace)."""
    B, T, H, K = q.shape
    V = v.shape[-1]
    TN, HN = types.shape[1], types.shape[2]
    dev = q.device
    n = seqs.n_seqs if seqs is not None else B
    total_chunks = seqs.total_chunks if seqs is not None else B * (-(-T // CHUNK_SIZE))
    L = _capi.lib()
    ws = torch.empty(L.natsl_linear_workspace_bytes(total_chunks, H), dtype=torch.uint8, device=dev)
    o = torch.empty(B, T, H, V, dtype=q.dtype, device=dev)
    ht = torch.empty(n, H, K, V, dtype=torch.float32, device=dev) if output_final_state else None
    hs = torch.empty(n, H, K, V, dtype=torch.float32, device=dev) if block_start_state else None
    gs = torch.empty(n, H, dtype=torch.float32, device=dev) if block_start_state else None
    sc = torch.empty(total_chunks, H, V, K, dtype=torch.bfloat16, device=dev) if chunk_states else None
    if h0 is not None:
        if tuple(h0.shape) != (n, H, K, V):
            raise ValueError(f"initial state must have shape {(n, H, K, V)}, got {tuple(h0.shape)}")
        h0 = h0.to(torch.float32).contiguous()
    sp, ns, tot = _seq_args(seqs, total_chunks)
    vn = torch.empty_like(v) if chunk_states and kind == 'gdn' else None
    common = (_capi.ptr(h0), _capi.ptr(o), _capi.ptr(ht), _capi.ptr(hs), _capi.ptr(gs), _capi.ptr(sc),
              *((_capi.ptr(vn),) if kind == 'gdn' else ()), _capi.ptr(types), _capi.dtype_code(types.dtype), B, T, H, HN, K, V, TN,
              block, float(scale), flags, _capi.ptr(ws), ws.numel(), _capi.dtype_code(q.dtype), sp, ns, tot,
              _capi.stream_ptr(dev))
    if kind == 'gdn':
        rc = L.natsl_gdn_chunk_fwd(_capi.ptr(q), _capi.ptr(k), _capi.ptr(v), _capi.ptr(g), _capi.ptr(beta), *common)
        _capi.check(rc, "natsl_gdn_chunk_fwd")
    else:
        rc = L.natsl_mamba_chunk_fwd(_capi.ptr(q), _capi.ptr(k), _capi.ptr(v), _capi.ptr(g), *common)
        _capi.check(rc, "natsl_mamba_chunk_fwd")
    if block_start_state:
        return o, ht, hs, gs
    if chunk_states:
        return o, ht, sc, (vn if kind == 'gdn' else v), ws
    return o, ht


def _mixed_forward_impl(kind, q_attn, k_attn, v_attn, q_lattn, k_lattn, v_lattn, initial_state, g, beta, nats_block_types,
                  scale_attn, scale_lattn, cu_seqlens, cu_seqlens_nats, nats_block_size, attn_sw_size,
                  attn_same_block: bool, lin_intra: bool, output_final_state: bool, decay_non_linear: bool,
                  incomplete_block_start_with_ht: bool, use_g_for_attn: bool, qk_l2norm: bool,
                  inference: bool = False, op_type_last_chunk=None, n_tokens_in_current_block: int = 0, return_aux: bool = False,
                  keep_chunk_states: bool = False, attn_prefix_valid: Optional[torch.Tensor] = None):
    """Shared forward of the mixed operators.  With inference=True it also returns the state at the
    start of the current selector block (4-tuple), as the reference's *_chunk_inference operators do.  With return_aux
    and keep_chunk_states the auxiliary dict also holds what the linear backward would otherwise recompute
    (`linear_saved`: chunk states, v_new, workspace).

    attn_prefix_valid (bool [B, NP, HN], inference only): k_attn and v_attn start with NP more whole blocks than the other
    tensors -- cached keys; block j of that prefix is visible to selector head h's queries where the flag is set.  The softmax
    branch then runs over prefix + tokens with no queries in the prefix (a chunked forward that continues a cache: the
    reference's attention operator sizes its output by the keys, src/nats/ops/attns/attns.py:1439,1491, and cannot)."""
    if nats_block_size < CHUNK_SIZE:
        raise AssertionError("nats_block_size must be at least the compute chunk (64)")   # mixed_attn_gdn.py:90
    if nats_block_size % CHUNK_SIZE:
        raise NotImplementedError("nats_block_size must be a multiple of 64")
    if attn_sw_size is not None:
        raise NotImplementedError("attn_sw_size is not used by the reference layers and is not built")
    if use_g_for_attn:
        raise NotImplementedError("use_g_for_attn is disabled in every reference layer and is not built")
    if lin_intra and not incomplete_block_start_with_ht:
        raise NotImplementedError("incomplete_block_start_with_ht=False is not built")
    if n_tokens_in_current_block != 0:
        raise NotImplementedError("n_tokens_in_current_block != 0 is never passed by the reference layers and is not built")
    if inference and (cu_seqlens is not None):
        raise NotImplementedError("packed sequences are not supported by the prefill hand-off")
    if not q_lattn.is_cuda:
        raise _capi.NatslError("the NAtS-L mixed operator runs on the GPU only (no CPU fallback)")
    io_dtype = q_lattn.dtype
    if io_dtype not in (torch.bfloat16, torch.float32):
        raise NotImplementedError(f"dtype {io_dtype} is not supported (bf16, or fp32 which is computed in bf16)")

    def prep(t):
        return None if t is None else t.detach().to(torch.bfloat16).contiguous()

    q_attn, k_attn, v_attn, q_lattn, k_lattn, v_lattn, beta = map(prep, (q_attn, k_attn, v_attn, q_lattn, k_lattn, v_lattn, beta))
    g = g.detach().to(torch.float32).contiguous()
    types = nats_block_types.detach()
    if types.dtype not in (torch.bfloat16, torch.float32):
        types = types.float()
    types = types.contiguous()
    dev = q_lattn.device
    T = q_lattn.shape[1]
    seqs = pack_sequences(cu_seqlens, cu_seqlens_nats, nats_block_size, dev)

    if attn_prefix_valid is not None:
        if not inference or seqs is not None:
            raise NotImplementedError("a key prefix is built for the prefill operators on unpacked input")
        NP = attn_prefix_valid.shape[1]
        n_prefix = NP * nats_block_size
        if k_attn.shape[1] != q_attn.shape[1] + n_prefix or v_attn.shape[1] != k_attn.shape[1]:
            raise ValueError(f"with a prefix of {NP} blocks the keys must hold {q_attn.shape[1] + n_prefix} tokens, got {k_attn.shape[1]}")
        pv = attn_prefix_valid.to(types.dtype)
        types_attn = torch.cat([torch.stack([pv, 1 - pv], -1), types], 1).contiguous()
        q_attn = torch.cat([q_attn.new_zeros(q_attn.shape[0], n_prefix, *q_attn.shape[2:]), q_attn], 1)
        r = route(types_attn, T + n_prefix, nats_block_size, None)
    else:
        n_prefix, types_attn = 0, types
        r = route(types, T, nats_block_size, seqs)
    cur = torch.cuda.current_stream(dev)
    n_chains = (seqs.n_seqs if seqs is not None else q_lattn.shape[0]) * q_lattn.shape[2]
    side = _get_attn_stream(dev) if _run_side_by_side(dev, n_chains, v_lattn.shape[-1]) else cur
    if side is not cur:
        side.wait_stream(cur)
    with torch.cuda.stream(side):
        _mark("softmax:start", side)
        o_attn, _lse, _ = parallel_attn_nats_fwd(
            q_attn, k_attn, v_attn, types_attn, r['nats_block_indices'], None, scale_attn, nats_block_size,
            compute_incomplete_chunk_scores=attn_same_block, n_nats_blocks=r['n_nats_blocks'], seqs=seqs)
        if n_prefix:
            o_attn = o_attn[:, n_prefix:]
        _mark("softmax:end", side)
    flags = (_capi.DECAY_NON_LINEAR if decay_non_linear else 0) | (_capi.QK_L2NORM if qk_l2norm else 0) | \
            (_capi.INTRA_CHUNK if lin_intra else 0)
    _mark("linear:start", cur)
    want_start = inference and output_final_state
    res = linear_chunk_fwd(kind, q_lattn, k_lattn, v_lattn, g, beta, initial_state, types, scale_lattn,
                           nats_block_size, flags, output_final_state, seqs, block_start_state=want_start,
                           chunk_states=keep_chunk_states and not want_start)
    o_lin, ht = res[0], res[1]
    _mark("linear:end", cur)
    if side is not cur:
        cur.wait_stream(side)
        # tensors allocated on the caller's stream and read on the side stream, and the side stream's own output
        # that the caller's stream goes on to use
        for t in (q_attn, k_attn, v_attn, types_attn, r['nats_block_indices'], r['n_nats_blocks']):
            t.record_stream(side)
        o_attn.record_stream(cur)
        _lse.record_stream(cur)
    if io_dtype != torch.bfloat16:
        o_lin, o_attn = o_lin.to(io_dtype), o_attn.to(io_dtype)
    if return_aux:
        aux = dict(q_attn=q_attn, k_attn=k_attn, v_attn=v_attn, q_lattn=q_lattn, k_lattn=k_lattn, v_lattn=v_lattn, beta=beta, g=g,
                   types=types, lse=_lse, nats_block_indices=r['nats_block_indices'], n_nats_blocks=r['n_nats_blocks'],
                   linear_saved=tuple(res[2:5]) if keep_chunk_states and not want_start else None)
        return o_lin, o_attn, ht, aux
    if not inference:
        return o_lin, o_attn, ht
    h_start = None
    if want_start:
        # State at the start of the current block (src/nats/ops/gated_delta_rule/chunk_fwd.py:178-206):
        # with an incomplete last block it is the state that entered that block; when the input ends on
        # a block boundary it is the state after the last block under its TRUE type -- the final state
        # if that type is linear, otherwise the entering state rolled forward by the block's decay.
        hs, gs = res[2], res[3]
        if T % nats_block_size != 0:
            h_start = hs
        else:
            if op_type_last_chunk is None:
                raise AssertionError("op_type_last_chunk is required when the input ends on a block boundary")
            H = ht.shape[1]
            lin = (op_type_last_chunk[..., 1] > 0)
            lin = lin.repeat_interleave(H // lin.shape[1], dim=1).view(ht.shape[0], H, 1, 1)
            rolled = hs * torch.exp(gs).view(ht.shape[0], H, 1, 1) if decay_non_linear else hs
            h_start = torch.where(lin, ht, rolled)
    return o_lin, o_attn, ht, h_start


class _MixedFunction(torch.autograd.Function):
    """The mixed operator with its backward (src/nats/ops/mixed_ops/mixed_attn_gdn.py:193-283,
    src/nats/ops/mixed_ops/mixed_attn_mamba.py:194-292): the softmax branch's gradients come from the HIP backward
    (natsl_softmax_sparse_bwd), the linear branch's from natsl_linear_chunk_bwd behind _linear_bwd.linear_chunk_backward; the
    selector's straight-through gradient is returned for nats_block_types, column 0 = softmax op, column 1 = linear op."""

    @staticmethod
    def forward(ctx, cfg, q_attn, k_attn, v_attn, q_lattn, k_lattn, v_lattn, initial_state, g, beta, nats_block_types):
        from ._linear_bwd import hip_backward_is_built
        keep = _keep_chunk_states(q_lattn, v_lattn, cfg['cu_seqlens']) and hip_backward_is_built(q_lattn.shape[-1], v_lattn.shape[-1])
        with torch.no_grad():
            o_lin, o_attn, ht, aux = _mixed_forward_impl(
                cfg['kind'], q_attn, k_attn, v_attn, q_lattn, k_lattn, v_lattn, initial_state, g, beta, nats_block_types,
                cfg['scale_attn'], cfg['scale_lattn'], cfg['cu_seqlens'], cfg['cu_seqlens_nats'], cfg['block'], None,
                cfg['attn_same_block'], cfg['lin_intra'],
                cfg['output_final_state'], cfg['decay_non_linear'], True, False, cfg['qk_l2norm'], return_aux=True,
                keep_chunk_states=keep)
        ctx.cfg = cfg
        ctx.in_dtypes = tuple(None if t is None else t.dtype for t in (q_attn, k_attn, v_attn, q_lattn, k_lattn, v_lattn,
                                                                       initial_state, g, beta, nats_block_types))
        ctx.has_h0 = initial_state is not None
        saved = [aux[n] for n in ('q_attn', 'k_attn', 'v_attn', 'q_lattn', 'k_lattn', 'v_lattn', 'g', 'types', 'lse',
                                  'nats_block_indices', 'n_nats_blocks')]
        saved += [o_attn.to(torch.bfloat16), aux['beta'] if aux['beta'] is not None else g.new_zeros(0),
                  initial_state if initial_state is not None else g.new_zeros(0)]
        ctx.n_linear_saved = 0
        if aux['linear_saved'] is not None:
            # (for 'mamba' the second entry is v_lattn itself, saved above already: the same tensor, no second copy)
            saved += list(aux['linear_saved'])
            ctx.n_linear_saved = len(aux['linear_saved'])
        ctx.save_for_backward(*saved)
        if ht is None:
            return o_lin, o_attn, None
        return o_lin, o_attn, ht

    @staticmethod
    def backward(ctx, do_lin, do_attn, dht):
        from ._linear_bwd import linear_chunk_backward
        from .attns import parallel_attn_nats_bwd
        cfg = ctx.cfg
        (q_a, k_a, v_a, q_l, k_l, v_l, g, types, lse, idx, nblk, o_attn, beta, h0) = ctx.saved_tensors[:14]
        linear_saved = tuple(ctx.saved_tensors[14:]) if ctx.n_linear_saved else None
        beta = beta if beta.numel() else None
        h0 = h0 if ctx.has_h0 else None
        B, NB, HN, _ = types.shape
        seqs = pack_sequences(cfg['cu_seqlens'], cfg['cu_seqlens_nats'], cfg['block'], types.device)
        if do_attn is not None:
            dq_a, dk_a, dv_a, _, dn_attn = parallel_attn_nats_bwd(
                q_a, k_a, v_a, o_attn, types, idx, nblk, None, lse, do_attn.to(torch.bfloat16).contiguous(), scale=cfg['scale_attn'],
                NAtS_block_size=cfg['block'], compute_incomplete_chunk_scores=cfg['attn_same_block'],
                compute_dnats_for_invalid_blocks_attn=cfg['dnats_invalid_attn'], seqs=seqs)
        else:
            dq_a, dk_a, dv_a = torch.zeros_like(q_a), torch.zeros_like(k_a), torch.zeros_like(v_a)
            dn_attn = torch.zeros(B, NB, HN, dtype=torch.float32, device=types.device)
        if do_lin is None:
            do_lin = torch.zeros(*q_l.shape[:3], v_l.shape[-1], dtype=torch.float32, device=q_l.device)
        lin_args = (cfg['scale_lattn'], cfg['block'], cfg['decay_non_linear'], cfg['qk_l2norm'], cfg['lin_intra'])
        dq_l, dk_l, dv_l, dg, dbeta, dh0, dn_lin = linear_chunk_backward(
            cfg['kind'], q_l, k_l, v_l, g, beta, h0, types, *lin_args, do_lin, dht, cfg['dnats_invalid_linear'], seqs,
            saved=linear_saved)
        d_types = torch.stack([dn_attn.float(), dn_lin.float()], -1)
        grads = [dq_a, dk_a, dv_a, dq_l, dk_l, dv_l, dh0, dg, dbeta, d_types]
        grads = [None if (t is None or dt is None) else t.to(dt) for t, dt in zip(grads, ctx.in_dtypes)]
        return (None, *grads)


def _host_list(x):
    return None if x is None else [int(t) for t in (x.tolist() if torch.is_tensor(x) else x)]


def mixed_forward(kind, q_attn, k_attn, v_attn, q_lattn, k_lattn, v_lattn, initial_state, g, beta, nats_block_types,
                  scale_attn, scale_lattn, cu_seqlens, cu_seqlens_nats, nats_block_size, attn_sw_size,
                  attn_same_block: bool, lin_intra: bool, output_final_state: bool, decay_non_linear: bool,
                  incomplete_block_start_with_ht: bool, use_g_for_attn: bool, qk_l2norm: bool,
                  inference: bool = False, op_type_last_chunk=None, n_tokens_in_current_block: int = 0,
                  dnats_invalid_attn: bool = False, dnats_invalid_linear: bool = False, attn_prefix_valid=None):
    """Entry of the mixed operators: the plain forward, or, when a tensor requires grad, the differentiable operator."""
    tensors = (q_attn, k_attn, v_attn, q_lattn, k_lattn, v_lattn, initial_state, g, beta, nats_block_types)
    # (the prefill operators are plain functions in the reference too: their outputs carry no gradient)
    if inference or not _wants_grad(*tensors):
        return _mixed_forward_impl(kind, q_attn, k_attn, v_attn, q_lattn, k_lattn, v_lattn, initial_state, g, beta,
                                   nats_block_types, scale_attn, scale_lattn, cu_seqlens, cu_seqlens_nats, nats_block_size,
                                   attn_sw_size, attn_same_block, lin_intra, output_final_state, decay_non_linear,
                                   incomplete_block_start_with_ht, use_g_for_attn, qk_l2norm, inference, op_type_last_chunk,
                                   n_tokens_in_current_block, attn_prefix_valid=attn_prefix_valid)
    if attn_prefix_valid is not None:
        raise NotImplementedError("a key prefix is built for the prefill operators (no gradient)")
    if attn_sw_size is not None or use_g_for_attn or not incomplete_block_start_with_ht:
        raise NotImplementedError("attn_sw_size / use_g_for_attn / incomplete_block_start_with_ht=False are not built")
    cfg = dict(kind=kind, scale_attn=float(scale_attn), scale_lattn=float(scale_lattn), block=int(nats_block_size),
               attn_same_block=bool(attn_same_block), lin_intra=bool(lin_intra), output_final_state=bool(output_final_state),
               decay_non_linear=bool(decay_non_linear), qk_l2norm=bool(qk_l2norm), dnats_invalid_attn=bool(dnats_invalid_attn),
               dnats_invalid_linear=bool(dnats_invalid_linear), cu_seqlens=_host_list(cu_seqlens),
               cu_seqlens_nats=_host_list(cu_seqlens_nats))
    return _MixedFunction.apply(cfg, *tensors)
