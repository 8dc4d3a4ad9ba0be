"""Backward of the linear-recurrent branches (Gated DeltaNet, Mamba2-style SSD) for training.

linear_chunk_backward_hip is the product path: the forward's per-chunk state and v_new outputs (kept by the differentiable
operator from its own forward, else the forward once more), then
natsl_linear_chunk_bwd (csrc/natsl_linear_bwd.hip: a reverse scan over the chunks and a per-chunk gradient kernel), and the
few lines of host glue around them (block sums of g, the per-block sums of the gate gradients).  It replaces
chunk_gated_delta_rule_nats_bwd (src/nats/ops/gated_delta_rule/chunk.py:170-332) and the Mamba counterpart
(src/nats/ops/mamba/chunk.py:112-260) in function.  linear_chunk_backward_torch is the same method as fp32 torch operations
on the GPU, for key widths the kernels are not built for and as the method's plain statement; both follow the
chunked algorithm of the forward kernels (csrc/natsl_linear.hip), so the gradients belong to the forward that was actually
computed, up to its bf16 rounding.

Per 64-token chunk c with entering state S_c (notation of the forward):
    X = v - W S_c,  v_new = T X,  o = Q~ S_c + P v_new,  S_{c+1} = e^{gamma_last} S_c + gate * K~^T v_new
(a block that is not typed linear ends in S = f * S_blockstart + gate_off * K~^T v_new instead, f = e^{sum of g over the
block} or 1).  Three steps (the torch formulation; the kernels split the work the same way):
  1. the states S_c of all chunks: the forward kernel run once more with its per-chunk state output (bf16, as the forward
     used them);
  2. the state gradients: the reverse recurrence
         dv_new = P^T dO + K~ dS',   dX = T^T dv_new,   dS_c = e^{gamma_last} dS' + Q~^T dO - W^T dX
     (dS' = gradient of S_{c+1}; at the end of a block that is not typed linear it goes to the block's first chunk times f
     instead of into the chain), one loop without autograd;
  3. everything else in ONE batched autograd call over all chunks at once: with S_c and dS' of every chunk as constants, the
     gradients of  sum_c <dO_c, o_c> + <dS'_c, S_{c+1}>  with respect to q, k, v, g, beta and the gates are the exact
     gradients of the whole recurrence (the chain rule split at the states).

The selector's straight-through gradient for the linear operator (src/nats/ops/common/chunk_o.py:438-443, :487-492) is the
inner product of the state gradient behind a chunk with that chunk's additive state update k~^T v_new: the derivative
with respect to a gate on the update.  It is taken with a gate tensor of ones (blocks typed linear) and, when the
gradient of the blocks that are NOT typed linear is asked for, a zero-valued gate on the update those blocks would have
made; per selector block and selector head the chunks and heads are summed (chunk_o.py:1571-1575).
"""
from __future__ import annotations

import torch

C = 64


def _chunks(x, NT):
    """[B,T,H,*] -> [B,H,NT,C,*], zero padded."""
    B, T = x.shape[:2]
    if NT * C != T:
        x = torch.cat([x, x.new_zeros(B, NT * C - T, *x.shape[2:])], 1)
    x = x.reshape(B, NT, C, *x.shape[2:])
    return x.permute(0, 3, 1, 2, *range(4, x.dim()))


def _chunk_local(kind, q, k, v, g, beta, scale, l2norm):
    """Everything of a chunk that does not depend on the state, for all chunks at once (differentiable):
    qe, kd [B,H,NT,C,K], P [B,H,NT,C,C], vc [B,H,NT,C,V], dec, glast [B,H,NT], and for the delta rule TmB [..,C,C], w [..,C,K]."""
    T = q.shape[1]
    NT = -(-T // C)
    delta = kind == 'gdn'
    if l2norm and delta:
        q = q * torch.rsqrt((q * q).sum(-1, keepdim=True) + 1e-6)
        k = k * torch.rsqrt((k * k).sum(-1, keepdim=True) + 1e-6)
    qc, kc, vc, gc = _chunks(q, NT), _chunks(k, NT), _chunks(v, NT), _chunks(g, NT)
    gam = gc.cumsum(-1)                                                     # [B,H,NT,C]
    tri = torch.tril(torch.ones(C, C, dtype=torch.bool, device=q.device))
    diff = gam.unsqueeze(-1) - gam.unsqueeze(-2)
    Lm = torch.where(tri, torch.exp(torch.where(tri, diff, torch.zeros_like(diff))), torch.zeros_like(diff))
    P = scale * (qc @ kc.transpose(-1, -2)) * Lm
    glast = gam[..., -1]                                                    # [B,H,NT]
    eg = torch.exp(gam).unsqueeze(-1)
    qe = scale * qc * eg
    dk = glast.unsqueeze(-1) - gam
    if not delta:
        dk = torch.clamp(dk, max=0.0)                                       # src/nats/ops/mamba/chunk_h.py:177
    kd = kc * torch.exp(dk).unsqueeze(-1)
    out = dict(qe=qe, kd=kd, P=P, vc=vc, dec=torch.exp(glast), glast=glast)
    if delta:
        bc = _chunks(beta, NT)
        A = torch.tril(bc.unsqueeze(-1) * (kc @ kc.transpose(-1, -2)) * Lm, -1)
        eye = torch.eye(C, dtype=q.dtype, device=q.device)
        Tm = torch.linalg.solve_triangular(eye + A, eye.expand_as(A).contiguous(), upper=False)
        out['TmB'] = Tm * bc.unsqueeze(-2)
        out['w'] = kc * eg
    return out


def linear_chunk_forward_torch(kind, q, k, v, g, beta, h0, lin, scale, block, decay, l2norm, intra, gate_on, gate_off):
    """Differentiable chunked forward (the whole recurrence under autograd; kept as the plain statement of the algorithm).
    q,k [B,T,H,K], v [B,T,H,V], g,beta [B,T,H] (fp32), h0 [B,H,K,V] or None, lin bool [B,NB,H] (block typed linear),
    gate_on / gate_off [B,NT,H] (ones / zeros).  -> (o [B,T,H,V], S [B,H,K,V])."""
    B, T, H, K = q.shape
    V = v.shape[-1]
    NT = -(-T // C)
    per = block // C
    delta = kind == 'gdn'
    m = _chunk_local(kind, q, k, v, g, beta, scale, l2norm)
    S = torch.zeros(B, H, K, V, dtype=q.dtype, device=q.device) if h0 is None else h0
    outs = []
    S_start, gsum = S, None
    for c in range(NT):
        if c % per == 0:
            S_start, gsum = S, torch.zeros(B, H, dtype=q.dtype, device=q.device)
        vn = m['TmB'][:, :, c] @ (m['vc'][:, :, c] - m['w'][:, :, c] @ S) if delta else m['vc'][:, :, c]
        o = m['qe'][:, :, c] @ S
        if intra:
            o = o + m['P'][:, :, c] @ vn
        outs.append(o)
        upd = m['kd'][:, :, c].transpose(-1, -2) @ vn                       # the chunk's additive state update
        gsum = gsum + m['glast'][:, :, c]
        S_up = m['dec'][:, :, c, None, None] * S + gate_on[:, c, :, None, None] * upd
        if (c + 1) % per == 0 or c == NT - 1:
            keep = lin[:, (c * C) // block][..., None, None]
            back = S_start * torch.exp(gsum)[..., None, None] if decay else S_start
            S = torch.where(keep, S_up, back + gate_off[:, c, :, None, None] * upd)
        else:
            S = S_up
    o = torch.stack(outs, 2)                                                # [B,H,NT,C,V]
    o = o.permute(0, 2, 3, 1, 4).reshape(B, NT * C, H, V)[:, :T]
    return o, S


def hip_backward_is_built(K: int, V: int) -> bool:
    """The head dims natsl_linear_chunk_bwd is built for."""
    return K in (64, 128, 192) and V % 64 == 0


def linear_chunk_backward(kind, q, k, v, g, beta, h0, types, scale, block, decay, l2norm, intra, do, dht,
                          dnats_for_invalid_blocks, seqs=None, saved=None):
    """Gradients of the chunked linear branch: -> (dq, dk, dv, dg fp32, dbeta or None, dh0 or None, dnats fp32 [B,NB,HN]).
    types [B,NB,HN,2]; do [B,T,H,V]; dht [N,H,K,V] or None; seqs: packed sequences (B = 1) or None; saved: what
    linear_chunk_fwd(..., chunk_states=True) returned after (o, final_state) on these same inputs, if the caller kept it.  The
    HIP kernels (natsl_linear_chunk_bwd) for K in 64/128/192 -- V a multiple of 64 as it is, other multiples of 16 behind zero
    columns --, else the torch formulation below, one sequence at a time.

    dnats_for_invalid_blocks with block > 64 raises NotImplementedError: for a block of several chunks that is not typed
    linear the reference sums a virtual key gradient v . dh over EVERY chunk of the block
    (src/nats/ops/common/chunk_o.py:446-491, summed per block at :1571), each against the dh its compacted reverse scan holds
    at that chunk (src/nats/ops/common/chunk_delta_h.py:492-509); that definition has not been restated here.  With one
    chunk per block it is the gradient of a zero gate on the block's state update, which is what this function returns."""
    if dnats_for_invalid_blocks and block > C:
        raise NotImplementedError(
            f"compute_dnats_for_invalid_blocks_linear_att=True is built for nats_block_size == {C} only (got {block}): "
            "pass compute_dnats_for_invalid_blocks_linear_att=False (the layers' default)")
    K, V = q.shape[-1], v.shape[-1]
    if hip_backward_is_built(K, V):
        return linear_chunk_backward_hip(kind, q, k, v, g, beta, h0, types, scale, block, decay, l2norm, intra, do, dht,
                                         dnats_for_invalid_blocks, seqs, saved)
    if hip_backward_is_built(K, 64) and V % 16 == 0:
        # Value widths the kernels are not built for (16..48, 96, ..): zero columns up to the next multiple of 64.  The state's
        # columns never mix, a zero column of v and dO stays zero through the whole recurrence and adds nothing to any sum
        # over V, so the gradients are exactly those of the narrower problem.
        pad = -V % 64
        padv = lambda t: None if t is None else torch.nn.functional.pad(t, (0, pad))
        res = linear_chunk_backward_hip(kind, q, k, padv(v), g, beta, padv(h0), types, scale, block, decay, l2norm, intra, padv(do),
                                        padv(dht), dnats_for_invalid_blocks, seqs, None)
        return (res[0], res[1], res[2][..., :V].contiguous(), res[3], res[4], None if res[5] is None else res[5][..., :V].contiguous(),
                res[6])
    if seqs is None:
        return linear_chunk_backward_torch(kind, q, k, v, g, beta, h0, types, scale, block, decay, l2norm, intra, do, dht,
                                           dnats_for_invalid_blocks)
    parts = []
    for i in range(seqs.n_seqs):
        a, b = seqs.cu_seqlens[i], seqs.cu_seqlens[i + 1]
        na, nb = seqs.cu_seqlens_nats[i], seqs.cu_seqlens_nats[i + 1]
        parts.append(linear_chunk_backward_torch(
            kind, q[:, a:b], k[:, a:b], v[:, a:b], g[:, a:b], None if beta is None else beta[:, a:b],
            None if h0 is None else h0[i:i + 1], types[:, na:nb], scale, block, decay, l2norm, intra, do[:, a:b],
            None if dht is None else dht[i:i + 1], dnats_for_invalid_blocks))
    cat = lambda j, dim: None if parts[0][j] is None else torch.cat([p[j] for p in parts], dim)
    return cat(0, 1), cat(1, 1), cat(2, 1), cat(3, 1), cat(4, 1), cat(5, 0), cat(6, 1)


_MAPS = {}


def _block_maps(B, T, block, seqs, dev):
    """Index tensors that tie tokens and chunks to selector blocks, flat over the sequences: for every block the first / one
    past the last token and chunk, the index of its last chunk, and for every token its block."""
    key = (B, T, block, None if seqs is None else tuple(seqs.cu_seqlens), str(dev))
    m = _MAPS.get(key)
    if m is not None:
        return m
    per = block // C
    bounds = [(i * T, (i + 1) * T) for i in range(B)] if seqs is None else list(zip(seqs.cu_seqlens[:-1], seqs.cu_seqlens[1:]))
    t0s, t1s, c0s, c1s, toks = [], [], [], [], []
    coff, boff = 0, 0
    for a, b in bounds:
        n = b - a
        nb, nc = -(-n // block), -(-n // C)
        j = torch.arange(nb)
        t0s.append(a + j * block)
        t1s.append(torch.clamp(a + (j + 1) * block, max=b))
        c0s.append(coff + j * per)
        c1s.append(torch.clamp(coff + (j + 1) * per, max=coff + nc))
        toks.append(boff + torch.arange(n) // block)
        coff += nc
        boff += nb
    m = tuple(torch.cat(x).to(dev) for x in (t0s, t1s, c0s, c1s, toks))
    if len(_MAPS) > 16:
        _MAPS.clear()
    _MAPS[key] = m
    return m


def _range_sums(x, first, end):
    """Sums of x[first[j]:end[j]] along dim 0 for every j (fp64 running sums: the same result every time)."""
    xt = x.double().t().contiguous()                      # [H, n]: the running sum along the contiguous dimension
    cs = torch.cat([xt.new_zeros(xt.shape[0], 1), xt.cumsum(1)], 1)
    return (cs[:, end] - cs[:, first]).t().float().contiguous()


def linear_chunk_backward_hip(kind, q, k, v, g, beta, h0, types, scale, block, decay, l2norm, intra, do, dht,
                              dnats_for_invalid_blocks, seqs=None, saved=None):
    """The backward as kernels: the forward once more (storing every chunk's entering state and v_new) unless the caller kept
    those from its own forward (`saved`), then the reverse scan and the per-chunk gradients (csrc/natsl_linear_bwd.hip)."""
    from . import _capi
    from ._mixed_common import linear_chunk_fwd
    from .nats_util import _seq_args
    B, T, H, K = q.shape
    V = v.shape[-1]
    NB, HN = types.shape[1], types.shape[2]
    N = B if seqs is None else seqs.n_seqs
    NTtot = B * (-(-T // C)) if seqs is None else seqs.total_chunks
    dev = q.device
    f32, bf16 = torch.float32, torch.bfloat16
    delta = kind == 'gdn'
    flags = (_capi.DECAY_NON_LINEAR if decay else 0) | (_capi.QK_L2NORM if l2norm else 0) | (_capi.INTRA_CHUNK if intra else 0)
    with torch.no_grad():
        ty = types.detach()
        ty = (ty if ty.dtype in (bf16, f32) else ty.float()).contiguous()
        qb, kb, vb = (t.detach().to(bf16).contiguous() for t in (q, k, v))
        gf = g.detach().to(f32).contiguous()
        bb = beta.detach().to(bf16).contiguous() if delta else None
        h0f = None if h0 is None else h0.detach().to(f32).contiguous()
        if saved is not None:
            states, v_new, ws = saved
        else:
            _, _, states, v_new, ws = linear_chunk_fwd(kind, qb, kb, vb, gf, bb, h0f, ty, scale, block, flags, False, seqs,
                                                       chunk_states=True)
        tok0, tok1, ch0, ch1, tok_blk = _block_maps(B, T, block, seqs, dev)
        # sum of g over every selector block [all blocks, H], from the chunk sums the forward left in its workspace (behind
        # the TmB and P areas: four vectors of 64 floats per chunk and head, the fourth {e^G, G, is_linear, ..}; they are
        # what the forward's own roll-back decay was made of)
        units = NTtot * H
        g_chunk = ws[units * (2 * C * C * 2):].view(f32).view(units, 4 * C)[:, 3 * C + 1].reshape(NTtot, H)
        one_chunk_blocks = block == C
        gsum = g_chunk.contiguous() if one_chunk_blocks else _range_sums(g_chunk, ch0, ch1).contiguous()
        d_states = torch.empty_like(states)
        dq, dk, dv = torch.empty_like(qb), torch.empty_like(kb), torch.empty_like(vb)
        dg = torch.empty(B, T, H, dtype=f32, device=dev)
        dbeta = torch.empty(B, T, H, dtype=f32, device=dev) if delta else None
        dbeta_parts = torch.empty(B, T, H, V // 16, dtype=f32, device=dev) if delta else None
        dh0 = torch.empty(N, H, K, V, dtype=f32, device=dev) if h0 is not None else None
        gate = torch.empty(NTtot, H, dtype=f32, device=dev)
        rb = torch.empty(NTtot, H, dtype=f32, device=dev)
        dof = do.detach().to(bf16).contiguous()
        dhtf = None if dht is None else dht.detach().to(f32).contiguous()
        P = _capi.ptr
        sp, ns, tot = _seq_args(seqs, NTtot)
        rc = _capi.lib().natsl_linear_chunk_bwd(
            1 if delta else 0, P(qb), P(kb), P(v_new), P(gf), P(bb), P(dof), P(dhtf), P(states), P(ty), _capi.dtype_code(ty.dtype),
            P(gsum), P(ws), P(d_states), P(dbeta_parts), P(dq), P(dk), P(dv), P(dg), P(dbeta), P(dh0), P(gate), P(rb),
            B, T, H, HN, K, V, NB, block, float(scale), flags, _capi.dtype_code(bf16), sp, ns, tot, _capi.stream_ptr(dev))
        _capi.check(rc, "natsl_linear_chunk_bwd")
        if decay:
            # the decay of a rolled-back block acts on every token of the block (rb is non-zero at such a block's last chunk)
            dg.view(B * T, H).add_(rb[ch1 - 1][tok_blk])
        lin = (torch.round(ty[..., 1].float()) == 1).repeat_interleave(H // HN, dim=2).view(-1, H)          # [all blocks, H]
        dn = torch.where(lin, gate if one_chunk_blocks else _range_sums(gate, ch0, ch1), torch.zeros_like(gsum))
        if dnats_for_invalid_blocks:
            # the (zero-valued) gate on the update a block that is not typed linear would have made (one chunk per block here)
            dn = dn + torch.where(lin, torch.zeros_like(gsum), gate[ch1 - 1])
        dn = dn.view(B, NB, HN, H // HN).sum(3)
    return (dq.to(q.dtype), dk.to(k.dtype), dv.to(v.dtype), dg, None if dbeta is None else dbeta.to(beta.dtype), dh0, dn)


def linear_chunk_backward_torch(kind, q, k, v, g, beta, h0, types, scale, block, decay, l2norm, intra, do, dht,
                                dnats_for_invalid_blocks):
    """The same gradients with torch operations (every shape)."""
    B, T, H, K = q.shape
    V = v.shape[-1]
    HN, NB = types.shape[2], types.shape[1]
    NT = -(-T // C)
    per = block // C
    f32 = torch.float32
    delta = kind == 'gdn'
    dev = q.device
    lin = (torch.round(types[..., 1].detach().float()) == 1).repeat_interleave(H // HN, dim=2)            # [B,NB,H]
    blk_of = torch.arange(NT, device=dev) * C // block                                                     # chunk -> block
    first_of = blk_of * per                                                                               # chunk -> first chunk of its block
    last = ((torch.arange(NT, device=dev) + 1) % per == 0) | (torch.arange(NT, device=dev) == NT - 1)      # chunk ends its block
    keep_c = lin[:, blk_of].permute(0, 2, 1)                                                               # [B,H,NT]: the chunk's block is typed linear
    rolled = last.view(1, 1, NT) & ~keep_c                                                                # the state is rolled back behind this chunk
    last_l = [((c + 1) % per == 0) or c == NT - 1 for c in range(NT)]
    first_l = [(c * C // block) * per for c in range(NT)]

    def block_factor(glast):
        # e^{sum of gamma_last over the chunks of the block} per chunk (the roll-back's decay), or 1
        if not decay:
            return torch.ones_like(glast)
        pad = NB * per - NT
        gl = torch.cat([glast, glast.new_zeros(B, H, pad)], -1) if pad else glast
        return torch.exp(gl.view(B, H, NB, per).sum(-1))[:, :, blk_of]

    with torch.no_grad():
        qf, kf, vf, gf = (t.detach().to(f32) for t in (q, k, v, g))
        bf = beta.detach().to(f32) if delta else None
        m = _chunk_local(kind, qf, kf, vf, gf, bf, scale, l2norm)
        dO = _chunks(do.detach().to(f32), NT)                                                             # [B,H,NT,C,V]
        f_c = block_factor(m['glast'])
        # ---- 1. the entering state of every chunk: the forward kernel run once more, storing them ------------------------
        from . import _capi
        from ._mixed_common import linear_chunk_fwd
        flags = (_capi.DECAY_NON_LINEAR if decay else 0) | (_capi.QK_L2NORM if l2norm else 0) | (_capi.INTRA_CHUNK if intra else 0)
        bf16 = torch.bfloat16
        ty = types.detach()
        ty = (ty if ty.dtype in (bf16, f32) else ty.float()).contiguous()
        st = linear_chunk_fwd(kind, q.detach().to(bf16).contiguous(), k.detach().to(bf16).contiguous(),
                              v.detach().to(bf16).contiguous(), g.detach().to(f32).contiguous(),
                              beta.detach().to(bf16).contiguous() if delta else None,
                              None if h0 is None else h0.detach().to(f32).contiguous(), ty, scale, block, flags,
                              False, None, chunk_states=True)[2]
        S_all = st.view(B, NT, H, V, K).permute(0, 2, 1, 4, 3).to(f32)                                     # [B,H,NT,K,V]
        del st
        # ---- 2. the gradient of the state behind every chunk ----------------------------------------------------------
        dSp = torch.empty(B, H, NT, K, V, dtype=f32, device=dev)
        dS = torch.zeros(B, H, K, V, dtype=f32, device=dev) if dht is None else dht.detach().to(f32)
        pending = None                                   # f * dS' of a rolled-back block, owed to the block's first chunk
        for c in range(NT - 1, -1, -1):
            dSp[:, :, c] = dS
            if last_l[c]:
                rb = rolled[:, :, c, None, None]
                pending = torch.where(rb, dS * f_c[:, :, c, None, None], torch.zeros_like(dS))
                dS_up = torch.where(rb, torch.zeros_like(dS), dS)
            else:
                dS_up = dS
            dvn = m['kd'][:, :, c] @ dS_up
            if intra:
                dvn = dvn + m['P'][:, :, c].transpose(-1, -2) @ dO[:, :, c]
            dS = m['dec'][:, :, c, None, None] * dS_up + m['qe'][:, :, c].transpose(-1, -2) @ dO[:, :, c]
            if delta:
                dX = m['TmB'][:, :, c].transpose(-1, -2) @ dvn
                dS = dS - m['w'][:, :, c].transpose(-1, -2) @ dX
            if c % per == 0:
                dS = dS + pending
        dh0 = dS if h0 is not None else None
        S_first = S_all[:, :, first_of]                                                                   # each chunk's block-start state
        del m

    # ---- 3. everything else: one batched autograd call with the states as constants ----------------------------------
    with torch.enable_grad():
        leaves = [t.detach().to(f32).requires_grad_(True) for t in (q, k, v, g)]
        qf, kf, vf, gf = leaves
        bf = beta.detach().to(f32).requires_grad_(True) if delta else None
        gate_on = torch.ones(B, NT, H, dtype=f32, device=dev, requires_grad=True)
        gate_off = torch.zeros(B, NT, H, dtype=f32, device=dev, requires_grad=dnats_for_invalid_blocks)
        m = _chunk_local(kind, qf, kf, vf, gf, bf, scale, l2norm)
        vn = m['TmB'] @ (m['vc'] - m['w'] @ S_all) if delta else m['vc']
        o = m['qe'] @ S_all
        if intra:
            o = o + m['P'] @ vn
        upd = m['kd'].transpose(-1, -2) @ vn
        S_up = m['dec'][..., None, None] * S_all + gate_on.permute(0, 2, 1)[..., None, None] * upd
        S_back = block_factor(m['glast'])[..., None, None] * S_first + gate_off.permute(0, 2, 1)[..., None, None] * upd
        S_next = torch.where(rolled[..., None, None], S_back, S_up)
        total = (o * dO).sum() + (S_next * dSp).sum()
        wrt = [qf, kf, vf, gf, gate_on]
        if bf is not None:
            wrt.append(bf)
        if dnats_for_invalid_blocks:
            wrt.append(gate_off)
        grads = list(torch.autograd.grad(total, wrt, allow_unused=True))
    dq, dk, dv, dg, dgate = grads[:5]
    rest = grads[5:]
    dbeta = rest.pop(0) if bf is not None else None
    # a gate acts where its block's update is kept (typed linear), the zero gate where it is not
    lin_c = lin.repeat_interleave(per, dim=1)[:, :NT]                                                     # per chunk
    dn = torch.where(lin_c, dgate, torch.zeros_like(dgate))
    if dnats_for_invalid_blocks:
        dgo = rest.pop(0)
        dn = dn + torch.where(lin_c, torch.zeros_like(dgo), dgo)
    pad = NB * per - NT
    if pad:
        dn = torch.cat([dn, dn.new_zeros(B, pad, H)], 1)
    dn = dn.view(B, NB, per, HN, H // HN).sum((2, 4))
    z = lambda t, like: torch.zeros_like(like) if t is None else t
    return (z(dq, qf).to(q.dtype), z(dk, kf).to(k.dtype), z(dv, vf).to(v.dtype), z(dg, gf),
            None if bf is None else z(dbeta, bf).to(beta.dtype), dh0, dn)
