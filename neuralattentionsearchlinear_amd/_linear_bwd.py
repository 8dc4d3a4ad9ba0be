"""Backward of the linear-recurrent branches (Gated DeltaNet, Mamba2-style SSD) for training.

NOT a HIP kernel yet: the gradients are obtained by re-running the chunked forward as differentiable torch operations on
the GPU (fp32, batched over sequences and heads, one step per 64-token chunk) and calling autograd on it.  It is the
same algorithm the forward kernels implement (csrc/natsl_linear.hip), so the gradients belong to the forward that was
actually computed, up to its bf16 rounding.  It replaces chunk_gated_delta_rule_nats_bwd
(src/nats/ops/gated_delta_rule/chunk.py:170-332) and the Mamba counterpart (src/nats/ops/mamba/chunk.py:112-260) in
function, not in speed.

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


def linear_chunk_forward_torch(kind, q, k, v, g, beta, h0, lin, scale, block, decay, l2norm, intra, gate_on, gate_off):
    """Differentiable chunked forward.  q,k [B,T,H,K], v [B,T,H,V], g,beta [B,T,H] (fp32), h0 [B,H,K,V] or None,
    lin bool [B,NB,H] (block typed linear), gate_on / gate_off [B,NT,H] (ones / zeros).  -> (o [B,T,H,V], S [B,H,K,V])."""
    B, T, H, K = q.shape
    V = v.shape[-1]
    NT = -(-T // C)
    per = block // C
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
    dec = torch.exp(glast)
    if delta:
        bc = _chunks(beta, NT)
        A = torch.tril(bc.unsqueeze(-1) * (kc @ kc.transpose(-1, -2)) * Lm, -1)
        eye = torch.eye(C, dtype=q.dtype, device=q.device)
        Tm = torch.linalg.solve_triangular(eye + A, eye.expand_as(A).contiguous(), upper=False)
        TmB = Tm * bc.unsqueeze(-2)
        w = kc * eg
    S = torch.zeros(B, H, K, V, dtype=q.dtype, device=q.device) if h0 is None else h0
    outs = []
    S_start, gsum = S, None
    for c in range(NT):
        if c % per == 0:
            S_start, gsum = S, torch.zeros(B, H, dtype=q.dtype, device=q.device)
        if delta:
            vn = TmB[:, :, c] @ (vc[:, :, c] - w[:, :, c] @ S)
        else:
            vn = vc[:, :, c]
        o = qe[:, :, c] @ S
        if intra:
            o = o + P[:, :, c] @ vn
        outs.append(o)
        upd = kd[:, :, c].transpose(-1, -2) @ vn                            # the chunk's additive state update
        gsum = gsum + glast[:, :, c]
        S_up = dec[:, :, c, None, None] * S + gate_on[:, c, :, None, None] * upd
        if (c + 1) % per == 0 or c == NT - 1:
            keep = lin[:, (c * C) // block][..., None, None]
            back = S_start * torch.exp(gsum)[..., None, None] if decay else S_start
            S = torch.where(keep, S_up, back + gate_off[:, c, :, None, None] * upd)
        else:
            S = S_up
    o = torch.stack(outs, 2)                                                # [B,H,NT,C,V]
    o = o.permute(0, 2, 3, 1, 4).reshape(B, NT * C, H, V)[:, :T]
    return o, S


def linear_chunk_backward(kind, q, k, v, g, beta, h0, types, scale, block, decay, l2norm, intra, do, dht,
                          dnats_for_invalid_blocks):
    """Gradients of the chunked linear branch: -> (dq, dk, dv, dg fp32, dbeta or None, dh0 or None, dnats fp32 [B,NB,HN]).
    types [B,NB,HN,2]; do [B,T,H,V]; dht [N,H,K,V] or None."""
    B, T, H, K = q.shape
    HN = types.shape[2]
    NT = -(-T // C)
    per = block // C
    f32 = torch.float32
    with torch.enable_grad():
        leaves = [t.detach().to(f32).requires_grad_(True) for t in (q, k, v, g)]
        qf, kf, vf, gf = leaves
        bf = beta.detach().to(f32).requires_grad_(True) if kind == 'gdn' else None
        hf = h0.detach().to(f32).requires_grad_(True) if h0 is not None else None
        lin = (torch.round(types[..., 1].detach().float()) == 1).repeat_interleave(H // HN, dim=2)       # [B,NB,H]
        gate_on = torch.ones(B, NT, H, dtype=f32, device=q.device, requires_grad=True)
        gate_off = torch.zeros(B, NT, H, dtype=f32, device=q.device, requires_grad=dnats_for_invalid_blocks)
        o, S = linear_chunk_forward_torch(kind, qf, kf, vf, gf, bf, hf, lin, scale, block, decay, l2norm, intra, gate_on, gate_off)
        outs, grads_out = [o], [do.to(f32)]
        if dht is not None:
            outs.append(S)
            grads_out.append(dht.to(f32))
        wrt = [qf, kf, vf, gf, gate_on]
        if bf is not None:
            wrt.append(bf)
        if hf is not None:
            wrt.append(hf)
        if dnats_for_invalid_blocks:
            wrt.append(gate_off)
        grads = list(torch.autograd.grad(outs, wrt, grads_out, allow_unused=True))
    dq, dk, dv, dg, dgate = grads[:5]
    rest = grads[5:]
    dbeta = rest.pop(0) if bf is not None else None
    dh0 = rest.pop(0) if hf is not None else None
    # a gate acts where its block's update is kept (typed linear), the zero gate where it is not
    lin_c = lin.repeat_interleave(per, dim=1)[:, :NT]                                                     # per chunk
    dn = torch.where(lin_c, dgate, torch.zeros_like(dgate))
    if dnats_for_invalid_blocks:
        dgo = rest.pop(0)
        dn = dn + torch.where(lin_c, torch.zeros_like(dgo), dgo)
    NB = types.shape[1]
    pad = NB * per - NT
    if pad:
        dn = torch.cat([dn, dn.new_zeros(B, pad, H)], 1)
    dn = dn.view(B, NB, per, HN, H // HN).sum((2, 4))
    z = lambda t, like: torch.zeros_like(like) if t is None else t
    return (z(dq, qf).to(q.dtype), z(dk, kf).to(k.dtype), z(dv, vf).to(v.dtype), z(dg, gf),
            None if bf is None else z(dbeta, bf).to(beta.dtype), dh0, dn)
