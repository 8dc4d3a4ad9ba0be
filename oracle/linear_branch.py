"""Oracle for the linear-recurrent branches: Gated DeltaNet and the Mamba2-style SSD.

TEST INFRASTRUCTURE ONLY -- see oracle/__init__.py.

Three restatements per branch, compared with each other in
tests/test_oracle_branches.py:

  token_recurrence      the reference's own decode semantics, one token at a
                        time with block roll-back
                        (src/nats/ops/gated_delta_rule/fused_recurrent.py:157-229,
                        src/nats/ops/mamba/fused_recurrent.py:150-207); fp64.
  chunked               chunk-parallel form with a running state; any block
                        size that is a multiple of 64, ragged T.  This is the
                        one timed as the CPU baseline.
  chunked_reference     the reference's pipeline stage by stage for block == 64:
                        local cumsum + carry over non-linear runs
                        (src/nats/ops/utils/cumsum.py:95-133), A / (I+A)^-1 / w,u
                        (src/nats/ops/common/chunk_scaled_dot_kkt.py:105-126,
                        src/nats/ops/utils/solve_tril.py, src/nats/ops/gated_delta_rule/wy_fast.py:128-153),
                        the h array written before each linear chunk
                        (src/nats/ops/common/chunk_delta_h.py:189-309) and the output
                        kernel reading h[starting_h_idx]
                        (src/nats/ops/common/chunk_o.py:93-215).

Further pins: all-linear types => textbook gated delta rule / scalar-decay
linear attention; g = 0, beta = 1 => plain delta rule; masking k, v, beta on
non-linear chunks reproduces the final state (the identity the reference's own
debug script uses, src/nats/ops/gated_delta_rule/chunk.py:622-630); splitting a
sequence at a block boundary and chaining final_state -> initial_state.
"""
from __future__ import annotations

import torch

CHUNK = 64


def l2norm(x: torch.Tensor, eps: float = 1e-6) -> torch.Tensor:
    """x * rsqrt(sum x^2 + eps), src/nats/ops/gated_delta_rule/fused_recurrent.py:165-169."""
    return x * torch.rsqrt((x * x).sum(-1, keepdim=True) + eps)


def _expand_types(lin_types: torch.Tensor, H: int) -> torch.Tensor:
    """[B,NB,HN] -> bool [B,NB,H]; selector head of h is h // (H//HN) (chunk_delta_h.py:83-84)."""
    HN = lin_types.shape[2]
    return torch.round(lin_types.float()).bool().repeat_interleave(H // HN, dim=2)


# --------------------------------------------------------------------------------------
# token-level recurrences (semantic definition)
# --------------------------------------------------------------------------------------
def gdn_token_recurrence(q, k, v, g, beta, lin_types, scale, h0=None, block=64, decay_non_linear=True,
                         l2norm_qk=True, dtype=torch.float64):
    """q,k [B,T,H,K]; v [B,T,H,V]; g,beta [B,T,H]; lin_types [B,NB,HN] -> (o [B,T,H,V], S [B,H,K,V]).

    Per token: S <- e^{g_t} S; delta = beta_t (v_t - S^T k_t); S <- S + k_t delta^T; o_t = scale S^T q_t.
    At the end of a block that is not linear-typed the state rolls back to its
    value at the block start, times exp(sum of the block's g) when
    decay_non_linear (fused_recurrent.py:221-228).
    """
    B, T, H, K = q.shape
    V = v.shape[-1]
    q, k, v, g, beta = (x.to(dtype) for x in (q, k, v, g, beta))
    if l2norm_qk:
        q, k = l2norm(q), l2norm(k)
    lin = _expand_types(lin_types, H)
    S = torch.zeros(B, H, K, V, dtype=dtype) if h0 is None else h0.to(dtype).clone()
    o = torch.zeros(B, T, H, V, dtype=dtype)
    S_start, gsum = S.clone(), torch.zeros(B, H, dtype=dtype)
    for t in range(T):
        if t % block == 0:
            S_start, gsum = S.clone(), torch.zeros(B, H, dtype=dtype)
        S = S * torch.exp(g[:, t])[..., None, None]
        kt, vt, qt = k[:, t], v[:, t], q[:, t]
        delta = beta[:, t][..., None] * (vt - torch.einsum('bhkv,bhk->bhv', S, kt))
        S = S + torch.einsum('bhk,bhv->bhkv', kt, delta)
        o[:, t] = scale * torch.einsum('bhkv,bhk->bhv', S, qt)
        gsum = gsum + g[:, t]
        if (t + 1) % block == 0 or t == T - 1:
            keep = lin[:, t // block][..., None, None]
            back = S_start * torch.exp(gsum)[..., None, None] if decay_non_linear else S_start
            S = torch.where(keep, S, back)
    return o, S


def mamba_token_recurrence(q, k, v, g, lin_types, scale, h0=None, block=64, decay_non_linear=True,
                           dtype=torch.float64):
    """S <- e^{g_t} S + k_t v_t^T; o_t = scale S^T q_t; same roll-back rule
    (src/nats/ops/mamba/fused_recurrent.py:150-207).  q = C, k = B, v = X*dt."""
    B, T, H, K = q.shape
    V = v.shape[-1]
    q, k, v, g = (x.to(dtype) for x in (q, k, v, g))
    lin = _expand_types(lin_types, H)
    S = torch.zeros(B, H, K, V, dtype=dtype) if h0 is None else h0.to(dtype).clone()
    o = torch.zeros(B, T, H, V, dtype=dtype)
    S_start, gsum = S.clone(), torch.zeros(B, H, dtype=dtype)
    for t in range(T):
        if t % block == 0:
            S_start, gsum = S.clone(), torch.zeros(B, H, dtype=dtype)
        S = S * torch.exp(g[:, t])[..., None, None] + torch.einsum('bhk,bhv->bhkv', k[:, t], v[:, t])
        o[:, t] = scale * torch.einsum('bhkv,bhk->bhv', S, q[:, t])
        gsum = gsum + g[:, t]
        if (t + 1) % block == 0 or t == T - 1:
            keep = lin[:, t // block][..., None, None]
            back = S_start * torch.exp(gsum)[..., None, None] if decay_non_linear else S_start
            S = torch.where(keep, S, back)
    return o, S


# --------------------------------------------------------------------------------------
# chunk-parallel form with a running state (general block size, ragged T)
# --------------------------------------------------------------------------------------
def _to_chunks(x, NT, C):
    """[B,T,H,*] -> [B,H,NT,C,*] zero padded."""
    B, T = x.shape[:2]
    pad = NT * C - T
    if pad:
        x = torch.cat([x, x.new_zeros(B, pad, *x.shape[2:])], 1)
    x = x.reshape(B, NT, C, *x.shape[2:])
    return x.permute(0, 3, 1, 2, *range(4, x.dim())).contiguous()


def _intra_chunk_terms(qh, kh, g_c, C):
    """gamma (inclusive local cumsum of g, chunk.py:52-54) and L_ij = exp(gamma_i-gamma_j) for i>=j."""
    gamma = g_c.cumsum(-1)
    diff = gamma.unsqueeze(-1) - gamma.unsqueeze(-2)
    tri = torch.tril(torch.ones(C, C, dtype=torch.bool))
    L = torch.where(tri, torch.exp(torch.where(tri, diff, torch.zeros_like(diff))), torch.zeros_like(diff))
    return gamma, L


def _scan(qe, w, u, kd, P, glast, lin, scale, h0, block, C, T, decay_non_linear, delta_rule, B, H, K, V, NT, dtype,
          intra=True, gate_on=None, gate_off=None):
    """gate_on / gate_off [B,NT,H] (default: ones / absent) multiply a chunk's additive state update where it is kept /
    add it, scaled, to the rolled-back state where it is not: d loss / d gate is the selector's straight-through gradient
    for the linear operator, <state gradient behind the chunk, k~^T v_new> (src/nats/ops/common/chunk_o.py:438-443 for
    blocks typed linear, :487-492 for the others when their gradient is asked for)."""
    S = torch.zeros(B, H, K, V, dtype=dtype) if h0 is None else h0.to(dtype).clone()
    o = torch.zeros(B, H, NT, C, V, dtype=dtype)
    S_start, gsum = S, torch.zeros(B, H, dtype=dtype)
    per = block // C
    for c in range(NT):
        if c % per == 0:
            S_start, gsum = S, torch.zeros(B, H, dtype=dtype)
        v_new = u[:, :, c] - w[:, :, c] @ S if delta_rule else u[:, :, c]
        o[:, :, c] = scale * (qe[:, :, c] @ S)
        if intra:
            o[:, :, c] += scale * (P[:, :, c] @ v_new)
        upd = kd[:, :, c].transpose(-1, -2) @ v_new
        if gate_on is not None:
            upd_on = gate_on[:, c, :, None, None] * upd
        else:
            upd_on = upd
        S = torch.exp(glast[:, :, c])[..., None, None] * S + upd_on
        gsum = gsum + glast[:, :, c]
        if (c + 1) % per == 0 or c == NT - 1:
            keep = lin[:, (c * C) // block][..., None, None]
            back = S_start * torch.exp(gsum)[..., None, None] if decay_non_linear else S_start
            if gate_off is not None:
                back = back + gate_off[:, c, :, None, None] * upd
            S = torch.where(keep, S, back)
    o = o.permute(0, 2, 3, 1, 4).reshape(B, NT * C, H, V)[:, :T]
    return o, S


def gdn_chunked(q, k, v, g, beta, lin_types, scale, h0=None, block=64, decay_non_linear=True, l2norm_qk=True,
                dtype=torch.float32, intra=True, gate_on=None, gate_off=None):
    """Chunk-parallel Gated DeltaNet forward (same result as gdn_token_recurrence).

    Per 64-token chunk: A = strict_lower(beta_i k_i.k_j e^{gamma_i-gamma_j}), Tm = (I+A)^-1,
    u = Tm(beta v), w = Tm(beta e^{gamma} k); with S the state entering the chunk:
    v_new = u - w S;  o = scale[(q e^{gamma}) S + tril(q k^T e^{gamma_i-gamma_j}) v_new];
    S' = e^{gamma_last} S + (k e^{gamma_last-gamma})^T v_new.  A block that is not
    linear-typed rolls S back at its end (times e^{sum g} when decay_non_linear).
    intra=False drops the intra-chunk term (mode 'attn', chunk_o.py:210-211).
    """
    B, T, H, K = q.shape
    V = v.shape[-1]
    C = CHUNK
    NT = -(-T // C)
    assert block % C == 0
    q, k, v, g, beta = (x.to(dtype) for x in (q, k, v, g, beta))
    if l2norm_qk:
        q, k = l2norm(q), l2norm(k)
    qc, kc, vc = _to_chunks(q, NT, C), _to_chunks(k, NT, C), _to_chunks(v, NT, C)
    gc, bc = _to_chunks(g, NT, C), _to_chunks(beta, NT, C)
    gamma, L = _intra_chunk_terms(qc, kc, gc, C)
    kk = kc @ kc.transpose(-1, -2)
    A = torch.tril(bc.unsqueeze(-1) * kk * L, -1)
    eye = torch.eye(C, dtype=dtype)
    Tm = torch.linalg.solve_triangular(eye + A, eye.expand_as(A).contiguous(), upper=False)
    u = Tm @ (bc.unsqueeze(-1) * vc)
    w = Tm @ ((bc * torch.exp(gamma)).unsqueeze(-1) * kc)
    P = (qc @ kc.transpose(-1, -2)) * L
    qe = qc * torch.exp(gamma).unsqueeze(-1)
    glast = gamma[..., -1]
    kd = kc * torch.exp(glast.unsqueeze(-1) - gamma).unsqueeze(-1)
    lin = _expand_types(lin_types, H)
    return _scan(qe, w, u, kd, P, glast, lin, scale, h0, block, C, T, decay_non_linear, True, B, H, K, V, NT, dtype,
                 intra, gate_on, gate_off)


def mamba_chunked(q, k, v, g, lin_types, scale, h0=None, block=64, decay_non_linear=True, dtype=torch.float32,
                  intra=True, gate_on=None, gate_off=None):
    """Chunk-parallel SSD forward: o = scale[(q e^{gamma}) S + tril(q k^T e^{gamma_i-gamma_j}) v],
    S' = e^{gamma_last} S + (k e^{min(gamma_last-gamma,0)})^T v
    (src/nats/ops/mamba/chunk_h.py:139-204, src/nats/ops/mamba/chunk_o.py:146-198)."""
    B, T, H, K = q.shape
    V = v.shape[-1]
    C = CHUNK
    NT = -(-T // C)
    assert block % C == 0
    q, k, v, g = (x.to(dtype) for x in (q, k, v, g))
    qc, kc, vc, gc = _to_chunks(q, NT, C), _to_chunks(k, NT, C), _to_chunks(v, NT, C), _to_chunks(g, NT, C)
    gamma, L = _intra_chunk_terms(qc, kc, gc, C)
    P = (qc @ kc.transpose(-1, -2)) * L
    qe = qc * torch.exp(gamma).unsqueeze(-1)
    glast = gamma[..., -1]
    kd = kc * torch.exp(torch.clamp(glast.unsqueeze(-1) - gamma, max=0.0)).unsqueeze(-1)
    lin = _expand_types(lin_types, H)
    return _scan(qe, None, vc, kd, P, glast, lin, scale, h0, block, C, T, decay_non_linear, False, B, H, K, V, NT,
                 dtype, intra, gate_on, gate_off)


# --------------------------------------------------------------------------------------
# the reference pipeline, stage by stage (block == chunk == 64, T multiple of 64)
# --------------------------------------------------------------------------------------
def gdn_chunked_reference(q, k, v, g, beta, lin_types, scale, h0=None, decay_non_linear=True, dtype=torch.float64):
    """Follows chunk_gated_delta_rule_nats_fwd (src/nats/ops/gated_delta_rule/chunk.py:22-167)
    with keep_wu_as_kv=True, compute_incomplete_chunk_scores=True,
    incomplete_block_start_with_ht=True.  Requires the last block to be linear-typed
    (the layer forces it, src/nats/layers/natsl_attn_gdn.py:553)."""
    B, T, H, K = q.shape
    V = v.shape[-1]
    C = CHUNK
    assert T % C == 0
    NT = T // C
    q, k, v, g, beta = (x.to(dtype) for x in (q, k, v, g, beta))
    q, k = l2norm(q), l2norm(k)
    lin = _expand_types(lin_types, H)                           # [B,NT,H]
    assert bool(lin[:, -1].all())
    # chunk.py:52-54  local cumsum
    gam = g.reshape(B, NT, C, H).cumsum(2)
    # cumsum.py:95-133  carry over the run of non-linear chunks that precedes each linear chunk
    phi = torch.zeros(B, NT, H, dtype=dtype)
    if decay_non_linear:
        for c in range(1, NT):
            prev_lin = lin[:, c - 1]
            phi[:, c] = torch.where(prev_lin, torch.zeros_like(phi[:, c]), phi[:, c - 1] + gam[:, c - 1, -1])
    gp = gam + phi.unsqueeze(2)                                 # g' [B,NT,C,H]
    qc, kc, vc = (x.reshape(B, NT, C, H, -1).permute(0, 3, 1, 2, 4) for x in (q, k, v))
    bc = beta.reshape(B, NT, C, H).permute(0, 3, 1, 2)
    gpc = gp.permute(0, 3, 1, 2)                                # [B,H,NT,C]
    diff = gpc.unsqueeze(-1) - gpc.unsqueeze(-2)
    strict = torch.tril(torch.ones(C, C, dtype=torch.bool), -1)
    incl = torch.tril(torch.ones(C, C, dtype=torch.bool))
    # chunk_scaled_dot_kkt.py:105-126
    A = torch.where(strict, bc.unsqueeze(-1) * (kc @ kc.transpose(-1, -2)) * torch.exp(diff * strict), torch.zeros((), dtype=dtype))
    # solve_tril.py:484-569
    Tm = torch.linalg.inv(torch.eye(C, dtype=dtype) + A)
    # wy_fast.py:128-153
    u = Tm @ (bc.unsqueeze(-1) * vc)
    w = Tm @ ((bc * torch.exp(gpc)).unsqueeze(-1) * kc)
    # chunk_delta_h.py:189-309: h stored BEFORE each linear chunk, state updated only there
    S = torch.zeros(B, H, K, V, dtype=dtype) if h0 is None else h0.to(dtype).clone()
    o = torch.zeros(B, H, NT, C, V, dtype=dtype)
    for b in range(B):
        for h in range(H):
            Sb = S[b, h]
            h_list = []
            for c in range(NT):
                if not lin[b, c, h]:
                    continue
                h_list.append(Sb.clone())
                v_new = u[b, h, c] - w[b, h, c] @ Sb
                gl = gpc[b, h, c, -1]
                Sb = torch.exp(gl) * Sb + kc[b, h, c].T @ (v_new * torch.exp(gl - gpc[b, h, c]).unsqueeze(-1))
            S[b, h] = Sb
            # chunk_o.py:93-215: chunk c reads h[#linear blocks that start before c*C]
            lin_ids = [c for c in range(NT) if lin[b, c, h]]
            for c in range(NT):
                i_th = sum(1 for j in lin_ids if j * C < c * C)
                Sp = h_list[i_th]
                v_new = u[b, h, c] - w[b, h, c] @ Sp             # linear chunks: same value as above
                Pm = torch.where(incl, (qc[b, h, c] @ kc[b, h, c].T) * torch.exp(diff[b, h, c] * incl), torch.zeros((), dtype=dtype))
                o[b, h, c] = scale * ((qc[b, h, c] * torch.exp(gpc[b, h, c]).unsqueeze(-1)) @ Sp + Pm @ v_new)
    return o.permute(0, 2, 3, 1, 4).reshape(B, T, H, V), S


def gdn_flops(n_chunks_total: float, n_linear_chunks: float, K: int, V: int, C: int = CHUNK) -> float:
    """Algorithmic FLOPs: 2C^2(3K+2V) + 6CKV + (2/3)C^3 per chunk-head; a chunk that is not
    linear-typed skips the state update (-2CKV)."""
    per = 2 * C * C * (3 * K + 2 * V) + 6 * C * K * V + (2.0 / 3.0) * C ** 3
    return per * n_chunks_total - 2 * C * K * V * (n_chunks_total - n_linear_chunks)


def mamba_flops(n_chunks_total: float, n_linear_chunks: float, K: int, V: int, C: int = CHUNK) -> float:
    per = 2 * C * C * (K + V) + 4 * C * K * V
    return per * n_chunks_total - 2 * C * K * V * (n_chunks_total - n_linear_chunks)


def linear_branch_bwd(kind, q, k, v, g, beta, lin_types, scale, do, dht=None, h0=None, block=64, decay_non_linear=True,
                      l2norm_qk=True, intra=True, dnats_for_invalid_blocks=False, dtype=torch.float64):
    """Gradients of the chunked linear branch by autograd through gdn_chunked / mamba_chunked in fp64:
    -> dict(dq, dk, dv, dg, dbeta, dh0, dnats [B,NB,HN]).  dnats: per selector block and head, the gate gradients of its
    chunks and heads summed (src/nats/ops/common/chunk_o.py:1571-1575); blocks not typed linear contribute their
    zero-gate gradient only when dnats_for_invalid_blocks."""
    B, T, H, K = q.shape
    NT = -(-T // CHUNK)
    per = block // CHUNK
    HN = lin_types.shape[2]
    leaf = lambda t: None if t is None else t.detach().to(dtype).requires_grad_(True)
    qf, kf, vf, gf, bf, hf = leaf(q), leaf(k), leaf(v), leaf(g), leaf(beta), leaf(h0)
    gate_on = torch.ones(B, NT, H, dtype=dtype, requires_grad=True)
    gate_off = torch.zeros(B, NT, H, dtype=dtype, requires_grad=True)
    if kind == 'gdn':
        o, S = gdn_chunked(qf, kf, vf, gf, bf, lin_types, scale, hf, block, decay_non_linear, l2norm_qk, dtype, intra, gate_on, gate_off)
    else:
        o, S = mamba_chunked(qf, kf, vf, gf, lin_types, scale, hf, block, decay_non_linear, dtype, intra, gate_on, gate_off)
    loss = (o * do.to(dtype)).sum()
    if dht is not None:
        loss = loss + (S * dht.to(dtype)).sum()
    loss.backward()
    lin_c = _expand_types(lin_types, H).repeat_interleave(per, dim=1)[:, :NT]
    # (a leaf nothing of the loss depends on -- one chunk without a final-state gradient -- has no gradient: zero)
    z_ = lambda t, like: torch.zeros_like(like) if (t is None or t.grad is None) else t.grad
    dn = torch.where(lin_c, z_(gate_on, gate_on), torch.zeros_like(gate_on))
    if dnats_for_invalid_blocks:
        dn = dn + torch.where(lin_c, torch.zeros_like(dn), z_(gate_off, gate_off))
    NB = lin_types.shape[1]
    if NB * per != NT:
        dn = torch.cat([dn, dn.new_zeros(B, NB * per - NT, H)], 1)
    dn = dn.view(B, NB, per, HN, H // HN).sum((2, 4))
    g_ = lambda t: None if t is None else z_(t, t)
    return dict(dq=g_(qf), dk=g_(kf), dv=g_(vf), dg=g_(gf), dbeta=g_(bf), dh0=g_(hf), dnats=dn)
