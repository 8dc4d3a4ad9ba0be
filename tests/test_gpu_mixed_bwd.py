"""GPU parity: backward of the mixed operators and a training step of the two layers.

Oracle: oracle.linear_branch.linear_branch_bwd (autograd through the chunked form in fp64, pinned on the CPU by the
token recurrence and by finite differences of the gates) and oracle.softmax_branch.softmax_branch_bwd.  Gradient tolerance
as for the softmax backward: rel-L2 5e-3, max-abs 2e-2 of the reference's largest magnitude.  The two per-token scalar
gradients of the linear branch, dg and dbeta, get rel-L2 1e-2: each is a sum of large terms of both signs (dg: the suffix sum
of <dq,q> - <dk,k> + ... plus the chunk's decay term; dbeta: <dX, v_new>), formed by kernels whose every operand (states,
state gradients, v_new, dX, the 64x64 weight tiles) is a bf16-rounded intermediate; measured 2e-3 .. 5.2e-3."""
import pytest
import torch
import torch.nn.functional as F

from oracle import linear_branch as LB
from oracle import softmax_branch as SB
from tests._util import make_gates, make_qkv, make_types, max_abs, rel_l2

pytestmark = pytest.mark.gpu
DEV = 'cuda:0'


def _close(a, b, what, rl_tol=5e-3):
    rl, ma, top = rel_l2(a, b), max_abs(a, b), float(b.abs().max())
    assert rl <= rl_tol and ma <= 2e-2 * max(top, 1.0), f"{what}: rel-L2 {rl:.3e}, max-abs {ma:.3e} (largest reference value {top:.3e})"


@pytest.mark.parametrize("kind,K,V,block,h0,invalid", [('gdn', 128, 128, 64, False, False), ('gdn', 64, 64, 64, True, True),
                                                        ('gdn', 128, 64, 128, True, False), ('mamba', 128, 64, 64, True, False),
                                                        ('mamba', 64, 64, 256, False, False), ('mamba', 64, 128, 64, False, True)])
def test_mixed_operator_backward(kind, K, V, block, h0, invalid):
    from neuralattentionsearchlinear_amd.mixed_attn_gdn import nats_mixed_attn_gdn
    from neuralattentionsearchlinear_amd.mixed_attn_mamba import nats_mixed_attn_mamba
    B, T, H, HN = 2, 512, 4, 2
    gen = torch.Generator().manual_seed(K + V)
    q, k, v = make_qkv(B, T, H, K, V, 11)
    if kind == 'mamba':
        q, k = F.normalize(q.float(), dim=-1).bfloat16(), F.normalize(k.float(), dim=-1).bfloat16()
    g, beta = make_gates(B, T, H, 12)
    ty = make_types(B, T // block, HN, 0.4, 13, torch.bfloat16)
    init = (torch.randn(B, H, K, V, generator=gen) * 0.3) if h0 else None
    do_l, do_a = (torch.randn(B, T, H, V, generator=gen).bfloat16() for _ in range(2))
    dht = torch.randn(B, H, K, V, generator=gen)
    scale_l = K ** -0.5 if kind == 'gdn' else 1.0
    # oracle
    rl = LB.linear_branch_bwd(kind, q, k, v, g, beta if kind == 'gdn' else None, ty[..., 1], scale_l, do_l, dht, init, block, True,
                              True, True, invalid)
    dq_a, dk_a, dv_a, dn_a, dn_mag = SB.softmax_branch_bwd(q, k, v, ty, do_a, K ** -0.5, block, True, with_magnitude=True)
    # the operator
    leaf = lambda t: None if t is None else t.to(DEV).requires_grad_(True)
    qa, ka, va, ql, kl, vl, gd, bd, hd, tyd = (leaf(t) for t in (q, k, v, q, k, v, g, beta, init, ty))
    nb = ty.to(torch.int32).sum(1).to(DEV)
    if kind == 'gdn':
        o_l, o_a, ht = nats_mixed_attn_gdn(qa, ka, va, ql, kl, vl, hd, gd, bd, tyd, nb, nats_block_size=block,
                                           ops_for_incomplete_chunks='all', output_final_state_gated_delta=True,
                                           decay_for_non_gdn_blocks=True, compute_dnats_for_invalid_blocks_linear_att=invalid)
    else:
        o_l, o_a, ht = nats_mixed_attn_mamba(qa, ka, va, ql, kl, vl, hd, gd, tyd, nb, scale_lattn=1.0, nats_block_size=block,
                                             ops_for_incomplete_chunks='all', output_final_state_mamba=True,
                                             decay_for_non_mamba_blocks=True, compute_dnats_for_invalid_blocks_linear_att=invalid)
    ((o_l.float() * do_l.to(DEV).float()).sum() + (o_a.float() * do_a.to(DEV).float()).sum() + (ht * dht.to(DEV)).sum()).backward()
    torch.cuda.synchronize()
    _close(ql.grad.float(), rl['dq'], "dq_lattn")
    _close(kl.grad.float(), rl['dk'], "dk_lattn")
    _close(vl.grad.float(), rl['dv'], "dv_lattn")
    _close(gd.grad.float(), rl['dg'], "dg", 1e-2)
    if kind == 'gdn':
        _close(bd.grad.float(), rl['dbeta'], "dbeta", 1e-2)
    if h0:
        _close(hd.grad.float(), rl['dh0'], "dh0")
    _close(qa.grad.float(), dq_a, "dq_attn")
    _close(ka.grad.float(), dk_a, "dk_attn")
    _close(va.grad.float(), dv_a, "dv_attn")
    dt = tyd.grad.float().cpu().double()
    err = (dt[..., 0] - dn_a).abs()
    assert bool((err <= 2e-3 * dn_mag + 1e-6).all()), f"dnats (softmax op): error {float(err.max()):.3e}"
    ref = rl['dnats']
    assert float((dt[..., 1] - ref).abs().max()) <= 2e-2 * max(float(ref.abs().max()), 1.0) and rel_l2(dt[..., 1], ref) <= 1e-2, \
        f"dnats (linear op): rel-L2 {rel_l2(dt[..., 1], ref):.3e}"
    if not invalid:
        nonlin = torch.round(ty[..., 1].float()) == 0
        assert float(dt[..., 1][nonlin].abs().max() if nonlin.any() else 0.0) == 0.0


@pytest.mark.parametrize("kind,invalid", [('gdn', False), ('mamba', True)])
def test_mixed_operator_backward_packed_sequences(kind, invalid):
    """Packed sequences: the gradients of every sequence equal the oracles' on that sequence alone (own initial state,
    own final-state gradient, own blocks)."""
    from neuralattentionsearchlinear_amd.mixed_attn_gdn import nats_mixed_attn_gdn
    from neuralattentionsearchlinear_amd.mixed_attn_mamba import nats_mixed_attn_mamba
    lens, H, HN, K, V, block = [320, 70, 512, 129], 4, 2, 64, 64, 64
    T, N = sum(lens), len(lens)
    cu = [0]
    for n in lens:
        cu.append(cu[-1] + n)
    gen = torch.Generator().manual_seed(77)
    q, k, v = make_qkv(1, T, H, K, V, 21)
    if kind == 'mamba':
        q, k = F.normalize(q.float(), dim=-1).bfloat16(), F.normalize(k.float(), dim=-1).bfloat16()
    g, beta = make_gates(1, T, H, 22)
    NB = sum(-(-n // block) for n in lens)
    ty = make_types(1, NB, HN, 0.4, 23, torch.bfloat16)
    init = torch.randn(N, H, K, V, generator=gen) * 0.3
    do_l, do_a = (torch.randn(1, T, H, V, generator=gen).bfloat16() for _ in range(2))
    dht = torch.randn(N, H, K, V, generator=gen)
    scale_l = K ** -0.5 if kind == 'gdn' else 1.0
    leaf = lambda t: None if t is None else t.to(DEV).requires_grad_(True)
    qa, ka, va, ql, kl, vl, gd, bd, hd, tyd = (leaf(t) for t in (q, k, v, q, k, v, g, beta, init, ty))
    cud = torch.tensor(cu, dtype=torch.int32, device=DEV)
    if kind == 'gdn':
        o_l, o_a, ht = nats_mixed_attn_gdn(qa, ka, va, ql, kl, vl, hd, gd, bd, tyd, None, cu_seqlens=cud, nats_block_size=block,
                                           ops_for_incomplete_chunks='all', output_final_state_gated_delta=True,
                                           decay_for_non_gdn_blocks=True, compute_dnats_for_invalid_blocks_linear_att=invalid)
    else:
        o_l, o_a, ht = nats_mixed_attn_mamba(qa, ka, va, ql, kl, vl, hd, gd, tyd, None, scale_lattn=1.0, cu_seqlens=cud,
                                             nats_block_size=block, ops_for_incomplete_chunks='all', output_final_state_mamba=True,
                                             decay_for_non_mamba_blocks=True, compute_dnats_for_invalid_blocks_linear_att=invalid)
    ((o_l.float() * do_l.to(DEV).float()).sum() + (o_a.float() * do_a.to(DEV).float()).sum() + (ht * dht.to(DEV)).sum()).backward()
    torch.cuda.synchronize()
    dt = tyd.grad.float().cpu().double()
    nb = 0
    for i, n in enumerate(lens):
        a, b, nbi = cu[i], cu[i + 1], -(-n // block)
        tyi = ty[:, nb:nb + nbi]
        rl = LB.linear_branch_bwd(kind, q[:, a:b], k[:, a:b], v[:, a:b], g[:, a:b], beta[:, a:b] if kind == 'gdn' else None,
                                  tyi[..., 1], scale_l, do_l[:, a:b], dht[i:i + 1], init[i:i + 1], block, True, True, True, invalid)
        dq_a, dk_a, dv_a, dn_a, dn_mag = SB.softmax_branch_bwd(q[:, a:b], k[:, a:b], v[:, a:b], tyi, do_a[:, a:b], K ** -0.5, block,
                                                               True, with_magnitude=True)
        w = f" of sequence {i}"
        _close(ql.grad[:, a:b].float(), rl['dq'], "dq_lattn" + w)
        _close(kl.grad[:, a:b].float(), rl['dk'], "dk_lattn" + w)
        _close(vl.grad[:, a:b].float(), rl['dv'], "dv_lattn" + w)
        _close(gd.grad[:, a:b].float(), rl['dg'], "dg" + w, 1e-2)
        if kind == 'gdn':
            _close(bd.grad[:, a:b].float(), rl['dbeta'], "dbeta" + w, 1e-2)
        _close(hd.grad[i:i + 1].float(), rl['dh0'], "dh0" + w)
        _close(qa.grad[:, a:b].float(), dq_a, "dq_attn" + w)
        _close(ka.grad[:, a:b].float(), dk_a, "dk_attn" + w)
        _close(va.grad[:, a:b].float(), dv_a, "dv_attn" + w)
        err = (dt[:, nb:nb + nbi, :, 0] - dn_a).abs()
        assert bool((err <= 2e-3 * dn_mag + 1e-6).all()), f"dnats (softmax op){w}: error {float(err.max()):.3e}"
        ref, got = rl['dnats'], dt[:, nb:nb + nbi, :, 1]
        assert float((got - ref).abs().max()) <= 2e-2 * max(float(ref.abs().max()), 1.0) and rel_l2(got, ref) <= 1e-2, \
            f"dnats (linear op){w}: rel-L2 {rel_l2(got, ref):.3e}"
        nb += nbi


@pytest.mark.parametrize("kind,geometry", [('gdn', None), ('mamba', None), ('gdn', '760M')])
def test_layer_training_step(kind, geometry):
    """One forward + backward of the layer in training mode: every parameter receives a finite gradient, and the gradients
    of everything outside the selector agree with autograd through the layer oracle on the same (injected) block types.
    The selector's own path (nats_layer) is the straight-through estimator of the operators, checked at operator level."""
    from oracle import layer as olayer
    from tests.test_gpu_layers import _layer_case
    layer, cfg, w, x = _layer_case(kind, geometry)   # ('760M': the published configuration's hidden size and head geometry)
    layer = layer.to(DEV).float().train()
    xd = x.to(DEV).requires_grad_(True)
    out = layer(xd)
    o = out[0] if isinstance(out, tuple) else out
    gy = torch.randn(o.shape, generator=torch.Generator().manual_seed(5))
    (o * gy.to(DEV)).sum().backward()
    torch.cuda.synchronize()
    with torch.no_grad():
        types, _, _ = layer.select_ops(xd.detach())
    ocfg = dict(cfg, num_nats_head=cfg['num_heads'], attn_qk_norm=(kind == 'gdn'), attn_with_short_conv=(kind == 'gdn'))
    wl = {k_: v_.detach().clone().float().requires_grad_(True) for k_, v_ in w.items()}
    fn = olayer.gdn_layer if kind == 'gdn' else olayer.mamba_layer
    # (the oracle rounds to bf16 where the operators do: their inputs and outputs; the cast passes gradients through)
    ref, _ = fn(wl, ocfg, x, types=types.cpu(), act_dtype=torch.bfloat16, round_at='ops')
    (ref * gy).sum().backward()
    for name, p_ in layer.named_parameters():
        assert p_.grad is not None and bool(torch.isfinite(p_.grad).all()), f"{name}: no finite gradient"
        if name.startswith('nats_layer'):
            assert float(p_.grad.abs().max()) > 0, "the selector receives no gradient"
            continue
        r_ = wl[name].grad
        rl_, top = rel_l2(p_.grad.float(), r_), float(r_.abs().max())
        assert rl_ <= 2e-2 and max_abs(p_.grad.float(), r_) <= 5e-2 * max(top, 1e-3), f"{name}: grad rel-L2 {rl_:.3e}"
    assert xd.grad is not None and bool(torch.isfinite(xd.grad).all())


def test_config0_backward_fp32_tensors():
    """The smallest configuration (B1 T256 H2 K=V=64, fp32 tensors) through loss.backward(): gradients come back in fp32,
    computed on bf16 copies like the forward, and match the oracle on the rounded inputs."""
    from neuralattentionsearchlinear_amd import nats_util
    from neuralattentionsearchlinear_amd.mixed_attn_gdn import nats_mixed_attn_gdn
    torch.manual_seed(0)
    B, T, H, D, block = 1, 256, 2, 64, 64
    q, k, v = (torch.randn(B, T, H, D).bfloat16().float() for _ in range(3))
    beta = torch.sigmoid(torch.randn(B, T, H)).bfloat16().float()
    g = -F.softplus(torch.randn(B, T, H))
    ty = make_types(B, T // block, H, 0.4, 3, torch.float32)
    do_l, do_a = (torch.randn(B, T, H, D).bfloat16().float() for _ in range(2))
    rl = LB.linear_branch_bwd('gdn', q, k, v, g, beta, ty[..., 1], D ** -0.5, do_l, None, None, block, True, True, True, False)
    dq_a, dk_a, dv_a, _, _ = SB.softmax_branch_bwd(q, k, v, ty, do_a, D ** -0.5, block, True, with_magnitude=True)
    leaf = lambda t: t.to(DEV).requires_grad_(True)
    qa, ka, va, ql, kl, vl, gd, bd = (leaf(t) for t in (q, k, v, q, k, v, g, beta))
    nb = ty.to(torch.int32).sum(1).to(DEV)
    o_l, o_a, _ = nats_mixed_attn_gdn(qa, ka, va, ql, kl, vl, None, gd, bd, ty.to(DEV), nb, nats_block_size=block,
                                      ops_for_incomplete_chunks='all', decay_for_non_gdn_blocks=True)
    assert o_l.dtype == torch.float32
    ((o_l * do_l.to(DEV)).sum() + (o_a * do_a.to(DEV)).sum()).backward()
    torch.cuda.synchronize()
    for t in (qa, ka, va, ql, kl, vl, gd, bd):
        assert t.grad is not None and t.grad.dtype == torch.float32
    _close(ql.grad, rl['dq'], "dq_lattn"); _close(kl.grad, rl['dk'], "dk_lattn"); _close(vl.grad, rl['dv'], "dv_lattn")
    _close(gd.grad, rl['dg'], "dg", 1e-2); _close(bd.grad, rl['dbeta'], "dbeta", 1e-2)
    _close(qa.grad, dq_a, "dq_attn"); _close(ka.grad, dk_a, "dk_attn"); _close(va.grad, dv_a, "dv_attn")


@pytest.mark.parametrize("kind,packed", [('gdn', False), ('mamba', False), ('gdn', True)])
def test_kept_chunk_states_give_the_recomputed_gradients(kind, packed):
    """_mixed_common.SAVE_CHUNK_STATES: the backward that starts from the forward's kept chunk states, v_new and workspace
    returns, bit for bit, what the backward that runs the forward's kernels once more returns."""
    import neuralattentionsearchlinear_amd._mixed_common as MC
    from neuralattentionsearchlinear_amd.mixed_attn_gdn import nats_mixed_attn_gdn
    from neuralattentionsearchlinear_amd.mixed_attn_mamba import nats_mixed_attn_mamba
    B, T, H, HN, K, V, block = (1, 704, 4, 2, 128, 128, 64) if packed else (2, 448, 4, 2, 128, 128, 64)
    gen = torch.Generator().manual_seed(5)
    q, k, v = make_qkv(B, T, H, K, V, 21)
    if kind == 'mamba':
        q, k = F.normalize(q.float(), dim=-1).bfloat16(), F.normalize(k.float(), dim=-1).bfloat16()
    g, beta = make_gates(B, T, H, 22)
    cu = [0, 200, 512, 704] if packed else None
    nblk = sum(-(-(b - a) // block) for a, b in zip(cu[:-1], cu[1:])) if packed else T // block
    ty = make_types(B, nblk, HN, 0.4, 23, torch.bfloat16)
    n = len(cu) - 1 if packed else B
    init = torch.randn(n, H, K, V, generator=gen) * 0.3
    do_l, do_a = (torch.randn(B, T, H, V, generator=gen).bfloat16().to(DEV) for _ in range(2))
    dht = torch.randn(n, H, K, V, generator=gen).to(DEV)
    kw = dict(cu_seqlens=torch.tensor(cu, dtype=torch.int32, device=DEV)) if packed else {}
    nb = None if packed else ty.to(torch.int32).sum(1).to(DEV)

    def grads(keep):
        old, MC.SAVE_CHUNK_STATES = MC.SAVE_CHUNK_STATES, keep
        try:
            leaf = lambda t: t.to(DEV).requires_grad_(True)
            qa, ka, va, ql, kl, vl, gd, bd, hd, tyd = (leaf(t) for t in (q, k, v, q, k, v, g, beta, init, ty))
            if kind == 'gdn':
                o_l, o_a, ht = nats_mixed_attn_gdn(qa, ka, va, ql, kl, vl, hd, gd, bd, tyd, nb, nats_block_size=block,
                                                   ops_for_incomplete_chunks='all', output_final_state_gated_delta=True,
                                                   decay_for_non_gdn_blocks=True, **kw)
            else:
                o_l, o_a, ht = nats_mixed_attn_mamba(qa, ka, va, ql, kl, vl, hd, gd, tyd, nb, scale_lattn=1.0, nats_block_size=block,
                                                     ops_for_incomplete_chunks='all', output_final_state_mamba=True,
                                                     decay_for_non_mamba_blocks=True, **kw)
            ((o_l.float() * do_l.float()).sum() + (o_a.float() * do_a.float()).sum() + (ht * dht).sum()).backward()
            torch.cuda.synchronize()
            leaves = [ql, kl, vl, gd, hd] + ([bd] if kind == 'gdn' else [])
            # (column 1 of the selector's gradient is the linear op's; column 0 comes from the softmax backward's atomic adds)
            return [o_l.detach(), ht.detach(), tyd.grad[..., 1]] + [t.grad for t in leaves]
        finally:
            MC.SAVE_CHUNK_STATES = old

    kept, again = grads(True), grads(False)
    for i, (a, b) in enumerate(zip(kept, again)):
        assert torch.equal(a, b), f"tensor {i} differs between the kept and the recomputed chunk states"
