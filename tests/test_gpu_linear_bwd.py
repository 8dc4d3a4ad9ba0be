"""GPU parity: the backward kernels of the two linear branches (natsl_linear_chunk_bwd: reverse scan + per-chunk gradients)
against autograd through the fp64 chunked oracle (oracle.linear_branch.linear_branch_bwd), and the torch formulation of the
same method against the same oracle.

Tolerance: rel-L2 5e-3 and max-abs 2e-2 of the reference's largest magnitude for dq, dk, dv, dh0; rel-L2 1e-2 for the
per-token scalars dg and dbeta and for the selector's gate gradient (sums of large terms of both signs over bf16-rounded
intermediates: the kernels round where the reference's do -- h, dh, v_new, dv are kept in the input dtype at
src/nats/ops/common/chunk_delta_h.py:681, 693, 775, 785)."""
import pytest
import torch
import torch.nn.functional as F

from oracle import linear_branch as LB
from tests._util import make_gates, make_qkv, make_types, max_abs, rel_l2

pytestmark = pytest.mark.gpu
DEV = 'cuda:0'

CASES = [
    # kind, B, T, H, HN, K, V, block, decay, intra, h0, dht, invalid
    ('gdn', 2, 512, 4, 2, 128, 128, 64, True, True, True, True, False),
    ('gdn', 1, 300, 4, 2, 64, 64, 128, True, True, False, True, False),     # ragged last chunk, incomplete last block
    ('gdn', 1, 640, 2, 1, 192, 384, 256, True, True, True, False, False),   # the 760M geometry
    ('gdn', 1, 512, 6, 6, 128, 256, 64, False, True, True, True, True),     # the 340M geometry, no decay on rolled-back blocks
    ('gdn', 1, 256, 2, 2, 128, 64, 64, True, False, True, True, True),      # no intra-chunk term
    ('mamba', 2, 512, 4, 2, 128, 64, 64, True, True, True, True, True),
    ('mamba', 1, 330, 4, 4, 64, 128, 128, False, True, False, True, False),
]


def _inputs(kind, B, T, H, HN, K, V, block, seed):
    q, k, v = make_qkv(B, T, H, K, V, seed)
    if kind == 'mamba':
        q, k = F.normalize(q.float(), dim=-1).bfloat16(), F.normalize(k.float(), dim=-1).bfloat16()
    g, beta = make_gates(B, T, H, seed + 1)
    ty = make_types(B, -(-T // block), HN, 0.4, seed + 2, torch.bfloat16)
    gen = torch.Generator().manual_seed(seed + 3)
    init = torch.randn(B, H, K, V, generator=gen) * 0.3
    do = torch.randn(B, T, H, V, generator=gen).bfloat16()
    dht = torch.randn(B, H, K, V, generator=gen) * 0.3      # the scale of the states themselves
    return q, k, v, g, beta, ty, init, do, dht


def _check(out, ref, kind, h0):
    names = ['dq', 'dk', 'dv', 'dg', 'dbeta', 'dh0']
    for name, got in zip(names, out[:6]):
        if name == 'dbeta' and kind != 'gdn':
            assert got is None
            continue
        if name == 'dh0' and not h0:
            assert got is None
            continue
        want = ref[name]
        tol = 1e-2 if name in ('dg', 'dbeta') else 5e-3
        rl, ma, top = rel_l2(got.float().cpu(), want), max_abs(got.float().cpu(), want), float(want.abs().max())
        assert rl <= tol and ma <= 2e-2 * max(top, 1.0), f"{name}: rel-L2 {rl:.3e}, max-abs {ma:.3e} (largest reference value {top:.3e})"
    dn, want = out[6].double().cpu(), ref['dnats']
    assert rel_l2(dn, want) <= 1e-2 and float((dn - want).abs().max()) <= 2e-2 * max(float(want.abs().max()), 1.0), \
        f"dnats: rel-L2 {rel_l2(dn, want):.3e}"


@pytest.mark.parametrize("which", ['hip', 'torch'])
@pytest.mark.parametrize("case", CASES, ids=lambda c: f"{c[0]}-T{c[2]}-K{c[5]}-V{c[6]}-b{c[7]}")
def test_linear_branch_backward(case, which):
    from neuralattentionsearchlinear_amd import _linear_bwd as B_
    kind, B, T, H, HN, K, V, block, decay, intra, h0, dht_on, invalid = case
    q, k, v, g, beta, ty, init, do, dht = _inputs(kind, B, T, H, HN, K, V, block, 100 + K + V)
    scale = K ** -0.5 if kind == 'gdn' else 1.0
    l2 = kind == 'gdn'
    ref = LB.linear_branch_bwd(kind, q, k, v, g, beta if kind == 'gdn' else None, ty[..., 1], scale, do, dht if dht_on else None,
                               init if h0 else None, block, decay, l2, intra, invalid)
    d = lambda t: t.to(DEV)
    fn = B_.linear_chunk_backward_hip if which == 'hip' else B_.linear_chunk_backward_torch
    out = fn(kind, d(q), d(k), d(v), d(g), d(beta) if kind == 'gdn' else None, d(init) if h0 else None, d(ty), scale, block, decay,
             l2, intra, d(do), d(dht) if dht_on else None, invalid)
    torch.cuda.synchronize()
    _check(out, ref, kind, h0)


@pytest.mark.parametrize("kind,wide", [('gdn', False), ('mamba', False), ('gdn', True), ('mamba', True)])
def test_packed_sequences_equal_separate_calls(kind, wide):
    """One call over packed sequences gives, bit for bit, what one call per sequence gives (own initial state, own
    final-state gradient, own blocks; ragged lengths).  The wide case has enough (sequence, head, column slice) chains for the
    reverse scan to run 64 state columns per workgroup in the packed call and 32 in the calls per sequence: the same bits."""
    from neuralattentionsearchlinear_amd import _linear_bwd as B_
    from neuralattentionsearchlinear_amd.nats_util import pack_sequences
    lens, H, HN, K, V, block = ([200, 64, 450, 129], 16, 4, 128, 256, 128) if wide else ([200, 64, 450, 129], 4, 2, 128, 64, 128)
    T = sum(lens)
    cu = [0]
    for n in lens:
        cu.append(cu[-1] + n)
    NB = sum(-(-n // block) for n in lens)
    q, k, v, g, beta, _, _, do, _ = _inputs(kind, 1, T, H, HN, K, V, block, 7)
    ty = make_types(1, NB, HN, 0.4, 9, torch.bfloat16)
    gen = torch.Generator().manual_seed(5)
    init = torch.randn(len(lens), H, K, V, generator=gen) * 0.3
    dht = torch.randn(len(lens), H, K, V, generator=gen) * 0.3
    d = lambda t: t.to(DEV)
    scale = K ** -0.5 if kind == 'gdn' else 1.0
    seqs = pack_sequences(cu, None, block, DEV)
    args = lambda sl, nsl, i: (kind, d(q[:, sl]), d(k[:, sl]), d(v[:, sl]), d(g[:, sl]), d(beta[:, sl]) if kind == 'gdn' else None,
                               d(init[i]), d(ty[:, nsl]), scale, block, True, kind == 'gdn', True, d(do[:, sl]), d(dht[i]), True)
    whole = B_.linear_chunk_backward_hip(*args(slice(None), slice(None), slice(None)), seqs)
    nb = 0
    for i, n in enumerate(lens):
        nbi = -(-n // block)
        part = B_.linear_chunk_backward_hip(*args(slice(cu[i], cu[i + 1]), slice(nb, nb + nbi), slice(i, i + 1)))
        for j, name in enumerate(['dq', 'dk', 'dv', 'dg', 'dbeta']):
            if part[j] is not None:
                assert torch.equal(whole[j][:, cu[i]:cu[i + 1]], part[j]), f"{name} of sequence {i}"
        assert torch.equal(whole[5][i:i + 1], part[5]), f"dh0 of sequence {i}"
        assert torch.equal(whole[6][:, nb:nb + nbi], part[6]), f"dnats of sequence {i}"
        nb += nbi


def _random_case(seed):
    import random
    r = random.Random(seed)
    kind = r.choice(['gdn', 'gdn', 'mamba'])
    K = r.choice([64, 128, 192])
    V = r.choice([64, 128]) if K < 192 else 64
    block = r.choice([64, 128, 256])
    H = r.choice([1, 2, 4])
    HN = r.choice([h for h in (1, 2, 4) if H % h == 0])
    T = r.choice([r.randrange(1, 64), r.randrange(65, 400), 64 * r.randrange(1, 7)])
    return (kind, r.choice([1, 2]), T, H, HN, K, V, block, r.random() < 0.7, r.random() < 0.85, r.random() < 0.5, r.random() < 0.5,
            r.random() < 0.5)


@pytest.mark.parametrize("seed", range(12))
def test_linear_branch_backward_random_shapes(seed):
    """Drawn shapes and options (ragged lengths down to a single token, all three key widths, blocks of 1, 2, 4 chunks,
    selector heads shared by several heads) against the fp64 oracle."""
    from neuralattentionsearchlinear_amd import _linear_bwd as B_
    case = _random_case(1000 + seed)
    kind, B, T, H, HN, K, V, block, decay, intra, h0, dht_on, invalid = case
    q, k, v, g, beta, ty, init, do, dht = _inputs(kind, B, T, H, HN, K, V, block, 500 + seed)
    scale = K ** -0.5 if kind == 'gdn' else 1.0
    l2 = kind == 'gdn'
    ref = LB.linear_branch_bwd(kind, q, k, v, g, beta if kind == 'gdn' else None, ty[..., 1], scale, do, dht if dht_on else None,
                               init if h0 else None, block, decay, l2, intra, invalid)
    d = lambda t: t.to(DEV)
    print(f"\ncase {case}", flush=True)
    out = B_.linear_chunk_backward_hip(kind, d(q), d(k), d(v), d(g), d(beta) if kind == 'gdn' else None, d(init) if h0 else None, d(ty),
                                       scale, block, decay, l2, intra, d(do), d(dht) if dht_on else None, invalid)
    torch.cuda.synchronize()
    _check(out, ref, kind, h0)


@pytest.mark.parametrize("kind,K,V", [('gdn', 64, 32), ('gdn', 128, 96), ('mamba', 128, 48)])
def test_value_widths_that_are_no_multiple_of_64(kind, K, V):
    """V = 16..48, 96, ..: the dispatcher runs the kernels on v, dO and the states padded with zero columns to the next multiple
    of 64 and cuts the gradients back; against the fp64 oracle on the narrow problem."""
    from neuralattentionsearchlinear_amd import _linear_bwd as B_
    B, T, H, HN, block = 2, 330, 4, 2, 64
    q, k, v, g, beta, ty, init, do, dht = _inputs(kind, B, T, H, HN, K, V, block, 900 + V)
    scale = K ** -0.5 if kind == 'gdn' else 1.0
    l2 = kind == 'gdn'
    ref = LB.linear_branch_bwd(kind, q, k, v, g, beta if kind == 'gdn' else None, ty[..., 1], scale, do, dht, init, block, True, l2, True, True)
    d = lambda t: t.to(DEV)
    assert not B_.hip_backward_is_built(K, V)
    out = B_.linear_chunk_backward(kind, d(q), d(k), d(v), d(g), d(beta) if kind == 'gdn' else None, d(init), d(ty), scale, block, True,
                                   l2, True, d(do), d(dht), True)
    torch.cuda.synchronize()
    assert out[2].shape[-1] == V and out[5].shape[-1] == V
    _check(out, ref, kind, True)
