"""GPU parity at the FULL sizes the path is specified on, through size-independent properties.

The fp32 oracle would take minutes to hours at these shapes, so the checks are properties that hold for
any correct implementation:
  * the softmax branch on single (sequence, head) slices against a dense fp32 masked softmax built from
    the oracle's visibility rule (tolerance: max-abs 2e-2, rel-L2 5e-3, as everywhere);
  * exact homogeneity: every output is linear in v, and scaling by a power of two is exact in bf16 and
    fp32, so o(2v) == 2 o(v) BIT FOR BIT, for the softmax, GDN and Mamba branches (up to denormal flushes);
  * state hand-off: a sequence run in one call equals the same sequence run as two calls with the first
    call's final state as the second's initial state (bit-exact: same chunk grid, fp32 state);
  * packed input: sequences packed into one row (cu_seqlens) give bit-identical outputs to separate calls (for the GDN
    output: identical up to the rounding of the intra-chunk matrix, which the two launch shapes form in different kernels).
"""
import pytest
import torch
import torch.nn.functional as F

from oracle import softmax_branch as SB
from tests import _util
from tests._util import make_types, record_parity

pytestmark = pytest.mark.gpu
DEV = 'cuda:0'


def assert_close(a, b, what=""):
    """tests._util.assert_close (max-abs 2e-2, rel-L2 5e-3), with the measured errors recorded."""
    ma, rl = _util.assert_close(a, b, what)
    record_parity(what, max_abs=ma, rel_l2=rl)
    return ma, rl


def _randn(shape, seed, dtype=torch.bfloat16):
    g = torch.Generator(device=DEV).manual_seed(seed)
    return torch.randn(*shape, device=DEV, generator=g, dtype=torch.float32).to(dtype)


def _inputs(B, T, H, K, V, seed):
    q, k, v = _randn((B, T, H, K), seed), _randn((B, T, H, K), seed + 1), _randn((B, T, H, V), seed + 2)
    g = -F.softplus(_randn((B, T, H), seed + 3, torch.float32))
    beta = torch.sigmoid(_randn((B, T, H), seed + 4, torch.float32)).to(torch.bfloat16)
    return q, k, v, g, beta


def _assert_doubles(o2, o1, what, one_in=1_000_000):
    """o2 == 2*o1 bit for bit, except where an intermediate product falls into the denormal range (flushed by
    the matrix cores): there the two runs may differ by one rounding.  Allow at most one element in a million
    (`one_in`), and only by a negligible amount."""
    d = (o2.float() - 2 * o1.float()).abs()
    bad = int((d != 0).sum())
    assert bad <= max(1, o1.numel() // one_in) and float(d.max()) <= 1e-4, f"{what}: {bad} elements differ, max {float(d.max()):.3e}"


def _linear(kind, q, k, v, g, beta, h0, types, block, scale, decay=True, seqs=None, final=True):
    from neuralattentionsearchlinear_amd import _capi
    from neuralattentionsearchlinear_amd._mixed_common import linear_chunk_fwd
    flags = (_capi.DECAY_NON_LINEAR if decay else 0) | _capi.INTRA_CHUNK | (_capi.QK_L2NORM if kind == 'gdn' else 0)
    with torch.no_grad():
        return linear_chunk_fwd(kind, q, k, v, g, beta, h0, types, scale, block, flags, final, seqs)


def _softmax(q, k, v, types, block, scale, same_block=True, seqs=None):
    from neuralattentionsearchlinear_amd import nats_util
    from neuralattentionsearchlinear_amd.attns import parallel_attn_nats_fwd
    with torch.no_grad():
        r = nats_util.route(types, q.shape[1], block, seqs)
        o, lse, _ = parallel_attn_nats_fwd(q, k, v, types, r['nats_block_indices'], None, scale, block,
                                           compute_incomplete_chunk_scores=same_block, n_nats_blocks=r['n_nats_blocks'], seqs=seqs)
    return o, lse


# --------------------------------------------------------------------------------------------
# c2: B8 T8192 H16 K=V=128, 25 % attention blocks
# --------------------------------------------------------------------------------------------
C2 = dict(B=8, T=8192, H=16, K=128, V=128, block=64, p=0.25)


@pytest.fixture(scope="module")
def c2():
    w = C2
    q, k, v, g, beta = _inputs(w['B'], w['T'], w['H'], w['K'], w['V'], 100)
    ty = make_types(w['B'], w['T'] // w['block'], w['H'], w['p'], 7, torch.bfloat16).to(DEV)
    return dict(q=q, k=k, v=v, g=g, beta=beta, ty=ty)


@pytest.mark.parametrize("same_block", [True, False])
def test_c2_softmax_slices_against_dense_fp32(c2, same_block):
    w = C2
    scale = w['K'] ** -0.5
    o, lse = _softmax(c2['q'], c2['k'], c2['v'], c2['ty'], w['block'], scale, same_block)
    for b, h in ((0, 0), (3, 5), (7, 15)):
        mask = SB.visibility_mask(c2['ty'][b, :, h, 0].float().cpu(), w['T'], w['block'], same_block).to(DEV)
        qf, kf, vf = (c2[n][b, :, h].float() for n in ('q', 'k', 'v'))
        s = (qf @ kf.T) * scale
        s = s.masked_fill(~mask, float('-inf'))
        seen = mask.any(-1)
        p = torch.softmax(s, -1).nan_to_num(0.0)          # rows that see no key give 0
        ref = p @ vf
        assert_close(o[b, :, h].float(), ref, f"c2 o_attn[{b},:,{h}] (own block {'visible' if same_block else 'hidden'}) against the dense fp32 masked softmax")
        lse_ref = torch.where(seen, torch.logsumexp(s, -1) * 1.4426950408889634, torch.zeros_like(seen, dtype=torch.float32))
        assert float((lse[b, :, h] - lse_ref).abs().max()) <= 2e-2, "lse (log2 units)"


def test_c2_softmax_backward_slices_against_dense_fp32(c2):
    """dq, dk, dv and the selector's gradient at the full c2 shape, on single (sequence, head) slices, against
    torch.autograd through the dense fp32 masked softmax (the oracle's visibility rule).  Gradient tolerance as in the
    backward's own tests: rel-L2 5e-3, max-abs 2e-2 of the reference's largest magnitude."""
    from neuralattentionsearchlinear_amd import nats_util
    from neuralattentionsearchlinear_amd.attns import parallel_attn_nats_bwd, parallel_attn_nats_fwd
    w = C2
    scale = w['K'] ** -0.5
    r = nats_util.route(c2['ty'], w['T'], w['block'])
    with torch.no_grad():
        o, lse, _ = parallel_attn_nats_fwd(c2['q'], c2['k'], c2['v'], c2['ty'], r['nats_block_indices'], None, scale, w['block'],
                                           compute_incomplete_chunk_scores=True, n_nats_blocks=r['n_nats_blocks'])
        do = _randn(o.shape, 55)
        dq, dk, dv, _, dn = parallel_attn_nats_bwd(c2['q'], c2['k'], c2['v'], o, c2['ty'], r['nats_block_indices'], r['n_nats_blocks'],
                                                   None, lse, do, scale=scale, NAtS_block_size=w['block'],
                                                   compute_incomplete_chunk_scores=True)
    for b, h in ((0, 0), (5, 9)):
        typ = c2['ty'][b, :, h, 0].float().cpu()
        mask = SB.visibility_mask(typ, w['T'], w['block'], True).to(DEV)
        qf, kf, vf = (c2[n][b, :, h].float().requires_grad_() for n in ('q', 'k', 'v'))
        s = ((qf @ kf.T) * scale).masked_fill(~mask, float('-inf'))
        p = torch.softmax(s, -1)
        (p @ vf).backward(do[b, :, h].float())
        for name, got, ref in (("dq", dq, qf.grad), ("dk", dk, kf.grad), ("dv", dv, vf.grad)):
            g_, r_ = got[b, :, h].float(), ref
            rl = float((g_ - r_).norm() / r_.norm())
            ma, top = float((g_ - r_).abs().max()), float(r_.abs().max())
            assert rl <= 5e-3 and ma <= 2e-2 * max(top, 1.0), f"{name}[{b},:,{h}]: rel-L2 {rl:.3e}, max-abs {ma:.3e} of {top:.3e}"
            record_parity(f"c2 softmax backward {name}[{b},:,{h}] against dense fp32 autograd", max_abs=ma, rel_l2=rl, largest_reference=top)
        # selector gradient of block j: sum of dS over (queries of later blocks) x (keys of block j), for blocks typed attention
        with torch.no_grad():
            dp = do[b, :, h].float() @ vf.detach().T
            delta = (do[b, :, h].float() * o[b, :, h].float()).sum(-1, keepdim=True)
            dS = p.detach() * (dp - delta)
            NB, Bs = w['T'] // w['block'], w['block']
            blk = torch.arange(w['T'], device=DEV) // Bs
            later = blk[:, None] > blk[None, :]
            dS_l = torch.where(later, dS, torch.zeros_like(dS))
            ref_dn = dS_l.sum(0).view(NB, Bs).sum(-1)
            mag = dS_l.abs().sum(0).view(NB, Bs).sum(-1)
            attn = (torch.round(typ) == 1).to(DEV)
            err = (dn[b, :, h].float() - torch.where(attn, ref_dn, torch.zeros_like(ref_dn))).abs()
            assert bool((err <= 2e-3 * mag + 1e-5).all()), f"dnats[{b},:,{h}]: error {float(err.max()):.3e} against magnitude {float(mag.max()):.3e}"


def test_c2_outputs_are_exactly_homogeneous_in_v(c2):
    w = C2
    scale = w['K'] ** -0.5
    o1, _ = _softmax(c2['q'], c2['k'], c2['v'], c2['ty'], w['block'], scale)
    o2, _ = _softmax(c2['q'], c2['k'], c2['v'] * 2, c2['ty'], w['block'], scale)
    assert torch.equal(o2, o1 * 2), "softmax branch: o(2v) != 2 o(v)"
    l1, s1 = _linear('gdn', c2['q'], c2['k'], c2['v'], c2['g'], c2['beta'], None, c2['ty'], w['block'], scale)
    l2, s2 = _linear('gdn', c2['q'], c2['k'], c2['v'] * 2, c2['g'], c2['beta'], None, c2['ty'], w['block'], scale)
    _assert_doubles(l2, l1, "GDN branch: o(2v) vs 2 o(v)")
    assert torch.equal(s2, s1 * 2), "GDN branch: S(2v) != 2 S(v)"
    assert torch.isfinite(l1.float()).all() and torch.isfinite(s1).all()


def test_c2_gdn_state_hand_off(c2):
    w = C2
    scale = w['K'] ** -0.5
    half = w['T'] // 2
    nb = half // w['block']
    o, s = _linear('gdn', c2['q'], c2['k'], c2['v'], c2['g'], c2['beta'], None, c2['ty'], w['block'], scale)
    sl = lambda t, a, b: t[:, a:b].contiguous()
    oa, sa = _linear('gdn', *(sl(c2[n], 0, half) for n in ('q', 'k', 'v', 'g', 'beta')), None, sl(c2['ty'], 0, nb), w['block'], scale)
    ob, sb = _linear('gdn', *(sl(c2[n], half, w['T']) for n in ('q', 'k', 'v', 'g', 'beta')), sa, sl(c2['ty'], nb, 2 * nb), w['block'], scale)
    assert torch.equal(o[:, :half], oa) and torch.equal(o[:, half:], ob), "outputs differ across the hand-off"
    assert torch.equal(s, sb), "final state differs across the hand-off"


# --------------------------------------------------------------------------------------------
# c1: B4 T4096 H16 K=V=128, every block linear
# --------------------------------------------------------------------------------------------
def test_c1_all_linear_matches_token_recurrence_on_a_slice():
    """All blocks linear: the chunked kernels must equal the plain token-by-token gated delta rule.  The
    recurrence (oracle) is run for two (sequence, head) slices only."""
    from oracle import linear_branch as LB
    B, T, H, K, V, block = 4, 4096, 16, 128, 128, 64
    q, k, v, g, beta = _inputs(B, T, H, K, V, 300)
    ty = make_types(B, T // block, H, 0.0, 1, torch.bfloat16).to(DEV)
    scale = K ** -0.5
    o, s = _linear('gdn', q, k, v, g, beta, None, ty, block, scale)
    for b, h in ((0, 0), (3, 11)):
        sl = lambda t: t[b:b + 1, :, h:h + 1].float().cpu()
        lin = torch.ones(1, T // block, 1)
        o_ref, s_ref = LB.gdn_token_recurrence(sl(q), sl(k), sl(v), sl(g), sl(beta), lin, scale, None, block=block)
        assert_close(o[b:b + 1, :, h:h + 1].float(), o_ref, f"c1 o_gdn[{b},:,{h}] against the fp64 token recurrence")
        assert_close(s[b:b + 1, h:h + 1], s_ref, f"c1 final_state[{b},{h}] against the fp64 token recurrence")


# --------------------------------------------------------------------------------------------
# c3: B1 T65536 H32 K=V=128, 10 % attention, also packed as 8192/16384/16384/24576
# --------------------------------------------------------------------------------------------
def test_c3_packed_equals_separate_calls():
    from neuralattentionsearchlinear_amd.nats_util import pack_sequences
    T, H, K, V, block = 65536, 32, 128, 128, 64
    lens = [8192, 16384, 16384, 24576]
    cu = [0]
    for n in lens:
        cu.append(cu[-1] + n)
    q, k, v, g, beta = _inputs(1, T, H, K, V, 500)
    parts = [make_types(1, n // block, H, 0.10, 20 + i, torch.bfloat16) for i, n in enumerate(lens)]
    ty = torch.cat(parts, 1).to(DEV)
    scale = K ** -0.5
    cud = torch.tensor(cu, dtype=torch.int64, device=DEV)
    seqs = pack_sequences(cud, None, block, torch.device(DEV))
    o_attn, lse = _softmax(q, k, v, ty, block, scale, True, seqs)
    o_lin, s = _linear('gdn', q, k, v, g, beta, None, ty, block, scale, seqs=seqs)
    assert s.shape == (len(lens), H, K, V)
    nb0 = 0
    for i, (a, b) in enumerate(zip(cu[:-1], cu[1:])):
        nb = (b - a) // block
        sl = lambda t: t[:, a:b].contiguous()
        tyi = ty[:, nb0:nb0 + nb].contiguous()
        oa, la = _softmax(sl(q), sl(k), sl(v), tyi, block, scale, True)
        ol, si = _linear('gdn', sl(q), sl(k), sl(v), sl(g), sl(beta), None, tyi, block, scale)
        assert torch.equal(o_attn[:, a:b], oa) and torch.equal(lse[:, a:b], la), f"softmax branch, sequence {i}"
        # (the packed call fills the machine and forms P inside the scan, a single sequence does not and takes P from the prep
        # kernel: the states are the same bits, the outputs agree to the rounding of P's bf16 tiles)
        assert torch.equal(s[i:i + 1], si), f"GDN branch, final state of sequence {i}"
        rl = float((o_lin[:, a:b].float() - ol.float()).norm() / ol.float().norm())
        assert rl <= 5e-4, f"GDN branch, sequence {i}: rel-L2 {rl:.3e} between the packed call and the call on the sequence alone"
        nb0 += nb


# --------------------------------------------------------------------------------------------
# c4: Mamba, B4 T8192 H32, state K=128, head V=64, selector block 256, 25 % attention
# --------------------------------------------------------------------------------------------
def test_c4_mamba_homogeneity_and_hand_off():
    B, T, H, K, V, block = 4, 8192, 32, 128, 64, 256
    q, k, v, g, _ = _inputs(B, T, H, K, V, 700)
    ty = make_types(B, T // block, H, 0.25, 3, torch.bfloat16).to(DEV)
    o, s = _linear('mamba', q, k, v, g, None, None, ty, block, 1.0)
    o2, s2 = _linear('mamba', q, k, v * 2, g, None, None, ty, block, 1.0)
    _assert_doubles(o2, o, "Mamba branch: o(2x) vs 2 o(x)")
    assert torch.equal(s2, s * 2), "Mamba branch: S(2x) != 2 S(x)"
    half, nb = T // 2, T // 2 // block
    sl = lambda t, a, b: t[:, a:b].contiguous()
    oa, sa = _linear('mamba', *(sl(t, 0, half) for t in (q, k, v, g)), None, None, sl(ty, 0, nb), block, 1.0)
    ob, sb = _linear('mamba', *(sl(t, half, T) for t in (q, k, v, g)), None, sa, sl(ty, nb, 2 * nb), block, 1.0)
    assert torch.equal(o[:, :half], oa) and torch.equal(o[:, half:], ob) and torch.equal(s, sb), "state hand-off"
    # the attention view of the same layer: K=128, V=64, block 256
    oa1, _ = _softmax(q, k, v, ty, block, K ** -0.5)
    oa2, _ = _softmax(q, k, v * 2, ty, block, K ** -0.5)
    assert torch.equal(oa2, oa1 * 2)
    mask = SB.visibility_mask(ty[1, :, 4, 0].float().cpu(), T, block, True).to(DEV)
    sc = (q[1, :, 4].float() @ k[1, :, 4].float().T) * K ** -0.5
    ref = torch.softmax(sc.masked_fill(~mask, float('-inf')), -1) @ v[1, :, 4].float()
    assert_close(oa1[1, :, 4].float(), ref, "c4 shape, N(0,1) inputs: o_attn[1,:,4] against the dense fp32 masked softmax")


# --------------------------------------------------------------------------------------------
# full-depth checks of the Gated-DeltaNet chain against the fp64 token recurrence, one (sequence, head)
# slice at a time (the recurrence runs on the host: a slice of 65 536 tokens takes a few seconds)
# --------------------------------------------------------------------------------------------
def _gdn_slice_against_token_recurrence(q, k, v, g, beta, ty, o, s, b, h, block, scale, t0=0, t1=None, s_index=None, what=""):
    """Slice (b, h), tokens [t0, t1) of the packed row, of the kernel's output `o` and final state `s` against the
    oracle's token-by-token recurrence in fp64 under the drawn block types.  Returns the measured errors."""
    from oracle import linear_branch as LB
    t1 = q.shape[1] if t1 is None else t1
    sl = lambda t: t[b:b + 1, t0:t1, h:h + 1].float().cpu()
    lin = ty[b:b + 1, t0 // block:-(-t1 // block), h:h + 1, 1].float().cpu()
    o_ref, s_ref = LB.gdn_token_recurrence(sl(q), sl(k), sl(v), sl(g), sl(beta), lin, scale, None, block=block)
    e_o = assert_close(o[b:b + 1, t0:t1, h:h + 1].float(), o_ref, f"{what} o_gdn[{b},{t0}:{t1},{h}]")
    si = b if s_index is None else s_index
    e_s = assert_close(s[si:si + 1, h:h + 1], s_ref, f"{what} final_state[{si},{h}]")
    # the tail of the chain on its own: an error that grows with depth shows here first
    tail = slice(t1 - t0 - 1024, t1 - t0)
    e_t = assert_close(o[b:b + 1, t0:t1, h:h + 1][:, tail].float(), o_ref[:, tail], f"{what} last 1024 tokens of o_gdn[{b},:,{h}]")
    print(f"\n{what} slice ({b},{h}) tokens {t0}:{t1}: o max-abs {e_o[0]:.2e} rel-L2 {e_o[1]:.2e}; "
          f"last 1024 tokens rel-L2 {e_t[1]:.2e}; final state max-abs {e_s[0]:.2e} rel-L2 {e_s[1]:.2e}", flush=True)
    return e_o, e_s


def test_c2_gdn_full_depth_slices_against_token_recurrence(c2):
    """c2 with the drawn mask (25 % attention blocks, decay across them): 128 chunks deep."""
    w = C2
    scale = w['K'] ** -0.5
    o, s = _linear('gdn', c2['q'], c2['k'], c2['v'], c2['g'], c2['beta'], None, c2['ty'], w['block'], scale)
    for b, h in ((0, 0), (6, 13)):
        _gdn_slice_against_token_recurrence(c2['q'], c2['k'], c2['v'], c2['g'], c2['beta'], c2['ty'], o, s, b, h, w['block'], scale, what="c2")


def test_c3_unpacked_single_sequence_against_the_oracle():
    """c3 as ONE sequence: B1 T65536 H32 K=V=128, 10 % attention blocks; 1024 chunks deep.
    Gated DeltaNet: two head slices against the fp64 token recurrence.  Softmax branch: the last 512 queries and a
    window in the middle of one head against the dense fp32 masked softmax over all 65 536 keys."""
    T, H, K, V, block = 65536, 32, 128, 128, 64
    q, k, v, g, beta = _inputs(1, T, H, K, V, 900)
    ty = make_types(1, T // block, H, 0.10, 31, torch.bfloat16).to(DEV)
    scale = K ** -0.5
    o_lin, s = _linear('gdn', q, k, v, g, beta, None, ty, block, scale)
    o_attn, lse = _softmax(q, k, v, ty, block, scale, True)
    assert torch.isfinite(o_lin.float()).all() and torch.isfinite(s).all() and torch.isfinite(o_attn.float()).all()
    for h in (0, 21):
        _gdn_slice_against_token_recurrence(q, k, v, g, beta, ty, o_lin, s, 0, h, block, scale, what="c3")
    h = 17
    mask_rows = SB.visibility_mask(ty[0, :, h, 0].float().cpu(), T, block, True)
    kf, vf = k[0, :, h].float(), v[0, :, h].float()
    for a, b_ in ((T - 512, T), (T // 2 - 256, T // 2 + 256)):
        m = mask_rows[a:b_].to(DEV)
        sc = ((q[0, a:b_, h].float() @ kf.T) * scale).masked_fill(~m, float('-inf'))
        ref = torch.softmax(sc, -1) @ vf
        assert_close(o_attn[0, a:b_, h].float(), ref, f"c3 o_attn[0,{a}:{b_},{h}]")
        lse_ref = torch.logsumexp(sc, -1) * 1.4426950408889634
        assert float((lse[0, a:b_, h] - lse_ref).abs().max()) <= 2e-2, "c3 lse (log2 units)"


def test_c3_packed_sequence_against_token_recurrence():
    """The packed c3 row (8192/16384/16384/24576 via cu_seqlens): the longest sequence's chain, cut out of the packed
    call's output, against the token recurrence started from a zero state at that sequence's first token."""
    from neuralattentionsearchlinear_amd.nats_util import pack_sequences
    T, H, K, V, block = 65536, 32, 128, 128, 64
    cu = [0, 8192, 24576, 40960, 65536]
    q, k, v, g, beta = _inputs(1, T, H, K, V, 500)
    ty = torch.cat([make_types(1, (b - a) // block, H, 0.10, 20 + i, torch.bfloat16) for i, (a, b) in enumerate(zip(cu[:-1], cu[1:]))], 1).to(DEV)
    scale = K ** -0.5
    seqs = pack_sequences(torch.tensor(cu, dtype=torch.int64, device=DEV), None, block, torch.device(DEV))
    o_lin, s = _linear('gdn', q, k, v, g, beta, None, ty, block, scale, seqs=seqs)
    _gdn_slice_against_token_recurrence(q, k, v, g, beta, ty, o_lin, s, 0, 9, block, scale, t0=cu[3], t1=cu[4], s_index=3, what="c3 packed")
    _gdn_slice_against_token_recurrence(q, k, v, g, beta, ty, o_lin, s, 0, 30, block, scale, t0=cu[1], t1=cu[2], s_index=1, what="c3 packed")


def _rel(a, b):
    a, b = a.double().cpu(), b.double().cpu()
    return float((a - b).norm() / (b.norm() + 1e-30))


def test_c2_gdn_backward_full_depth(c2):
    """The linear branch's backward kernels at c2 (128 chunks deep, the drawn mask, decay across attention blocks):
    (i) two (batch, head) slices against autograd through the fp64 chunked oracle on that slice alone (heads and batch
    entries are independent chains); (ii) the whole result against the torch formulation of the same method;
    (iii) the gradients are linear in dO: doubling dO doubles them bit for bit.
    Tolerances as in tests/test_gpu_linear_bwd.py: rel-L2 5e-3 for dq, dk, dv, 1e-2 for the per-token scalars dg, dbeta."""
    from oracle import linear_branch as LB
    from neuralattentionsearchlinear_amd import _linear_bwd as B_
    w = C2
    scale = w['K'] ** -0.5
    do = _randn((w['B'], w['T'], w['H'], w['V']), 300)
    args = ('gdn', c2['q'], c2['k'], c2['v'], c2['g'], c2['beta'], None, c2['ty'], scale, w['block'], True, True, True)
    with torch.no_grad():
        got = B_.linear_chunk_backward_hip(*args, do, None, False)
        got2 = B_.linear_chunk_backward_hip(*args, do * 2, None, False)
        ref = B_.linear_chunk_backward_torch(*args, do, None, False)
    names = ['dq', 'dk', 'dv', 'dg', 'dbeta']
    for j, name in enumerate(names):
        assert torch.isfinite(got[j].float()).all(), name
        # (a gradient passes through many more products than an output, and the state gradient's share from far-away chunks
        # decays through the denormal range on its way to zero: a few elements in 100 000, by less than 1e-7)
        _assert_doubles(got2[j], got[j], f"{name}(2 dO) vs 2 {name}(dO)", 20_000)
        assert float((got2[j].float() - 2 * got[j].float()).abs().max()) <= 1e-7, name
        r = _rel(got[j], ref[j])
        assert r <= (1e-2 if name in ('dg', 'dbeta') else 5e-3), f"{name} against the torch formulation: rel-L2 {r:.3e}"
    r = _rel(got[6], ref[6])
    assert r <= 1e-2, f"dnats against the torch formulation: rel-L2 {r:.3e}"
    for b, h in ((0, 0), (6, 13)):
        sl = lambda t: t[b:b + 1, :, h:h + 1].cpu()
        o = LB.linear_branch_bwd('gdn', sl(c2['q']), sl(c2['k']), sl(c2['v']), sl(c2['g']), sl(c2['beta']), c2['ty'][b:b + 1, :, h:h + 1, 1].cpu(),
                                 scale, sl(do), None, None, w['block'], True, True, True, False)
        errs = {}
        for j, name in enumerate(names):
            errs[name] = _rel(got[j][b:b + 1, :, h:h + 1], o[name])
            assert errs[name] <= (1e-2 if name in ('dg', 'dbeta') else 5e-3), f"{name}[{b},:,{h}] against the fp64 oracle: rel-L2 {errs[name]:.3e}"
        e_n = _rel(got[6][b:b + 1, :, h:h + 1], o['dnats'])
        assert e_n <= 1e-2, f"dnats[{b},:,{h}] against the fp64 oracle: rel-L2 {e_n:.3e}"
        print(f"\nc2 backward slice ({b},{h}): " + "  ".join(f"{n} {e:.2e}" for n, e in errs.items()) + f"  dnats {e_n:.2e}", flush=True)
        record_parity(f"c2 GDN backward slice ({b},{h}) against the fp64 oracle, rel-L2", **errs, dnats=e_n)


def _c4_draw(seed=1700):
    """c4's own distributions: dt = softplus(N(0,1) - 4); A = -exp(U(0, log 16)) per head; B, C ~ N(0,1) in ONE group shared by
    all heads (k = B, q = C, state dim 128); X ~ N(0,1), head dim 64; the operator takes v = X dt and g = A dt
    (src/nats/layers/natsl_attn_mamba2.py:472-474); selector blocks of 256 tokens, 25 % typed attention."""
    B, T, H, K, V, block = 4, 8192, 32, 128, 64, 256
    dt = F.softplus(_randn((B, T, H), seed, torch.float32) - 4.0)
    gen = torch.Generator(device=DEV).manual_seed(seed + 1)
    A = -torch.exp(torch.rand(H, device=DEV, generator=gen) * torch.log(torch.tensor(16.0)))
    q = _randn((B, T, 1, K), seed + 2).expand(B, T, H, K).contiguous()
    k = _randn((B, T, 1, K), seed + 3).expand(B, T, H, K).contiguous()
    x = _randn((B, T, H, V), seed + 4)
    v = (x.float() * dt.unsqueeze(-1)).to(torch.bfloat16)
    g = A.view(1, 1, H) * dt
    ty = make_types(B, T // block, H, 0.25, 17, torch.bfloat16).to(DEV)
    return dict(q=q, k=k, v=v, g=g, ty=ty, x=x, B=B, T=T, H=H, K=K, V=V, block=block)


def test_c4_mamba_config_draw_slices_against_token_recurrence():
    """c4 as its configuration draws it (un-normalised B and C shared across heads, small dt, strong per-head decay): two
    (sequence, head) slices of the Mamba branch's output and the final SSM state against the fp64 token recurrence, and
    one slice of the softmax branch (K = 128, V = 64, block 256) against the dense fp32 masked softmax."""
    from oracle import linear_branch as LB
    d = _c4_draw()
    T, K, block = d['T'], d['K'], d['block']
    o, s = _linear('mamba', d['q'], d['k'], d['v'], d['g'], None, None, d['ty'], block, 1.0)
    assert torch.isfinite(o.float()).all() and torch.isfinite(s).all()
    for b, h in ((0, 0), (3, 26)):
        sl = lambda t: t[b:b + 1, :, h:h + 1].float().cpu()
        lin = d['ty'][b:b + 1, :, h:h + 1, 1].float().cpu()
        o_ref, s_ref = LB.mamba_token_recurrence(sl(d['q']), sl(d['k']), sl(d['v']), sl(d['g']), lin, 1.0, None, block=block)
        # the outputs here reach far beyond 1 (|B.C| ~ 11 per key, tens of keys in the decay window): the absolute bound scales
        top = float(o_ref.abs().max())
        ma, rl = _util.max_abs(o[b:b + 1, :, h:h + 1].float(), o_ref), _util.rel_l2(o[b:b + 1, :, h:h + 1].float(), o_ref)
        record_parity(f"c4 o_mamba[{b},:,{h}] against the fp64 token recurrence", max_abs=ma, rel_l2=rl, largest_reference=top)
        assert rl <= _util.REL_L2_TOL and ma <= _util.MAX_ABS_TOL * max(top, 1.0), f"o_mamba[{b},:,{h}]: rel-L2 {rl:.3e}, max-abs {ma:.3e} of {top:.3e}"
        top = float(s_ref.abs().max())
        ma, rl = _util.max_abs(s[b:b + 1, h:h + 1], s_ref), _util.rel_l2(s[b:b + 1, h:h + 1], s_ref)
        record_parity(f"c4 final SSM state[{b},{h}] against the fp64 token recurrence", max_abs=ma, rel_l2=rl, largest_reference=top)
        assert rl <= _util.REL_L2_TOL and ma <= _util.MAX_ABS_TOL * max(top, 1.0), f"final state[{b},{h}]: rel-L2 {rl:.3e}, max-abs {ma:.3e} of {top:.3e}"
    # the attention view reads the un-scaled X (src/nats/layers/natsl_attn_mamba2.py:391-393, :442)
    oa, _ = _softmax(d['q'], d['k'], d['x'], d['ty'], block, K ** -0.5)
    b, h = 2, 9
    mask = SB.visibility_mask(d['ty'][b, :, h, 0].float().cpu(), T, block, True).to(DEV)
    sc = (d['q'][b, :, h].float() @ d['k'][b, :, h].float().T) * K ** -0.5
    ref = torch.softmax(sc.masked_fill(~mask, float('-inf')), -1) @ d['x'][b, :, h].float()
    assert_close(oa[b, :, h].float(), ref, f"c4 o_attn[{b},:,{h}] against the dense fp32 masked softmax")


def test_c4_mamba_backward_slices():
    """The linear branch's backward in its Mamba form at c4 (32 blocks of 4 chunks, the configuration's draw): two
    (sequence, head) slices of dq, dk, dv, dg and the selector's gradient against autograd through the fp64 chunked oracle
    on that slice alone, and exact linearity in dO.  Tolerances as in tests/test_gpu_linear_bwd.py."""
    from oracle import linear_branch as LB
    from neuralattentionsearchlinear_amd import _linear_bwd as B_
    d = _c4_draw()
    do = _randn((d['B'], d['T'], d['H'], d['V']), 1800)
    args = ('mamba', d['q'], d['k'], d['v'], d['g'], None, None, d['ty'], 1.0, d['block'], True, False, True)
    with torch.no_grad():
        got = B_.linear_chunk_backward_hip(*args, do, None, False)
        got2 = B_.linear_chunk_backward_hip(*args, do * 2, None, False)
    names = ['dq', 'dk', 'dv', 'dg']
    for j, name in enumerate(names):
        assert torch.isfinite(got[j].float()).all(), name
        _assert_doubles(got2[j], got[j], f"{name}(2 dO) vs 2 {name}(dO)", 20_000)
    for b, h in ((0, 0), (3, 26)):
        sl = lambda t: t[b:b + 1, :, h:h + 1].cpu()
        o = LB.linear_branch_bwd('mamba', sl(d['q']), sl(d['k']), sl(d['v']), sl(d['g']), None, d['ty'][b:b + 1, :, h:h + 1, 1].cpu(),
                                 1.0, sl(do), None, None, d['block'], True, False, True, False)
        errs = {}
        for j, name in enumerate(names):
            errs[name] = _rel(got[j][b:b + 1, :, h:h + 1], o[name])
            assert errs[name] <= (1e-2 if name == 'dg' else 5e-3), f"{name}[{b},:,{h}] against the fp64 oracle: rel-L2 {errs[name]:.3e}"
        e_n = _rel(got[6][b:b + 1, :, h:h + 1], o['dnats'])
        assert e_n <= 1e-2, f"dnats[{b},:,{h}] against the fp64 oracle: rel-L2 {e_n:.3e}"
        record_parity(f"c4 Mamba backward slice ({b},{h}) against the fp64 oracle, rel-L2", **errs, dnats=e_n)
