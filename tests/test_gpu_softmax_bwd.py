"""GPU parity: backward of the softmax branch through the C ABI vs oracle/softmax_branch.softmax_branch_bwd
(fp64 on the same bf16-rounded inputs).  Tolerance for gradients: rel-L2 5e-3 as for the outputs; the absolute part of
the outputs' tolerance does not transfer (gradients are not O(1)), so max-abs is checked against 2e-2 of the
reference's largest magnitude."""
import pytest
import torch

from oracle import softmax_branch as sb
from tests._util import make_qkv, make_types, max_abs, rel_l2

pytestmark = pytest.mark.gpu
DEV = 'cuda:0'


def _close(a, b, what):
    rl, ma, top = rel_l2(a, b), max_abs(a, b), float(b.abs().max())
    assert rl <= 5e-3 and ma <= 2e-2 * max(top, 1.0), f"{what}: rel-L2 {rl:.3e}, max-abs {ma:.3e} (largest reference value {top:.3e})"


def _run(B, T, HQ, H, HN, K, V, block, p_attn, same_block, seed, through_autograd=False, dnats_invalid=False):
    from neuralattentionsearchlinear_amd import nats_util
    from neuralattentionsearchlinear_amd.attns import parallel_attn_nats_bwd, parallel_attn_nats_fwd, parallel_nats_attn
    q, k, v = make_qkv(B, T, H, K, V, seed, HQ=HQ)
    do = torch.randn(B, T, HQ, V, generator=torch.Generator().manual_seed(seed + 7)).bfloat16()
    ty = make_types(B, -(-T // block), HN, p_attn, seed + 1, torch.bfloat16)
    scale = K ** -0.5
    dq_r, dk_r, dv_r, dn_r, dn_mag = sb.softmax_branch_bwd(q, k, v, ty, do, scale, block, same_block, with_magnitude=True,
                                                           dnats_invalid=dnats_invalid)
    qd, kd, vd, dod, tyd = (t.to(DEV) for t in (q, k, v, do, ty))
    r = nats_util.route(tyd, T, block)
    if through_autograd:
        qd, kd, vd = (t.requires_grad_() for t in (qd, kd, vd))
        tyd = tyd.requires_grad_()
        o, _ = parallel_nats_attn(qd, kd, vd, None, tyd, r['nats_block_indices'], r['n_nats_blocks'], scale,
                                  NAtS_block_size=block, compute_incomplete_chunk_scores=same_block,
                                  compute_dnats_for_invalid_blocks_attn=dnats_invalid)
        o.backward(dod)
        dq, dk, dv, dn = qd.grad, kd.grad, vd.grad, tyd.grad[..., 0]
        assert float(tyd.grad[..., 1:].abs().max()) == 0.0
    else:
        o, lse, _ = parallel_attn_nats_fwd(qd, kd, vd, tyd, r['nats_block_indices'], None, scale, block,
                                           compute_incomplete_chunk_scores=same_block, n_nats_blocks=r['n_nats_blocks'])
        dq, dk, dv, _, dn = parallel_attn_nats_bwd(qd, kd, vd, o, tyd, r['nats_block_indices'], r['n_nats_blocks'], None, lse, dod,
                                                   scale=scale, NAtS_block_size=block, compute_incomplete_chunk_scores=same_block,
                                                   compute_dnats_for_invalid_blocks_attn=dnats_invalid)
    torch.cuda.synchronize()
    _close(dq.float(), dq_r, "dq")
    _close(dk.float(), dk_r, "dk")
    _close(dv.float(), dv_r, "dv")
    # dnats sums thousands of signed terms that largely cancel (to exactly 0 when a query sees one earlier block and
    # nothing else): the error is measured against the sum of their magnitudes
    err = (dn.float().cpu().double() - dn_r).abs()
    assert bool((err <= 2e-3 * dn_mag + 1e-6).all()), f"dnats: error {float(err.max()):.3e} against a magnitude of {float(dn_mag.max()):.3e}"
    lin = torch.round(ty[..., 0].float()) == 0
    if not dnats_invalid:
        assert float(dn.float().cpu()[lin].abs().max() if lin.any() else 0.0) == 0.0, "blocks not typed attention get no gradient"


@pytest.mark.parametrize("same_block", [True, False])
@pytest.mark.parametrize("K,V", [(128, 128), (64, 64), (64, 128), (128, 64)])
def test_softmax_bwd_small(K, V, same_block):
    _run(2, 512, 4, 4, 4, K, V, 64, 0.4, same_block, seed=0)


def test_softmax_bwd_gqa_and_selector_groups():
    _run(1, 768, 8, 4, 2, 128, 128, 64, 0.5, True, seed=3)
    _run(1, 512, 8, 2, 8, 64, 64, 64, 0.5, True, seed=4)       # more selector heads than kv heads


def test_softmax_bwd_ragged_length():
    _run(2, 600, 2, 2, 2, 128, 128, 64, 0.5, True, seed=5)
    _run(1, 100, 2, 2, 2, 64, 64, 64, 0.5, True, seed=6)


@pytest.mark.parametrize("block", [128, 256])
def test_softmax_bwd_large_blocks(block):
    _run(1, 1024, 2, 2, 2, 128, 64, block, 0.5, True, seed=7)
    _run(1, 1024, 2, 2, 2, 128, 64, block, 0.5, False, seed=8)


def test_softmax_bwd_all_attention_and_all_linear():
    _run(1, 512, 2, 2, 2, 128, 128, 64, 1.0, True, seed=9)
    _run(1, 512, 2, 2, 2, 128, 128, 64, 0.0, True, seed=10)


def test_softmax_bwd_through_autograd():
    _run(2, 384, 4, 2, 2, 128, 128, 64, 0.5, True, seed=11, through_autograd=True)


def test_softmax_bwd_many_pairs_and_long_walks():
    """More (sequence, kv head) pairs than XCDs and walks of tens of query tiles: the dk/dv kernel's ring of tiles in its
    steady state, several pairs per XCD; then grouped query heads (the ring restarts for every head of the group)."""
    _run(2, 2048, 16, 16, 16, 128, 128, 64, 0.3, True, seed=20)
    _run(2, 1024, 16, 8, 4, 64, 128, 64, 0.4, False, seed=21)
    _run(1, 1000, 8, 8, 8, 128, 64, 128, 0.5, True, seed=22)     # ragged last tile, blocks of two chunks


def test_softmax_bwd_repeatable_and_workspace_reuse():
    """The dk/dv kernel takes its units from work queues in whatever order the workgroups arrive: dq, dk, dv must not
    depend on it (bit-identical from launch to launch; dnats is summed with float atomics and may differ in the last
    bits).  The queue counters live in the caller's workspace and are reset by every call: the same buffer, dirty from
    the previous call and then filled with ones, serves the next."""
    from neuralattentionsearchlinear_amd import _capi, nats_util
    from neuralattentionsearchlinear_amd.attns import parallel_attn_nats_fwd
    B, T, HQ, H, HN, K, V, block = 2, 1536, 16, 8, 8, 128, 128, 64
    q, k, v = (t.to(DEV) for t in make_qkv(B, T, H, K, V, 31, HQ=HQ))
    do = torch.randn(B, T, HQ, V, generator=torch.Generator().manual_seed(32)).bfloat16().to(DEV)
    ty = make_types(B, T // block, HN, 0.4, 33, torch.bfloat16).to(DEV)
    scale = K ** -0.5
    r = nats_util.route(ty, T, block)
    o, lse, _ = parallel_attn_nats_fwd(q, k, v, ty, r['nats_block_indices'], None, scale, block,
                                       compute_incomplete_chunk_scores=True, n_nats_blocks=r['n_nats_blocks'])
    L = _capi.lib()
    ws_bytes = L.natsl_softmax_bwd_workspace_bytes(B, T, HQ)
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device=DEV)
    outs = []
    for rep in range(3):
        dq, dk, dv = torch.empty_like(q), torch.empty_like(k), torch.empty_like(v)
        dn = torch.zeros(B, T // block, HQ, dtype=torch.float32, device=DEV)
        if rep == 2:
            ws.fill_(1)
        rc = L.natsl_softmax_sparse_bwd(
            _capi.ptr(q), _capi.ptr(k), _capi.ptr(v), _capi.ptr(o), _capi.ptr(lse), _capi.ptr(do), _capi.ptr(dq), _capi.ptr(dk),
            _capi.ptr(dv), _capi.ptr(dn), _capi.ptr(ty), _capi.dtype_code(ty.dtype), _capi.ptr(r['nats_block_indices']),
            _capi.ptr(r['n_nats_blocks']), B, T, HQ, H, HN, K, V, T // block, block, float(scale), 1, _capi.dtype_code(q.dtype),
            _capi.ptr(ws), ws_bytes, None, 0, 0, 0, _capi.stream_ptr(q.device))
        _capi.check(rc, "natsl_softmax_sparse_bwd")
        torch.cuda.synchronize()
        outs.append((dq, dk, dv, dn))
    for rep in (1, 2):
        for name, a, b in zip(("dq", "dk", "dv"), outs[0], outs[rep]):
            assert torch.equal(a, b), f"{name} differs between launches 0 and {rep}"
        assert float((outs[0][3] - outs[rep][3]).abs().max()) <= 1e-3 * float(outs[0][3].abs().max() + 1.0)


@pytest.mark.parametrize("same_block", [True, False])
@pytest.mark.parametrize("K,V", [(128, 128), (64, 128)])
def test_softmax_bwd_dnats_of_blocks_that_are_not_attention(K, V, same_block):
    """compute_dnats_for_invalid_blocks_attn=True: every block gets a selector gradient; dq, dk, dv are unchanged."""
    _run(2, 512, 4, 4, 4, K, V, 64, 0.4, same_block, seed=20, dnats_invalid=True)


def test_softmax_bwd_dnats_of_blocks_that_are_not_attention_other_shapes():
    _run(1, 768, 8, 4, 2, 128, 128, 128, 0.5, True, seed=21, dnats_invalid=True)          # grouped heads, two chunks per block
    _run(2, 600, 2, 2, 2, 64, 64, 64, 0.3, True, seed=22, dnats_invalid=True)             # ragged
    _run(1, 512, 2, 2, 2, 128, 128, 64, 0.0, True, seed=23, dnats_invalid=True)           # nothing typed attention
    _run(2, 512, 4, 4, 4, 128, 128, 64, 0.4, True, seed=24, through_autograd=True, dnats_invalid=True)


@pytest.mark.parametrize("dnats_invalid", [False, True])
@pytest.mark.parametrize("lens,HQ,H,HN,K,V,block", [
    ([200, 64, 1000, 333, 3], 8, 2, 4, 128, 128, 64),      # ragged lengths, a three-token sequence, grouped heads
    ([512, 300, 129], 4, 4, 4, 64, 128, 128),              # lengths around the 128-query tile of the dq kernel
    ([2048, 1536], 16, 16, 16, 128, 64, 256),
])
def test_softmax_backward_packed_sequences(lens, HQ, H, HN, K, V, block, dnats_invalid):
    """Packed sequences (cu_seqlens): every sequence's gradients equal the oracle's on that sequence alone."""
    from neuralattentionsearchlinear_amd import nats_util
    from neuralattentionsearchlinear_amd.attns import parallel_nats_attn
    T = sum(lens)
    cu = [0]
    for n in lens:
        cu.append(cu[-1] + n)
    q, k, v = make_qkv(1, T, H, K, V, 41, HQ=HQ)
    do = torch.randn(1, T, HQ, V, generator=torch.Generator().manual_seed(48)).bfloat16()
    TN = sum(-(-n // block) for n in lens)
    ty = make_types(1, TN, HN, 0.4, 42, torch.bfloat16)
    scale = K ** -0.5
    qd, kd, vd, dod, tyd = (t.to(DEV) for t in (q, k, v, do, ty))
    seqs = nats_util.pack_sequences(cu, None, block, DEV)
    r = nats_util.route(tyd, T, block, seqs=seqs)
    qd, kd, vd, tyd = (t.requires_grad_() for t in (qd, kd, vd, tyd))
    o, _ = parallel_nats_attn(qd, kd, vd, None, tyd, r['nats_block_indices'], r['n_nats_blocks'], scale,
                              cu_seqlens=torch.tensor(cu, dtype=torch.int32), NAtS_block_size=block,
                              compute_incomplete_chunk_scores=True, compute_dnats_for_invalid_blocks_attn=dnats_invalid)
    o.backward(dod)
    torch.cuda.synchronize()
    nb = 0
    for i, n in enumerate(lens):
        a, b, nbi = cu[i], cu[i + 1], -(-n // block)
        tyi = ty[:, nb:nb + nbi]
        dq_r, dk_r, dv_r, dn_r, dn_mag = sb.softmax_branch_bwd(q[:, a:b], k[:, a:b], v[:, a:b], tyi, do[:, a:b], scale, block, True,
                                                               with_magnitude=True, dnats_invalid=dnats_invalid)
        _close(qd.grad[:, a:b].float(), dq_r, f"dq of sequence {i}")
        _close(kd.grad[:, a:b].float(), dk_r, f"dk of sequence {i}")
        _close(vd.grad[:, a:b].float(), dv_r, f"dv of sequence {i}")
        err = (tyd.grad[:, nb:nb + nbi, :, 0].float().cpu().double() - dn_r).abs()
        assert bool((err <= 2e-3 * dn_mag + 1e-6).all()), f"dnats of sequence {i}: error {float(err.max()):.3e}"
        nb += nbi
