"""GPU parity of the persistent softmax kernel (whole 256-query tiles, at least two per CU): against the oracle,
bit for bit against the per-tile kernel (same chunk order, same arithmetic), and its work queues across launches."""
import os

import pytest
import torch

from oracle import softmax_branch as sb
from tests._util import assert_close, make_qkv, make_types

pytestmark = pytest.mark.gpu


def _inputs(B, T, HQ, H, HN, K, V, block, p_attn, seed, dev):
    q, k, v = make_qkv(B, T, H, K, V, seed, HQ=HQ)
    ty = make_types(B, -(-T // block), HN, p_attn, seed + 1, torch.bfloat16)
    return q, k, v, ty, q.to(dev), k.to(dev), v.to(dev), ty.to(dev)


def _call(qd, kd, vd, tyd, K, block, same_block, persistent=True):
    from neuralattentionsearchlinear_amd import nats_util
    from neuralattentionsearchlinear_amd.attns import parallel_attn_nats_fwd
    r = nats_util.route(tyd, qd.shape[1], block)
    old = os.environ.pop("NATSL_SOFTMAX_NO_STREAM", None)
    if not persistent:
        os.environ["NATSL_SOFTMAX_NO_STREAM"] = "1"
    try:
        o, lse, _ = parallel_attn_nats_fwd(qd, kd, vd, tyd, r['nats_block_indices'], None, K ** -0.5, block,
                                           compute_incomplete_chunk_scores=same_block, n_nats_blocks=r['n_nats_blocks'])
    finally:
        os.environ.pop("NATSL_SOFTMAX_NO_STREAM", None)
        if old is not None:
            os.environ["NATSL_SOFTMAX_NO_STREAM"] = old
    return o, lse


def _enough_tiles(B, HQ, T):
    cus = torch.cuda.get_device_properties(0).multi_processor_count
    return T % 256 == 0 and B * HQ * (T // 256) >= 2 * cus


@pytest.mark.parametrize("same_block", [True, False])
@pytest.mark.parametrize("K,V", [(128, 128), (64, 64), (64, 128), (128, 64)])
def test_persistent_kernel_against_the_oracle(K, V, same_block):
    B, T, HQ, H, HN, block = 4, 2048, 16, 4, 8, 64
    dev = torch.device('cuda:0')
    assert _enough_tiles(B, HQ, T), "shape does not reach the persistent kernel on this GPU"
    q, k, v, ty, qd, kd, vd, tyd = _inputs(B, T, HQ, H, HN, K, V, block, 0.3, 11, dev)
    o_ref, lse_ref = sb.softmax_branch(q, k, v, ty, K ** -0.5, block, same_block)
    o, lse = _call(qd, kd, vd, tyd, K, block, same_block)
    torch.cuda.synchronize()
    assert_close(o.float(), o_ref, "o_attn")
    assert_close(lse, lse_ref, "lse")


@pytest.mark.parametrize("B,T,HQ,H,HN,K,V,block,p_attn,same_block", [
    (8, 8192, 16, 16, 16, 128, 128, 64, 0.25, True),     # the benchmark shape
    (2, 8192, 16, 4, 8, 128, 128, 128, 0.3, True),       # grouped kv heads and selector heads
    (4, 4096, 32, 32, 32, 64, 64, 256, 0.5, False),      # only earlier attention blocks visible
    (3, 2048, 24, 8, 24, 64, 128, 512, 0.4, True),       # blocks larger than a tile, head count not a multiple of 8
    (2, 4096, 16, 16, 16, 128, 64, 2048, 0.5, True),     # 32 chunks from the block start
    (8, 4096, 16, 16, 16, 128, 128, 64, 1.0, True),      # dense causal
    (8, 4096, 16, 16, 16, 128, 128, 64, 0.0, True),      # nothing but the own block
    (8, 4096, 16, 16, 16, 128, 128, 64, 0.0, False),     # nothing visible at all
    (1, 65536, 8, 8, 8, 128, 128, 64, 0.1, True),        # longest admitted sequence: 1024 blocks in the list
])
def test_persistent_kernel_equals_the_per_tile_kernel(B, T, HQ, H, HN, K, V, block, p_attn, same_block):
    dev = torch.device('cuda:0')
    assert _enough_tiles(B, HQ, T), "shape does not reach the persistent kernel on this GPU"
    _, _, _, _, qd, kd, vd, tyd = _inputs(B, T, HQ, H, HN, K, V, block, p_attn, 23, dev)
    o1, l1 = _call(qd, kd, vd, tyd, K, block, same_block, persistent=False)
    o2, l2 = _call(qd, kd, vd, tyd, K, block, same_block, persistent=True)
    torch.cuda.synchronize()
    assert torch.equal(o1, o2)
    assert torch.equal(l1, l2)


def test_persistent_kernel_queues_across_launches_and_streams():
    """The ticket counters are shared device state: set back by every launch, one slot per launch in rotation."""
    B, T, HQ, H, HN, K, V, block = 4, 4096, 16, 16, 16, 128, 128, 64
    dev = torch.device('cuda:0')
    assert _enough_tiles(B, HQ, T)
    _, _, _, _, qd, kd, vd, tyd = _inputs(B, T, HQ, H, HN, K, V, block, 0.25, 5, dev)
    _, _, _, _, qe, ke, ve, tye = _inputs(B, T, HQ, H, HN, K, V, block, 0.5, 6, dev)
    o_ref, l_ref = _call(qd, kd, vd, tyd, K, block, True, persistent=False)
    o_ref2, l_ref2 = _call(qe, ke, ve, tye, K, block, True, persistent=False)
    torch.cuda.synchronize()
    for _ in range(70):   # more launches than there are slots
        o, l = _call(qd, kd, vd, tyd, K, block, True)
    torch.cuda.synchronize()
    assert torch.equal(o, o_ref) and torch.equal(l, l_ref)
    s1, s2 = torch.cuda.Stream(), torch.cuda.Stream()   # default priority
    s1.wait_stream(torch.cuda.current_stream())
    s2.wait_stream(torch.cuda.current_stream())
    outs = []
    for _ in range(4):
        with torch.cuda.stream(s1):
            outs.append((_call(qd, kd, vd, tyd, K, block, True), (o_ref, l_ref)))
        with torch.cuda.stream(s2):
            outs.append((_call(qe, ke, ve, tye, K, block, True), (o_ref2, l_ref2)))
    s1.synchronize()
    s2.synchronize()
    for (o, l), (orf, lrf) in outs:
        assert torch.equal(o, orf) and torch.equal(l, lrf)
