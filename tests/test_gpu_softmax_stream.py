"""GPU parity of the persistent softmax kernel (whole 256-query tiles, at least two per CU): against the oracle,
bit for bit against the per-tile kernel (same chunk order, same arithmetic), and its work queues across launches."""
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
    """The softmax branch through the C ABI: natsl_softmax_sparse_fwd (picks the persistent kernel for these shapes), or
    natsl_softmax_sparse_fwd_per_tile (one workgroup per query tile, the same results)."""
    from neuralattentionsearchlinear_amd import _capi, nats_util
    r = nats_util.route(tyd, qd.shape[1], block)
    B, T, HQ, _ = qd.shape
    H, V = kd.shape[2], vd.shape[-1]
    TN, HN = tyd.shape[1], tyd.shape[2]
    o = torch.empty(B, T, HQ, V, dtype=vd.dtype, device=qd.device)
    lse = torch.empty(B, T, HQ, dtype=torch.float32, device=qd.device)
    L = _capi.lib()
    fn = L.natsl_softmax_sparse_fwd if persistent else L.natsl_softmax_sparse_fwd_per_tile
    if persistent:
        assert L.natsl_softmax_fwd_variant(B, T, HQ, H, block, 0) == 2, "shape does not reach the persistent kernel on this GPU"
    rc = fn(_capi.ptr(qd), _capi.ptr(kd), _capi.ptr(vd), _capi.ptr(o), _capi.ptr(lse), _capi.ptr(tyd), _capi.dtype_code(tyd.dtype),
            _capi.ptr(r['nats_block_indices']), _capi.ptr(r['n_nats_blocks']), B, T, HQ, H, HN, K, V, TN, block, float(K ** -0.5),
            int(bool(same_block)), _capi.dtype_code(qd.dtype), None, 0, 0, _capi.stream_ptr(qd.device))
    _capi.check(rc, "natsl_softmax_sparse_fwd")
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
    """The ticket counters are shared device state: one slot per launch in rotation, zeroed on the launch's stream right
    before it."""
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


def test_persistent_kernel_in_a_captured_graph():
    """The launch (queue fill kernel + persistent kernel) replays from a HIP graph: every replay, with eager work and
    synchronisations between the replays, gives the eager result."""
    B, T, HQ, H, HN, K, V, block = 4, 4096, 16, 16, 16, 128, 128, 64
    dev = torch.device('cuda:0')
    assert _enough_tiles(B, HQ, T)
    _, _, _, _, qd, kd, vd, tyd = _inputs(B, T, HQ, H, HN, K, V, block, 0.25, 7, dev)
    from neuralattentionsearchlinear_amd import _capi, nats_util
    r = nats_util.route(tyd, T, block)
    o_ref, l_ref = _call(qd, kd, vd, tyd, K, block, True, persistent=False)
    o = torch.empty_like(o_ref)
    lse = torch.empty_like(l_ref)
    L = _capi.lib()

    def launch():
        rc = L.natsl_softmax_sparse_fwd(_capi.ptr(qd), _capi.ptr(kd), _capi.ptr(vd), _capi.ptr(o), _capi.ptr(lse), _capi.ptr(tyd),
                                        _capi.dtype_code(tyd.dtype), _capi.ptr(r['nats_block_indices']), _capi.ptr(r['n_nats_blocks']),
                                        B, T, HQ, H, HN, K, V, tyd.shape[1], block, float(K ** -0.5), 1, _capi.dtype_code(qd.dtype),
                                        None, 0, 0, _capi.stream_ptr(dev))
        _capi.check(rc, "natsl_softmax_sparse_fwd")

    launch()   # first use on the device outside the capture
    torch.cuda.synchronize()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g):
        launch()
    for i in range(4):
        o.fill_(float('nan'))
        lse.fill_(float('nan'))
        g.replay()
        torch.cuda.synchronize()
        assert torch.equal(o, o_ref) and torch.equal(lse, l_ref), f"replay {i}"
        if i & 1:
            _call(qd, kd, vd, tyd, K, block, True)   # an eager launch between replays, on the same stream
            torch.cuda.synchronize()
