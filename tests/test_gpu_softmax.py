"""GPU parity: softmax branch through the C ABI vs the oracle."""
import pytest
import torch

from oracle import routing as R
from oracle import softmax_branch as sb
from tests._util import assert_close, make_qkv, make_types

pytestmark = pytest.mark.gpu


def _run(B, T, HQ, H, HN, K, V, block, p_attn, same_block, seed):
    from neuralattentionsearchlinear_amd import nats_util
    from neuralattentionsearchlinear_amd.attns import parallel_attn_nats_fwd
    dev = torch.device('cuda:0')
    q, k, v = make_qkv(B, T, H, K, V, seed, HQ=HQ)
    NB = -(-T // block)
    ty = make_types(B, NB, HN, p_attn, seed + 1, torch.bfloat16)
    scale = K ** -0.5
    o_ref, lse_ref = sb.softmax_branch(q, k, v, ty, scale, block, same_block)
    tyd = ty.to(dev)
    r = nats_util.route(tyd, T, block)
    assert torch.equal(r['nats_block_indices'].cpu(), R.block_indices(ty))
    o, lse, _ = parallel_attn_nats_fwd(q.to(dev), k.to(dev), v.to(dev), tyd, r['nats_block_indices'], None, scale, block,
                                       compute_incomplete_chunk_scores=same_block, n_nats_blocks=r['n_nats_blocks'])
    torch.cuda.synchronize()
    assert_close(o.float(), o_ref, "o_attn")
    assert_close(lse, lse_ref, "lse")


@pytest.mark.parametrize("same_block", [True, False])
@pytest.mark.parametrize("K,V", [(128, 128), (64, 64), (64, 128), (128, 64)])
def test_softmax_small(K, V, same_block):
    _run(2, 512, 4, 4, 4, K, V, 64, 0.4, same_block, seed=0)


def test_softmax_gqa_and_selector_groups():
    _run(1, 768, 8, 4, 2, 128, 128, 64, 0.5, True, seed=3)


def test_softmax_ragged_length():
    _run(2, 600, 2, 2, 2, 128, 128, 64, 0.5, True, seed=5)
    _run(1, 100, 2, 2, 2, 64, 64, 64, 0.5, True, seed=6)


@pytest.mark.parametrize("block", [128, 256, 512])
def test_softmax_large_blocks(block):
    _run(1, 1024, 2, 2, 2, 128, 64, block, 0.5, True, seed=7)
    _run(1, 1024, 2, 2, 2, 128, 64, block, 0.5, False, seed=8)


def test_softmax_all_attention_and_all_linear():
    _run(1, 512, 2, 2, 2, 128, 128, 64, 1.0, True, seed=9)
    _run(1, 512, 2, 2, 2, 128, 128, 64, 0.0, True, seed=10)
    _run(1, 512, 2, 2, 2, 128, 128, 64, 0.0, False, seed=11)


# ---- the 256-query tile on 8 waves: chosen once B*HQ*ceil(T/256) >= 256, which the cases above never reach ----
@pytest.mark.parametrize("same_block", [True, False])
@pytest.mark.parametrize("K,V", [(128, 128), (64, 64), (64, 128), (128, 64)])
def test_softmax_wide_tiles(K, V, same_block):
    _run(4, 1024, 32, 32, 32, K, V, 64, 0.3, same_block, seed=20)


def test_softmax_wide_tiles_gqa_ragged_and_dense():
    _run(4, 1024, 32, 8, 4, 128, 128, 64, 0.5, True, seed=21)      # grouped kv heads and selector heads
    _run(4, 1000, 32, 32, 32, 128, 128, 64, 0.4, True, seed=22)    # the last tile of every sequence is ragged
    _run(8, 300, 32, 32, 32, 128, 64, 64, 0.4, False, seed=23)     # ... and cut below 256 queries
    _run(4, 1024, 32, 32, 32, 128, 128, 64, 1.0, True, seed=24)    # every block attention-typed: the longest chunk loops
    _run(4, 1024, 32, 32, 32, 128, 128, 64, 0.0, True, seed=25)    # none: only the tile's own chunks


@pytest.mark.parametrize("block", [128, 256, 512])
def test_softmax_wide_tiles_large_blocks(block):
    _run(4, 1024, 32, 32, 32, 128, 64, block, 0.5, True, seed=26)
    _run(4, 1024, 32, 32, 32, 128, 64, block, 0.5, False, seed=27)


@pytest.mark.parametrize("T", [64, 128, 192, 256, 320, 576])
def test_softmax_wide_tiles_short_sequences(T):
    """8-wave shape on sequences of one to three tiles: fewer chunks than the staging rings hold, waves with no query
    at all (T < 256), a full tile followed by a ragged one (320, 576)."""
    _run(16, T, 32, 32, 32, 128, 128, 64, 0.5, True, seed=40 + T)
    _run(16, T, 32, 16, 8, 64, 128, 64, 0.5, False, seed=41 + T)


def test_softmax_wide_tiles_block_of_three_chunks():
    """Selector blocks of 192 tokens: blocks do not line up with the 256-query tiles and hold an odd number of chunks."""
    _run(4, 1536, 32, 32, 32, 128, 128, 192, 0.5, True, seed=50)
    _run(4, 1536, 32, 8, 8, 128, 64, 192, 0.5, False, seed=51)


def test_softmax_wide_tiles_packed():
    """Packed sequences on the 8-wave shape: every sequence attends within itself; sequence ends fall inside tiles."""
    from neuralattentionsearchlinear_amd import nats_util
    from neuralattentionsearchlinear_amd.attns import parallel_attn_nats_fwd
    dev = torch.device('cuda:0')
    cu, HQ, K, V, block = [0, 1000, 2500, 4096], 32, 128, 128, 64
    T = cu[-1]
    q, k, v = make_qkv(1, T, HQ, K, V, 30, HQ=HQ)
    parts = [make_types(1, -(-(b - a) // block), HQ, 0.4, 31 + i, torch.bfloat16) for i, (a, b) in enumerate(zip(cu[:-1], cu[1:]))]
    ty = torch.cat(parts, 1)
    scale = K ** -0.5
    refs = [sb.softmax_branch(q[:, a:b], k[:, a:b], v[:, a:b], t, scale, block, True) for (a, b), t in zip(zip(cu[:-1], cu[1:]), parts)]
    o_ref, lse_ref = torch.cat([r[0] for r in refs], 1), torch.cat([r[1] for r in refs], 1)
    seqs = nats_util.pack_sequences(cu, None, block, dev)
    tyd = ty.to(dev)
    r = nats_util.route(tyd, T, block, seqs=seqs)
    o, lse, _ = parallel_attn_nats_fwd(q.to(dev), k.to(dev), v.to(dev), tyd, r['nats_block_indices'], None, scale, block,
                                       compute_incomplete_chunk_scores=True, n_nats_blocks=r['n_nats_blocks'], seqs=seqs)
    torch.cuda.synchronize()
    assert_close(o.float(), o_ref, "o_attn")
    assert_close(lse, lse_ref, "lse")
