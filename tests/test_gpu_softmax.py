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
