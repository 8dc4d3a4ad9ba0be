"""GPU parity (bit-exact): selector, pooling and routing tables through the C ABI vs the oracle."""
import pytest
import torch

from oracle import routing as R
from tests._util import make_types
from tests.test_oracle_routing import _bf16_neighbours

pytestmark = pytest.mark.gpu


def _dev():
    return torch.device('cuda:0')


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_hard_select_random(dtype):
    from neuralattentionsearchlinear_amd import nats_util
    g = torch.Generator().manual_seed(0)
    logits = torch.randn(8, 128, 16, 2, generator=g).to(dtype)
    ref = R.hard_select(logits)
    ty, nb = nats_util.hard_select(logits.to(_dev()))
    assert torch.equal(ty.cpu(), ref)
    assert torch.equal(nb.cpu(), R.n_blocks(ref))
    ty2, nb2 = nats_util.hard_select(logits.to(_dev()), force_last_block=True)
    ref2 = R.force_last_block(ref)
    assert torch.equal(ty2.cpu(), ref2)
    assert torch.equal(nb2.cpu(), R.n_blocks(ref2))


def test_hard_select_bf16_near_ties_exhaustive():
    """every positive/negative normal bf16 paired with its 0..6-ulp neighbours, both orders"""
    from neuralattentionsearchlinear_amd import nats_util
    lg = _bf16_neighbours(6)
    lg = torch.cat([lg, lg.flip(-1)], 0)
    n = lg.shape[0]
    ref = R.hard_select(lg)
    ty, _ = nats_util.hard_select(lg.view(1, n, 1, 2).to(_dev()))
    assert torch.equal(ty.cpu().view(n, 2), ref)


def test_hard_select_fp32_near_ties():
    from neuralattentionsearchlinear_amd import nats_util
    g = torch.Generator().manual_seed(1)
    x0 = torch.randn(200000, generator=g)
    ulps = torch.randint(-3, 4, (200000,), generator=g)
    x1 = (x0.view(torch.int32) + ulps.int()).view(torch.float32)
    lg = torch.stack([x0, x1], -1)
    ref = R.hard_select(lg)
    ty, _ = nats_util.hard_select(lg.view(1, -1, 1, 2).to(_dev()))
    assert torch.equal(ty.cpu().view(-1, 2), ref)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("B,T,D,block", [(2, 512, 256, 64), (3, 200, 96, 64), (1, 1000, 130, 256)])
def test_mean_pool(B, T, D, block, dtype):
    from neuralattentionsearchlinear_amd import nats_util
    g = torch.Generator().manual_seed(2)
    x = torch.randn(B, T, D, generator=g).to(dtype)
    ref = R.mean_pool(x, block)
    out = nats_util.mean_pooling(x.to(_dev()), block)
    # sums of <=256 values in fp32: the summation order may differ, so allow 1 ulp of the output dtype
    tol = 2 ** -7 if dtype == torch.bfloat16 else 1e-6
    assert float((out.cpu().float() - ref.float()).abs().max()) <= tol * float(ref.float().abs().max())


@pytest.mark.parametrize("B,TN,HN,block,p", [(1, 4, 1, 64, 0.5), (8, 128, 16, 64, 0.25), (2, 1024, 4, 64, 0.1), (3, 33, 5, 256, 0.6), (2, 16, 2, 128, 0.0), (2, 16, 2, 64, 1.0)])
def test_route_tables(B, TN, HN, block, p):
    from neuralattentionsearchlinear_amd import nats_util
    T = TN * block
    for dtype in (torch.bfloat16, torch.float32):
        ty = make_types(B, TN, HN, p, seed=TN + HN, dtype=dtype)
        ref = R.route(ty, T, block)
        got = nats_util.route(ty.to(_dev()), T, block, tables=True)
        torch.cuda.synchronize()
        assert torch.equal(got['nats_block_indices'].cpu(), ref['nats_block_indices'])
        assert torch.equal(got['n_nats_blocks'].cpu(), ref['n_nats_blocks'])
        assert torch.equal(got['linear_chunk_offsets'].cpu(), ref['linear_chunk_offsets'])
        n = int(ref['linear_chunk_offsets'][-1])
        assert torch.equal(got['chunk_indices_linear_buffer'][:n].cpu(), ref['chunk_indices_linear'])
        assert torch.equal(got['starting_h_idx'].cpu(), ref['starting_h_idx'])
        assert torch.equal(got['attn_n_iters'].cpu(), ref['attn_n_iters'])
        # the torch re-statements of the two host helpers agree too
        ci = nats_util.prepare_nats_block_indices(got['n_nats_blocks'][..., 1], block, 64)
        assert torch.equal(ci.cpu().int(), ref['chunk_indices_linear'])
        off = nats_util.prepare_nats_chunk_offsets(got['n_nats_blocks'], None, block, 64, 1)
        assert torch.equal(off.cpu(), ref['linear_chunk_offsets'])


def test_route_known_answer():
    from neuralattentionsearchlinear_amd import nats_util
    types = torch.tensor([[1, 0], [0, 1], [1, 0], [1, 1]], dtype=torch.float32).view(1, 4, 1, 2)
    got = nats_util.route(types.to(_dev()), 256, 64, tables=True)
    assert got['nats_block_indices'][0, :, 0, 0].tolist() == [0, 2, 3, 4]
    assert got['nats_block_indices'][0, :, 0, 1].tolist() == [1, 3, 4, 4]
    assert got['n_nats_blocks'][0, 0].tolist() == [3, 2]
    assert got['linear_chunk_offsets'].tolist() == [0, 2]
    assert got['starting_h_idx'][0, :, 0].tolist() == [0, 0, 1, 1]
    assert got['attn_n_iters'][0, :, 0].tolist() == [0, 1]
