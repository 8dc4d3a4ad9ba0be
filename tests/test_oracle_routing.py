"""Pins the oracle's selector and routing tables (CPU only)."""
import numpy as np
import torch

from oracle import routing as R


def test_known_answer_routing():
    # hand-derived: attention column [1,0,1,1], linear column [0,1,0,1] (last block forced to both)
    types = torch.tensor([[1, 0], [0, 1], [1, 0], [1, 1]], dtype=torch.float32).view(1, 4, 1, 2)
    r = R.route(types, T=256, block=64)
    assert r['nats_block_indices'][0, :, 0, 0].tolist() == [0, 2, 3, 4]
    assert r['nats_block_indices'][0, :, 0, 1].tolist() == [1, 3, 4, 4]
    assert r['n_nats_blocks'][0, 0].tolist() == [3, 2]
    assert r['chunk_indices_linear'].tolist() == [[0, 0], [0, 1]]
    assert r['linear_chunk_offsets'].tolist() == [0, 2]
    assert r['starting_h_idx'][0, :, 0].tolist() == [0, 0, 1, 1]
    assert r['attn_n_iters'][0, :, 0].tolist() == [0, 1]


def test_reference_docstring_example():
    # src/nats/ops/nats_util.py:134: 8 chunks, linear chunks [2,5] -> by the code at :161
    types = torch.zeros(1, 8, 1, 2)
    types[0, [2, 5], 0, 1] = 1
    idx = R.block_indices(types)
    assert R.starting_h_idx(idx, 512, 64)[0, :, 0].tolist() == [0, 0, 0, 1, 1, 1, 2, 2]


def test_tables_vectorised_vs_loops():
    g = torch.Generator().manual_seed(0)
    for (B, TN, HN, block) in [(2, 8, 3, 64), (1, 16, 2, 64), (3, 6, 1, 128), (2, 4, 2, 256)]:
        types = (torch.rand(B, TN, HN, 2, generator=g) < 0.5).float()
        types = R.force_last_block(types)
        T = TN * block
        idx = R.block_indices(types)
        assert torch.equal(idx, R.block_indices_loop(types))
        assert torch.equal(R.starting_h_idx(idx, T, block), R.starting_h_idx_loop(types, T, block))
        assert torch.equal(R.attn_n_iters(idx, T, block), R.attn_n_iters_loop(types, T, block))
        nb = R.n_blocks(types)
        assert torch.equal(nb.long(), types.long().sum(1))
        off = R.linear_chunk_offsets(nb[..., 1], block)
        ci = R.chunk_indices_linear(nb[..., 1], block)
        assert off[-1].item() == len(ci)
        # rows grouped by flat (b,hn), second column counts up from 0
        for bh in range(B * HN):
            rows = ci[off[bh]:off[bh + 1]]
            assert (rows[:, 0] == bh).all() and rows[:, 1].tolist() == list(range(len(rows)))


def test_hard_select_is_exact_one_hot():
    g = torch.Generator().manual_seed(1)
    for dt in (torch.float32, torch.bfloat16, torch.float16):
        logits = torch.randn(4, 32, 8, 2, generator=g).to(dt)
        y = R.hard_select(logits)
        assert set(np.unique(y.float().numpy()).tolist()) <= {0.0, 1.0}
        assert torch.equal(y.float().sum(-1), torch.ones(4, 32, 8))


def _bf16_neighbours(n_steps):
    """all positive normal bf16 x0 paired with x0 + j ulps, j = 0..n_steps (and the negatives)."""
    bits = torch.arange(0x0080, 0x7F00, dtype=torch.int32)          # positive normals
    pairs = []
    for j in range(0, n_steps + 1):
        hi = torch.clamp(bits + j, max=0x7F7F)
        pairs.append(torch.stack([bits, hi], -1))
    p = torch.cat(pairs, 0).to(torch.int16)
    pos = p.view(torch.bfloat16)
    return torch.cat([pos, -pos.flip(-1)], 0)                        # keep x0 <= x1 ordering for negatives too


def test_hard_select_bf16_tie_trap():
    """argmax is over the ROUNDED softmax: when both probabilities round to 0.5 the first
    index (attention) wins although logit[1] > logit[0].  The closed form of the tie set
    (exact arithmetic) is d = x1 - x0 <= ln(0.5009765625/0.4990234375) = 0.00390625508...;
    torch's fp32 softmax agrees with that threshold on every near-tie bf16 pair."""
    lg = _bf16_neighbours(6)
    y = R.hard_select(lg)
    x0, x1 = lg[:, 0].double(), lg[:, 1].double()
    d = x1 - x0
    thr = float(np.log(0.5009765625 / 0.4990234375))
    expect_attn = (d <= thr)
    assert torch.equal(y[:, 0] == 1, expect_attn)
    # the trap is real: some pairs have logit[1] > logit[0] yet select index 0
    assert int(((d > 0) & (y[:, 0] == 1)).sum()) > 0
    # symmetric direction: x0 > x1 always selects 0
    y2 = R.hard_select(lg.flip(-1))
    assert bool((y2[:, 0] == 1).all())


def test_mean_pool_divisor():
    x = torch.arange(2 * 100 * 3, dtype=torch.float32).view(2, 100, 3)
    p = R.mean_pool(x, 64)
    assert p.shape == (2, 2, 3)
    assert torch.allclose(p[:, 0], x[:, :64].mean(1))
    assert torch.allclose(p[:, 1], x[:, 64:].mean(1))       # divisor 36, not 64
