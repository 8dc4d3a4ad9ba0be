"""Pins oracle/cache.py (CPU): the incremental model against the whole-sequence definition on random splits, and
both against the invariants the reference's own cache checks state (src/nats/models/utils.py:855-1047), with the
reference's sizes and its token-index pattern (key value = token index + 1)."""
import pytest
import torch

from oracle import cache as C


def _pattern(B, T, H, D):
    return (torch.arange(T) + 1).view(1, T, 1, 1).repeat(B, 1, H, D).float()


def _types(B, NB, HN, seed):
    g = torch.Generator().manual_seed(seed)
    idx = torch.randn(B, NB, HN, 2, generator=g).max(-1, keepdim=True)[1]
    return torch.zeros(B, NB, HN, 2).scatter_(-1, idx, 1.0)


@pytest.mark.parametrize("T", [1078, 1728, 64, 63, 200])
def test_whole_sequence_layout_holds_the_reference_invariants(T):
    B, H, HN, D, bs = 4, 8, 4, 2, 64                                   # src/nats/models/utils.py:856-861
    k = _pattern(B, T, H, D)
    ty = _types(B, -(-T // bs), HN, T)
    st = C.whole_sequence(k, k.clone(), ty, bs)
    n_max = st['n_max']
    for b in range(B):
        for h1 in range(HN):
            for h2 in range(H // HN):
                h = h2 + h1 * (H // HN)
                i_cache = 0
                for j in range(T // bs):
                    if ty[b, j, h1, 0]:
                        want = k[b, j * bs:(j + 1) * bs, h, 0]
                        got = st['keys'][b, i_cache * bs:(i_cache + 1) * bs, h, 0]
                        assert torch.equal(want, got)                                       # :893-897
                        assert bool(st['valid'][b, i_cache, h1])                            # :898
                        i_cache += 1
                assert i_cache == int(st['n_attn_blocks'][b, h1])
                assert not bool(st['valid'][b, i_cache:n_max, h1].any())                    # :906-907
                tail = st['keys'][b, n_max * bs:(n_max + 1) * bs, h, 0]
                n_tail = T % bs
                assert torch.equal(tail[:n_tail], k[b, T - n_tail:, h, 0])                  # :900-901
                assert float(tail[n_tail:].abs().sum()) == 0                                # :902-903


@pytest.mark.parametrize("T1,T2,step", [(1728, 45, None), (1777, 195, 1), (1078, 300, 7), (10, 200, 64)])
def test_pieces_equal_whole(T1, T2, step):
    """One piece == two pieces == token by token (src/nats/models/utils.py:910-1047)."""
    B, H, HN, D, bs = 2, 4, 2, 2, 64
    T = T1 + T2
    k = _pattern(B, T, H, D)
    v = -k
    ty = _types(B, -(-T // bs), HN, T1)
    if T >= 30 * bs:
        ty[:, 29] = 0                                                                        # :997
    whole = C.whole_sequence(k, v, ty, bs)
    m = C.CacheModel(bs)
    t = 0
    pieces = [T1] + ([T2] if step is None else [step] * (T2 // step) + ([T2 % step] if T2 % step else []))
    for n in pieces:
        first_block = (t - t % bs) // bs
        nb = -(-(t % bs + n) // bs)
        m.feed(k[:, t:t + n], v[:, t:t + n], ty[:, first_block:first_block + nb])
        t += n
    st = m.state()
    assert st['n_max'] == whole['n_max'] and st['n_tail'] == whole['n_tail']
    assert torch.equal(st['keys'], whole['keys']) and torch.equal(st['values'], whole['values'])
    G = H // HN
    assert torch.equal(st['n_attn_blocks_per_kv_head'][:, ::G], whole['n_attn_blocks'])


def test_next_query_mask():
    B, H, HN, D, bs, T = 2, 4, 2, 2, 64, 64 * 5 + 9
    k = _pattern(B, T, H, D)
    ty = _types(B, 6, HN, 1)
    st = C.whole_sequence(k, k, ty, bs)
    m = C.next_query_mask(st, bs)
    assert m.shape == (B, HN, 1, st['n_max'] * bs + 10)
    for b in range(B):
        for hn in range(HN):
            c = int(st['n_attn_blocks'][b, hn])
            assert int(m[b, hn, 0].sum()) == c * bs + 10
            assert bool(m[b, hn, 0, :c * bs].all()) and bool(m[b, hn, 0, st['n_max'] * bs:].all())
