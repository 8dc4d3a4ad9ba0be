"""GPU parity of the K/V cache (natsl_kv_compact behind NAtSLayerCache) against oracle/cache.py, bit-exact, and
of generation through the hybrid layers (one prefill, then decode steps) against the same layer's forward
over the whole sequence."""
import pytest
import torch

from oracle import cache as C
from tests.test_gpu_layers import _layer_case
from tests._util import max_abs, rel_l2

pytestmark = pytest.mark.gpu
DEV = 'cuda:0'


def _types(B, NB, HN, seed, p_attn=0.5, dtype=torch.float32):
    g = torch.Generator().manual_seed(seed)
    a = (torch.rand(B, NB, HN, generator=g) < p_attn).float()
    return torch.stack([a, 1 - a], -1).to(dtype)


def _feed(cache, k, v, ty, pieces, bs):
    """Drive the cache the way the layers do: update_attn_cache, (the operators), update."""
    t = 0
    views = []
    for n in pieces:
        first_block = (t - t % bs) // bs
        total = t % bs + n
        types = ty[:, first_block:first_block + -(-total // bs)] if total >= bs else torch.ones_like(ty[:, :1])
        kk, vv = k[:, t:t + n].contiguous(), v[:, t:t + n].contiguous()
        views.append(cache.update_attn_cache((kk, vv), types))
        cache.update(attn_state=(kk, vv), nats_block_types=types, n_new_tokens=n)
        t += n
    return views


def _check(cache, want, bs, G, zero_tail=True):
    nmax = want['n_max']
    assert cache.n_attn_blocks_max == nmax and cache._n_tokens_in_nats_block == want['n_tail']
    assert cache.n_attn_tokens_max == nmax * bs + want['n_tail']
    assert torch.equal(cache.n_attn_blocks.cpu(), want['n_attn_blocks'])
    valid = cache.valid_attn_tokens.cpu()
    assert torch.equal(valid[:, :nmax + 1], want['valid']) and not bool(valid[:, nmax + 1:].any())
    # only what the validity flags expose is compared: dropped blocks may leave stale tokens behind
    vis = want['valid'].repeat_interleave(bs, 1).repeat_interleave(G, 2)                         # [B, tokens, HKV]
    if not zero_tail:
        vis[:, nmax * bs + want['n_tail']:] = False            # decode steps reuse dropped blocks' memory for the incomplete block
    for got, ref in ((cache.attn_k, want['keys']), (cache.attn_v, want['values'])):
        got = got[:, :(nmax + 1) * bs].cpu()
        assert torch.equal(got * vis.unsqueeze(-1), ref * vis.unsqueeze(-1))
    if want['n_tail'] and zero_tail:
        tail = cache.attn_k[:, nmax * bs + want['n_tail']:(nmax + 1) * bs]
        assert float(tail.float().abs().sum()) == 0, "the incomplete block must be zero padded"


@pytest.mark.parametrize("dtype,tdtype", [(torch.bfloat16, torch.bfloat16), (torch.float32, torch.float32), (torch.bfloat16, torch.float32)])
@pytest.mark.parametrize("T,K,V,HKV,HN,bs", [(1078, 64, 128, 8, 4, 64), (1728, 128, 128, 4, 4, 64), (64, 64, 64, 2, 1, 64),
                                             (40, 64, 64, 2, 2, 64), (1100, 128, 64, 4, 2, 256), (640, 256, 512, 2, 2, 64)])
def test_prefill_compaction(T, K, V, HKV, HN, bs, dtype, tdtype):
    from neuralattentionsearchlinear_amd.cache import NAtSLayerCache
    B = 3
    g = torch.Generator().manual_seed(T + K)
    k, v = torch.randn(B, T, HKV, K, generator=g).to(dtype), torch.randn(B, T, HKV, V, generator=g).to(dtype)
    ty = _types(B, -(-T // bs), HN, T, dtype=tdtype)
    cache = NAtSLayerCache(nats_block_size=bs, op_for_incomplete_chunk='all')
    (kv, vv), = _feed(cache, k.to(DEV), v.to(DEV), ty.to(DEV), [T], bs)
    assert kv.shape[1] == T                                             # the first forward attends to its own keys
    _check(cache, C.whole_sequence(k, v, ty.float(), bs), bs, HKV // HN)
    assert cache.attn_k.shape[1] <= (int(cache.n_attn_blocks_max) + 2) * bs, "the cache must not keep the dropped blocks"


@pytest.mark.parametrize("T1,T2,step", [(1728, 45, 1), (1777, 195, 1), (1078, 130, 7), (10, 200, 1), (0, 150, 3), (640, 640, 63)])
def test_pieces_equal_whole(T1, T2, step):
    """One prefill and then decode steps reach the cache of the whole sequence
    (the reference states this at src/nats/models/utils.py:910-1047)."""
    from neuralattentionsearchlinear_amd.cache import NAtSLayerCache
    B, HKV, HN, K, V, bs = 2, 4, 2, 64, 128, 64
    T = T1 + T2
    g = torch.Generator().manual_seed(T)
    k, v = torch.randn(B, T, HKV, K, generator=g).bfloat16(), torch.randn(B, T, HKV, V, generator=g).bfloat16()
    ty = _types(B, -(-T // bs), HN, T1 + 1, dtype=torch.bfloat16)
    if T >= 30 * bs:
        ty[:, 29, :, 0] = 0                                             # as the reference's check does (:997)
    pieces, t = ([T1] if T1 else []), T1
    while t < T:                                                        # decode steps never cross a block boundary
        n = min(step, T - t, bs - t % bs)
        pieces.append(n); t += n
    cache = NAtSLayerCache(nats_block_size=bs, op_for_incomplete_chunk='all')
    kd, vd = k.to(DEV), v.to(DEV)
    views = _feed(cache, kd, vd, ty.to(DEV), pieces, bs)
    want = C.whole_sequence(k, v, ty.float(), bs)
    _check(cache, want, bs, HKV // HN, zero_tail=False)
    # what the last step's attention saw: the kept blocks, the incomplete block and its own token(s)
    kv, _ = views[-1]
    before = C.whole_sequence(k[:, :T - pieces[-1]], v[:, :T - pieces[-1]], ty[:, :-(-(T - pieces[-1]) // bs) or 1].float(), bs) \
        if T - pieces[-1] > 0 else None
    if before is not None and len(pieces) > 1:
        assert kv.shape[1] == before['n_max'] * bs + before['n_tail'] + pieces[-1]
        assert torch.equal(kv[:, -pieces[-1]:].cpu(), k[:, T - pieces[-1]:])


def test_mask_of_the_next_token():
    from neuralattentionsearchlinear_amd.cache import NAtSLayerCache
    B, HKV, HN, K, bs, T = 2, 4, 2, 64, 64, 64 * 6 + 9
    g = torch.Generator().manual_seed(9)
    k = torch.randn(B, T + 3, HKV, K, generator=g).bfloat16()
    ty = _types(B, 7, HN, 2)
    cache = NAtSLayerCache(nats_block_size=bs, op_for_incomplete_chunk='all')
    kd = k.to(DEV)
    _feed(cache, kd[:, :T], kd[:, :T], ty.to(DEV), [T], bs)
    want = C.whole_sequence(k[:, :T], k[:, :T], ty, bs)
    one = torch.ones(B, 1, HN, 2, device=DEV)
    kv, _ = cache.update_attn_cache((kd[:, T:T + 1].contiguous(), kd[:, T:T + 1].contiguous()), one)
    m = cache.generate_msk(1, one, True)
    assert m.dtype == torch.bool and m.shape[-1] == kv.shape[1]
    assert torch.equal(m.cpu(), C.next_query_mask(want, bs))
    cache.update(attn_state=(kd[:, T:T + 1], kd[:, T:T + 1]), nats_block_types=one, n_new_tokens=1)
    # three tokens at once, still inside the block: kept blocks, then causal inside the block
    kv, _ = cache.update_attn_cache((kd[:, T + 1:T + 3].contiguous(), kd[:, T + 1:T + 3].contiguous()), one)
    m = cache.generate_msk(2, one, True).cpu()
    assert m.shape == (B, HN, 2, kv.shape[1])
    base = C.next_query_mask(want, bs)[:, :, 0]                           # columns up to token T included
    assert torch.equal(m[:, :, 0, :-1], torch.cat([base, torch.ones(B, HN, 1, dtype=torch.bool)], -1))
    assert not bool(m[:, :, 0, -1].any()) and bool(m[:, :, 1, -2:].all())


@pytest.mark.parametrize("kind,T0,T,geometry,ops", [(k_, a, b, None, 'all') for k_ in ('gdn', 'mamba') for a, b in ((320, 420), (266, 400), (64, 130))]
                         + [('gdn', 200, 270, '760M', 'all'), ('gdn', 30, 140, None, 'all')]
                         # the mode in which the linear operator skips the incomplete block: its tokens read the state that
                         # entered the block, and the state advances when the block is complete
                         + [(k_, a, b, None, 'attn') for k_ in ('gdn', 'mamba') for a, b in ((320, 420), (266, 400), (30, 140))]
                         # the mode in which the softmax operator skips the incomplete block
                         + [('gdn', 266, 400, None, 'gated_delta_net'), ('mamba', 30, 140, None, 'mamba')])
def test_layer_generation_matches_whole_forward(kind, T0, T, geometry, ops):
    """Prefill T0 tokens with a cache, decode up to T token by token (two tokens at a time where the block allows
    it): every output must match the layer's forward over the first T0 tokens resp. the whole sequence at the same
    positions; the selector decisions of the two runs must be identical."""
    from neuralattentionsearchlinear_amd.cache import NAtSCache, NAtSMamba2Cache
    layer, cfg, w, _ = _layer_case(kind, geometry, ops)
    layer.layer_idx = 0
    layer = layer.to(DEV).to(torch.bfloat16).eval()
    bs = layer.nats_block_size
    torch.manual_seed(T)
    x = torch.randn(2, T, cfg['hidden_size']).to(DEV).to(torch.bfloat16)
    first = lambda out: out[0] if isinstance(out, tuple) else out
    with torch.no_grad():
        whole = first(layer(x))
        types_whole, _, _ = layer.select_ops(x, force_last_block=False)
        holder = NAtSCache() if kind == 'gdn' else NAtSMamba2Cache()
        kw = dict(past_key_values=holder, use_cache=True) if kind == 'gdn' else dict(cache_params=holder, use_cache=True)
        outs = [first(layer(x[:, :T0], **kw))]
        t = T0
        while t < T:
            n = 2 if (t % bs) in (10, 20) and t + 2 <= T else 1
            outs.append(first(layer(x[:, t:t + n], **kw)))
            t += n
    cache = holder[0] if kind == 'gdn' else holder.nats_cache[0]
    # same selector decisions: the kept-block counts follow from them
    n_complete = T // bs
    want_counts = (types_whole[:, :n_complete, :, 0] == 1).sum(1)
    assert torch.equal(cache.n_attn_blocks, want_counts), "the cached run typed a block differently from the whole forward"
    assert cache.n_observed_tokens == T and cache._n_tokens_in_nats_block == T % bs
    got = torch.cat(outs, 1).float()
    # the prefill part is compared with a forward over exactly those tokens only where no later token matters:
    # a whole-sequence forward types complete blocks only, so positions in blocks completed by the prefill agree
    ma, rl = max_abs(got[:, T0:], whole[:, T0:].float()), rel_l2(got[:, T0:], whole[:, T0:].float())
    assert rl <= 2e-2, f"decoded tokens: rel-L2 {rl:.3e}, max-abs {ma:.3e}"
    rl0 = rel_l2(got[:, :T0], whole[:, :T0].float())
    assert rl0 <= 2e-2, f"prefilled tokens: rel-L2 {rl0:.3e}"


def test_single_token_steps_after_a_prefill_are_repeatable():
    from neuralattentionsearchlinear_amd.cache import NAtSCache
    layer, cfg, w, x = _layer_case('gdn')
    layer.layer_idx = 0
    layer = layer.to(DEV).to(torch.bfloat16).eval()
    xd = x.to(DEV).bfloat16()
    cache = NAtSCache()
    with torch.no_grad():
        layer(xd[:, :100], past_key_values=cache, use_cache=True)
        # a refused step leaves the cache as it was: the same tokens fed one at a time afterwards give what an
        # untouched cache gives
        fresh = NAtSCache()
        layer(xd[:, :100], past_key_values=fresh, use_cache=True)
        for t in range(100, 104):
            a = layer(xd[:, t:t + 1], past_key_values=cache, use_cache=True)[0]
            b = layer(xd[:, t:t + 1], past_key_values=fresh, use_cache=True)[0]
            assert torch.equal(a, b), f"token {t} differs after a refused step"


@pytest.mark.parametrize("kind", ['gdn', 'mamba'])
def test_decode_step_across_a_block_boundary(kind):
    """A decode step of several tokens that crosses a selector-block boundary (36 cached tokens of the block + 40 new ones)
    gives what the same tokens give one at a time, and leaves the cache in the same state."""
    from neuralattentionsearchlinear_amd.cache import NAtSCache, NAtSMamba2Cache
    layer, cfg, w, x = _layer_case(kind)
    layer.layer_idx = 0
    layer = layer.to(DEV).to(torch.bfloat16).eval()
    xd = x.to(DEV).bfloat16()
    first = lambda out: out[0] if isinstance(out, tuple) else out
    mk = (lambda: NAtSCache()) if kind == 'gdn' else (lambda: NAtSMamba2Cache())
    kw = lambda h: dict(past_key_values=h, use_cache=True) if kind == 'gdn' else dict(cache_params=h, use_cache=True)
    with torch.no_grad():
        a_h, b_h = mk(), mk()
        layer(xd[:, :100], **kw(a_h))
        layer(xd[:, :100], **kw(b_h))
        a = first(layer(xd[:, 100:140], **kw(a_h)))
        b = torch.cat([first(layer(xd[:, t:t + 1], **kw(b_h))) for t in range(100, 140)], 1)
        assert a.shape == b.shape
        assert rel_l2(a.float(), b.float()) <= 1e-3, f"rel-L2 {rel_l2(a.float(), b.float()):.3e}"
        ca, cb = (h[0] if kind == 'gdn' else h.nats_cache[0] for h in (a_h, b_h))
        assert ca.n_observed_tokens == cb.n_observed_tokens == 140 and ca._n_tokens_in_nats_block == cb._n_tokens_in_nats_block == 12
        assert torch.equal(ca.n_attn_blocks, cb.n_attn_blocks)
        # and the two caches go on alike
        a2, b2 = first(layer(xd[:, 140:141], **kw(a_h))), first(layer(xd[:, 140:141], **kw(b_h)))
        assert rel_l2(a2.float(), b2.float()) <= 1e-3


@pytest.mark.parametrize("kind,ops,T0,T1", [('gdn', 'all', 100, 300), ('mamba', 'all', 100, 300), ('gdn', 'all', 128, 319),
                                            ('gdn', 'all', 30, 94), ('gdn', 'gated_delta_net', 100, 300), ('mamba', 'mamba', 70, 290),
                                            ('gdn', 'attn', 100, 300), ('mamba', 'attn', 192, 256)])
def test_long_continuation_on_a_filled_cache(kind, ops, T0, T1):
    """64 or more new tokens on a cache that already holds tokens (a second prompt) run through the chunked operators -- the
    linear branch from the state that entered the incomplete block, the softmax branch with the kept blocks as a key prefix:
    outputs close to the tokens fed one at a time and to the whole forward, the same cache afterwards."""
    from neuralattentionsearchlinear_amd.cache import NAtSCache, NAtSMamba2Cache
    layer, cfg, w, x = _layer_case(kind, None, ops)
    layer.layer_idx = 0
    layer = layer.to(DEV).to(torch.bfloat16).eval()
    xd = x.to(DEV).bfloat16()                                           # 320 tokens
    first = lambda out: out[0] if isinstance(out, tuple) else out
    mk = (lambda: NAtSCache()) if kind == 'gdn' else (lambda: NAtSMamba2Cache())
    kw = lambda h: dict(past_key_values=h, use_cache=True) if kind == 'gdn' else dict(cache_params=h, use_cache=True)
    with torch.no_grad():
        whole = first(layer(xd))
        a_h, b_h = mk(), mk()
        layer(xd[:, :T0], **kw(a_h))
        layer(xd[:, :T0], **kw(b_h))
        a = first(layer(xd[:, T0:T1], **kw(a_h)))                       # at once
        b = torch.cat([first(layer(xd[:, t:t + 1], **kw(b_h))) for t in range(T0, T1)], 1)
        # and both caches go on to give the same next token
        a2, b2 = (first(layer(xd[:, T1:T1 + 1], **kw(h))) for h in (a_h, b_h)) if T1 < xd.shape[1] else (None, None)
    assert a.shape == b.shape == (2, T1 - T0, xd.shape[-1])
    assert rel_l2(a.float(), b.float()) <= 1e-2, f"against single-token steps: rel-L2 {rel_l2(a.float(), b.float()):.3e}"
    assert rel_l2(a.float(), whole[:, T0:T1].float()) <= 2e-2, f"against the whole forward: rel-L2 {rel_l2(a.float(), whole[:, T0:T1].float()):.3e}"
    ca, cb = (h[0] if kind == 'gdn' else h.nats_cache[0] for h in (a_h, b_h))
    assert torch.equal(ca.n_attn_blocks, cb.n_attn_blocks)
    if a2 is not None:
        assert ca.n_observed_tokens == cb.n_observed_tokens == T1 + 1
        assert rel_l2(a2.float(), b2.float()) <= 1e-2, f"the next token: rel-L2 {rel_l2(a2.float(), b2.float()):.3e}"
