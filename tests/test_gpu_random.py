"""Randomised sweep of the mixed GDN operator against the oracle: ragged lengths (down to a single token),
block sizes 64..256, selector head groups, packed batches, every incomplete-block mode, attention rates from 0
to 1, with and without an initial state.  Same tolerances as everywhere (max-abs 2e-2, rel-L2 5e-3)."""
import random

import pytest

from tests.test_gpu_mixed import _gdn_case

pytestmark = pytest.mark.gpu


def _draw(seed):
    rnd = random.Random(1000 + seed)
    K, V = rnd.choice([(64, 64), (128, 128), (64, 128), (128, 64)])
    H = rnd.choice([2, 4, 6])
    HN = rnd.choice([h for h in (1, 2, 3, H) if H % h == 0])
    block = rnd.choice([64, 64, 128, 192, 256])
    mode = rnd.choice(['all', 'all', 'attn', 'gated_delta_net'])
    p = rnd.choice([0.0, 0.2, 0.5, 0.8, 1.0])
    h0 = rnd.random() < 0.5
    if rnd.random() < 0.35:
        n = rnd.randint(2, 4)
        lens = [rnd.choice([1, 37, 64, 65, 130, 200, 333]) for _ in range(n)]
        cu = [0]
        for x in lens:
            cu.append(cu[-1] + x)
        return dict(B=1, T=cu[-1], H=H, K=K, V=V, p_attn=p, mode=mode, block=block, HN=HN, h0=h0, cu=cu)
    T = rnd.choice([1, 2, 63, 64, 65, 127, 128, 129, 200, 256, 300, 449, 512, 640])
    return dict(B=rnd.randint(1, 3), T=T, H=H, K=K, V=V, p_attn=p, mode=mode, block=block, HN=HN, h0=h0, cu=None)


@pytest.mark.parametrize("seed", range(32))
def test_random_case(seed):
    c = _draw(seed)
    _gdn_case(c['B'], c['T'], c['H'], c['K'], c['V'], c['p_attn'], seed=seed, mode=c['mode'], block=c['block'], HN=c['HN'],
              h0=c['h0'], cu=c['cu'])
