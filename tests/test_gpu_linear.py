"""GPU parity: Gated DeltaNet and Mamba2-SSD branches through the C ABI vs the oracle.

Tolerance (stated for the path): outputs and final states max-abs <= 2e-2 and relative L2 <= 5e-3
against the fp32 oracle evaluated on the same bf16-rounded inputs."""
import pytest
import torch
import torch.nn.functional as F

from oracle import linear_branch as lb
from tests._util import assert_close, make_gates, make_qkv, make_types

pytestmark = pytest.mark.gpu
DEV = 'cuda:0'


def _gdn(B, T, H, HN, K, V, block, p_attn, decay, seed, h0=False, intra=True, l2=True, scale=None):
    from neuralattentionsearchlinear_amd import _capi
    from neuralattentionsearchlinear_amd._mixed_common import linear_chunk_fwd
    q, k, v = make_qkv(B, T, H, K, V, seed)
    g, beta = make_gates(B, T, H, seed + 1)
    NB = -(-T // block)
    ty = make_types(B, NB, HN, p_attn, seed + 2, torch.bfloat16)
    init = torch.randn(B, H, K, V, generator=torch.Generator().manual_seed(seed + 3)) * 0.5 if h0 else None
    scale = K ** -0.5 if scale is None else scale
    if not l2:
        q, k = (F.normalize(q.float(), dim=-1).bfloat16(), F.normalize(k.float(), dim=-1).bfloat16())
    o_ref, S_ref = lb.gdn_chunked(q, k, v, g, beta, ty[..., 1], scale, init, block, decay, l2, torch.float32, intra)
    flags = (_capi.DECAY_NON_LINEAR if decay else 0) | (_capi.QK_L2NORM if l2 else 0) | (_capi.INTRA_CHUNK if intra else 0)
    o, S = linear_chunk_fwd('gdn', q.to(DEV), k.to(DEV), v.to(DEV), g.to(DEV), beta.to(DEV),
                            None if init is None else init.to(DEV), ty.to(DEV), scale, block, flags, True, None)
    torch.cuda.synchronize()
    assert_close(o.float(), o_ref, "o_gdn")
    assert_close(S, S_ref, "final_state")


def _mamba(B, T, H, HN, K, V, block, p_attn, decay, seed, h0=False):
    from neuralattentionsearchlinear_amd import _capi
    from neuralattentionsearchlinear_amd._mixed_common import linear_chunk_fwd
    g_ = torch.Generator().manual_seed(seed)
    # the Mamba layer L2-normalises C and B outside the op, x*dt is small, g = A*dt
    q = F.normalize(torch.randn(B, T, H, K, generator=g_), dim=-1).bfloat16()
    k = F.normalize(torch.randn(B, T, H, K, generator=g_), dim=-1).bfloat16()
    dt = F.softplus(torch.randn(B, T, H, generator=g_) - 4)
    A = -torch.exp(torch.rand(H, generator=g_) * torch.log(torch.tensor(16.0)))
    v = (torch.randn(B, T, H, V, generator=g_) * dt[..., None]).bfloat16()
    g = A * dt
    NB = -(-T // block)
    ty = make_types(B, NB, HN, p_attn, seed + 2, torch.bfloat16)
    init = torch.randn(B, H, K, V, generator=g_) * 0.1 if h0 else None
    o_ref, S_ref = lb.mamba_chunked(q, k, v, g, ty[..., 1], 1.0, init, block, decay, torch.float32)
    flags = (_capi.DECAY_NON_LINEAR if decay else 0) | _capi.INTRA_CHUNK
    o, S = linear_chunk_fwd('mamba', q.to(DEV), k.to(DEV), v.to(DEV), g.to(DEV), None,
                            None if init is None else init.to(DEV), ty.to(DEV), 1.0, block, flags, True, None)
    torch.cuda.synchronize()
    assert_close(o.float(), o_ref, "o_mamba")
    assert_close(S, S_ref, "final_state")


@pytest.mark.parametrize("decay", [True, False])
@pytest.mark.parametrize("K,V", [(128, 128), (64, 64), (128, 256), (64, 32)])
def test_gdn_small(K, V, decay):
    _gdn(2, 512, 4, 4, K, V, 64, 0.4, decay, seed=0)


def test_gdn_all_linear_with_initial_state():
    _gdn(2, 1024, 4, 4, 128, 128, 64, 0.0, True, seed=1, h0=True)


def test_gdn_mostly_attention():
    _gdn(1, 1024, 4, 2, 128, 128, 64, 0.9, True, seed=2, h0=True)


def test_gdn_ragged_length():
    _gdn(2, 600, 2, 2, 128, 128, 64, 0.4, True, seed=3)
    _gdn(1, 70, 2, 2, 64, 64, 64, 0.4, True, seed=4, h0=True)


@pytest.mark.parametrize("block", [128, 256])
def test_gdn_large_blocks(block):
    _gdn(2, 1024, 2, 2, 128, 64, block, 0.5, True, seed=5, h0=True)
    _gdn(2, 1024, 2, 2, 128, 64, block, 0.5, False, seed=6)


def test_gdn_without_intra_term_and_without_l2norm():
    _gdn(1, 512, 2, 2, 128, 128, 64, 0.4, True, seed=7, intra=False)
    _gdn(1, 512, 2, 2, 128, 128, 64, 0.4, True, seed=8, l2=False)


def test_gdn_odd_head_counts():
    _gdn(3, 256, 6, 3, 128, 128, 64, 0.3, True, seed=9)      # chains not a multiple of 8


@pytest.mark.parametrize("decay", [True, False])
@pytest.mark.parametrize("K,V,block", [(128, 64, 256), (128, 64, 64), (64, 128, 128)])
def test_mamba(K, V, block, decay):
    _mamba(2, 1024, 4, 2, K, V, block, 0.3, decay, seed=10, h0=True)


def test_mamba_ragged():
    _mamba(1, 333, 2, 2, 128, 64, 64, 0.3, True, seed=11)


# ---- the 760M configuration's head geometry: key dim 192, value dim 384 (reference experiments/configs/natsl_760M.json) ----
@pytest.mark.parametrize("decay", [True, False])
def test_gdn_key_dim_192(decay):
    _gdn(2, 512, 4, 2, 192, 384, 64, 0.4, decay, seed=20, h0=True)


def test_gdn_key_dim_192_other_shapes():
    _gdn(1, 300, 2, 2, 192, 192, 128, 0.5, True, seed=21)            # ragged, block of two chunks
    _gdn(1, 512, 2, 2, 192, 48, 64, 0.3, True, seed=22, l2=False)    # narrow value dim


def test_mamba_key_dim_192():
    _mamba(2, 512, 4, 2, 192, 384, 64, 0.3, True, seed=23, h0=True)


# ---- the scan's three workgroup widths: 64 columns when that still gives one workgroup per CU, else 32, else 16; the small
# shapes above all take 16 ----
def _cus():
    return torch.cuda.get_device_properties(0).multi_processor_count


def test_gdn_scan_with_32_columns_per_workgroup():
    B, H, V = 4, 16, 128
    assert B * H * (V // 32) >= _cus() > B * H * (V // 64)
    _gdn(B, 320, H, 8, 128, V, 64, 0.4, True, seed=24, h0=True)
    _gdn(4, 256, 6, 3, 192, 384, 64, 0.4, True, seed=25)             # key dim 192 never takes 64 columns


def test_gdn_and_mamba_scan_with_64_columns_per_workgroup():
    B, H, V = 8, 16, 128
    assert B * H * (V // 64) >= _cus()
    _gdn(B, 320, H, 16, 128, V, 64, 0.3, True, seed=26, h0=True)
    _gdn(B, 256, H, 4, 64, V, 128, 0.5, False, seed=27)
    _gdn(B, 200, H, 8, 128, V, 64, 0.4, True, seed=29, intra=False)      # (this launch forms P in the scan and does not use it)
    _mamba(B, 256, H, 8, 128, V, 64, 0.3, True, seed=28, h0=True)


@pytest.mark.parametrize("K", [128, 64])
def test_gdn_p_formed_by_the_scan_agrees_with_p_from_the_prep(K):
    """A four-wave launch that fills the machine forms P inside the scan (the prep reads k only); a call that also returns the
    chunk states for a backward takes P from the prep kernel through the workspace.  Same inputs: the states are bit-identical
    (P does not enter them), the outputs agree to the rounding of P's bf16 tiles."""
    from neuralattentionsearchlinear_amd import _capi
    from neuralattentionsearchlinear_amd._mixed_common import linear_chunk_fwd
    B, T, H, V, block = 8, 448, 16, 128, 64
    assert B * H * (V // 64) >= _cus()
    q, k, v = make_qkv(B, T, H, K, V, 40)
    g, beta = make_gates(B, T, H, 41)
    ty = make_types(B, T // block, H, 0.3, 42, torch.bfloat16)
    flags = _capi.DECAY_NON_LINEAR | _capi.QK_L2NORM | _capi.INTRA_CHUNK
    args = [t.to(DEV) for t in (q, k, v, g, beta)]
    o1, s1 = linear_chunk_fwd('gdn', *args, None, ty.to(DEV), K ** -0.5, block, flags, True, None)
    o2, s2 = linear_chunk_fwd('gdn', *args, None, ty.to(DEV), K ** -0.5, block, flags, True, None, chunk_states=True)[:2]
    assert torch.equal(s1, s2)
    rl = float((o1.float() - o2.float()).norm() / o2.float().norm())
    assert 0 < rl <= 5e-4, rl          # (0 would mean both calls took the same path)
