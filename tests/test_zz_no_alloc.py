"""The entry point that allocates nothing: natsl_attn_masked_fwd_static against natsl_attn_masked_fwd, through the C ABI.

Same kernels, same split count, so the outputs must be IDENTICAL bit for bit.  Two calls in a row, the second with a
smaller input (fewer keys, fewer queries): the scratch array keeps the first call's contents, which must not leak."""
import ctypes

import pytest
import torch

pytestmark = pytest.mark.gpu
DEV = 'cuda:0'


def _case(B, TQ, TK, HQ, HKV, HM, K, V, seed):
    g = torch.Generator(device=DEV).manual_seed(seed)
    rn = lambda *s: torch.randn(*s, device=DEV, generator=g).bfloat16()
    q, k, v = rn(B, TQ, HQ, K), rn(B, TK, HKV, K), rn(B, TK, HKV, V)
    mask = (torch.rand(B, HM, TQ, TK, device=DEV, generator=g) < 0.7).to(torch.uint8)
    mask[0, 0, 0] = 0                                   # one query that sees nothing
    return q, k, v, mask.contiguous()


def _run(static, q, k, v, mask, K, V):
    from neuralattentionsearchlinear_amd import _capi
    L = _capi.lib()
    B, TQ, HQ, _ = q.shape
    TK, HKV, HM = k.shape[1], k.shape[2], mask.shape[1]
    o = torch.full((B, TQ, HQ, V), float('nan'), device=DEV, dtype=torch.bfloat16)
    scale = K ** -0.5
    P = _capi.ptr
    if static:
        rc = L.natsl_attn_masked_fwd_static(P(q), P(k), P(v), P(mask), P(o), B, TQ, TK, HQ, HKV, HM, K, V, scale, _capi.BF16,
                                            _capi.stream_ptr(q.device))
        _capi.check(rc, "natsl_attn_masked_fwd_static")
    else:
        need = L.natsl_attn_masked_workspace_bytes(B, TQ, TK, HQ, V)
        ws = torch.empty(max(need, 1), dtype=torch.uint8, device=DEV)
        rc = L.natsl_attn_masked_fwd(P(q), P(k), P(v), P(mask), P(o), B, TQ, TK, HQ, HKV, HM, K, V, scale, _capi.BF16, P(ws), need,
                                     0, 0, _capi.stream_ptr(q.device))
        _capi.check(rc, "natsl_attn_masked_fwd")
    torch.cuda.synchronize()
    return o, need if not static else None


def test_static_entry_equals_the_workspace_entry_on_two_calls_in_a_row():
    from neuralattentionsearchlinear_amd import _capi
    L = _capi.lib()
    assert L.natsl_attn_masked_static_scratch_bytes() == 256 << 10
    big = _case(4, 1, 3000, 16, 8, 8, 128, 128, 1)       # keys split over several workgroups per query
    small = _case(2, 1, 1100, 8, 8, 4, 128, 128, 2)      # fewer queries, fewer keys, fewer splits
    for q, k, v, mask in (big, small):
        ref, need = _run(False, q, k, v, mask, 128, 128)
        assert need > 0, "the case must use the split scratch"
        out, _ = _run(True, q, k, v, mask, 128, 128)
        assert torch.isfinite(out.float()).all()
        assert torch.equal(out, ref), f"static entry differs: max {float((out.float() - ref.float()).abs().max()):.3e}"
        assert bool((out[0, 0, 0] == 0).all())           # mask head 0, query 0 sees no key
    # against the dense definition as well (the workspace entry's own tests pin it; one check here)
    q, k, v, mask = small
    out, _ = _run(True, q, k, v, mask, 128, 128)
    G, GM = q.shape[2] // k.shape[2], q.shape[2] // mask.shape[1]
    kf, vf = k.float().repeat_interleave(G, 2), v.float().repeat_interleave(G, 2)
    s = torch.einsum('bqhd,bkhd->bhqk', q.float(), kf) * 128 ** -0.5
    m = mask.bool().repeat_interleave(GM, 1)
    p = torch.softmax(s.masked_fill(~m, float('-inf')), -1).nan_to_num(0.0)
    ref = torch.einsum('bhqk,bkhd->bqhd', p, vf)
    assert float((out.float() - ref).abs().max()) <= 2e-2 and float((out.float() - ref).norm() / ref.norm()) <= 5e-3


def test_static_entry_refuses_a_shape_beyond_its_scratch():
    from neuralattentionsearchlinear_amd import _capi
    L = _capi.lib()
    # 256 queries x 16 splits x (2 + 128) floats = 266 240 bytes, just above the 262 144 the library holds: refused on the
    # host, nothing is launched (the pointers are never dereferenced)
    B, TQ, TK, HQ, V = 8, 32, 65536, 1, 128
    need = L.natsl_attn_masked_workspace_bytes(B, TQ, TK, HQ, V)
    assert need > L.natsl_attn_masked_static_scratch_bytes()
    p = ctypes.c_void_p(256)
    rc = L.natsl_attn_masked_fwd_static(p, p, p, p, p, B, TQ, TK, HQ, 1, 1, 128, V, 0.1, _capi.BF16, _capi.stream_ptr(torch.device(DEV)))
    assert rc == -3 and b"built-in buffer" in L.natsl_last_error()
