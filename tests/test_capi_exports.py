"""CPU-only: the C-ABI library builds, loads, and exports every function include/natsl.h declares;
argument validation runs on the host before any launch."""
import ctypes
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared():
    text = open(os.path.join(ROOT, "include", "natsl.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(natsl_[a-z_0-9]+)\s*\(", text)))


def _lib():
    from neuralattentionsearchlinear_amd import _capi
    if not os.path.exists(_capi.LIB_PATH):
        from neuralattentionsearchlinear_amd import _build
        _build.build()
    return _capi.lib()


def test_header_symbols_are_exported():
    names = _declared()
    assert len(names) >= 10
    L = _lib()
    missing = [n for n in names if not hasattr(L, n)]
    assert not missing, missing
    from neuralattentionsearchlinear_amd import _capi
    assert sorted(_capi.exported_symbols()) == names          # the ctypes table covers the whole header
    assert L.natsl_version() >= 100


def test_argument_validation_needs_no_gpu():
    L = _lib()
    # null pointers / bad shapes are rejected on the host, before any launch
    assert L.natsl_hard_select(None, None, None, 1, 4, 2, 1, 0, None, 0, 0, None) == -1
    assert b"null" in L.natsl_last_error()
    assert L.natsl_route(ctypes.c_void_p(16), 1, 1, 4, 2, 256, 32, None, None, None, None, None, None, None, 0, 0, None) == -2
    assert b"multiple of 64" in L.natsl_last_error()
    assert L.natsl_linear_workspace_bytes(16384, 16) == 16384 * 16 * (2 * 64 * 64 * 2 + 4 * 64 * 4)
    p = ctypes.c_void_p(256)
    rc = L.natsl_softmax_sparse_fwd(p, p, p, p, p, p, 1, p, p, 1, 256, 4, 4, 4, 96, 96, 4, 64, 0.1, 1, 1, None, 0, 0, None)
    assert rc == -2 and b"head dims" in L.natsl_last_error()
    rc = L.natsl_gdn_chunk_fwd(p, p, p, p, p, None, p, None, None, None, None, None, p, 1, 1, 256, 4, 4, 128, 128, 4, 64, 0.1, 7, p, 16, 1,
                               None, 0, 0, None)
    assert rc == -3 and b"workspace" in L.natsl_last_error()
    # the softmax backward's 32-bit row offsets: T * HQ * max(K, V) * 2 bytes must stay below 2^32 -- refused on the host,
    # before any kernel is launched (T = 2^20 tokens x 32 heads x 128 x 2 bytes = 2^33)
    rc = L.natsl_softmax_sparse_bwd(p, p, p, p, p, p, p, p, p, p, p, 1, p, p, 1, 1 << 20, 32, 32, 32, 128, 128, 1 << 14, 64, 0.1, 1, 1,
                                    p, ctypes.c_size_t(1 << 40), None, 0, 0, 0, None)
    assert rc == -2 and b"32-bit" in L.natsl_last_error()


def test_no_cpu_fallback():
    import torch
    from neuralattentionsearchlinear_amd import _capi
    from neuralattentionsearchlinear_amd.mixed_attn_gdn import nats_mixed_attn_gdn
    x = torch.zeros(1, 64, 1, 64, dtype=torch.bfloat16)
    g = torch.zeros(1, 64, 1)
    ty = torch.ones(1, 1, 1, 2)
    with pytest.raises(_capi.NatslError):
        nats_mixed_attn_gdn(x, x, x, x, x, x, None, g, g.bfloat16(), ty, None)


def test_product_does_not_import_the_oracle():
    pkg = os.path.join(ROOT, "neuralattentionsearchlinear_amd")
    for dirpath, _, files in os.walk(pkg):
        for f in files:
            if f.endswith((".py", ".hip", ".h")):
                src = open(os.path.join(dirpath, f)).read()
                assert "oracle" not in src.replace("no CPU fallback", ""), f"{f} mentions the oracle"


def test_backward_entry_rejects_what_is_not_built():
    """Argument errors come back as codes from the host, before any launch."""
    import ctypes
    from neuralattentionsearchlinear_amd import _capi
    L = _capi.lib()
    p = ctypes.c_void_p(256)
    args = lambda K, V, block: (1, p, p, p, p, p, p, None, p, p, 1, p, p, p, p, p, p, p, p, p, None, p, p, 1, 256, 4, 4, K, V, 256 // block, block,
                                0.1, 7, 1, None, 0, 0, None)
    assert L.natsl_linear_chunk_bwd(*args(96, 64, 64)) == -2 and b"K=96" in L.natsl_last_error()
    assert L.natsl_linear_chunk_bwd(*args(128, 48, 64)) == -2 and b"V=48" in L.natsl_last_error()
    # both forms read the forward's workspace (the Mamba form its scale vectors)
    for delta_rule in (1, 0):
        a = list(args(128, 64, 64))
        a[0], a[12] = delta_rule, None
        assert L.natsl_linear_chunk_bwd(*a) == -1 and b"null pointer" in L.natsl_last_error()


def test_invalid_block_gradient_is_refused_for_blocks_of_several_chunks():
    """The linear branch's selector gradient for blocks NOT typed linear is built for one chunk per block only: a
    larger block with the flag set raises before anything is launched."""
    import torch
    from neuralattentionsearchlinear_amd._linear_bwd import linear_chunk_backward
    q = torch.zeros(1, 128, 2, 64, dtype=torch.bfloat16)
    ty = torch.zeros(1, 1, 2, 2, dtype=torch.bfloat16)
    with pytest.raises(NotImplementedError, match="nats_block_size == 64"):
        linear_chunk_backward('gdn', q, q, q, torch.zeros(1, 128, 2), torch.zeros(1, 128, 2, dtype=torch.bfloat16), None, ty, 1.0, 128,
                              True, True, True, q, None, True)


def test_chunk_state_saving_follows_the_byte_budget():
    """_mixed_common.SAVE_CHUNK_STATES = None keeps the linear branch's chunk states for the backward only while they fit
    SAVE_CHUNK_STATES_MAX_BYTES; True / False force it."""
    import torch
    import neuralattentionsearchlinear_amd._mixed_common as MC
    small = torch.empty(1, 512, 4, 128, device='meta')
    big = torch.empty(8, 8192, 16, 128, device='meta')
    old = MC.SAVE_CHUNK_STATES
    try:
        MC.SAVE_CHUNK_STATES = None
        assert MC._keep_chunk_states(small, small, None) and not MC._keep_chunk_states(big, big, None)
        MC.SAVE_CHUNK_STATES = True
        assert MC._keep_chunk_states(big, big, None)
        MC.SAVE_CHUNK_STATES = False
        assert not MC._keep_chunk_states(small, small, None)
    finally:
        MC.SAVE_CHUNK_STATES = old
