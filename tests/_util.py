"""Shared helpers for the GPU parity tests."""
import os

import torch
import torch.nn.functional as F


def rel_l2(a, b):
    a, b = a.double().cpu(), b.double().cpu()
    return float((a - b).norm() / b.norm().clamp_min(1e-30))


def max_abs(a, b):
    return float((a.double().cpu() - b.double().cpu()).abs().max())


MAX_ABS_TOL = 2e-2     # tolerance stated for outputs and final states
REL_L2_TOL = 5e-3


def assert_close(a, b, what=""):
    ma, rl = max_abs(a, b), rel_l2(a, b)
    assert ma <= MAX_ABS_TOL and rl <= REL_L2_TOL, f"{what}: max-abs {ma:.3e} (tol {MAX_ABS_TOL}), rel-L2 {rl:.3e} (tol {REL_L2_TOL})"
    return ma, rl


def record_parity(what, **errors):
    """Appends one line of measured errors to the text file the environment variable NATSL_PARITY_LOG names (no file when it
    is unset): the full-size tests call this, so that a run leaves the measured figures behind and not only pass / fail."""
    path = os.environ.get("NATSL_PARITY_LOG")
    if path:
        with open(path, "a") as f:
            f.write(f"{what}: " + "  ".join(f"{k} {v:.3e}" for k, v in errors.items()) + "\n")


def make_types(B, NB, HN, p_attn, seed, dtype=torch.float32, force_last=True):
    g = torch.Generator().manual_seed(seed)
    lin = (torch.rand(B, NB, HN, generator=g) >= p_attn).float()
    ty = torch.stack([1 - lin, lin], -1)
    if force_last:
        ty[:, -1] = 1
    return ty.to(dtype)


def make_qkv(B, T, H, K, V, seed, dtype=torch.bfloat16, HQ=None):
    g = torch.Generator().manual_seed(seed)
    q = torch.randn(B, T, HQ or H, K, generator=g).to(dtype)
    k = torch.randn(B, T, H, K, generator=g).to(dtype)
    v = torch.randn(B, T, H, V, generator=g).to(dtype)
    return q, k, v


def make_gates(B, T, H, seed, dtype=torch.bfloat16):
    g = torch.Generator().manual_seed(seed)
    beta = torch.sigmoid(torch.randn(B, T, H, generator=g)).to(dtype)
    gl = -F.softplus(torch.randn(B, T, H, generator=g))
    return gl, beta
