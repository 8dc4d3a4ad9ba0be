"""Small torch modules the two hybrid layers are built from.

The reference takes these from flash-linear-attention (ShortConvolution, RMSNorm, L2Norm) and from
src/nats/modules/fused_norm_gate.py (FusedMultiInputRMSNormGated); parameter names are kept so that
reference checkpoints load.  Projections and the short convolution stay torch ops (rocBLAS / MIOpen);
the two-input norm-gate runs the HIP kernel natsl_norm_gate_fwd.
"""
from __future__ import annotations

from typing import Optional

import torch
import torch.nn as nn
import torch.nn.functional as F

from . import _capi


class RMSNorm(nn.Module):
    def __init__(self, hidden_size: int, eps: float = 1e-5):
        super().__init__()
        self.eps = eps
        self.weight = nn.Parameter(torch.ones(hidden_size))

    def forward(self, x):
        xf = x.float()
        y = xf * torch.rsqrt(xf.pow(2).mean(-1, keepdim=True) + self.eps) * self.weight.float()
        return y.to(x.dtype)


class L2Norm(nn.Module):
    def __init__(self, eps: float = 1e-6):
        super().__init__()
        self.eps = eps

    def forward(self, x):
        xf = x.float()
        return (xf * torch.rsqrt(xf.pow(2).sum(-1, keepdim=True) + self.eps)).to(x.dtype)


class ShortConvolution(nn.Conv1d):
    """Depthwise causal convolution over time with optional SiLU; weight [hidden, 1, kernel] as in fla."""

    def __init__(self, hidden_size: int, kernel_size: int, bias: bool = False, activation: Optional[str] = 'silu'):
        super().__init__(hidden_size, hidden_size, kernel_size, groups=hidden_size, bias=bias, padding=kernel_size - 1)
        if activation not in (None, 'silu', 'swish'):
            raise ValueError(f"unsupported activation {activation}")
        self.hidden_size = hidden_size
        self.activation = activation

    def forward(self, x, cache=None, output_final_state: bool = False, cu_seqlens=None):
        if cu_seqlens is not None:
            raise NotImplementedError("packed sequences are not supported by this ShortConvolution")
        B, T, D = x.shape
        xt = x.transpose(1, 2)
        W = self.kernel_size[0]
        if cache is not None:
            xt = torch.cat([cache.to(xt.dtype), xt], -1)
            y = F.conv1d(xt, self.weight, self.bias, groups=D)[..., -T:]
        else:
            y = F.conv1d(xt, self.weight, self.bias, padding=W - 1, groups=D)[..., :T]
        final = None
        if output_final_state:
            src = xt if cache is not None else F.pad(xt, (W, 0))
            final = src[..., -W:].contiguous()
        if self.activation is not None:
            y = F.silu(y)
        return y.transpose(1, 2), final


class FusedMultiInputRMSNormGated(nn.Module):
    """y = (rms(x1)*weight1*xw[...,0] + rms(x2)*weight2*xw[...,1]) * g*sigmoid(g)
    (forward of src/nats/modules/fused_norm_gate.py:1354-1429 with x-weights and both affine weights)."""

    def __init__(self, hidden_size: int, elementwise_affine: bool = True, eps: float = 1e-5, activation: str = 'swish'):
        super().__init__()
        if activation not in ('swish', 'silu'):
            raise NotImplementedError("only the swish/silu gate is built")
        if not elementwise_affine:
            raise NotImplementedError("elementwise_affine=False is not built")
        self.hidden_size, self.eps, self.activation = hidden_size, eps, activation
        self.weight1 = nn.Parameter(torch.ones(hidden_size))
        self.weight2 = nn.Parameter(torch.ones(hidden_size))

    def forward(self, x1, x2, g, x_weights_after_norm=None):
        if x_weights_after_norm is None:
            x_weights_after_norm = torch.ones(*x1.shape[:-1], 2, dtype=x1.dtype, device=x1.device)
        return two_inputs_rms_norm_gated(x1, x2, g, x_weights_after_norm, self.weight1, self.weight2, self.eps)


def _norm_gate_fwd(x1, x2, g, x_weights, weight1, weight2, eps):
    io_dtype = x1.dtype
    D = x1.shape[-1]
    to = lambda t: t.detach().to(torch.bfloat16).contiguous()
    a, b, gg, xw = to(x1), to(x2.reshape(x1.shape)), to(g.reshape(x1.shape)), to(x_weights)
    w1, w2 = weight1.detach().contiguous(), weight2.detach().contiguous()
    if w1.dtype != w2.dtype or w1.dtype not in (torch.float32, torch.bfloat16):
        w1, w2 = w1.float(), w2.float()
    y = torch.empty_like(a)
    rows = a.numel() // D
    rc = _capi.lib().natsl_norm_gate_fwd(_capi.ptr(a), _capi.ptr(b), _capi.ptr(gg), _capi.ptr(xw), _capi.ptr(w1), _capi.ptr(w2),
                                         _capi.ptr(y), rows, D, _capi.BF16, float(eps), _capi.dtype_code(w1.dtype),
                                         _capi.stream_ptr(a.device))
    _capi.check(rc, "natsl_norm_gate_fwd")
    return y.to(io_dtype)


class _NormGate(torch.autograd.Function):
    """The HIP forward with a backward for training: the gradients are those of the same formula evaluated as fp32 torch
    operations (elementwise work plus two row reductions; replaces the backward of
    src/nats/modules/fused_norm_gate.py:185-420 in function)."""

    @staticmethod
    def forward(ctx, x1, x2, g, x_weights, weight1, weight2, eps):
        ctx.save_for_backward(x1, x2, g, x_weights, weight1, weight2)
        ctx.eps = eps
        return _norm_gate_fwd(x1, x2, g, x_weights, weight1, weight2, eps)

    @staticmethod
    def backward(ctx, dy):
        saved = ctx.saved_tensors
        with torch.enable_grad():
            x1, x2, g, xw, w1, w2 = (t.detach().float().requires_grad_(True) for t in saved)
            r1 = x1 * torch.rsqrt((x1 * x1).mean(-1, keepdim=True) + ctx.eps) * w1
            r2 = x2.reshape(x1.shape) * torch.rsqrt((x2.reshape(x1.shape) ** 2).mean(-1, keepdim=True) + ctx.eps) * w2
            gate = g.reshape(x1.shape)
            y = (r1 * xw[..., 0:1] + r2 * xw[..., 1:2]) * gate * torch.sigmoid(gate)
            grads = torch.autograd.grad(y, (x1, x2, g, xw, w1, w2), dy.float())
        return tuple(gr.to(t.dtype) for gr, t in zip(grads, saved)) + (None,)


def two_inputs_rms_norm_gated(x1, x2, g, x_weights, weight1, weight2, eps: float = 1e-5):
    if not x1.is_cuda:
        raise _capi.NatslError("the norm-gate runs on the GPU only (no CPU fallback)")
    if torch.is_grad_enabled() and any(t.requires_grad for t in (x1, x2, g, x_weights, weight1, weight2)):
        return _NormGate.apply(x1, x2, g, x_weights, weight1, weight2, eps)
    return _norm_gate_fwd(x1, x2, g, x_weights, weight1, weight2, eps)
