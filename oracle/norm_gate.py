"""Oracle for the layer tail: two-input RMSNorm, per-head mix weights, swish gate.

TEST INFRASTRUCTURE ONLY -- see oracle/__init__.py.

Restates the forward of FusedMultiInputRMSNormGated with both weights and
x-weights present (src/nats/modules/fused_norm_gate.py:116-182):
    y = (rms(x1)*w1*xw[...,0] + rms(x2)*w2*xw[...,1]) * gate*sigmoid(gate),
    rms(x) = x * rsqrt(mean(x^2) + eps)        (kernel :122-123 is authoritative).
Pin: closed form; torch.nn.functional.rms_norm is the library cross-check.
"""
import torch


def two_input_rmsnorm_gated(x1, x2, gate, x_weights, w1, w2, eps=1e-5, dtype=torch.float32):
    x1, x2, gate, xw = x1.to(dtype), x2.to(dtype), gate.to(dtype), x_weights.to(dtype)
    r1 = x1 * torch.rsqrt((x1 * x1).mean(-1, keepdim=True) + eps) * w1.to(dtype)
    r2 = x2 * torch.rsqrt((x2 * x2).mean(-1, keepdim=True) + eps) * w2.to(dtype)
    y = r1 * xw[..., 0:1] + r2 * xw[..., 1:2]
    return y * gate * torch.sigmoid(gate)
