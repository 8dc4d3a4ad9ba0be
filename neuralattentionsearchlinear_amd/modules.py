"""Small torch modules the two hybrid layers are built from.

The reference takes these from flash-linear-attention (ShortConvolution, RMSNorm, L2Norm) and from
src/nats/modules/fused_norm_gate.py (FusedMultiInputRMSNormGated); parameter names are kept so that
reference checkpoints load.  Projections stay torch ops (rocBLAS); the short convolution, the RMS / L2 row norms and the
two-input norm-gate run HIP kernels in the forward (natsl_short_conv_fwd, natsl_row_norm_fwd, natsl_norm_gate_fwd) and in
the backward (natsl_short_conv_bwd, natsl_row_norm_bwd, natsl_norm_gate_bwd) wherever the forward does; the torch formulas
below cover CPU tensors and widths the kernels are not built for.
"""
from __future__ import annotations

from typing import Optional

import torch
import torch.nn as nn
import torch.nn.functional as F

from . import _capi


_ROW_NORM_WIDTHS = (32, 64, 96, 128, 192, 256, 384, 512)
_NORM_GATE_WIDTHS = (32, 64, 96, 128, 192, 256, 384, 512)


def _row_norm_torch(x, weight, eps, l2):
    xf = x.float()
    ss = xf.pow(2).sum(-1, keepdim=True) if l2 else xf.pow(2).mean(-1, keepdim=True)
    y = xf * torch.rsqrt(ss + eps)
    if weight is not None:
        y = y * weight.float()
    return y.to(x.dtype)


def _row_norm_fwd(x, weight, eps, l2):
    """natsl_row_norm_fwd on [..., D] (fp32 arithmetic, result in x's dtype)."""
    D = x.shape[-1]
    xc = x.detach().contiguous()
    w = None if weight is None else weight.detach().contiguous()
    if w is not None and w.dtype not in (torch.float32, torch.bfloat16):
        w = w.float()
    y = torch.empty_like(xc)
    rc = _capi.lib().natsl_row_norm_fwd(_capi.ptr(xc), _capi.ptr(w), _capi.ptr(y), xc.numel() // D, D, float(eps), int(l2),
                                        _capi.dtype_code(xc.dtype), _capi.dtype_code(w.dtype) if w is not None else _capi.F32,
                                        _capi.stream_ptr(xc.device))
    _capi.check(rc, "natsl_row_norm_fwd")
    return y


class _RowNorm(torch.autograd.Function):
    """The HIP forward and backward (natsl_row_norm_fwd / natsl_row_norm_bwd)."""

    @staticmethod
    def forward(ctx, x, weight, eps, l2):
        ctx.save_for_backward(x, weight)
        ctx.eps, ctx.l2 = eps, l2
        return _row_norm_fwd(x, weight, eps, l2)

    @staticmethod
    def backward(ctx, dy):
        x, weight = ctx.saved_tensors
        D = x.shape[-1]
        xc, dyc = x.detach().contiguous(), dy.detach().to(x.dtype).contiguous()
        w = None if weight is None else weight.detach().contiguous()
        if w is not None and w.dtype not in (torch.float32, torch.bfloat16):
            w = w.float()
        rows = xc.numel() // D
        L = _capi.lib()
        dx = torch.empty_like(xc)
        dw = None if w is None else torch.empty(D, dtype=torch.float32, device=xc.device)
        ws = None if w is None else torch.empty(L.natsl_row_norm_bwd_workspace_bytes(rows, D), dtype=torch.uint8, device=xc.device)
        rc = L.natsl_row_norm_bwd(_capi.ptr(xc), _capi.ptr(w), _capi.ptr(dyc), _capi.ptr(dx), _capi.ptr(dw), _capi.ptr(ws),
                                  0 if ws is None else ws.numel(), rows, D, float(ctx.eps), int(ctx.l2), _capi.dtype_code(xc.dtype),
                                  _capi.dtype_code(w.dtype) if w is not None else _capi.F32, _capi.stream_ptr(xc.device))
        _capi.check(rc, "natsl_row_norm_bwd")
        return dx, (None if w is None else dw.to(weight.dtype)), None, None


def row_norm(x, weight, eps: float, l2: bool):
    """RMSNorm (l2=False, optional weight) or L2 normalisation (l2=True) of the last dimension: the HIP kernel for f32 / bf16
    tensors on the GPU with a supported width, else the same formula as torch operations."""
    if not (x.is_cuda and x.dtype in (torch.float32, torch.bfloat16) and x.shape[-1] in _ROW_NORM_WIDTHS and x.numel() > 0):
        return _row_norm_torch(x, weight, eps, l2)
    if torch.is_grad_enabled() and (x.requires_grad or (weight is not None and weight.requires_grad)):
        return _RowNorm.apply(x, weight, eps, l2)
    return _row_norm_fwd(x, weight, eps, l2)


class RMSNorm(nn.Module):
    def __init__(self, hidden_size: int, eps: float = 1e-5):
        super().__init__()
        self.eps = eps
        self.weight = nn.Parameter(torch.ones(hidden_size))

    def forward(self, x):
        return row_norm(x, self.weight, self.eps, False)


class L2Norm(nn.Module):
    def __init__(self, eps: float = 1e-6):
        super().__init__()
        self.eps = eps

    def forward(self, x):
        return row_norm(x, None, self.eps, True)


def _short_conv_torch(x, weight, bias, cache, activation):
    """[B,T,D] -> [B,T,D]: the causal depthwise convolution as torch operations (weight [D,1,W])."""
    B, T, D = x.shape
    W = weight.shape[-1]
    xt = x.transpose(1, 2)
    if cache is not None:
        xt = torch.cat([cache.to(xt.dtype), xt], -1)
        y = F.conv1d(xt, weight, bias, groups=D)[..., -T:]
    else:
        y = F.conv1d(xt, weight, bias, padding=W - 1, groups=D)[..., :T]
    if activation is not None:
        y = F.silu(y)
    return y.transpose(1, 2)


def _short_conv_fwd(x, weight, bias, cache, activation, want_state=False):
    """natsl_short_conv_fwd: token-major in, token-major out, no transposed copies -> (y, next state [B,D,W] or None)."""
    B, T, D = x.shape
    W = weight.shape[-1]
    xc, w, b, st = _conv_operands(x, weight, bias, cache)
    y = torch.empty_like(xc)
    nxt = torch.empty(B, D, W, dtype=xc.dtype, device=xc.device) if want_state else None
    rc = _capi.lib().natsl_short_conv_fwd(_capi.ptr(xc), _capi.ptr(w), _capi.ptr(b), _capi.ptr(st), _capi.ptr(y), _capi.ptr(nxt), B, T, D,
                                          W, 0 if activation is None else 1, _capi.dtype_code(xc.dtype), _capi.dtype_code(w.dtype),
                                          _capi.dtype_code(st.dtype) if st is not None else _capi.F32, _capi.stream_ptr(xc.device))
    _capi.check(rc, "natsl_short_conv_fwd")
    return y, nxt


def _conv_operands(x, weight, bias, cache):
    B, T, D = x.shape
    W = weight.shape[-1]
    xc = x.detach().contiguous()
    w = weight.detach().reshape(D, W).contiguous()
    b = None if bias is None else bias.detach().to(w.dtype).contiguous()
    if w.dtype not in (torch.float32, torch.bfloat16):
        w, b = w.float(), (None if b is None else b.float())
    st = None
    if cache is not None:
        st = cache.detach().contiguous()
        if st.dtype not in (torch.float32, torch.bfloat16):
            st = st.float()
    return xc, w, b, st


class _ShortConv(torch.autograd.Function):
    """The HIP forward with the HIP backward (natsl_short_conv_bwd: dx, and dweight / dbias reduced in a fixed order)."""

    @staticmethod
    def forward(ctx, x, weight, bias, cache, activation):
        ctx.save_for_backward(x, weight, bias, cache)
        ctx.activation = activation
        return _short_conv_fwd(x, weight, bias, cache, activation)[0]

    @staticmethod
    def backward(ctx, dy):
        x, weight, bias, cache = ctx.saved_tensors
        B, T, D = x.shape
        W = weight.shape[-1]
        xc, w, b, st = _conv_operands(x, weight, bias, cache)
        dyc = dy.detach().to(xc.dtype).contiguous()
        dx = torch.empty_like(xc)
        dw = torch.empty(D, W, dtype=torch.float32, device=xc.device)
        db = torch.empty(D, dtype=torch.float32, device=xc.device) if bias is not None else None
        L = _capi.lib()
        ws_bytes = L.natsl_short_conv_bwd_workspace_bytes(B, T, D, W)
        ws = torch.empty(ws_bytes, dtype=torch.uint8, device=xc.device)
        rc = L.natsl_short_conv_bwd(_capi.ptr(xc), _capi.ptr(w), _capi.ptr(b), _capi.ptr(st), _capi.ptr(dyc), _capi.ptr(dx), _capi.ptr(dw),
                                    _capi.ptr(db), _capi.ptr(ws), ws_bytes, B, T, D, W, 0 if ctx.activation is None else 1,
                                    _capi.dtype_code(xc.dtype), _capi.dtype_code(w.dtype),
                                    _capi.dtype_code(st.dtype) if st is not None else _capi.F32, _capi.stream_ptr(xc.device))
        _capi.check(rc, "natsl_short_conv_bwd")
        return (dx.to(x.dtype), dw.view(weight.shape).to(weight.dtype), None if bias is None else db.to(bias.dtype), None, None)


class ShortConvolution(nn.Conv1d):
    """Depthwise causal convolution over time with optional SiLU; weight [hidden, 1, kernel] as in fla.  On the GPU the
    forward is the HIP kernel natsl_short_conv_fwd (kernel sizes 2-4, hidden % 8 == 0, f32 / bf16), else torch's conv1d."""

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
        W = self.kernel_size[0]
        hip = x.is_cuda and W in (2, 3, 4) and D % 8 == 0 and x.dtype in (torch.float32, torch.bfloat16) and x.numel() > 0
        final = None
        if not hip:
            y = _short_conv_torch(x, self.weight, self.bias, cache, self.activation)
        elif torch.is_grad_enabled() and (x.requires_grad or self.weight.requires_grad):
            y = _ShortConv.apply(x, self.weight, self.bias, cache, self.activation)
        else:
            y, final = _short_conv_fwd(x, self.weight, self.bias, cache, self.activation, want_state=output_final_state)
        if output_final_state and final is None:
            # the last W inputs, [B,D,W]: what the next call sees before its first token
            tail = x[:, -W:].transpose(1, 2)
            if T < W:
                prev = cache.to(x.dtype)[..., -(W - T):] if cache is not None else x.new_zeros(B, D, W - T)
                tail = torch.cat([prev, tail], -1)
            final = tail.contiguous()
        return y, final


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
    """The HIP forward and backward (natsl_norm_gate_fwd / natsl_norm_gate_bwd; the backward replaces that of
    src/nats/modules/fused_norm_gate.py:185-420 in function).  Widths without a kernel: the gradients of the same formula as
    fp32 torch operations."""

    @staticmethod
    def forward(ctx, x1, x2, g, x_weights, weight1, weight2, eps):
        ctx.save_for_backward(x1, x2, g, x_weights, weight1, weight2)
        ctx.eps = eps
        return _norm_gate_fwd(x1, x2, g, x_weights, weight1, weight2, eps)

    @staticmethod
    def backward(ctx, dy):
        saved = ctx.saved_tensors
        x1, x2, g, xw, w1, w2 = saved
        D = x1.shape[-1]
        if D in _NORM_GATE_WIDTHS and x1.numel() > 0:
            # natsl_norm_gate_bwd: one pass over the rows, the weight gradients through per-workgroup partial sums
            to = lambda t: t.detach().to(torch.bfloat16).contiguous()
            a, b, gg, xwb, d = to(x1), to(x2.reshape(x1.shape)), to(g.reshape(x1.shape)), to(xw), to(dy.reshape(x1.shape))
            wa, wb = w1.detach().contiguous(), w2.detach().contiguous()
            if wa.dtype != wb.dtype or wa.dtype not in (torch.float32, torch.bfloat16):
                wa, wb = wa.float(), wb.float()
            rows = a.numel() // D
            L = _capi.lib()
            da, db, dg = torch.empty_like(a), torch.empty_like(a), torch.empty_like(a)
            dxw = torch.empty(rows, 2, dtype=torch.float32, device=a.device)
            dw = torch.empty(2, D, dtype=torch.float32, device=a.device)
            ws = torch.empty(L.natsl_norm_gate_bwd_workspace_bytes(rows, D), dtype=torch.uint8, device=a.device)
            P = _capi.ptr
            rc = L.natsl_norm_gate_bwd(P(a), P(b), P(gg), P(xwb), P(wa), P(wb), P(d), P(da), P(db), P(dg), P(dxw), P(dw[0]), P(dw[1]),
                                       P(ws), ws.numel(), rows, D, _capi.BF16, float(ctx.eps), _capi.dtype_code(wa.dtype),
                                       _capi.stream_ptr(a.device))
            _capi.check(rc, "natsl_norm_gate_bwd")
            return (da.to(x1.dtype), db.view(x2.shape).to(x2.dtype), dg.view(g.shape).to(g.dtype), dxw.view(xw.shape).to(xw.dtype),
                    dw[0].to(w1.dtype), dw[1].to(w2.dtype), None)
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
