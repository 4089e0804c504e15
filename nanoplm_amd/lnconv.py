"""LayerNorm fused into the conv's forward: ``conv(layer_norm(x))`` (``+ x``) in one pass over x.

For a conv that takes the place of a sub-module of the reference's pre-norm encoder layer
(src/nanoplm/pretraining/models/modern_bert/modeling.py:404-414)::

    x = x + self.attn(self.attn_norm(x), ...)      # attn_norm: nn.LayerNorm(hidden), modeling.py:264-266

``ln_varlen_dwconv(x, cu_seqlens, ln_weight, ln_bias, weight, bias, residual=True)`` returns
``x + conv(layer_norm(x))`` from one read of x and one write of y: the kernel's blocks own whole rows (rows of at
most 2 KiB: C <= 1024 in bf16, 512 in fp32; K in {3,5,7,9}), take the row statistics from the tile they have staged
and normalise as they read. The normalised tensor is never stored; the kernel leaves (mean, rstd) per row for the
backward, which recomputes it: the backward is a composition (normalise with elementwise ops in fp32, this library's
conv backward, ATen's LayerNorm backward), so the fusion saves forward traffic and the activation memory of the
normalised tensor, not backward traffic. Shapes the fused kernel is not built for (the library says so with its
return code) run ``F.layer_norm`` and the plain HIP conv.
"""
from __future__ import annotations

from typing import Optional

import torch
import torch.nn.functional as F

from . import _lib
from .dwconv import _DTYPES, _launch_on, _ptr, varlen_dwconv_bwd, varlen_dwconv_fwd


def _check(x, cu_seqlens, ln_weight, ln_bias, weight, bias):
    if x.dim() != 2:
        raise ValueError("x must be [T, C]")
    if not x.is_cuda:
        raise RuntimeError(f"ln_varlen_dwconv runs only on a ROCm device (x is on {x.device}); there is no CPU implementation")
    T, C = x.shape
    if weight.dim() != 2 or weight.shape[0] != C:
        raise ValueError(f"weight must be [C={C}, K], got {tuple(weight.shape)}")
    for name, t in (("ln_weight", ln_weight), ("ln_bias", ln_bias), ("bias", bias)):
        if t is not None and tuple(t.shape) != (C,):
            raise ValueError(f"{name} must be [C={C}], got {tuple(t.shape)}")
    if ln_weight is None:
        raise ValueError("ln_weight is required (pass ones for a LayerNorm without affine parameters)")
    if cu_seqlens.dtype != torch.int32 or cu_seqlens.dim() != 1 or cu_seqlens.numel() < 1:
        raise TypeError("cu_seqlens must be a 1-D int32 tensor with at least one entry")
    return T, C, weight.shape[1], cu_seqlens.numel() - 1


def ln_dwconv_fwd(x, cu_seqlens, ln_weight, ln_bias, weight, bias=None, *, eps: float = 1e-5, residual: bool = False,
                  want_stats: bool = True):
    """Raw forward (no autograd): ``(y, stats)`` with y = conv(layer_norm(x)) (+ x) in x's dtype and stats
    ``[T, 2]`` fp32 = (mean, rstd) per row (None without ``want_stats``). The LayerNorm parameters are used in the
    conv weight's dtype."""
    T, C, K, S = _check(x, cu_seqlens, ln_weight, ln_bias, weight, bias)
    lib = _lib.load()
    x = x.contiguous()
    weight = weight.contiguous()
    wdt = weight.dtype
    ln_weight = ln_weight.to(wdt).contiguous()
    ln_bias = None if ln_bias is None else ln_bias.to(wdt).contiguous()
    bias = None if bias is None else bias.to(wdt).contiguous()
    y = torch.empty_like(x)
    stats = torch.empty((T, 2), dtype=torch.float32, device=x.device) if want_stats else None
    with _launch_on(x) as dev:
        rc = lib.nplm_dwconv_ln_fwd(_ptr(x), _ptr(cu_seqlens.contiguous()), _ptr(ln_weight), _ptr(ln_bias), float(eps),
                                    _ptr(weight), _ptr(bias), _ptr(y), _ptr(stats), T, C, K, S, _DTYPES[x.dtype],
                                    _DTYPES[wdt], _lib.RESIDUAL if residual else 0, dev.stream)
    if rc == -_lib.EUNSUPPORTED:
        xf = x.float()
        var, mean = torch.var_mean(xf, dim=-1, unbiased=False, keepdim=True)
        rstd = torch.rsqrt(var + eps)
        n = (xf - mean) * rstd * ln_weight.float()
        if ln_bias is not None:
            n = n + ln_bias.float()
        y = varlen_dwconv_fwd(n, cu_seqlens, weight, bias)
        if residual:
            y = y + xf
        return y.to(x.dtype), (torch.cat([mean, rstd], dim=1) if want_stats else None)
    _lib.check(rc, "nplm_dwconv_ln_fwd")
    return y, stats


class LnVarlenDWConv1dFunction(torch.autograd.Function):
    """y = conv(layer_norm(x; ln_weight, ln_bias); weight, bias) (+ x). Forward fused; backward composed (see the
    module docstring): gradients for x, ln_weight, ln_bias, weight, bias."""

    @staticmethod
    def forward(ctx, x, cu_seqlens, ln_weight, ln_bias, weight, bias, eps, residual):
        y, stats = ln_dwconv_fwd(x, cu_seqlens, ln_weight, ln_bias, weight, bias, eps=eps, residual=residual)
        ctx.save_for_backward(x, cu_seqlens, ln_weight, ln_bias, weight, stats)
        ctx.has_bias = bias is not None
        ctx.bias_dtype = None if bias is None else bias.dtype
        ctx.eps, ctx.residual = eps, residual
        return y

    @staticmethod
    def backward(ctx, dy):
        x, cu, ln_weight, ln_bias, weight, stats = ctx.saved_tensors
        C = x.shape[1]
        mean, rstd = stats[:, 0:1].contiguous(), stats[:, 1:2].contiguous()     # ATen reads them as dense [T, 1]
        xf = x.float()
        gf = ln_weight.float()
        n = (xf - mean) * rstd * gf
        if ln_bias is not None:
            n = n + ln_bias.float()
        dyf = dy.float().contiguous()
        dn, dw, db = varlen_dwconv_bwd(n, dyf, cu, weight)
        bf = None if ln_bias is None else ln_bias.float()
        dx, dg, dbeta = torch.ops.aten.native_layer_norm_backward(dn, xf, [C], mean, rstd, gf, bf,
                                                                  [True, True, ln_bias is not None])
        if ctx.residual:
            dx = dx + dyf
        return (dx.to(x.dtype), None, dg.to(ln_weight.dtype), None if ln_bias is None else dbeta.to(ln_bias.dtype),
                dw.to(weight.dtype), db.to(ctx.bias_dtype) if ctx.has_bias else None, None, None)


def ln_varlen_dwconv(x, cu_seqlens, ln_weight, ln_bias, weight, bias=None, *, eps: float = 1e-5, residual: bool = False):
    """Differentiable ``conv(layer_norm(x))`` (``+ x`` with ``residual``) over packed sequences."""
    return LnVarlenDWConv1dFunction.apply(x, cu_seqlens, ln_weight, ln_bias, weight, bias, eps, residual)


def ln_supported(x: torch.Tensor, weight: torch.Tensor) -> bool:
    """Whether the fused forward takes this call (K in {3,5,7,9}, rows of at most 2 KiB in multiples of 16 bytes,
    16-byte aligned contiguous x on a ROCm device). Informational: ``ln_dwconv_fwd`` finds out from the library."""
    if not (isinstance(x, torch.Tensor) and x.is_cuda and x.dim() == 2 and x.dtype in _DTYPES and weight.dtype in _DTYPES):
        return False
    rb = x.shape[1] * x.element_size()
    return weight.shape[1] in (3, 5, 7, 9) and rb % 16 == 0 and rb <= 2048 and x.is_contiguous() and x.data_ptr() % 16 == 0
