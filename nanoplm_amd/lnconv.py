"""LayerNorm fused into the conv's forward: ``conv(layer_norm(x))`` (``+ x``) in one pass over x.

For a conv that takes the place of a sub-module of the reference's pre-norm encoder layer
(src/nanoplm/pretraining/models/modern_bert/modeling.py:404-438)::

    x = x + self.attn(self.attn_norm(x), ...)      # attn_norm: nn.LayerNorm(hidden), modeling.py:408-414

``ln_varlen_dwconv(x, cu_seqlens, ln_weight, ln_bias, weight, bias, residual=True)`` returns
``x + conv(layer_norm(x))``; the normalised tensor is never stored (K in {3,5,7,9}, rows in multiples of 16 bytes):

* rows of at most 2 KiB (C <= 1024 in bf16, 512 in fp32) and fp32 rows of at most 4 KiB (C <= 1024: the residual
  stream of the reference under ``torch.autocast`` is fp32): one kernel, one read of x and one write of y; its blocks
  own whole rows, take the row statistics from the tile they have staged and normalise as they read;
* other rows of at most 8 KiB: a row-statistics kernel, then the conv kernel normalising as it reads with the
  statistics given;
* the forward leaves (mean, rstd) per row for the backward, whose conv kernel normalises x again as it reads it and
  sums the LayerNorm parameter gradients beside dw and db; for rows of at most 4 KiB its waves also exchange the row
  sums of the LayerNorm input gradient and write dx themselves (one kernel), for wider rows it hands the gradient of
  the normalised tensor (fp32) to one more pass over the rows.

Other shapes (the library says so with its return code) compose elementwise normalisation, the plain HIP conv and
ATen's LayerNorm backward.
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


def _param_dtype(weight, ln_weight, ln_bias):
    """The one dtype the kernels take every parameter in: the conv weight's when the LayerNorm parameters share it,
    else fp32 (the wider of the two; casting the other way would round the fp32 parameters to bf16)."""
    for t in (ln_weight, ln_bias):
        if t is not None and t.dtype != weight.dtype:
            return torch.float32
    return weight.dtype


def ln_dwconv_fwd(x, cu_seqlens, ln_weight, ln_bias, weight, bias=None, *, eps: float = 1e-5, residual: bool = False,
                  want_stats: bool = True):
    """Raw forward (no autograd): ``(y, stats)`` with y = conv(layer_norm(x)) (+ x) in x's dtype and stats
    ``[T, 2]`` fp32 = (mean, rstd) per row (None without ``want_stats``). The kernels take the LayerNorm parameters
    and the conv parameters in one dtype: when they differ (fp32 ``nn.LayerNorm`` parameters beside bf16 taps, say), all
    of them go in as fp32 for this call, so that no parameter is rounded."""
    T, C, K, S = _check(x, cu_seqlens, ln_weight, ln_bias, weight, bias)
    lib = _lib.load()
    x = x.contiguous()
    wdt = _param_dtype(weight, ln_weight, ln_bias)
    weight = weight.to(wdt).contiguous()
    ln_weight = ln_weight.to(wdt).contiguous()
    ln_bias = None if ln_bias is None else ln_bias.to(wdt).contiguous()
    bias = None if bias is None else bias.to(wdt).contiguous()
    y = torch.empty_like(x)
    stats = torch.empty((T, 2), dtype=torch.float32, device=x.device)    # also what the two kernels of wide rows share
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
    return y, (stats if want_stats else None)


def ln_dwconv_bwd(x, dy, cu_seqlens, stats, ln_weight, ln_bias, weight, *, residual: bool = False, grads_bf16: bool = False):
    """Raw backward of :func:`ln_dwconv_fwd`: ``(dx, dln_weight, dln_bias, dw, db)``; dx in x's dtype, the rest fp32
    (dln_bias None without ``ln_bias``). ``stats`` is the forward's ``[T, 2]`` (mean, rstd).

    With ``grads_bf16`` the four parameter gradients come back in bf16, rounded once by the reduction kernel.

    Fused shapes: the conv backward normalises x as it reads it (the normalised tensor is never stored) and sums the
    LayerNorm parameter gradients beside dw and db; dx comes from the same kernel (rows of at most 4 KiB) or from one
    more pass over (x, dn, dy). Other shapes compose
    elementwise normalisation in fp32, the plain HIP conv backward and ATen's LayerNorm backward."""
    T, C, K, S = _check(x, cu_seqlens, ln_weight, ln_bias, weight, None)
    if dy.shape != x.shape or dy.dtype != x.dtype or dy.device != x.device:
        raise ValueError("dy must match x in shape, dtype and device")
    if stats is None or tuple(stats.shape) != (T, 2) or stats.dtype != torch.float32:
        raise ValueError(f"stats must be the forward's [T={T}, 2] fp32 (mean, rstd)")
    lib = _lib.load()
    x = x.contiguous()
    dy = dy.contiguous()
    stats = stats.contiguous()
    wdt = _param_dtype(weight, ln_weight, ln_bias)
    weight = weight.to(wdt).contiguous()
    lnw = ln_weight.to(wdt).contiguous()
    lnb = None if ln_bias is None else ln_bias.to(wdt).contiguous()
    act = _DTYPES[x.dtype]
    nbytes = int(lib.nplm_dwconv_ln_bwd_workspace_bytes(T, C, K, act)) if T > 0 else 0
    if nbytes > 0 or T == 0:
        dx = torch.empty_like(x)
        gdt = torch.bfloat16 if grads_bf16 else torch.float32
        dw = torch.empty((C, K), dtype=gdt, device=x.device)
        db = torch.empty((C,), dtype=gdt, device=x.device)
        dg = torch.empty((C,), dtype=gdt, device=x.device)
        dbeta = None if ln_bias is None else torch.empty((C,), dtype=gdt, device=x.device)
        with _launch_on(x) as dev:
            workspace = torch.empty((max(nbytes, 256),), dtype=torch.uint8, device=x.device)
            rc = lib.nplm_dwconv_ln_bwd(_ptr(x), _ptr(dy), _ptr(cu_seqlens.contiguous()), _ptr(stats), _ptr(lnw), _ptr(lnb),
                                        _ptr(weight), _ptr(dx), _ptr(dw), _ptr(db), _ptr(dg), _ptr(dbeta), _ptr(workspace),
                                        workspace.numel(), T, C, K, S, act, _DTYPES[wdt],
                                        (_lib.RESIDUAL if residual else 0) | (_lib.GRADS_BF16 if grads_bf16 else 0), dev.stream)
        if rc != -_lib.EUNSUPPORTED:
            _lib.check(rc, "nplm_dwconv_ln_bwd")
            return dx, dg, dbeta, dw, db
    mean, rstd = stats[:, 0:1].contiguous(), stats[:, 1:2].contiguous()     # ATen reads them as dense [T, 1]
    xf = x.float()
    gf = lnw.float()
    n = (xf - mean) * rstd * gf
    if lnb is not None:
        n = n + lnb.float()
    dyf = dy.float()
    dn, dw, db = varlen_dwconv_bwd(n, dyf, cu_seqlens, weight)
    dx, dg, dbeta = torch.ops.aten.native_layer_norm_backward(dn, xf, [C], mean, rstd, gf, None if lnb is None else lnb.float(),
                                                              [True, True, lnb is not None])
    if residual:
        dx = dx + dyf
    if grads_bf16:
        dg, dw, db = dg.bfloat16(), dw.bfloat16(), db.bfloat16()
        dbeta = None if dbeta is None else dbeta.bfloat16()
    return dx.to(x.dtype), dg, (dbeta if lnb is not None else None), dw, db


def _all_bf16(ln_weight, ln_bias, weight, bias_dtype) -> bool:
    """Every parameter is bf16: their gradients can come in bf16 straight from the reduction kernel."""
    return (weight.dtype == torch.bfloat16 and ln_weight.dtype == torch.bfloat16 and bias_dtype in (None, torch.bfloat16)
            and (ln_bias is None or ln_bias.dtype == torch.bfloat16))


class LnVarlenDWConv1dFunction(torch.autograd.Function):
    """y = conv(layer_norm(x; ln_weight, ln_bias); weight, bias) (+ x): gradients for x, ln_weight, ln_bias, weight,
    bias. Forward and backward fused where the library has the kernels (see the module docstring)."""

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
        if dy.dtype != x.dtype:
            dy = dy.to(x.dtype)
        dx, dg, dbeta, dw, db = ln_dwconv_bwd(x, dy, cu, stats, ln_weight, ln_bias, weight, residual=ctx.residual,
                                              grads_bf16=_all_bf16(ln_weight, ln_bias, weight, ctx.bias_dtype))
        return (dx, None, dg.to(ln_weight.dtype), None if ln_bias is None else dbeta.to(ln_bias.dtype),
                dw.to(weight.dtype), db.to(ctx.bias_dtype) if ctx.has_bias else None, None, None)


def ln_varlen_dwconv(x, cu_seqlens, ln_weight, ln_bias, weight, bias=None, *, eps: float = 1e-5, residual: bool = False):
    """Differentiable ``conv(layer_norm(x))`` (``+ x`` with ``residual``) over packed sequences."""
    return LnVarlenDWConv1dFunction.apply(x, cu_seqlens, ln_weight, ln_bias, weight, bias, eps, residual)


# ---------------------------------------------------------------------------------------------
# torch.library registration of the pair, so that a compiled model (torch.compile(dynamic=False),
# src/nanoplm/pretraining/pure_pipeline.py:519-524) keeps one graph. Neither op synchronises the host.
# ---------------------------------------------------------------------------------------------
@torch.library.custom_op("nanoplm_amd::ln_dwconv_fwd", mutates_args=(), device_types="cuda")
def ln_dwconv_fwd_op(x: torch.Tensor, cu_seqlens: torch.Tensor, ln_weight: torch.Tensor, ln_bias: Optional[torch.Tensor],
                     weight: torch.Tensor, bias: Optional[torch.Tensor], eps: float = 1e-5,
                     residual: bool = False) -> tuple[torch.Tensor, torch.Tensor]:
    """(y, stats)."""
    y, stats = ln_dwconv_fwd(x, cu_seqlens, ln_weight, ln_bias, weight, bias, eps=eps, residual=residual)
    return y, stats


@ln_dwconv_fwd_op.register_fake
def _(x, cu_seqlens, ln_weight, ln_bias, weight, bias, eps=1e-5, residual=False):
    return torch.empty_like(x, memory_format=torch.contiguous_format), x.new_empty((x.shape[0], 2), dtype=torch.float32)


@torch.library.custom_op("nanoplm_amd::ln_dwconv_bwd", mutates_args=(), device_types="cuda")
def ln_dwconv_bwd_op(x: torch.Tensor, dy: torch.Tensor, cu_seqlens: torch.Tensor, stats: torch.Tensor, ln_weight: torch.Tensor,
                     ln_bias: Optional[torch.Tensor], weight: torch.Tensor, residual: bool = False,
                     grads_bf16: bool = False) -> tuple[torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor]:
    """(dx, dln_weight, dln_bias, dw, db); dln_bias is zeros [C] without ``ln_bias`` (an op returns tensors only)."""
    dx, dg, dbeta, dw, db = ln_dwconv_bwd(x, dy, cu_seqlens, stats, ln_weight, ln_bias, weight, residual=residual,
                                          grads_bf16=grads_bf16)
    if dbeta is None:
        dbeta = torch.zeros_like(dg)
    return dx, dg, dbeta, dw, db


@ln_dwconv_bwd_op.register_fake
def _(x, dy, cu_seqlens, stats, ln_weight, ln_bias, weight, residual=False, grads_bf16=False):
    C, K = weight.shape
    f = lambda *shape: x.new_empty(shape, dtype=torch.bfloat16 if grads_bf16 else torch.float32)
    return torch.empty_like(x, memory_format=torch.contiguous_format), f(C), f(C), f(C, K), f(C)


def _ln_setup_context(ctx, inputs, output):
    x, cu_seqlens, ln_weight, ln_bias, weight, bias, eps, residual = inputs
    ctx.save_for_backward(x, cu_seqlens, ln_weight, ln_bias, weight, output[1])
    ctx.bias_dtype = None if bias is None else bias.dtype
    ctx.residual = bool(residual)
    ctx.set_materialize_grads(False)


def _ln_backward(ctx, dy, _dstats):
    x, cu_seqlens, ln_weight, ln_bias, weight, stats = ctx.saved_tensors
    if dy is None:
        dy = torch.zeros_like(x)
    if dy.dtype != x.dtype:
        dy = dy.to(x.dtype)
    dx, dg, dbeta, dw, db = ln_dwconv_bwd_op(x, dy.contiguous(), cu_seqlens, stats, ln_weight, ln_bias, weight, ctx.residual,
                                             _all_bf16(ln_weight, ln_bias, weight, ctx.bias_dtype))
    return (dx, None, dg.to(ln_weight.dtype), None if ln_bias is None else dbeta.to(ln_bias.dtype), dw.to(weight.dtype),
            None if ctx.bias_dtype is None else db.to(ctx.bias_dtype), None, None)


ln_dwconv_fwd_op.register_autograd(_ln_backward, setup_context=_ln_setup_context)


def ln_varlen_dwconv_compilable(x, cu_seqlens, ln_weight, ln_bias, weight, bias=None, *, eps: float = 1e-5,
                                residual: bool = False):
    """Same result as :func:`ln_varlen_dwconv`, routed through the registered custom ops (traceable)."""
    return ln_dwconv_fwd_op(x, cu_seqlens, ln_weight, ln_bias, weight, bias, eps, residual)[0]


def ln_supported(x: torch.Tensor, weight: torch.Tensor) -> bool:
    """Whether the fused kernels take this call (K in {3,5,7,9}, rows of at most 8 KiB in multiples of 16 bytes,
    16-byte aligned contiguous x on a ROCm device). Informational: ``ln_dwconv_fwd`` finds out from the library."""
    if not (isinstance(x, torch.Tensor) and x.is_cuda and x.dim() == 2 and x.dtype in _DTYPES and weight.dtype in _DTYPES):
        return False
    rb = x.shape[1] * x.element_size()
    return weight.shape[1] in (3, 5, 7, 9) and rb % 16 == 0 and rb <= 8192 and x.is_contiguous() and x.data_ptr() % 16 == 0
