"""Gated depthwise conv: ``conv(x_proj * silu(gate))`` with the gate product fused into the kernels.

For a conv placed inside the reference's SwiGLU MLP
(src/nanoplm/pretraining/models/modern_bert/modeling.py:300-302)::

    x_proj, gate = self.Wi(x).chunk(2, dim=-1)
    h = F.silu(gate) * x_proj            # [T, intermediate]
    h = conv(h, cu_seqlens)              # <- here
    return self.Wo(self.drop(h))

``gated_varlen_dwconv(z, cu_seqlens, weight, bias)`` takes ``z = self.Wi(x)`` (``[T, 2C]``: x_proj in
columns ``[0, C)``, gate in ``[C, 2C)``) and returns ``conv(h)`` ``[T, C]`` without ever writing ``h``:
the forward reads z once and writes y, the backward reads z and dy and writes dz = [d x_proj | d gate],
dw and db. Shapes the fused kernels are not built for (the library says so with its return code) run the
same HIP conv after the gate product is formed with ordinary elementwise GPU ops.
"""
from __future__ import annotations

from typing import Optional

import torch

from . import _lib
from .dwconv import _DTYPES, _launch_on, _ptr, varlen_dwconv_bwd, varlen_dwconv_fwd


def gated_supported(z: torch.Tensor, weight: torch.Tensor) -> bool:
    """Whether the fused kernels take this call (an odd kernel size up to 31, rows of C*elemsize >= 1 KiB
    in multiples of 16 bytes, 16-byte aligned contiguous z on a ROCm device). Informational: the entry
    points below find out from the library's return code."""
    if not (isinstance(z, torch.Tensor) and z.is_cuda and z.dim() == 2 and z.shape[1] % 2 == 0):
        return False
    if z.dtype not in _DTYPES or weight.dtype not in _DTYPES or not z.is_contiguous() or z.data_ptr() % 16:
        return False
    T, C2 = z.shape
    K = weight.shape[1]
    return int(_lib.load().nplm_dwconv_gated_bwd_workspace_bytes(max(T, 1), C2 // 2, K, _DTYPES[z.dtype])) > 0


def _check(z, cu_seqlens, weight, bias):
    if z.dim() != 2 or z.shape[1] % 2:
        raise ValueError("z must be [T, 2C]: x_proj columns followed by gate columns")
    if not z.is_cuda:
        raise RuntimeError(f"gated_varlen_dwconv runs only on a ROCm device (z is on {z.device}); there is no CPU implementation")
    T, C = z.shape[0], z.shape[1] // 2
    if tuple(weight.shape[:1]) != (C,) or weight.dim() != 2:
        raise ValueError(f"weight must be [C={C}, K], got {tuple(weight.shape)}")
    if bias is not None and tuple(bias.shape) != (C,):
        raise ValueError(f"bias must be [C={C}], got {tuple(bias.shape)}")
    if cu_seqlens.dtype != torch.int32 or cu_seqlens.dim() != 1 or cu_seqlens.numel() < 1:
        raise TypeError("cu_seqlens must be a 1-D int32 tensor with at least one entry")
    return T, C, weight.shape[1], cu_seqlens.numel() - 1


def _gate_terms(z):
    """fp32 pieces of h = x_proj * silu(gate): (x_proj, gate * sigmoid(gate), sigmoid(gate), gate)."""
    u, g = z.chunk(2, dim=-1)
    uf, gf = u.float(), g.float()
    sg = torch.sigmoid(gf)
    return uf, gf * sg, sg, gf


def gated_dwconv_fwd(z, cu_seqlens, weight, bias=None, *, residual: bool = False):
    """Raw forward (no autograd): y [T, C] = conv(z[:, :C] * silu(z[:, C:])).

    Fused kernels where the library has them; a shape it reports as unsupported (other kernel sizes, rows
    under 1 KiB or not a multiple of 16 bytes, a view that is not 16-byte aligned) forms the gate product
    with elementwise GPU ops and runs the plain HIP conv on it (h is then rounded once to z's dtype)."""
    T, C, K, S = _check(z, cu_seqlens, weight, bias)
    lib = _lib.load()
    z = z.contiguous()
    weight = weight.contiguous()
    if bias is not None:
        bias = bias.to(weight.dtype).contiguous()
    y = torch.empty((T, C), dtype=z.dtype, device=z.device)
    with _launch_on(z) as dev:
        rc = lib.nplm_dwconv_gated_fwd(_ptr(z), _ptr(cu_seqlens.contiguous()), _ptr(weight), _ptr(bias), _ptr(y), T, C, K, S,
                                       _DTYPES[z.dtype], _DTYPES[weight.dtype], _lib.RESIDUAL if residual else 0,
                                       dev.stream)
    if rc == -_lib.EUNSUPPORTED:
        uf, gs, _, _ = _gate_terms(z)
        return varlen_dwconv_fwd((uf * gs).to(z.dtype), cu_seqlens, weight, bias, residual=residual)
    _lib.check(rc, "nplm_dwconv_gated_fwd")
    return y


def gated_dwconv_bwd(z, dy, cu_seqlens, weight, *, residual: bool = False, grads_bf16: bool = False):
    """Raw backward: (dz [T, 2C] in z's dtype, dw [C, K] fp32, db [C] fp32); unsupported shapes as in the forward.
    With ``grads_bf16`` dw and db come back in bf16, rounded once by the reduction kernel that forms them."""
    T, C, K, S = _check(z, cu_seqlens, weight, None)
    if tuple(dy.shape) != (T, C) or dy.dtype != z.dtype or dy.device != z.device:
        raise ValueError("dy must be [T, C] in z's dtype on z's device")
    lib = _lib.load()
    z = z.contiguous()
    dy = dy.contiguous()
    weight = weight.contiguous()
    act = _DTYPES[z.dtype]
    with _launch_on(z) as dev:
        nbytes = int(lib.nplm_dwconv_gated_bwd_workspace_bytes(T, C, K, act))
        rc = -_lib.EUNSUPPORTED
        if nbytes > 0 or T == 0:
            dz = torch.empty_like(z)
            gdt = torch.bfloat16 if grads_bf16 else torch.float32
            dw = torch.empty((C, K), dtype=gdt, device=z.device)
            db = torch.empty((C,), dtype=gdt, device=z.device)
            ws = torch.empty((max(nbytes, 256),), dtype=torch.uint8, device=z.device)
            rc = lib.nplm_dwconv_gated_bwd(_ptr(z), _ptr(dy), _ptr(cu_seqlens.contiguous()), _ptr(weight), _ptr(dz), _ptr(dw),
                                           _ptr(db), _ptr(ws), ws.numel(), T, C, K, S, act, _DTYPES[weight.dtype],
                                           (_lib.RESIDUAL if residual else 0) | (_lib.GRADS_BF16 if grads_bf16 else 0),
                                           dev.stream)
    if rc == -_lib.EUNSUPPORTED:
        uf, gs, sg, gf = _gate_terms(z)
        dh, dw, db = varlen_dwconv_bwd((uf * gs).to(z.dtype), dy, cu_seqlens, weight, residual=residual, grads_bf16=grads_bf16)
        dhf = dh.float()
        dz = torch.cat((dhf * gs, dhf * uf * sg * (1.0 + gf * (1.0 - sg))), dim=-1).to(z.dtype)
        return dz, dw, db
    _lib.check(rc, "nplm_dwconv_gated_bwd")
    return dz, dw, db


class GatedVarlenDWConv1dFunction(torch.autograd.Function):
    """``apply(z, cu_seqlens, weight, bias, residual) -> y``; backward returns ``(dz, None, dw, db, None)``."""

    @staticmethod
    def forward(ctx, z, cu_seqlens, weight, bias=None, residual=False):
        y = gated_dwconv_fwd(z, cu_seqlens, weight, bias, residual=bool(residual))
        ctx.save_for_backward(z, cu_seqlens, weight)
        ctx.bias_dtype = None if bias is None else bias.dtype
        ctx.residual = bool(residual)
        return y

    @staticmethod
    def backward(ctx, dy):
        z, cu_seqlens, weight = ctx.saved_tensors
        if dy.dtype != z.dtype:
            dy = dy.to(z.dtype)
        grads_bf16 = weight.dtype == torch.bfloat16 and ctx.bias_dtype in (None, torch.bfloat16)
        dz, dw, db = gated_dwconv_bwd(z, dy, cu_seqlens, weight, residual=ctx.residual, grads_bf16=grads_bf16)
        return (dz if ctx.needs_input_grad[0] else None, None,
                dw.to(weight.dtype) if ctx.needs_input_grad[2] else None,
                db.to(ctx.bias_dtype) if (ctx.bias_dtype is not None and ctx.needs_input_grad[3]) else None, None)


def gated_varlen_dwconv(z: torch.Tensor, cu_seqlens: torch.Tensor, weight: torch.Tensor,
                        bias: Optional[torch.Tensor] = None, residual: bool = False) -> torch.Tensor:
    """``conv(z[:, :C] * silu(z[:, C:]))`` over packed sequences, ``[T, 2C] -> [T, C]``.

    Under ``torch.compile`` the call goes through the registered custom ops (opaque to the tracer, no graph
    break, any shape); otherwise through the autograd Function. Both run the same two raw entry points."""
    if torch.compiler.is_compiling():
        return gated_dwconv_fwd_op(z, cu_seqlens, weight, bias, residual)
    return GatedVarlenDWConv1dFunction.apply(z, cu_seqlens, weight, bias, residual)


# ---------------------------------------------------------------------------------------------
# torch.library registration of the fused pair, so that a compiled model
# (torch.compile(dynamic=False), src/nanoplm/pretraining/pure_pipeline.py:519-524) keeps one graph.
# ---------------------------------------------------------------------------------------------
@torch.library.custom_op("nanoplm_amd::gated_dwconv_fwd", mutates_args=(), device_types="cuda")
def gated_dwconv_fwd_op(z: torch.Tensor, cu_seqlens: torch.Tensor, weight: torch.Tensor,
                        bias: Optional[torch.Tensor], residual: bool = False) -> torch.Tensor:
    return gated_dwconv_fwd(z, cu_seqlens, weight, bias, residual=residual)


@gated_dwconv_fwd_op.register_fake
def _(z, cu_seqlens, weight, bias, residual=False):
    return z.new_empty((z.shape[0], z.shape[1] // 2))


@torch.library.custom_op("nanoplm_amd::gated_dwconv_bwd", mutates_args=(), device_types="cuda")
def gated_dwconv_bwd_op(z: torch.Tensor, dy: torch.Tensor, cu_seqlens: torch.Tensor, weight: torch.Tensor,
                        residual: bool = False, grads_bf16: bool = False) -> tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    dz, dw, db = gated_dwconv_bwd(z, dy, cu_seqlens, weight, residual=residual, grads_bf16=grads_bf16)
    return dz, dw, db


@gated_dwconv_bwd_op.register_fake
def _(z, dy, cu_seqlens, weight, residual=False, grads_bf16=False):
    C, K = weight.shape
    gdt = torch.bfloat16 if grads_bf16 else torch.float32
    return (torch.empty_like(z, memory_format=torch.contiguous_format),
            z.new_empty((C, K), dtype=gdt), z.new_empty((C,), dtype=gdt))


def _gated_setup_context(ctx, inputs, output):
    z, cu_seqlens, weight, bias, residual = inputs
    ctx.save_for_backward(z, cu_seqlens, weight)
    ctx.bias_dtype = None if bias is None else bias.dtype
    ctx.residual = bool(residual)


def _gated_backward(ctx, dy):
    z, cu_seqlens, weight = ctx.saved_tensors
    if dy.dtype != z.dtype:
        dy = dy.to(z.dtype)
    grads_bf16 = weight.dtype == torch.bfloat16 and ctx.bias_dtype in (None, torch.bfloat16)
    dz, dw, db = gated_dwconv_bwd_op(z, dy.contiguous(), cu_seqlens, weight, ctx.residual, grads_bf16)
    return dz, None, dw.to(weight.dtype), (None if ctx.bias_dtype is None else db.to(ctx.bias_dtype)), None


gated_dwconv_fwd_op.register_autograd(_gated_backward, setup_context=_gated_setup_context)
