"""Varlen depthwise 1-D convolution over packed sequences: autograd Function and nn.Module.

Drop-in surface for the conv on the packed path of the encoder layer
(reference call site: src/nanoplm/pretraining/models/modern_bert/modeling.py:421-439, which passes
``x:[total_tokens, hidden]`` and int32 ``cu_seqlens`` (collator.py:322-325) to its sub-modules):

    y = VarlenDWConv1dFunction.apply(x, cu_seqlens, weight, bias)
    conv = VarlenDWConv1d(channels=C, kernel_size=K);  y = conv(x, cu_seqlens)

``residual=True`` (function argument / module option) fuses the residual connection a caller would
write as ``x = x + conv(x, cu_seqlens)``: the kernels compute ``x + conv(x)`` and ``dy + conv^T(dy)``
directly, which saves the elementwise add's three passes over [T, C] in each direction.

All arithmetic runs in hand-written HIP kernels reached through the C ABI of libnplm_dwconv.so.
There is deliberately no CPU or pure-PyTorch implementation here: tensors that are not on a ROCm
device, or a missing shared library, raise.
"""
from __future__ import annotations

import math
from typing import Optional

import torch
from torch import nn

from . import _lib

_DTYPES = {torch.float32: _lib.F32, torch.bfloat16: _lib.BF16}


def _ptr(t: Optional[torch.Tensor]) -> Optional[int]:
    return None if t is None else t.data_ptr()


def _validate(x, cu_seqlens, weight, bias):
    """Shape/dtype/device checks shared by forward and backward. Returns (T, C, K, S)."""
    if not isinstance(x, torch.Tensor) or x.dim() != 2:
        raise ValueError("x must be a 2-D tensor [T, C] of packed tokens")
    if x.dtype not in _DTYPES:
        raise TypeError(f"x must be float32 or bfloat16, got {x.dtype}")
    if not x.is_cuda:
        raise RuntimeError("varlen_dwconv runs only on a ROCm device (x is on "
                           f"{x.device}); there is no CPU implementation")
    T, C = x.shape
    if weight.dim() != 2 or weight.shape[0] != C:
        raise ValueError(f"weight must be [C={C}, K], got {tuple(weight.shape)}")
    K = weight.shape[1]
    if K % 2 == 0:
        raise ValueError(f"kernel size must be odd for centred 'same' padding, got K={K}")
    if weight.dtype not in _DTYPES:
        raise TypeError(f"weight must be float32 or bfloat16, got {weight.dtype}")
    if bias is not None and tuple(bias.shape) != (C,):
        raise ValueError(f"bias must be [C={C}], got {tuple(bias.shape)}")
    if cu_seqlens.dtype != torch.int32 or cu_seqlens.dim() != 1 or cu_seqlens.numel() < 1:
        raise TypeError("cu_seqlens must be a 1-D int32 tensor with at least one entry")
    for name, t in (("cu_seqlens", cu_seqlens), ("weight", weight), ("bias", bias)):
        if t is not None and t.device != x.device:
            raise RuntimeError(f"{name} is on {t.device}, x is on {x.device}")
    return T, C, K, cu_seqlens.numel() - 1


def _with_flags(tuning: _lib.Tuning, flags: int) -> _lib.Tuning:
    t = _lib.Tuning.from_buffer_copy(tuning)
    t.flags = flags
    return t


def varlen_dwconv_fwd(x, cu_seqlens, weight, bias=None, *, residual: bool = False,
                      tuning: Optional[_lib.Tuning] = None):
    """y = conv(x), or x + conv(x) with ``residual`` (same dtype as x). Raw forward without autograd."""
    T, C, K, S = _validate(x, cu_seqlens, weight, bias)
    lib = _lib.load()
    x = x.contiguous()
    weight = weight.contiguous()
    cu_seqlens = cu_seqlens.contiguous()
    if bias is not None:
        bias = bias.to(weight.dtype).contiguous()
    y = torch.empty_like(x)
    with torch.cuda.device(x.device):
        stream = torch.cuda.current_stream().cuda_stream
        flags = _lib.RESIDUAL if residual else 0
        args = (_ptr(x), _ptr(cu_seqlens), _ptr(weight), _ptr(bias), _ptr(y), T, C, K, S,
                _DTYPES[x.dtype], _DTYPES[weight.dtype])
        if tuning is None:
            rc = lib.nplm_dwconv_fwd_ex(*args, flags, stream)
        else:
            rc = lib.nplm_dwconv_fwd_tuned(*args, stream, _with_flags(tuning, flags))
    _lib.check(rc, "nplm_dwconv_fwd")
    return y


def bwd_workspace_bytes(T: int, C: int, K: int, dtype: torch.dtype) -> int:
    """Bytes of workspace the backward needs for these sizes (host arithmetic only)."""
    return int(_lib.load().nplm_dwconv_bwd_workspace_bytes(T, C, K, _DTYPES[dtype]))


def varlen_dwconv_bwd(x, dy, cu_seqlens, weight, *, need_dx=True, need_dw=True, residual: bool = False,
                      tuning: Optional[_lib.Tuning] = None, workspace: Optional[torch.Tensor] = None):
    """(dx, dw, db): dx in x's dtype (or None), dw [C,K] and db [C] in fp32 (or None, None).

    With ``residual`` dx is the gradient of x + conv(x), i.e. dy + conv^T(dy); dw and db do not change."""
    T, C, K, S = _validate(x, cu_seqlens, weight, None)
    if dy.shape != x.shape or dy.dtype != x.dtype or dy.device != x.device:
        raise ValueError("dy must match x in shape, dtype and device")
    lib = _lib.load()
    x = x.contiguous()
    dy = dy.contiguous()
    weight = weight.contiguous()
    cu_seqlens = cu_seqlens.contiguous()
    act = _DTYPES[x.dtype]
    dx = torch.empty_like(x) if need_dx else None
    dw = torch.empty((C, K), dtype=torch.float32, device=x.device) if need_dw else None
    db = torch.empty((C,), dtype=torch.float32, device=x.device) if need_dw else None
    with torch.cuda.device(x.device):
        if need_dw and workspace is None:
            if tuning is None:
                nbytes = int(lib.nplm_dwconv_bwd_workspace_bytes(T, C, K, act))
            else:
                nbytes = int(lib.nplm_dwconv_bwd_slabs(T, C, K, act, tuning)) * (K + 1) * C * 4
            workspace = torch.empty((max(nbytes, 256),), dtype=torch.uint8, device=x.device)
        stream = torch.cuda.current_stream().cuda_stream
        flags = _lib.RESIDUAL if residual else 0
        args = (_ptr(x), _ptr(dy), _ptr(cu_seqlens), _ptr(weight), _ptr(dx), _ptr(dw), _ptr(db),
                _ptr(workspace), 0 if workspace is None else workspace.numel() * workspace.element_size(),
                T, C, K, S, act, _DTYPES[weight.dtype])
        if tuning is None:
            rc = lib.nplm_dwconv_bwd_ex(*args, flags, stream)
        else:
            rc = lib.nplm_dwconv_bwd_tuned(*args, stream, _with_flags(tuning, flags))
    _lib.check(rc, "nplm_dwconv_bwd")
    return dx, dw, db


def check_cu_seqlens(cu_seqlens: torch.Tensor, T: int) -> None:
    """Debug helper: verify cu[0] == 0, non-decreasing, cu[-1] == T (synchronises the stream)."""
    if not cu_seqlens.is_cuda or cu_seqlens.dtype != torch.int32:
        raise TypeError("cu_seqlens must be an int32 tensor on a ROCm device")
    lib = _lib.load()
    with torch.cuda.device(cu_seqlens.device):
        rc = lib.nplm_dwconv_check_cu(_ptr(cu_seqlens.contiguous()), cu_seqlens.numel() - 1, T,
                                      torch.cuda.current_stream().cuda_stream)
    _lib.check(rc, "nplm_dwconv_check_cu")


class VarlenDWConv1dFunction(torch.autograd.Function):
    """``apply(x, cu_seqlens, weight, bias[, residual]) -> y``; backward returns ``(dx, None, dw, db[, None])``.

    dw and db are reduced and produced in fp32 by the kernels and cast to the parameters' dtypes
    only here. Under ``torch.autocast`` the op takes its inputs as they come (bf16 activations
    with fp32 parameters is a supported combination), so no cast kernels are inserted.
    """

    @staticmethod
    def forward(ctx, x, cu_seqlens, weight, bias=None, residual=False):
        y = varlen_dwconv_fwd(x, cu_seqlens, weight, bias, residual=bool(residual))
        ctx.save_for_backward(x, cu_seqlens, weight)
        ctx.bias_dtype = None if bias is None else bias.dtype
        ctx.residual = bool(residual)
        return y

    @staticmethod
    def backward(ctx, dy):
        x, cu_seqlens, weight = ctx.saved_tensors
        need_dx = ctx.needs_input_grad[0]
        need_dw = ctx.needs_input_grad[2] or (ctx.bias_dtype is not None and ctx.needs_input_grad[3])
        if dy.dtype != x.dtype:
            dy = dy.to(x.dtype)
        dx, dw, db = varlen_dwconv_bwd(x, dy, cu_seqlens, weight, need_dx=need_dx, need_dw=need_dw,
                                       residual=ctx.residual)
        if dw is not None:
            dw = dw.to(weight.dtype) if ctx.needs_input_grad[2] else None
            db = db.to(ctx.bias_dtype) if (ctx.bias_dtype is not None and ctx.needs_input_grad[3]) else None
        return dx, None, dw, db, None


def varlen_dwconv(x, cu_seqlens, weight, bias=None, residual: bool = False):
    """Functional form of :class:`VarlenDWConv1dFunction`."""
    return VarlenDWConv1dFunction.apply(x, cu_seqlens, weight, bias, residual)


class VarlenDWConv1d(nn.Module):
    """Depthwise conv over packed sequences: ``forward(x:[T,C], cu_seqlens:int32[S+1]) -> [T,C]``.

    ``weight`` is ``[C, K]`` (tap k multiplies row ``t + k - (K-1)//2``), ``bias`` is ``[C]``.
    Rows outside a sequence read as zero; nothing crosses a sequence boundary.
    ``residual=True`` makes the module return ``x + conv(x)`` from the same single pass.
    """

    def __init__(self, channels: int, kernel_size: int, bias: bool = True, residual: bool = False,
                 device=None, dtype=None):
        super().__init__()
        if kernel_size < 1 or kernel_size % 2 == 0:
            raise ValueError(f"kernel_size must be odd and positive, got {kernel_size}")
        self.channels = channels
        self.kernel_size = kernel_size
        self.residual = bool(residual)
        self.weight = nn.Parameter(torch.empty((channels, kernel_size), device=device, dtype=dtype))
        self.bias = nn.Parameter(torch.empty((channels,), device=device, dtype=dtype)) if bias else None
        self.reset_parameters()

    def reset_parameters(self) -> None:
        # variance 1/K per tap, small bias: the distributions the benchmark configs draw from
        nn.init.normal_(self.weight, mean=0.0, std=1.0 / math.sqrt(self.kernel_size))
        if self.bias is not None:
            nn.init.normal_(self.bias, mean=0.0, std=0.02)

    def forward(self, x: torch.Tensor, cu_seqlens: torch.Tensor) -> torch.Tensor:
        if torch.compiler.is_compiling():
            # under torch.compile the opaque custom ops keep the graph whole
            return varlen_dwconv_fwd_op(x, cu_seqlens, self.weight, self.bias, self.residual)
        return VarlenDWConv1dFunction.apply(x, cu_seqlens, self.weight, self.bias, self.residual)

    def extra_repr(self) -> str:
        return (f"channels={self.channels}, kernel_size={self.kernel_size}, bias={self.bias is not None}, "
                f"residual={self.residual}")


# ---------------------------------------------------------------------------------------------
# torch.library registration: the same two kernels as opaque custom ops, so that
# torch.compile(model, dynamic=False) (src/nanoplm/pretraining/pure_pipeline.py:519-524) traces
# through a model that contains the conv without a graph break. Neither op synchronises the host;
# cu_seqlens may be the static collator's fixed-length tensor (collator.py:430-450).
# ---------------------------------------------------------------------------------------------
@torch.library.custom_op("nanoplm_amd::varlen_dwconv_fwd", mutates_args=(), device_types="cuda")
def varlen_dwconv_fwd_op(x: torch.Tensor, cu_seqlens: torch.Tensor, weight: torch.Tensor,
                         bias: Optional[torch.Tensor], residual: bool = False) -> torch.Tensor:
    return varlen_dwconv_fwd(x, cu_seqlens, weight, bias, residual=residual)


@varlen_dwconv_fwd_op.register_fake
def _(x, cu_seqlens, weight, bias, residual=False):
    return torch.empty_like(x, memory_format=torch.contiguous_format)


@torch.library.custom_op("nanoplm_amd::varlen_dwconv_bwd", mutates_args=(), device_types="cuda")
def varlen_dwconv_bwd_op(x: torch.Tensor, dy: torch.Tensor, cu_seqlens: torch.Tensor, weight: torch.Tensor,
                         residual: bool = False) -> tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    """(dx, dw, db) with dw [C,K] and db [C] in fp32."""
    dx, dw, db = varlen_dwconv_bwd(x, dy, cu_seqlens, weight, residual=residual)
    return dx, dw, db


@varlen_dwconv_bwd_op.register_fake
def _(x, dy, cu_seqlens, weight, residual=False):
    C, K = weight.shape
    return (torch.empty_like(x, memory_format=torch.contiguous_format),
            x.new_empty((C, K), dtype=torch.float32), x.new_empty((C,), dtype=torch.float32))


def _op_setup_context(ctx, inputs, output):
    x, cu_seqlens, weight, bias, residual = inputs
    ctx.save_for_backward(x, cu_seqlens, weight)
    ctx.bias_dtype = None if bias is None else bias.dtype
    ctx.residual = bool(residual)


def _op_backward(ctx, dy):
    x, cu_seqlens, weight = ctx.saved_tensors
    if dy.dtype != x.dtype:
        dy = dy.to(x.dtype)
    dx, dw, db = varlen_dwconv_bwd_op(x, dy.contiguous(), cu_seqlens, weight, ctx.residual)
    return dx, None, dw.to(weight.dtype), (None if ctx.bias_dtype is None else db.to(ctx.bias_dtype)), None


varlen_dwconv_fwd_op.register_autograd(_op_backward, setup_context=_op_setup_context)


def varlen_dwconv_compilable(x, cu_seqlens, weight, bias=None, residual: bool = False):
    """Same result as :func:`varlen_dwconv`, routed through the registered custom ops (traceable)."""
    return varlen_dwconv_fwd_op(x, cu_seqlens, weight, bias, residual)
