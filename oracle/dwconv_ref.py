"""Reference path and cross-checks for the varlen depthwise conv -- TEST INFRASTRUCTURE ONLY.

The product (nanoplm_amd) never imports this module. It holds three independent statements of
the same operator, used to pin one another and then to check the HIP kernels:

* ``ref_dwconv_varlen`` / ``ref_dwconv_varlen_grads`` -- the reference path: a Python loop over the
  sequences of the packed tensor calling ``torch.nn.functional.conv1d(..., padding=(K-1)//2,
  groups=C)`` and autograd for the gradients. The reference snapshot (peymanvahidi/nanoplm 0.1.6)
  holds no convolution, so this loop follows no reference function; its arithmetic is torch's
  (``torch>=2.8.0``, /root/reference/pyproject.toml:39). Tensor layout and ``cu_seqlens`` follow
  /root/reference/src/nanoplm/pretraining/models/modern_bert/modeling.py:339 and
  /root/reference/src/nanoplm/pretraining/collator.py:308-325.
* ``c_oracle_fwd`` / ``c_oracle_bwd`` -- ctypes bindings of oracle/dwconv_oracle.c (definition,
  double accumulation, OpenMP), fast enough for the full benchmark sizes.
* ``brute_force`` -- pure-Python loops in exact rational-free float64, for tiny cases.

Parity status: pinned by tests/test_oracle.py (library routine vs C vs brute force, closed forms,
adjoint identities, finite differences, golden vectors).
"""
from __future__ import annotations

import ctypes
import os
import subprocess

import numpy as np
import torch
import torch.nn.functional as F

_HERE = os.path.dirname(os.path.abspath(__file__))
_C_LIB_PATH = os.path.join(_HERE, "build", "libdwconv_oracle.so")
_c_lib = None


# --------------------------------------------------------------------------------------------
# reference path: per-sequence F.conv1d
# --------------------------------------------------------------------------------------------
def ref_dwconv_varlen(x, cu_seqlens, weight, bias=None, compute_dtype=torch.float32, residual=False):
    """y[T, C] of the per-sequence conv1d loop, computed in ``compute_dtype`` on x's device.

    ``residual``: the caller-side residual connection ``x + conv(x)`` written as a separate add, the
    way an encoder layer applies its sub-modules (modeling.py:421-439)."""
    T, C = x.shape
    K = weight.shape[1]
    assert K % 2 == 1, "same-length output needs an odd kernel size"
    cu = [int(v) for v in cu_seqlens.tolist()]
    assert cu[0] == 0 and cu[-1] == T, "cu_seqlens must start at 0 and end at T"
    xw = x.to(compute_dtype)
    ww = weight.to(compute_dtype)[:, None, :]
    bw = None if bias is None else bias.to(compute_dtype)
    outs = []
    for s, e in zip(cu[:-1], cu[1:]):
        if e == s:
            continue
        xs = xw[s:e].transpose(0, 1)[None]                      # [1, C, L]
        ys = F.conv1d(xs, ww, bw, padding=(K - 1) // 2, groups=C)
        outs.append(ys[0].transpose(0, 1))
    if not outs:
        return xw.new_zeros((0, C))
    y = torch.cat(outs, dim=0)
    return xw + y if residual else y


def ref_dwconv_varlen_grads(x, cu_seqlens, weight, bias, dy, compute_dtype=torch.float32, residual=False):
    """(y, dx, dw, db) of the reference path via autograd, all in ``compute_dtype``."""
    xr = x.detach().to(compute_dtype).requires_grad_(True)
    wr = weight.detach().to(compute_dtype).requires_grad_(True)
    br = None if bias is None else bias.detach().to(compute_dtype).requires_grad_(True)
    y = ref_dwconv_varlen(xr, cu_seqlens, wr, br, compute_dtype, residual)
    y.backward(dy.to(compute_dtype))
    db = None if br is None else br.grad
    return y.detach(), xr.grad, wr.grad, db


def ref_gated_dwconv_grads(z, cu_seqlens, weight, bias, dy, compute_dtype=torch.float64, residual=False):
    """(y, dz, dw, db) of the reference MLP's gate product followed by the conv loop:
    ``x_proj, gate = z.chunk(2, -1); h = F.silu(gate) * x_proj`` (modeling.py:300-302), then
    ``ref_dwconv_varlen(h)``, gradients by autograd, everything in ``compute_dtype``."""
    zr = z.detach().to(compute_dtype).requires_grad_(True)
    wr = weight.detach().to(compute_dtype).requires_grad_(True)
    br = None if bias is None else bias.detach().to(compute_dtype).requires_grad_(True)
    x_proj, gate = zr.chunk(2, dim=-1)
    h = F.silu(gate) * x_proj
    y = ref_dwconv_varlen(h, cu_seqlens, wr, br, compute_dtype, residual)
    if dy is None:
        return y.detach()
    y.backward(dy.to(compute_dtype))
    return y.detach(), zr.grad, wr.grad, (None if br is None else br.grad)


def ref_ln_dwconv_grads(x, cu_seqlens, ln_weight, ln_bias, weight, bias, dy, eps=1e-5, compute_dtype=torch.float64,
                        residual=False):
    """(y, dx, d ln_weight, d ln_bias, dw, db) of a conv sub-module in the reference's pre-norm layer
    (``x + attn(attn_norm(x))``, modeling.py:404-438, the norm a ``torch.nn.LayerNorm`` over the hidden dimension,
    modeling.py:408-414): ``F.layer_norm`` over the channels, then ``ref_dwconv_varlen``, plus the raw x with
    ``residual``; gradients by autograd, everything in ``compute_dtype``. With ``dy=None`` only y."""
    xr = x.detach().to(compute_dtype).requires_grad_(True)
    gr = ln_weight.detach().to(compute_dtype).requires_grad_(True)
    hr = None if ln_bias is None else ln_bias.detach().to(compute_dtype).requires_grad_(True)
    wr = weight.detach().to(compute_dtype).requires_grad_(True)
    br = None if bias is None else bias.detach().to(compute_dtype).requires_grad_(True)
    n = F.layer_norm(xr, (xr.shape[1],), gr, hr, eps)
    y = ref_dwconv_varlen(n, cu_seqlens, wr, br, compute_dtype, False)
    if residual:
        y = y + xr
    if dy is None:
        return y.detach()
    y.backward(dy.to(compute_dtype))
    return (y.detach(), xr.grad, gr.grad, None if hr is None else hr.grad, wr.grad, None if br is None else br.grad)


# --------------------------------------------------------------------------------------------
# C oracle (definition, double accumulation)
# --------------------------------------------------------------------------------------------
def build_c_oracle(force=False):
    """Compile oracle/dwconv_oracle.c with gcc (a few hundred ms)."""
    if force or not os.path.exists(_C_LIB_PATH):
        subprocess.run(["make", "-B", "-C", _HERE], check=True, capture_output=True)
    return _C_LIB_PATH


def _load_c():
    global _c_lib
    if _c_lib is None:
        build_c_oracle()
        lib = ctypes.CDLL(_C_LIB_PATH)
        fp = ctypes.POINTER(ctypes.c_float)
        dp = ctypes.POINTER(ctypes.c_double)
        ip = ctypes.POINTER(ctypes.c_int32)
        lib.nplm_oracle_dwconv_fwd.argtypes = [fp, ip, fp, fp, dp, ctypes.c_int64, ctypes.c_int32,
                                               ctypes.c_int32, ctypes.c_int32]
        lib.nplm_oracle_dwconv_fwd.restype = ctypes.c_int
        lib.nplm_oracle_dwconv_bwd.argtypes = [fp, fp, ip, fp, dp, dp, dp, ctypes.c_int64, ctypes.c_int32,
                                               ctypes.c_int32, ctypes.c_int32]
        lib.nplm_oracle_dwconv_bwd.restype = ctypes.c_int
        _c_lib = lib
    return _c_lib


def _f32(t):
    return np.ascontiguousarray(t.detach().to("cpu", torch.float32).numpy())


def _ptr(a, ct):
    return None if a is None else a.ctypes.data_as(ctypes.POINTER(ct))


def c_oracle_fwd(x, cu_seqlens, weight, bias=None, residual=False):
    """float64 y[T, C] (torch, CPU) from the C restatement; inputs are upcast to fp32 first.
    ``residual`` adds x (in float64) to the result."""
    lib = _load_c()
    xa, wa = _f32(x), _f32(weight)
    ba = None if bias is None else _f32(bias)
    cua = np.ascontiguousarray(cu_seqlens.detach().cpu().numpy().astype(np.int32))
    T, C = xa.shape
    K = wa.shape[1]
    y = np.empty((T, C), dtype=np.float64)
    rc = lib.nplm_oracle_dwconv_fwd(_ptr(xa, ctypes.c_float), _ptr(cua, ctypes.c_int32), _ptr(wa, ctypes.c_float),
                                    _ptr(ba, ctypes.c_float), _ptr(y, ctypes.c_double), T, C, K, len(cua) - 1)
    if rc:
        raise ValueError("C oracle rejected its inputs (cu_seqlens malformed or K even)")
    if residual:
        y += xa
    return torch.from_numpy(y)


def c_oracle_bwd(x, dy, cu_seqlens, weight, residual=False):
    """float64 (dx[T,C], dw[C,K], db[C]) from the C restatement; ``residual`` adds dy to dx."""
    lib = _load_c()
    xa, ga, wa = _f32(x), _f32(dy), _f32(weight)
    cua = np.ascontiguousarray(cu_seqlens.detach().cpu().numpy().astype(np.int32))
    T, C = xa.shape
    K = wa.shape[1]
    dx = np.empty((T, C), dtype=np.float64)
    dw = np.empty((C, K), dtype=np.float64)
    db = np.empty((C,), dtype=np.float64)
    rc = lib.nplm_oracle_dwconv_bwd(_ptr(xa, ctypes.c_float), _ptr(ga, ctypes.c_float), _ptr(cua, ctypes.c_int32),
                                    _ptr(wa, ctypes.c_float), _ptr(dx, ctypes.c_double), _ptr(dw, ctypes.c_double),
                                    _ptr(db, ctypes.c_double), T, C, K, len(cua) - 1)
    if rc:
        raise ValueError("C oracle rejected its inputs (cu_seqlens malformed or K even)")
    if residual:
        dx += ga
    return torch.from_numpy(dx), torch.from_numpy(dw), torch.from_numpy(db)


# --------------------------------------------------------------------------------------------
# brute force (tiny inputs only)
# --------------------------------------------------------------------------------------------
def brute_force(x, cu_seqlens, weight, bias, dy=None):
    """Pure-Python float64 loops over (sequence, row, channel, tap). Returns y or (y, dx, dw, db)."""
    xa = x.detach().cpu().double().numpy()
    wa = weight.detach().cpu().double().numpy()
    ba = None if bias is None else bias.detach().cpu().double().numpy()
    cu = [int(v) for v in cu_seqlens.tolist()]
    T, C = xa.shape
    K = wa.shape[1]
    P = (K - 1) // 2
    y = np.zeros((T, C))
    for s, e in zip(cu[:-1], cu[1:]):
        for t in range(s, e):
            for c in range(C):
                acc = 0.0 if ba is None else ba[c]
                for k in range(K):
                    j = t + k - P
                    if s <= j < e:
                        acc += wa[c, k] * xa[j, c]
                y[t, c] = acc
    if dy is None:
        return torch.from_numpy(y)
    ga = dy.detach().cpu().double().numpy()
    dx = np.zeros((T, C))
    dw = np.zeros((C, K))
    db = np.zeros((C,))
    # scatter form (each forward product sends its gradient to both operands): deliberately a
    # different loop structure from the gather form used by the C oracle and the kernels
    for s, e in zip(cu[:-1], cu[1:]):
        for t in range(s, e):
            for c in range(C):
                db[c] += ga[t, c]
                for k in range(K):
                    j = t + k - P
                    if s <= j < e:
                        dx[j, c] += wa[c, k] * ga[t, c]
                        dw[c, k] += xa[j, c] * ga[t, c]
    return torch.from_numpy(y), torch.from_numpy(dx), torch.from_numpy(dw), torch.from_numpy(db)
