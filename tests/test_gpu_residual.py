"""Fused residual connection (y = x + conv(x), dx = dy + conv^T(dy)) against the oracle, through the
C ABI (nplm_dwconv_fwd_ex / nplm_dwconv_bwd_ex) and the autograd surface. The residual is the one an
encoder layer applies around its sub-modules (modeling.py:421-439)."""
import pytest
import torch

import nanoplm_amd as npa
from nanoplm_amd import _lib
from nanoplm_amd.workloads import cu_from_lengths
from oracle import dwconv_ref as O
from tests.gpu_util import assert_act_close, assert_red_close, workload_with_oracle

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
LENS_MIX = [1, 2, 3, 8, 0, 1, 150, 0, 5, 7, 6, 1, 64, 63, 65, 2, 300, 4]


def _case(lens, C, K, dt, wdt, seed):
    g = torch.Generator().manual_seed(seed)
    lens = torch.tensor(lens)
    T = int(lens.sum())
    x = torch.randn(T, C, generator=g).to(dt)
    w = (torch.randn(C, K, generator=g) * K ** -0.5).to(wdt)
    b = (torch.randn(C, generator=g) * 0.02).to(wdt)
    dy = torch.randn(T, C, generator=g).to(dt)
    return x, cu_from_lengths(lens), w, b, dy


def _check(x, cu, w, b, dy, what, tuning=None):
    y64 = O.c_oracle_fwd(x, cu, w, b, residual=True)
    dx64, dw64, db64 = O.c_oracle_bwd(x, dy, cu, w, residual=True)
    xd, cud, wd, bd, dyd = (t.to(DEV) for t in (x, cu, w, b, dy))
    y = npa.varlen_dwconv_fwd(xd, cud, wd, bd, residual=True, tuning=tuning)
    dx, dw, db = npa.varlen_dwconv_bwd(xd, dyd, cud, wd, residual=True, tuning=tuning)
    assert_act_close(y, y64, x.dtype, what + " y")
    assert_act_close(dx, dx64, x.dtype, what + " dx")
    assert_red_close(dw, dw64, what + " dw")
    assert_red_close(db, db64, what + " db")
    return y, dx, dw, db


@pytest.mark.parametrize("K", [1, 3, 7, 9, 11, 15, 31])
@pytest.mark.parametrize("dt", [torch.bfloat16, torch.float32])
def test_residual_kernel_sizes(K, dt):
    """LDS-staged (K <= 9), sliding-window (15, 31) and runtime-K (11) kernels."""
    print(f"[case] residual K={K} {dt}", flush=True)
    _check(*_case(LENS_MIX, 256 if K != 7 else 1024, K, dt, dt, seed=100 + K), f"residual K={K} {dt}")


@pytest.mark.parametrize("algo", [1, 2])
def test_residual_both_kernel_families_at_boundary_stress(algo):
    wl, *_ = workload_with_oracle(5, 20000, 1024)
    _check(wl.x, wl.cu_seqlens, wl.weight, wl.bias, wl.dy, f"residual algo={algo}", tuning=_lib.Tuning(algo=algo))


def test_residual_with_fp32_weights_under_bf16_activations():
    _check(*_case(LENS_MIX, 512, 7, torch.bfloat16, torch.float32, seed=5), "residual bf16/fp32")


def test_zero_weights_give_the_identity_exactly():
    """w = 0, b = 0: y == x and dx == dy bit for bit (the centre weight is exactly 1)."""
    x, cu, w, b, dy = _case(LENS_MIX, 1024, 7, torch.bfloat16, torch.bfloat16, seed=3)
    xd, cud, dyd = x.to(DEV), cu.to(DEV), dy.to(DEV)
    wz = torch.zeros_like(w).to(DEV)
    y = npa.varlen_dwconv_fwd(xd, cud, wz, None, residual=True)
    dx, dw, db = npa.varlen_dwconv_bwd(xd, dyd, cud, wz, residual=True)
    assert torch.equal(y, xd) and torch.equal(dx, dyd)
    # dw/db are those of the plain convolution
    _, dw0, db0 = npa.varlen_dwconv_bwd(xd, dyd, cud, wz)
    assert torch.equal(dw, dw0) and torch.equal(db, db0)


def test_residual_equals_centre_weight_plus_one_for_fp32():
    """x + conv(x; w) == conv(x; w + delta_centre): same kernels, so bit-identical when w + 1 is exact."""
    x, cu, w, b, dy = _case(LENS_MIX, 256, 5, torch.float32, torch.float32, seed=8)
    w = (w * 1024).round() / 1024           # w + 1 exactly representable
    w1 = w.clone()
    w1[:, 2] += 1.0
    xd, cud, bd, dyd = x.to(DEV), cu.to(DEV), b.to(DEV), dy.to(DEV)
    y_res = npa.varlen_dwconv_fwd(xd, cud, w.to(DEV), bd, residual=True)
    y_ref = npa.varlen_dwconv_fwd(xd, cud, w1.to(DEV), bd)
    dx_res, dw_res, _ = npa.varlen_dwconv_bwd(xd, dyd, cud, w.to(DEV), residual=True)
    dx_ref, dw_ref, _ = npa.varlen_dwconv_bwd(xd, dyd, cud, w1.to(DEV))
    assert torch.equal(y_res, y_ref) and torch.equal(dx_res, dx_ref) and torch.equal(dw_res, dw_ref)


def test_residual_module_autograd_matches_separate_add():
    """Module with residual=True against the unfused x + conv(x) through the same op (fp32: 1e-5)."""
    torch.manual_seed(0)
    lens = torch.tensor([17, 1, 250, 3, 90])
    cu = cu_from_lengths(lens).to(DEV)
    T = int(lens.sum())
    conv = npa.VarlenDWConv1d(256, 7, residual=True, device=DEV)
    plain = npa.VarlenDWConv1d(256, 7, device=DEV)
    plain.load_state_dict(conv.state_dict())
    x1 = torch.randn(T, 256, device=DEV, requires_grad=True)
    x2 = x1.detach().clone().requires_grad_(True)
    gy = torch.randn(T, 256, device=DEV)
    conv(x1, cu).backward(gy)
    (x2 + plain(x2, cu)).backward(gy)
    torch.testing.assert_close(x1.grad, x2.grad, rtol=1e-5, atol=1e-5)
    torch.testing.assert_close(conv.weight.grad, plain.weight.grad, rtol=1e-5, atol=1e-4)
    torch.testing.assert_close(conv.bias.grad, plain.bias.grad, rtol=1e-5, atol=1e-4)
    assert "residual=True" in repr(conv)


def test_residual_compiles_without_graph_breaks():
    lens = torch.tensor([40, 2, 300, 58])
    cu = cu_from_lengths(lens).to(DEV)
    T = int(lens.sum())
    conv = npa.VarlenDWConv1d(128, 7, residual=True, device=DEV, dtype=torch.bfloat16)
    x = torch.randn(T, 128, device=DEV, dtype=torch.bfloat16, requires_grad=True)
    eager = conv(x, cu)
    compiled = torch.compile(conv, backend="aot_eager", fullgraph=True, dynamic=False)
    out = compiled(x, cu)
    assert torch.equal(out, eager)
    out.float().sum().backward()
    assert x.grad is not None and torch.isfinite(x.grad.float()).all()


def test_unknown_flag_bits_are_rejected_before_any_launch():
    lib = _lib.load()
    x = torch.zeros(8, 64, device=DEV)
    cu = torch.tensor([0, 8], dtype=torch.int32, device=DEV)
    w = torch.zeros(64, 3, device=DEV)
    rc = lib.nplm_dwconv_fwd_ex(x.data_ptr(), cu.data_ptr(), w.data_ptr(), None, x.data_ptr(), 8, 64, 3, 1, 0, 0,
                                0x80, torch.cuda.current_stream().cuda_stream)
    assert rc == -9 and "flags" in _lib.strerror(rc)
