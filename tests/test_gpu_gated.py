"""Gated conv (conv over x_proj * silu(gate), the SwiGLU product of modeling.py:300-302, fused into the
kernels) against the float64 oracle, through the C ABI entry points and the autograd surface."""
import pytest
import torch
import torch.nn.functional as F

import nanoplm_amd as npa
from nanoplm_amd import _lib
from nanoplm_amd.workloads import cu_from_lengths, make_workload
from oracle import dwconv_ref as O
from tests.gpu_util import assert_act_close, assert_red_close

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
LENS_MIX = [1, 2, 3, 8, 0, 1, 150, 0, 5, 7, 6, 1, 64, 63, 65, 2, 300, 4, 17, 512]


def _case(lens, C, K, dt, wdt, seed):
    g = torch.Generator().manual_seed(seed)
    T = int(sum(lens))
    z = torch.randn(T, 2 * C, generator=g).to(dt)
    w = (torch.randn(C, K, generator=g) * K ** -0.5).to(wdt)
    b = (torch.randn(C, generator=g) * 0.02).to(wdt)
    dy = torch.randn(T, C, generator=g).to(dt)
    return z, cu_from_lengths(torch.tensor(lens)), w, b, dy


def _check(z, cu, w, b, dy, what, residual=False):
    y64, dz64, dw64, db64 = O.ref_gated_dwconv_grads(z, cu, w, b, dy, torch.float64, residual)
    zd, cud, wd, bd, dyd = (t.to(DEV) for t in (z, cu, w, b, dy))
    assert npa.gated_supported(zd, wd)
    y = npa.gated_dwconv_fwd(zd, cud, wd, bd, residual=residual)
    dz, dw, db = npa.gated_dwconv_bwd(zd, dyd, cud, wd, residual=residual)
    assert y.shape == dy.shape and dz.shape == z.shape
    assert_act_close(y, y64, z.dtype, what + " y")
    assert_act_close(dz, dz64, z.dtype, what + " dz")
    assert_red_close(dw, dw64, what + " dw")
    assert_red_close(db, db64, what + " db")


@pytest.mark.parametrize("K", [3, 5, 7, 9])
@pytest.mark.parametrize("dt,C", [(torch.bfloat16, 1024), (torch.bfloat16, 520), (torch.float32, 256), (torch.float32, 768),
                                   (torch.bfloat16, 1152), (torch.float32, 576)])
def test_gated_kernel_sizes_and_widths(K, dt, C):
    print(f"[case] gated K={K} C={C} {dt}", flush=True)
    _check(*_case(LENS_MIX, C, K, dt, dt, seed=K + C), f"gated K={K} C={C} {dt}")


LENS_LONG = LENS_MIX + [40, 33, 31, 30, 29, 16, 15, 14, 0, 1, 1, 700]


@pytest.mark.parametrize("K", [15, 31])
@pytest.mark.parametrize("dt,wdt,C", [(torch.bfloat16, torch.bfloat16, 1024), (torch.bfloat16, torch.float32, 2048),
                                       (torch.bfloat16, torch.bfloat16, 520), (torch.float32, torch.float32, 256),
                                       (torch.float32, torch.float32, 776), (torch.bfloat16, torch.bfloat16, 1152)])
def test_long_gated_kernel_sizes_and_widths(K, dt, wdt, C):
    """K = 15 and 31 (the intermediate-width configuration is C = 2048, K = 31): the forward forms the gate product in
    LDS once per staged element (rows of at least 512 bytes: every wave gates its share of a 128-row tile and then runs
    the taps; narrower rows: loader waves gate 32-row tiles); the backward is the role-split kernel with the gate in
    both roles (rows of at least 512 bytes) or the sliding-window kernel with the gate on its centre rows (C = 256 in
    bf16 would be; 520 takes column blocks of which the last is nearly empty)."""
    print(f"[case] long gated K={K} C={C} {dt} w {wdt}", flush=True)
    _check(*_case(LENS_LONG, C, K, dt, wdt, seed=K + C), f"gated K={K} C={C} {dt}")
    _check(*_case(LENS_LONG[::-1], C, K, dt, wdt, seed=K + C + 1), f"gated residual K={K} C={C} {dt}", residual=True)


def test_long_gated_is_deterministic_and_takes_the_boundary_stress_mix():
    wl = make_workload(5, T=20011, C=1024, with_dy=True)        # lengths of 1..8 mixed with 400..512, odd T
    g = torch.Generator().manual_seed(19)
    z = torch.randn(wl.T, 2048, generator=g).bfloat16()
    w = (torch.randn(1024, 31, generator=g) * 31 ** -0.5).bfloat16()
    _check(z, wl.cu_seqlens, w, wl.bias, wl.dy, "long gated boundary stress")
    zd, cud, wd, dyd = z.to(DEV), wl.cu_seqlens.to(DEV), w.to(DEV), wl.dy.to(DEV)
    a = npa.gated_dwconv_bwd(zd, dyd, cud, wd)
    b = npa.gated_dwconv_bwd(zd, dyd, cud, wd)
    assert all(torch.equal(p, q) for p, q in zip(a, b))
    assert torch.equal(npa.gated_dwconv_fwd(zd, cud, wd, None), npa.gated_dwconv_fwd(zd, cud, wd, None))


@pytest.mark.parametrize("C,K,dt", [(1024, 7, torch.bfloat16), (2048, 31, torch.bfloat16), (1024, 15, torch.bfloat16),
                                     (512, 31, torch.float32), (1152, 5, torch.bfloat16)])
def test_nonfinite_gate_inputs_reach_only_the_taps_their_products_belong_to(C, K, dt):
    """As for the plain conv (test_gpu_parity): h = x_proj * silu(gate) of a sequence of L rows feeds the taps with
    |k - P| < L only, so an Inf in x_proj or a NaN in gate of one- and two-row sequences must leave the other taps of dw
    and all of db bit for bit as they are without it; the boundary paths of the gated kernels mask by selection."""
    lens = [40, 1, 2, 50, 1, 300, 2, 30, 7, 1, 213, 2, 64, 1, 33, 700, 2, 1]
    P = (K - 1) // 2
    z, cu, w, b, dy = _case(lens, C, K, dt, dt, seed=C + K)
    cul = cu.tolist()
    zd, cud, wd, dyd = (t.to(DEV) for t in (z, cu, w, dy))
    _, dw0, db0 = npa.gated_dwconv_bwd(zd, dyd, cud, wd)
    for what, L, col0, val in (("Inf in x_proj of one-row sequences", 1, 0, float("inf")),
                               ("NaN in gate of two-row sequences", 2, C, float("nan"))):
        z2 = z.clone()
        for i, n in enumerate(lens):
            if n == L:
                z2[cul[i]:cul[i + 1], col0:col0 + C] = val
        _, dw, db = npa.gated_dwconv_bwd(z2.to(DEV), dyd, cud, wd)
        touched = torch.tensor([abs(k - P) <= L - 1 for k in range(K)])
        assert bool((~torch.isfinite(dw[:, touched])).all()), f"{what}: a tap the rows feed stayed finite"
        assert torch.equal(dw[:, ~touched], dw0[:, ~touched]), f"{what}: a tap the rows do not feed changed"
        assert torch.equal(db, db0), f"{what}: db changed"


@pytest.mark.parametrize("C,K,dt", [(2048, 31, torch.bfloat16), (1024, 15, torch.bfloat16), (512, 31, torch.float32),
                                     (1024, 7, torch.bfloat16)])
def test_gated_forward_keeps_nonfinite_rows_inside_their_sequence(C, K, dt):
    """The forward at K = 15 and 31 turns whole staged tiles, halo rows of neighbouring sequences included, into
    h = x_proj * silu(gate) in LDS before any tap is taken: an Inf or NaN there must stay out of every other sequence's
    rows (taps across a boundary are skipped, never multiplied by zero), which must come out bit for bit as without it."""
    lens = [40, 1, 2, 50, 1, 300, 2, 30, 7, 1, 213, 2, 64, 1, 33, 700, 2, 1, 129, 127]
    z, cu, w, b, dy = _case(lens, C, K, dt, dt, seed=C + K + 3)
    cul = cu.tolist()
    zd, cud, wd, bd = (t.to(DEV) for t in (z, cu, w, b))
    y0 = npa.gated_dwconv_fwd(zd, cud, wd, bd)
    for what, pick, col0, val in (("Inf in x_proj", lambda i, n: n <= 2, 0, float("inf")),
                                  ("NaN in gate", lambda i, n: i % 3 == 0, C, float("nan"))):
        z2 = z.clone()
        poisoned = torch.zeros(z.shape[0], dtype=torch.bool)
        for i, n in enumerate(lens):
            if pick(i, n):
                z2[cul[i]:cul[i + 1], col0:col0 + C] = val
                poisoned[cul[i]:cul[i + 1]] = True
        y = npa.gated_dwconv_fwd(z2.to(DEV), cud, wd, bd).cpu()
        assert torch.equal(y[~poisoned], y0.cpu()[~poisoned]), f"{what}: a row of another sequence changed"
        assert bool((~torch.isfinite(y[poisoned].float())).all()), f"{what}: a row of a poisoned sequence stayed finite"


@pytest.mark.parametrize("C,K", [(1024, 7), (2048, 31), (100, 7)])
def test_gated_parameter_gradients_straight_in_bf16(C, K):
    """NPLM_DWCONV_GRADS_BF16 on the gated backward (fused kernels and the composed fallback): the cast of the fp32 result."""
    z, cu, w, b, dy = _case(LENS_MIX, C, K, torch.bfloat16, torch.bfloat16, seed=C + K)
    zd, cud, wd, dyd = (t.to(DEV) for t in (z, cu, w, dy))
    dz, dw, db = npa.gated_dwconv_bwd(zd, dyd, cud, wd)
    dz2, dw2, db2 = npa.gated_dwconv_bwd(zd, dyd, cud, wd, grads_bf16=True)
    assert dw2.dtype == torch.bfloat16 and db2.dtype == torch.bfloat16
    assert torch.equal(dz, dz2) and torch.equal(dw.bfloat16(), dw2) and torch.equal(db.bfloat16(), db2)


def test_gated_intermediate_width_with_fp32_weights_and_residual():
    _check(*_case(LENS_MIX, 2048, 7, torch.bfloat16, torch.float32, seed=4), "gated C=2048 bf16/fp32")
    _check(*_case(LENS_MIX, 1024, 7, torch.bfloat16, torch.bfloat16, seed=6), "gated residual", residual=True)


def test_gated_boundary_stress_and_partial_last_tile():
    wl = make_workload(5, T=20011, C=1024, with_dy=True)        # lengths of 1..8 mixed with 400..512, odd T
    g = torch.Generator().manual_seed(9)
    z = torch.randn(wl.T, 2048, generator=g).bfloat16()
    _check(z, wl.cu_seqlens, wl.weight, wl.bias, wl.dy, "gated boundary stress")


def test_gated_autograd_matches_the_unfused_composition_and_is_deterministic():
    z, cu, w, b, dy = _case(LENS_MIX, 1024, 7, torch.float32, torch.float32, seed=12)
    cud, dyd = cu.to(DEV), dy.to(DEV)
    z1 = z.to(DEV).requires_grad_(True)
    w1 = w.to(DEV).requires_grad_(True)
    b1 = b.to(DEV).requires_grad_(True)
    y1 = npa.gated_varlen_dwconv(z1, cud, w1, b1)
    y1.backward(dyd)
    z2 = z.to(DEV).requires_grad_(True)
    w2 = w.to(DEV).requires_grad_(True)
    b2 = b.to(DEV).requires_grad_(True)
    u, g = z2.chunk(2, dim=-1)
    y2 = npa.varlen_dwconv((F.silu(g) * u).contiguous(), cud, w2, b2)
    y2.backward(dyd)
    torch.testing.assert_close(y1, y2, rtol=1e-5, atol=1e-5)
    torch.testing.assert_close(z1.grad, z2.grad, rtol=1e-4, atol=1e-5)
    torch.testing.assert_close(w1.grad, w2.grad, rtol=1e-5, atol=1e-3)
    torch.testing.assert_close(b1.grad, b2.grad, rtol=1e-5, atol=1e-3)
    # second run: bit-identical
    z3 = z.to(DEV).requires_grad_(True)
    w3 = w.to(DEV).requires_grad_(True)
    y3 = npa.gated_varlen_dwconv(z3, cud, w3, b.to(DEV))
    y3.backward(dyd)
    assert torch.equal(y3, y1) and torch.equal(z3.grad, z1.grad) and torch.equal(w3.grad, w1.grad)


def _composed_case_matches(z, cu, w, b, dy, what):
    """A shape without fused kernels: the raw entry points and the autograd surface compose the unfused ops; h is
    rounded to z's dtype on this route, so bf16 gets a bf16-sized allowance on top of the conv's own tolerance."""
    y64, dz64, dw64, db64 = O.ref_gated_dwconv_grads(z, cu, w, b, dy, torch.float64)
    zd, cud, wd, bd, dyd = (t.to(DEV) for t in (z, cu, w, b, dy))
    z1 = zd.clone().requires_grad_(True)
    w1 = wd.clone().requires_grad_(True)
    b1 = bd.clone().requires_grad_(True)
    y = npa.gated_varlen_dwconv(z1, cud, w1, b1)
    y.backward(dyd)
    tol = 4e-2 if z.dtype == torch.bfloat16 else 1e-4
    scale = lambda r: max(1.0, float(r.abs().max()))
    assert float((y.detach().cpu().double() - y64).abs().max()) <= tol * scale(y64), what
    assert float((z1.grad.cpu().double() - dz64).abs().max()) <= tol * scale(dz64), what
    assert float((w1.grad.cpu().double() - dw64).abs().max()) <= 2 * tol * scale(dw64), what
    assert float((b1.grad.cpu().double() - db64).abs().max()) <= 2 * tol * scale(db64), what
    return zd, cud, wd, bd, dyd


def test_unsupported_shapes_compose_and_the_abi_says_so():
    z, cu, w, b, dy = _case([5, 40, 3], 100, 7, torch.bfloat16, torch.bfloat16, seed=1)     # 200-byte rows
    zd, cud, wd, bd, _ = _composed_case_matches(z, cu, w, b, dy, "200-byte rows")
    assert not npa.gated_supported(zd, wd)
    lib = _lib.load()
    out = torch.empty(48, 100, device=DEV, dtype=torch.bfloat16)
    rc = lib.nplm_dwconv_gated_fwd(zd.data_ptr(), cud.data_ptr(), wd.data_ptr(), None, out.data_ptr(), 48, 100, 7, 3, 1, 1, 0,
                                   torch.cuda.current_stream().cuda_stream)
    assert rc == -_lib.EUNSUPPORTED and "gated" in _lib.strerror(rc)
    c33 = _case([30, 30], 1024, 33, torch.bfloat16, torch.bfloat16, seed=2)  # K = 33: above the largest built size
    assert not npa.gated_supported(c33[0].to(DEV), c33[2].to(DEV))
    _composed_case_matches(*c33, "K=33")
    _composed_case_matches(*_case([30, 7, 30], 512, 35, torch.float32, torch.float32, seed=3), "K=35 fp32")


@pytest.mark.parametrize("K,Kx,C,dt,wdt", [(11, 15, 1024, torch.bfloat16, torch.bfloat16), (13, 15, 256, torch.float32, torch.float32),
                                           (1, 3, 1152, torch.bfloat16, torch.bfloat16), (21, 31, 2048, torch.bfloat16, torch.float32),
                                           (29, 31, 520, torch.bfloat16, torch.bfloat16)])
def test_gated_kernel_sizes_without_kernels_of_their_own_run_as_the_next_size_with_zero_taps(K, Kx, C, dt, wdt):
    """As for the plain conv: an odd K <= 31 other than 3, 5, 7, 9, 15, 31 runs on the fused gated kernels of the next of
    3, 15, 31 with zero outer taps; every output equals the call with explicitly padded [C, Kx] taps bit for bit (dw: its
    inner K columns) and the oracle to the usual tolerances."""
    print(f"[case] gated K={K} as {Kx} C={C} {dt} w {wdt}", flush=True)
    z, cu, w, b, dy = _case(LENS_LONG, C, K, dt, wdt, seed=K + C)
    _check(z, cu, w, b, dy, f"gated K={K} C={C}")
    off = (Kx - K) // 2
    wx = torch.zeros(C, Kx, dtype=wdt)
    wx[:, off:off + K] = w
    zd, cud, wd, wxd, bd, dyd = (t.to(DEV) for t in (z, cu, w, wx, b, dy))
    for res in (False, True):
        assert torch.equal(npa.gated_dwconv_fwd(zd, cud, wd, bd, residual=res), npa.gated_dwconv_fwd(zd, cud, wxd, bd, residual=res))
        dz, dw, db = npa.gated_dwconv_bwd(zd, dyd, cud, wd, residual=res)
        dzx, dwx, dbx = npa.gated_dwconv_bwd(zd, dyd, cud, wxd, residual=res)
        assert dw.shape == (C, K)
        assert torch.equal(dz, dzx) and torch.equal(dw, dwx[:, off:off + K]) and torch.equal(db, dbx)


def test_offset_view_of_z_composes_instead_of_failing():
    """z that is contiguous but starts 8 bytes off a 16-byte boundary: the fused kernels decline, the call still works,
    eagerly and through the registered ops."""
    z, cu, w, b, dy = _case([40, 3, 200, 13], 1024, 7, torch.bfloat16, torch.bfloat16, seed=5)
    T = z.shape[0]
    buf = torch.zeros(T * 2048 + 8, dtype=torch.bfloat16, device=DEV)
    zv = buf[4:4 + T * 2048].view(T, 2048)
    zv.copy_(z)
    assert zv.is_contiguous() and zv.data_ptr() % 16 == 8
    cud, wd, bd, dyd = (t.to(DEV) for t in (cu, w, b, dy))
    y_al = npa.gated_dwconv_fwd(z.to(DEV), cud, wd, bd)
    y = npa.gated_dwconv_fwd(zv, cud, wd, bd)
    y_op = npa.gated_dwconv_fwd_op(zv, cud, wd, bd)
    assert torch.equal(y, y_op)
    def close(a, b):      # h is rounded to bf16 on the composed route: about one bf16 rounding of the result
        a, b = a.float(), b.float()
        return bool(((a - b).abs() <= 2.0 ** -6 * b.abs() + 3e-2).all())

    assert close(y, y_al)
    dz, dw, db = npa.gated_dwconv_bwd(zv, dyd, cud, wd)
    dz_al, dw_al, db_al = npa.gated_dwconv_bwd(z.to(DEV), dyd, cud, wd)
    assert close(dz, dz_al)
    torch.testing.assert_close(dw, dw_al, rtol=2e-2, atol=0.5)
    torch.testing.assert_close(db, db_al, rtol=1e-5, atol=1e-3)


@pytest.mark.parametrize("C,K", [(2048, 31), (1024, 11), (100, 7)])
def test_every_gated_shape_compiles_without_graph_breaks(C, K):
    """Intermediate width with the long kernel, a kernel size without fused kernels and narrow rows: under
    torch.compile(fullgraph=True) each is one opaque op, whichever route the library takes inside it."""
    print(f"[case] gated compile C={C} K={K}", flush=True)
    z, cu, w, b, dy = _case([40, 3, 200, 13, 300], C, K, torch.bfloat16, torch.bfloat16, seed=C + K)
    zd, cud, dyd = z.to(DEV), cu.to(DEV), dy.to(DEV)
    conv = npa.VarlenDWConv1d(C, K, device=DEV, dtype=torch.bfloat16)
    with torch.no_grad():
        conv.weight.copy_(w.to(DEV))
        conv.bias.copy_(b.to(DEV))

    class MLPTail(torch.nn.Module):
        def __init__(self):
            super().__init__()
            self.conv = conv

        def forward(self, zz, cc):
            return self.conv.forward_gated(zz, cc)

    def run(mod):
        conv.zero_grad()
        zin = zd.clone().requires_grad_(True)
        y = mod(zin, cud)
        y.backward(dyd)
        return y.detach(), zin.grad, conv.weight.grad.clone(), conv.bias.grad.clone()

    m = MLPTail()
    eager = run(m)
    torch._dynamo.reset()
    compiled = run(torch.compile(m, backend="aot_eager", fullgraph=True, dynamic=False))
    for a, bb in zip(eager, compiled):
        assert torch.equal(a, bb)
    y64, dz64, _, _ = O.ref_gated_dwconv_grads(z, cu, w, b, dy, torch.float64)
    assert float((eager[0].cpu().double() - y64).abs().max()) <= 4e-2 * max(1.0, float(y64.abs().max()))
    assert float((eager[1].cpu().double() - dz64).abs().max()) <= 4e-2 * max(1.0, float(dz64.abs().max()))


def test_gated_ops_pass_opcheck_and_compile_without_graph_breaks():
    z, cu, w, b, dy = _case([40, 3, 200, 13], 1024, 7, torch.bfloat16, torch.bfloat16, seed=21)
    zd, cud, wd, bd, dyd = (t.to(DEV) for t in (z, cu, w, b, dy))
    torch.library.opcheck(npa.gated_dwconv_fwd_op, (zd, cud, wd, bd), test_utils=("test_schema", "test_faketensor"))
    torch.library.opcheck(npa.gated_dwconv_bwd_op, (zd, dyd, cud, wd), test_utils=("test_schema", "test_faketensor"))

    class MLPTail(torch.nn.Module):
        def __init__(self):
            super().__init__()
            self.conv = npa.VarlenDWConv1d(1024, 7, device=DEV, dtype=torch.bfloat16)

        def forward(self, zz, cc):
            return self.conv.forward_gated(zz, cc)

    m = MLPTail()
    z1 = zd.clone().requires_grad_(True)
    eager = m(z1, cud)
    eager.backward(dyd)
    compiled = torch.compile(m, backend="aot_eager", fullgraph=True, dynamic=False)
    z2 = zd.clone().requires_grad_(True)
    m.zero_grad()
    out = compiled(z2, cud)
    out.backward(dyd)
    assert torch.equal(out, eager) and torch.equal(z2.grad, z1.grad)
