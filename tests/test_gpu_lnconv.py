"""LayerNorm fused into the conv's forward and backward (a conv sub-module of the reference's pre-norm layer,
modeling.py:404-438) against the float64 oracle, through the C ABI entry points and the autograd surface."""
import pytest
import torch

import nanoplm_amd as npa
from nanoplm_amd import _lib
from nanoplm_amd.workloads import cu_from_lengths, make_workload
from oracle import dwconv_ref as O
from tests.gpu_util import assert_act_close, assert_red_close

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
LENS_MIX = [1, 2, 3, 8, 0, 1, 150, 0, 5, 7, 6, 1, 64, 63, 65, 2, 300, 4, 17, 512, 23, 24, 25, 47, 48, 49]


def _case(lens, C, K, dt, wdt, seed, ln_bias=True):
    g = torch.Generator().manual_seed(seed)
    T = int(sum(lens))
    x = (torch.randn(T, C, generator=g) * (1 + torch.rand(T, 1, generator=g) * 3) + torch.randn(T, 1, generator=g)).to(dt)
    gam = (1 + 0.3 * torch.randn(C, generator=g)).to(wdt)
    bet = (0.2 * torch.randn(C, generator=g)).to(wdt) if ln_bias else None
    w = (torch.randn(C, K, generator=g) * K ** -0.5).to(wdt)
    b = (torch.randn(C, generator=g) * 0.02).to(wdt)
    dy = torch.randn(T, C, generator=g).to(dt)
    return x, cu_from_lengths(torch.tensor(lens)), gam, bet, w, b, dy


def _check_fwd(x, cu, gam, bet, w, b, what, residual=False, fused=True):
    y64 = O.ref_ln_dwconv_grads(x, cu, gam, bet, w, b, None, 1e-5, torch.float64, residual)
    xd, cud, gd, wd, bd = (t.to(DEV) for t in (x, cu, gam, w, b))
    hd = None if bet is None else bet.to(DEV)
    assert npa.ln_supported(xd, wd) == fused
    y, stats = npa.ln_dwconv_fwd(xd, cud, gd, hd, wd, bd, residual=residual)
    assert_act_close(y, y64, x.dtype, what + " y")
    x64 = x.double()
    mean = x64.mean(1)
    rstd = 1 / torch.sqrt(x64.var(1, unbiased=False) + 1e-5)
    torch.testing.assert_close(stats[:, 0].cpu().double(), mean, rtol=1e-5, atol=1e-5)
    torch.testing.assert_close(stats[:, 1].cpu().double(), rstd, rtol=1e-5, atol=1e-6)
    return y


@pytest.mark.parametrize("K", [3, 5, 7, 9])
@pytest.mark.parametrize("dt,wdt,C", [(torch.bfloat16, torch.bfloat16, 1024), (torch.bfloat16, torch.float32, 768),
                                       (torch.float32, torch.float32, 512), (torch.float32, torch.float32, 384),
                                       (torch.bfloat16, torch.bfloat16, 8), (torch.float32, torch.bfloat16, 100),
                                       (torch.bfloat16, torch.bfloat16, 512)])
def test_fused_layernorm_forward_kernel_sizes_and_widths(K, dt, wdt, C):
    """Whole rows in one 2 KiB column block: full and partial rows, one chunk per row, both dtypes, mixed
    parameter dtypes; lengths around the 24-row tiles and the 12-row wave windows, empty sequences."""
    print(f"[case] ln K={K} C={C} {dt} w {wdt}", flush=True)
    _check_fwd(*_case(LENS_MIX, C, K, dt, wdt, seed=K + C)[:6], f"ln K={K} C={C} {dt}")
    _check_fwd(*_case(LENS_MIX[::-1], C, K, dt, wdt, seed=K + C + 1, ln_bias=False)[:6], f"ln residual K={K} C={C} {dt}",
               residual=True)


def test_fused_layernorm_forward_is_deterministic_and_takes_the_boundary_stress_mix():
    wl = make_workload(5, T=20011, C=1024, with_dy=False)        # lengths of 1..8 mixed with 400..512, odd T
    g = torch.Generator().manual_seed(5)
    gam = (1 + 0.3 * torch.randn(1024, generator=g)).bfloat16()
    bet = (0.2 * torch.randn(1024, generator=g)).bfloat16()
    y = _check_fwd(wl.x, wl.cu_seqlens, gam, bet, wl.weight, wl.bias, "ln boundary stress", residual=True)
    a = [t.to(DEV) for t in (wl.x, wl.cu_seqlens, gam, bet, wl.weight, wl.bias)]
    y2, _ = npa.ln_dwconv_fwd(*a, residual=True)
    assert torch.equal(y, y2)


@pytest.mark.parametrize("C", [1024, 644, 516, 772])
def test_fp32_rows_of_up_to_4_kib_take_the_whole_row_forward_on_the_boundary_stress_mix(C):
    """The fp32 residual stream (rows of 4 KiB at hidden 1024; 644 channels leave the last wave-columns of the 3 KiB
    column block partly and wholly empty; 516 and 772 channels put 16 bytes into the last 1 KiB piece of the 3 KiB and
    the 4 KiB block): one kernel, which needs no statistics buffer; a bf16 row of that size goes through the two-kernel
    path and does need one."""
    wl = make_workload(5, T=9973, C=C, with_dy=False)
    g = torch.Generator().manual_seed(C)
    x = (wl.x.float() * (1 + 3 * torch.rand(wl.T, 1, generator=g)) + torch.randn(wl.T, 1, generator=g))
    gam = 1 + 0.3 * torch.randn(C, generator=g)
    bet = 0.2 * torch.randn(C, generator=g)
    w, b = wl.weight.float(), wl.bias.float()
    y = _check_fwd(x, wl.cu_seqlens, gam, bet, w, b, f"ln fp32 C={C} boundary stress", residual=True)
    a = [t.to(DEV) for t in (x, wl.cu_seqlens, gam, bet, w, b)]
    y2, _ = npa.ln_dwconv_fwd(*a, residual=True)
    assert torch.equal(y, y2)
    lib = _lib.load()
    y3 = torch.empty_like(y2)
    args = lambda t, o, act: (t.data_ptr(), a[1].data_ptr(), a[2].data_ptr(), a[3].data_ptr(), 1e-5, a[4].data_ptr(), a[5].data_ptr(),
                              o.data_ptr(), None, wl.T, t.shape[1], wl.K, wl.S, act, 0, 1, None)
    assert lib.nplm_dwconv_ln_fwd(*args(a[0], y3, 0)) == 0
    torch.cuda.synchronize()
    assert torch.equal(y2, y3)
    if C == 1024:
        xb = torch.cat([a[0], a[0]], 1).bfloat16()          # bf16 rows of 4 KiB
        gb = torch.cat([a[2], a[2]]); hb = torch.cat([a[3], a[3]]); wb = torch.cat([a[4], a[4]]); bb = torch.cat([a[5], a[5]])
        rc = lib.nplm_dwconv_ln_fwd(xb.data_ptr(), a[1].data_ptr(), gb.data_ptr(), hb.data_ptr(), 1e-5, wb.data_ptr(), bb.data_ptr(),
                                    torch.empty_like(xb).data_ptr(), None, wl.T, 2048, wl.K, wl.S, 1, 0, 1, None)
        assert rc == -1                                      # NPLM_DWCONV_ENULL


WIDE = [(torch.bfloat16, torch.bfloat16, 2048), (torch.float32, torch.float32, 1024), (torch.float32, torch.bfloat16, 768),
        (torch.bfloat16, torch.float32, 1536), (torch.float32, torch.float32, 2048), (torch.bfloat16, torch.bfloat16, 1032),
        (torch.float32, torch.float32, 644), (torch.float32, torch.bfloat16, 516), (torch.float32, torch.float32, 772)]


@pytest.mark.parametrize("K", [3, 5, 7, 9])
@pytest.mark.parametrize("dt,wdt,C", WIDE)
def test_layernorm_forward_of_wide_rows(K, dt, wdt, C):
    """Rows of more than 2 KiB (up to 8 KiB). fp32 rows of up to 4 KiB: the whole-row kernel with 8 wave-columns; the
    others: the row-statistics kernel, then the conv forward that normalises as it reads: 2, 3, 6 and 8 column blocks,
    the last one partly filled, rows of 4 and 8 chunks per lane."""
    print(f"[case] ln wide K={K} C={C} {dt} w {wdt}", flush=True)
    _check_fwd(*_case(LENS_MIX, C, K, dt, wdt, seed=K + C)[:6], f"ln wide K={K} C={C} {dt}")
    _check_fwd(*_case(LENS_MIX[::-1], C, K, dt, wdt, seed=K + C + 1, ln_bias=False)[:6], f"ln wide residual K={K} C={C} {dt}",
               residual=True)


@pytest.mark.parametrize("K", [3, 7, 9])
@pytest.mark.parametrize("dt,wdt,C", WIDE)
def test_layernorm_backward_of_wide_rows(K, dt, wdt, C):
    """Rows of more than 2 KiB: the one-kernel backward (up to 4 KiB: 16 wave-columns of 4 bytes per lane, or, in fp32,
    8 or 6 wave-columns of 8 bytes in two row groups) and the two-kernel path (conv backward leaving the normalised
    tensor's gradient in fp32, then the row pass for dx)."""
    print(f"[case] ln bwd wide K={K} C={C} {dt} w {wdt}", flush=True)
    _check_bwd(*_case(LENS_MIX, C, K, dt, wdt, seed=K + C), f"ln bwd wide K={K} C={C} {dt}")
    _check_bwd(*_case(LENS_MIX[::-1], C, K, dt, wdt, seed=K + C + 1, ln_bias=False), f"ln bwd wide residual K={K} C={C} {dt}",
               residual=True)


def test_shapes_outside_the_fused_kernel_compose_layer_norm_and_the_conv():
    for (C, K, dt) in ((4104, 7, torch.bfloat16), (2052, 7, torch.float32), (1024, 15, torch.bfloat16), (1020, 7, torch.bfloat16)):
        print(f"[case] ln composed C={C} K={K} {dt}", flush=True)
        _check_fwd(*_case([5, 40, 3, 0, 90], C, K, dt, dt, seed=C + K)[:6], f"ln composed C={C} K={K}", residual=True, fused=False)


@pytest.mark.parametrize("dt,C,residual", [(torch.bfloat16, 1024, True), (torch.float32, 512, False), (torch.bfloat16, 2048, True),
                                           (torch.float32, 1024, True), (torch.bfloat16, 4104, True)])
def test_autograd_through_the_fused_kernels(dt, C, residual):
    """Gradients of x, the LayerNorm parameters and the conv parameters against the float64 oracle (whole-row kernels,
    wide rows, and as the last case a width the fused kernels do not take: same surface, composed ops)."""
    x, cu, gam, bet, w, b, dy = _case(LENS_MIX, C, 7, dt, torch.float32, seed=C)
    y64, dx64, dg64, dh64, dw64, db64 = O.ref_ln_dwconv_grads(x, cu, gam, bet, w, b, dy, 1e-5, torch.float64, residual)
    xd = x.to(DEV).requires_grad_(True)
    params = [t.to(DEV).requires_grad_(True) for t in (gam, bet, w, b)]
    y = npa.ln_varlen_dwconv(xd, cu.to(DEV), params[0], params[1], params[2], params[3], residual=residual)
    y.backward(dy.to(DEV))
    assert_act_close(y.detach(), y64, dt, "y")
    assert_act_close(xd.grad, dx64, dt, "dx")
    assert_red_close(params[0].grad, dg64, "d ln_weight")
    assert_red_close(params[1].grad, dh64, "d ln_bias")
    assert_red_close(params[2].grad, dw64, "dw")
    assert_red_close(params[3].grad, db64, "db")


def _check_bwd(x, cu, gam, bet, w, b, dy, what, residual=False, fused=True):
    _, dx64, dg64, dh64, dw64, db64 = O.ref_ln_dwconv_grads(x, cu, gam, bet, w, b, dy, 1e-5, torch.float64, residual)
    xd, cud, gd, wd, dyd = (t.to(DEV) for t in (x, cu, gam, w, dy))
    hd = None if bet is None else bet.to(DEV)
    T, C = x.shape
    ws = _lib.load().nplm_dwconv_ln_bwd_workspace_bytes(T, C, w.shape[1], 1 if x.dtype == torch.bfloat16 else 0)
    assert (ws > 0) == fused, f"{what}: workspace {ws}"
    _, stats = npa.ln_dwconv_fwd(xd, cud, gd, hd, wd, None, residual=residual)
    out = npa.ln_dwconv_bwd(xd, dyd, cud, stats, gd, hd, wd, residual=residual)
    dx, dg, dh, dw, db = out
    assert_act_close(dx, dx64, x.dtype, what + " dx")
    assert_red_close(dg.cpu(), dg64, what + " d ln_weight")
    assert_red_close(dw.cpu(), dw64, what + " dw")
    assert_red_close(db.cpu(), db64, what + " db")
    if bet is None:
        assert dh is None
    else:
        assert_red_close(dh.cpu(), dh64, what + " d ln_bias")
    return out


@pytest.mark.parametrize("K", [3, 5, 7, 9])
@pytest.mark.parametrize("dt,wdt,C", [(torch.bfloat16, torch.bfloat16, 1024), (torch.bfloat16, torch.float32, 768),
                                       (torch.float32, torch.float32, 512), (torch.float32, torch.float32, 384),
                                       (torch.bfloat16, torch.bfloat16, 8), (torch.float32, torch.bfloat16, 100)])
def test_fused_layernorm_backward_kernel_sizes_and_widths(K, dt, wdt, C):
    """The one-kernel backward for rows a block owns: the conv backward normalises x as it reads, sums the LayerNorm
    parameter gradients, exchanges the row sums between its waves and writes dx. Full and partly filled rows, one
    16-byte chunk per row, both dtypes, mixed parameter dtypes, with and without the LayerNorm bias and the residual
    connection; lengths around the 16-row tiles and 8-row wave windows, empty sequences."""
    print(f"[case] ln bwd K={K} C={C} {dt} w {wdt}", flush=True)
    _check_bwd(*_case(LENS_MIX, C, K, dt, wdt, seed=K + C), f"ln bwd K={K} C={C} {dt}")
    _check_bwd(*_case(LENS_MIX[::-1], C, K, dt, wdt, seed=K + C + 1, ln_bias=False), f"ln bwd residual K={K} C={C} {dt}",
               residual=True)


@pytest.mark.parametrize("dt,C", [(torch.bfloat16, 1024), (torch.bfloat16, 2048), (torch.float32, 768)])
def test_fp32_layernorm_parameters_beside_bf16_taps_are_not_rounded(dt, C):
    """nn.LayerNorm keeps fp32 parameters under autocast while the conv's taps may be bf16 (FSDP mixed precision):
    every parameter then goes into the kernels as fp32, so the result is that of the fp32 LayerNorm parameters (an
    oracle run with gamma and beta rounded to bf16 differs from it by more than the tolerance on d ln_weight)."""
    x, cu, gam, bet, w, b, dy = _case(LENS_MIX, C, 7, dt, torch.bfloat16, seed=C + 3)
    g = torch.Generator().manual_seed(C)
    gam = 1 + 0.3 * torch.randn(C, generator=g)          # fp32, not representable in bf16
    bet = 0.2 * torch.randn(C, generator=g)
    _check_fwd(x, cu, gam, bet, w, b, f"mixed ln dtypes C={C} {dt}", residual=True)
    _check_bwd(x, cu, gam, bet, w, b, dy, f"mixed ln dtypes bwd C={C} {dt}", residual=True)


@pytest.mark.parametrize("dt,C", [(torch.bfloat16, 1024), (torch.bfloat16, 2048), (torch.bfloat16, 3072), (torch.bfloat16, 4104)])
def test_layernorm_parameter_gradients_straight_in_bf16(dt, C):
    """NPLM_DWCONV_GRADS_BF16 on the LayerNorm-fused backward (one-kernel, two-kernel and composed paths): all four
    parameter gradients equal the cast of the fp32 results; through autograd bf16 parameters get bf16 gradients."""
    x, cu, gam, bet, w, b, dy = _case(LENS_MIX, C, 7, dt, torch.bfloat16, seed=C + 9)
    xd, cud, gd, hd, wd, dyd = (t.to(DEV) for t in (x, cu, gam, bet, w, dy))
    _, stats = npa.ln_dwconv_fwd(xd, cud, gd, hd, wd, None, residual=True)
    ref = npa.ln_dwconv_bwd(xd, dyd, cud, stats, gd, hd, wd, residual=True)
    got = npa.ln_dwconv_bwd(xd, dyd, cud, stats, gd, hd, wd, residual=True, grads_bf16=True)
    assert torch.equal(ref[0], got[0])
    for a, g in zip(ref[1:], got[1:]):
        assert g.dtype == torch.bfloat16 and torch.equal(a.bfloat16(), g)
    xr = xd.clone().requires_grad_(True)
    params = [t.clone().requires_grad_(True) for t in (gd, hd, wd, b.to(DEV))]
    npa.ln_varlen_dwconv(xr, cud, *params, residual=True).backward(dyd)
    assert all(p.grad.dtype == torch.bfloat16 for p in params)
    assert torch.equal(params[2].grad, got[3]) and torch.equal(params[0].grad, got[1])


def test_fused_layernorm_backward_is_deterministic_and_takes_the_boundary_stress_mix():
    wl = make_workload(5, T=20011, C=1024, with_dy=True)        # lengths of 1..8 mixed with 400..512, odd T
    g = torch.Generator().manual_seed(6)
    gam = (1 + 0.3 * torch.randn(1024, generator=g)).bfloat16()
    bet = (0.2 * torch.randn(1024, generator=g)).bfloat16()
    a = (wl.x, wl.cu_seqlens, gam, bet, wl.weight, wl.bias, wl.dy)
    o1 = _check_bwd(*a, "ln bwd boundary stress", residual=True)
    o2 = _check_bwd(*a, "ln bwd boundary stress again", residual=True)
    for p, q in zip(o1, o2):
        assert torch.equal(p, q)


def test_backward_of_shapes_outside_the_fused_kernels_is_composed():
    for (C, K, dt) in ((4104, 7, torch.bfloat16), (1024, 15, torch.bfloat16), (1020, 7, torch.bfloat16)):
        print(f"[case] ln bwd composed C={C} K={K} {dt}", flush=True)
        _check_bwd(*_case([5, 40, 3, 0, 90], C, K, dt, dt, seed=C + K), f"ln bwd composed C={C} K={K}", residual=True, fused=False)


def test_layernorm_backward_refuses_a_short_workspace_and_zero_fills_for_no_tokens():
    lib = _lib.load()
    x, cu, gam, bet, w, b, dy = (t.to(DEV) for t in _case([5, 9], 512, 7, torch.float32, torch.float32, seed=2))
    _, stats = npa.ln_dwconv_fwd(x, cu, gam, bet, w, None)
    need = lib.nplm_dwconv_ln_bwd_workspace_bytes(14, 512, 7, 0)
    assert need >= (7 + 1 + 2) * 512 * 4           # one token block's partial sums (whole rows: no dn buffer)
    assert lib.nplm_dwconv_ln_bwd_workspace_bytes(14, 2048, 7, 0) >= 14 * 2048 * 4       # rows of 8 KiB: dn in fp32 as well
    outs = [torch.empty_like(x)] + [torch.full((512, 7), 3.0, device=DEV)] + [torch.full((512,), 3.0, device=DEV) for _ in range(3)]
    ws = torch.empty(need, dtype=torch.uint8, device=DEV)
    p = lambda t: None if t is None else t.data_ptr()
    common = (p(x), p(dy), p(cu), p(stats), p(gam), p(bet), p(w), *(p(o) for o in outs))
    assert lib.nplm_dwconv_ln_bwd(*common, p(ws), need - 256, 14, 512, 7, 2, 0, 0, 0, None) == -6      # NPLM_DWCONV_EWORKSPACE
    assert lib.nplm_dwconv_ln_bwd(*common, p(ws), need, 14, 512, 7, 2, 0, 0, 8, None) == -9         # NPLM_DWCONV_EFLAGS
    assert lib.nplm_dwconv_ln_bwd(*common, None, 0, 0, 512, 7, 0, 0, 0, 0, None) == 0
    torch.cuda.synchronize()
    for o in outs[1:]:
        assert torch.count_nonzero(o).item() == 0


@pytest.mark.parametrize("backend", ["aot_eager", "inductor"])
def test_layernorm_conv_compiles_into_one_graph(backend):
    """The custom-op pair under torch.compile(dynamic=False) as the reference compiles its model
    (pure_pipeline.py:519-524), a pre-norm sub-module in a bf16 residual stream: x + conv(norm(x)), then a Linear.
    The compiled graph calls the same kernels as eager: every output and gradient bit-equal under aot_eager; Inductor
    may fuse and re-round the elementwise ops around the opaque ops, so it is held to the eager result's tolerance."""
    C, K = 1024, 7
    x, cu, gam, bet, w, b, dy = (t.to(DEV) for t in _case(LENS_MIX, C, K, torch.bfloat16, torch.bfloat16, seed=11))
    torch.manual_seed(3)
    lin = torch.nn.Linear(C, C, bias=False).to(DEV).bfloat16()
    params = [t.clone().requires_grad_(True) for t in (gam, bet, w, b)]

    def block(x, cu):
        h = npa.ln_varlen_dwconv_compilable(x, cu, params[0], params[1], params[2], params[3], residual=True)
        return lin(h)

    def run(fn):
        for p in params + [lin.weight]:
            p.grad = None
        xin = x.clone().requires_grad_(True)
        y = fn(xin, cu)
        y.backward(dy)
        return [y.detach(), xin.grad] + [p.grad.clone() for p in params + [lin.weight]]

    eager = run(block)
    torch._dynamo.reset()
    compiled = run(torch.compile(block, backend=backend, fullgraph=True, dynamic=False))
    for name, a, c in zip(("y", "dx", "d ln_weight", "d ln_bias", "dw", "db", "d lin"), eager, compiled):
        if backend == "aot_eager":
            assert torch.equal(a, c), name
        else:
            err = float((a.float() - c.float()).abs().max() / a.float().abs().max().clamp_min(1e-30))
            assert err <= 2.0 ** -7, (name, err)
    # and the op pair agrees with the autograd.Function surface
    xin = x.clone().requires_grad_(True)
    y = lin(npa.ln_varlen_dwconv(xin, cu, *[p.detach() for p in params], residual=True))
    assert torch.equal(y.detach(), eager[0])


def test_layernorm_conv_ops_pass_opcheck():
    x, cu, gam, bet, w, b, dy = (t.to(DEV) for t in _case([5, 40, 3, 0, 90], 512, 5, torch.float32, torch.float32, seed=12))
    torch.library.opcheck(npa.ln_dwconv_fwd_op, (x, cu, gam, bet, w, b, 1e-5, True), test_utils=("test_schema", "test_faketensor"))
    _, stats = npa.ln_dwconv_fwd(x, cu, gam, bet, w, b)
    torch.library.opcheck(npa.ln_dwconv_bwd_op, (x, dy, cu, stats, gam, None, w, False),
                          test_utils=("test_schema", "test_faketensor"))


@pytest.mark.parametrize("dt,C", [(torch.bfloat16, 1024), (torch.float32, 1024)])
def test_layernorm_conv_replays_correctly_from_a_hip_graph(dt, C):
    """Forward and backward of both widths (whole-row kernels; statistics kernel + normalising conv + row pass) captured
    once and replayed with new contents in the static buffers, with eager work and synchronisation between the
    replays; every replay equals the eager result bit for bit."""
    K = 7
    x0, cu, gam, bet, w, b, dy0 = (t.to(DEV) for t in _case([100, 3, 512, 1, 408], C, K, dt, torch.float32, seed=21))
    sx, sdy = torch.zeros_like(x0), torch.zeros_like(dy0)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):                      # warm-up outside capture
        _, st = npa.ln_dwconv_fwd(sx, cu, gam, bet, w, b, residual=True)
        npa.ln_dwconv_bwd(sx, sdy, cu, st, gam, bet, w, residual=True)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        gy, gst = npa.ln_dwconv_fwd(sx, cu, gam, bet, w, b, residual=True)
        gout = npa.ln_dwconv_bwd(sx, sdy, cu, gst, gam, bet, w, residual=True)
    g = torch.Generator(device=DEV).manual_seed(5)
    for it in range(4):
        x = (torch.randn(x0.shape, device=DEV, generator=g) * 2 + 0.5).to(dt)
        dy = torch.randn(x0.shape, device=DEV, generator=g).to(dt)
        sx.copy_(x)
        sdy.copy_(dy)
        graph.replay()
        torch.cuda.synchronize()
        ey, est = npa.ln_dwconv_fwd(x, cu, gam, bet, w, b, residual=True)
        eout = npa.ln_dwconv_bwd(x, dy, cu, est, gam, bet, w, residual=True)
        torch.cuda.synchronize()
        assert torch.equal(gy, ey) and torch.equal(gst, est), f"replay {it}"
        for a, e in zip(gout, eout):
            assert torch.equal(a, e), f"replay {it}"


@pytest.mark.parametrize("dt", [torch.bfloat16, torch.float32])
def test_layernorm_conv_at_the_headline_size_against_the_composed_ops(dt):
    """T=131072, C=1024, K=7 with configuration 3's lengths, in bf16 (8192 tiles, every block 32 rounds) and as the fp32
    residual stream (rows of 4 KiB: 18725 forward tiles of 7 rows and 21846 backward tiles of 6, the last round partly
    empty): the fused forward and the one-kernel backward against the same operator composed on the GPU in fp32 (torch's
    LayerNorm, this library's fp32 conv kernels, which the other tests hold to the oracle, ATen's LayerNorm backward):
    bf16 outputs within one bf16 rounding of the fp32 result where it is not tiny, fp32 outputs to 1e-4, parameter
    gradients to 1e-4 of their largest value; and twice the same bits."""
    import dataclasses
    wl = make_workload(3, with_dy=True)
    if dt == torch.float32:
        wl = dataclasses.replace(wl, x=wl.x.float(), dy=wl.dy.float(), dtype=torch.float32)
    d = wl.to(DEV)
    g = torch.Generator().manual_seed(9)
    gam = (1 + 0.3 * torch.randn(wl.C, generator=g)).to(DEV)
    bet = (0.2 * torch.randn(wl.C, generator=g)).to(DEV)
    w32, b32 = d.weight.float(), d.bias.float()
    y, st = npa.ln_dwconv_fwd(d.x, d.cu_seqlens, gam, bet, w32, b32, residual=True)
    out = npa.ln_dwconv_bwd(d.x, d.dy, d.cu_seqlens, st, gam, bet, w32, residual=True)
    y2, st2 = npa.ln_dwconv_fwd(d.x, d.cu_seqlens, gam, bet, w32, b32, residual=True)
    out2 = npa.ln_dwconv_bwd(d.x, d.dy, d.cu_seqlens, st2, gam, bet, w32, residual=True)
    assert torch.equal(y, y2) and all(torch.equal(a, b) for a, b in zip(out, out2))
    xf = d.x.float().requires_grad_(True)
    gp, bp = gam.clone().requires_grad_(True), bet.clone().requires_grad_(True)
    wp, bbp = w32.clone().requires_grad_(True), b32.clone().requires_grad_(True)
    n = torch.nn.functional.layer_norm(xf, (wl.C,), gp, bp, 1e-5)
    yr = xf + npa.varlen_dwconv(n, d.cu_seqlens, wp, bbp)
    yr.backward(d.dy.float())

    def act_close(got, ref, what):
        err = (got.float() - ref).abs()
        bound = ref.abs() * 2.0 ** -8 + 2e-2 * (ref.abs() < 8) if dt == torch.bfloat16 else 1e-4 * (1 + ref.abs())
        bad = int((err > bound).sum())
        assert bad == 0, f"{what}: {bad} elements beyond the bound (max err {float(err.max()):.3e})"

    act_close(y, yr.detach(), "y")
    act_close(out[0], xf.grad, "dx")
    for got, ref, what in ((out[1], gp.grad, "d ln_weight"), (out[2], bp.grad, "d ln_bias"), (out[3], wp.grad, "dw"), (out[4], bbp.grad, "db")):
        rel = float((got - ref).abs().max() / ref.abs().max())
        assert rel <= 1e-4, (what, rel)


def test_layernorm_conv_takes_the_static_collators_cu_seqlens():
    """Fixed-length cu_seqlens as the static-shape collator builds it (collator.py:430-450): real sequences, pad
    pseudo-sequences up to the flat length, trailing zero-length entries; whole-row kernels and wide rows."""
    from nanoplm_amd.workloads import static_packed_cu
    g = torch.Generator().manual_seed(41)
    lens = torch.randint(20, 300, (12,), generator=g)
    real = cu_from_lengths(lens)
    F_rows = int(real[-1]) + 700
    cu = static_packed_cu(real, F_rows, 256, cu_len=24)
    assert int(cu[-1]) == F_rows and int((cu[1:] == cu[:-1]).sum()) > 0
    lens_all = (cu[1:] - cu[:-1]).tolist()
    for dt, C in ((torch.bfloat16, 1024), (torch.float32, 1024)):
        x, _, gam, bet, w, b, dy = _case(lens_all, C, 7, dt, torch.float32, seed=C + 1)
        _check_fwd(x, cu, gam, bet, w, b, f"ln static cu {dt}", residual=True)
        _check_bwd(x, cu, gam, bet, w, b, dy, f"ln bwd static cu {dt}", residual=True)


def test_module_prenorm_door_matches_the_functional_form():
    C, K = 512, 5
    x, cu, gam, bet, w, b, dy = (t.to(DEV) for t in _case(LENS_MIX, C, K, torch.float32, torch.float32, seed=31))
    conv = npa.VarlenDWConv1d(C, K, residual=True).to(DEV)
    norm = torch.nn.LayerNorm(C, eps=1e-5, bias=False).to(DEV)
    with torch.no_grad():
        conv.weight.copy_(w)
        conv.bias.copy_(b)
        norm.weight.copy_(gam)
    xin = x.clone().requires_grad_(True)
    y = conv.forward_prenorm(xin, cu, norm)
    y.backward(dy)
    y64, dx64, dg64, _, dw64, db64 = O.ref_ln_dwconv_grads(x.cpu(), cu.cpu(), gam.cpu(), None, w.cpu(), b.cpu(), dy.cpu(), 1e-5,
                                                            torch.float64, True)
    assert_act_close(y.detach(), y64, torch.float32, "prenorm door y")
    assert_act_close(xin.grad, dx64, torch.float32, "prenorm door dx")
    assert_red_close(norm.weight.grad, dg64, "prenorm door d ln_weight")
    assert_red_close(conv.weight.grad, dw64, "prenorm door dw")
    assert_red_close(conv.bias.grad, db64, "prenorm door db")
    with pytest.raises(ValueError):
        conv.forward_prenorm(xin, cu, torch.nn.LayerNorm(C + 8).to(DEV))


def test_unsupported_arguments_are_refused():
    x, cu, gam, bet, w, b, dy = _case([5, 9], 64, 7, torch.float32, torch.float32, seed=1)
    with pytest.raises(RuntimeError):
        npa.ln_dwconv_fwd(x, cu, gam, bet, w, b)                      # CPU tensors
    with pytest.raises(ValueError):
        npa.ln_dwconv_fwd(x.to(DEV), cu.to(DEV), gam[:-1].to(DEV), None, w.to(DEV), None)
