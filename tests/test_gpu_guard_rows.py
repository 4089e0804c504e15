"""Nothing is written outside the outputs: every activation-sized output (y, dx, dz, the LayerNorm statistics) is a
slice of a larger allocation with guard rows in front of it and behind it, the parameter gradients sit between guard
elements, T is not a multiple of any tile height, and after each call through the C ABI the guards are bit for bit
what they were while the outputs equal those of the same call on ordinary tensors.

The kernels drop the rows of a last, partial tile either by an explicit row test or by the range check of the buffer
descriptor they store through (its size is that of the T rows, not of the allocation), so a store that relied on the
allocation's end instead would land in the guard rows here. All writes stay inside one allocation: nothing can fault.
"""
import pytest
import torch

import nanoplm_amd as npa
from nanoplm_amd import _lib
from nanoplm_amd.workloads import cu_from_lengths

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
G = 70                      # guard rows on either side of an activation-sized output
# 3011 rows: not a multiple of 6, 7, 8, 10, 12, 16, 20, 30, 32, 40, 48, 64, 96 or 128
LENS = [300, 1, 17, 512, 2, 64, 63, 700, 5, 129, 33, 1, 400, 250, 31, 15, 16, 200, 272]
assert sum(LENS) == 3011


def _code(dt):
    return _lib.BF16 if dt == torch.bfloat16 else _lib.F32


class Guarded:
    """A [rows, cols] output inside a larger allocation filled with a value no kernel produces."""

    def __init__(self, rows, cols, dtype):
        self.buf = torch.full(((rows + 2 * G) * cols,), -12345.0, dtype=dtype, device=DEV)
        self.before = self.buf.clone()
        self.lo, self.hi = G * cols, (G + rows) * cols
        self.view = self.buf[self.lo:self.hi].view(rows, cols) if cols > 1 else self.buf[self.lo:self.hi]

    def ptr(self):
        return self.view.data_ptr()

    def check(self, expected, what):
        torch.cuda.synchronize()
        assert torch.equal(self.buf[:self.lo], self.before[:self.lo]), f"{what}: written in front of the output"
        assert torch.equal(self.buf[self.hi:], self.before[self.hi:]), f"{what}: written behind the output"
        assert torch.equal(self.view.reshape(-1), expected.reshape(-1)), f"{what}: differs from the call on ordinary tensors"


def _inputs(C, K, dt, wdt, seed, width=1):
    g = torch.Generator().manual_seed(seed)
    T = sum(LENS)
    x = torch.randn(T, width * C, generator=g).to(dt).to(DEV)
    dy = torch.randn(T, C, generator=g).to(dt).to(DEV)
    w = (torch.randn(C, K, generator=g) * K ** -0.5).to(wdt).to(DEV)
    b = (torch.randn(C, generator=g) * 0.02).to(wdt).to(DEV)
    return x, dy, cu_from_lengths(torch.tensor(LENS)).to(DEV), w, b


PLAIN = [(1024, 7, torch.bfloat16), (2048, 31, torch.bfloat16), (1024, 15, torch.bfloat16), (768, 3, torch.bfloat16),
         (256, 7, torch.float32), (512, 31, torch.float32), (100, 11, torch.bfloat16), (520, 31, torch.bfloat16),
         (1152, 9, torch.bfloat16), (24, 5, torch.float32)]


@pytest.mark.parametrize("C,K,dt", PLAIN)
@pytest.mark.parametrize("residual", [False, True])
def test_plain_conv_writes_its_outputs_only(C, K, dt, residual):
    print(f"[case] guard rows, plain C={C} K={K} {dt} residual={residual}", flush=True)
    lib = _lib.load()
    x, dy, cu, w, b = _inputs(C, K, dt, dt, C + K)
    T, S = x.shape[0], cu.numel() - 1
    flags = _lib.RESIDUAL if residual else 0
    stream = torch.cuda.current_stream().cuda_stream
    y_ref = npa.varlen_dwconv_fwd(x, cu, w, b, residual=residual)
    dx_ref, dw_ref, db_ref = npa.varlen_dwconv_bwd(x, dy, cu, w, residual=residual)
    y, dx = Guarded(T, C, dt), Guarded(T, C, dt)
    dw, db = Guarded(C * K, 1, torch.float32), Guarded(C, 1, torch.float32)
    _lib.check(lib.nplm_dwconv_fwd_ex(x.data_ptr(), cu.data_ptr(), w.data_ptr(), b.data_ptr(), y.ptr(), T, C, K, S,
                                      _code(dt), _code(dt), flags, stream), "nplm_dwconv_fwd_ex")
    y.check(y_ref, "y")
    ws = torch.empty(max(int(lib.nplm_dwconv_bwd_workspace_bytes(T, C, K, _code(dt))), 256), dtype=torch.uint8, device=DEV)
    _lib.check(lib.nplm_dwconv_bwd_ex(x.data_ptr(), dy.data_ptr(), cu.data_ptr(), w.data_ptr(), dx.ptr(), dw.ptr(), db.ptr(),
                                      ws.data_ptr(), ws.numel(), T, C, K, S, _code(dt), _code(dt), flags, stream),
               "nplm_dwconv_bwd_ex")
    dx.check(dx_ref, "dx")
    dw.check(dw_ref, "dw")
    db.check(db_ref, "db")
    # dx alone and dw/db alone take other kernels at K = 15 and 31
    dx2 = Guarded(T, C, dt)
    _lib.check(lib.nplm_dwconv_bwd_ex(x.data_ptr(), dy.data_ptr(), cu.data_ptr(), w.data_ptr(), dx2.ptr(), None, None,
                                      ws.data_ptr(), ws.numel(), T, C, K, S, _code(dt), _code(dt), flags, stream),
               "nplm_dwconv_bwd_ex (dx only)")
    dx2.check(npa.varlen_dwconv_bwd(x, dy, cu, w, need_dw=False, residual=residual)[0], "dx alone")


@pytest.mark.parametrize("C,K,dt", [(1024, 7, torch.bfloat16), (2048, 31, torch.bfloat16), (1024, 15, torch.bfloat16),
                                     (1152, 5, torch.bfloat16), (256, 31, torch.float32), (768, 9, torch.float32),
                                     (520, 15, torch.bfloat16)])
def test_gated_conv_writes_its_outputs_only(C, K, dt):
    print(f"[case] guard rows, gated C={C} K={K} {dt}", flush=True)
    lib = _lib.load()
    z, dy, cu, w, b = _inputs(C, K, dt, dt, C + K + 1, width=2)
    assert npa.gated_supported(z, w)
    T, S = z.shape[0], cu.numel() - 1
    stream = torch.cuda.current_stream().cuda_stream
    y_ref = npa.gated_dwconv_fwd(z, cu, w, b)
    dz_ref, dw_ref, db_ref = npa.gated_dwconv_bwd(z, dy, cu, w)
    y, dz = Guarded(T, C, dt), Guarded(T, 2 * C, dt)
    dw, db = Guarded(C * K, 1, torch.float32), Guarded(C, 1, torch.float32)
    _lib.check(lib.nplm_dwconv_gated_fwd(z.data_ptr(), cu.data_ptr(), w.data_ptr(), b.data_ptr(), y.ptr(), T, C, K, S,
                                         _code(dt), _code(dt), 0, stream), "nplm_dwconv_gated_fwd")
    y.check(y_ref, "gated y")
    ws = torch.empty(max(int(lib.nplm_dwconv_gated_bwd_workspace_bytes(T, C, K, _code(dt))), 256), dtype=torch.uint8, device=DEV)
    _lib.check(lib.nplm_dwconv_gated_bwd(z.data_ptr(), dy.data_ptr(), cu.data_ptr(), w.data_ptr(), dz.ptr(), dw.ptr(), db.ptr(),
                                         ws.data_ptr(), ws.numel(), T, C, K, S, _code(dt), _code(dt), 0, stream),
               "nplm_dwconv_gated_bwd")
    dz.check(dz_ref, "dz")
    dw.check(dw_ref, "gated dw")
    db.check(db_ref, "gated db")


@pytest.mark.parametrize("C,K,dt", [(1024, 7, torch.bfloat16), (768, 7, torch.float32), (1024, 7, torch.float32),
                                     (2048, 5, torch.bfloat16), (512, 9, torch.float32), (640, 3, torch.bfloat16),
                                     (1536, 7, torch.float32)])
def test_layernorm_fused_conv_writes_its_outputs_only(C, K, dt):
    """Rows of one 2 KiB column block, of 3 and 4 KiB (whole-row kernels) and wider ones (statistics kernel + conv,
    conv backward + row pass through the fp32 workspace)."""
    print(f"[case] guard rows, layernorm C={C} K={K} {dt}", flush=True)
    lib = _lib.load()
    x, dy, cu, w, b = _inputs(C, K, dt, dt, C + K + 2)
    assert npa.ln_supported(x, w)
    g = torch.Generator().manual_seed(C)
    gam = (1 + 0.1 * torch.randn(C, generator=g)).to(dt).to(DEV)
    bet = (0.1 * torch.randn(C, generator=g)).to(dt).to(DEV)
    T, S = x.shape[0], cu.numel() - 1
    stream = torch.cuda.current_stream().cuda_stream
    y_ref, st_ref = npa.ln_dwconv_fwd(x, cu, gam, bet, w, b, residual=True)
    ref = npa.ln_dwconv_bwd(x, dy, cu, st_ref, gam, bet, w, residual=True)
    y, dx, st = Guarded(T, C, dt), Guarded(T, C, dt), Guarded(T, 2, torch.float32)
    dw, db = Guarded(C * K, 1, torch.float32), Guarded(C, 1, torch.float32)
    dg, dbt = Guarded(C, 1, torch.float32), Guarded(C, 1, torch.float32)
    _lib.check(lib.nplm_dwconv_ln_fwd(x.data_ptr(), cu.data_ptr(), gam.data_ptr(), bet.data_ptr(), 1e-5, w.data_ptr(),
                                      b.data_ptr(), y.ptr(), st.ptr(), T, C, K, S, _code(dt), _code(dt), _lib.RESIDUAL, stream),
               "nplm_dwconv_ln_fwd")
    y.check(y_ref, "layernorm y")
    st.check(st_ref, "row statistics")
    ws = torch.empty(max(int(lib.nplm_dwconv_ln_bwd_workspace_bytes(T, C, K, _code(dt))), 256), dtype=torch.uint8, device=DEV)
    _lib.check(lib.nplm_dwconv_ln_bwd(x.data_ptr(), dy.data_ptr(), cu.data_ptr(), st_ref.data_ptr(), gam.data_ptr(), bet.data_ptr(),
                                      w.data_ptr(), dx.ptr(), dw.ptr(), db.ptr(), dg.ptr(), dbt.ptr(), ws.data_ptr(), ws.numel(),
                                      T, C, K, S, _code(dt), _code(dt), _lib.RESIDUAL, stream), "nplm_dwconv_ln_bwd")
    # ln_dwconv_bwd returns dx, d ln_weight, d ln_bias, dw, db
    for got, want, what in zip((dx, dg, dbt, dw, db), ref, ("dx", "d ln_weight", "d ln_bias", "dw", "db")):
        got.check(want, "layernorm " + what)
