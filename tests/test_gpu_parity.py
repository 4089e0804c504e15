"""GPU parity of the HIP kernels (called through the C ABI) against the CPU oracle.

Every test here needs a real MI355X. Inputs are the seeded configurations of
nanoplm_amd.workloads at their full sizes, the committed golden vectors, and edge cases; the oracle
is oracle/ (C restatement with double accumulation, pinned by tests/test_oracle.py).
"""
import numpy as np
import pytest
import torch

import nanoplm_amd as npa
from nanoplm_amd import _lib
from nanoplm_amd.workloads import cu_from_lengths, make_workload, static_packed_cu
from oracle import dwconv_ref as O

from gpu_util import assert_act_close, assert_red_close, error_stats, record_parity, workload_with_oracle

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _run_all(wl_dev):
    y = npa.varlen_dwconv_fwd(wl_dev.x, wl_dev.cu_seqlens, wl_dev.weight, wl_dev.bias)
    dx, dw, db = npa.varlen_dwconv_bwd(wl_dev.x, wl_dev.dy, wl_dev.cu_seqlens, wl_dev.weight)
    torch.cuda.synchronize()
    return y, dx, dw, db


def test_library_is_loaded_from_the_tree():
    lib = _lib.load()
    assert lib.nplm_dwconv_version() >= 100
    assert torch.cuda.is_available() and "gfx950" in torch.cuda.get_device_properties(0).gcnArchName


# ---- the five configurations at full size ---------------------------------------------------------
@pytest.mark.parametrize("index", [1, 2, 3, 5, 4])
def test_configuration_matches_oracle(index):
    print(f"[case] configuration {index}", flush=True)
    wl, y64, dx64, dw64, db64 = workload_with_oracle(index)
    d = wl.to(DEV)
    y, dx, dw, db = _run_all(d)
    e_y = assert_act_close(y, y64, wl.dtype, f"cfg{index} y")
    e_dx = assert_act_close(dx, dx64, wl.dtype, f"cfg{index} dx")
    e_dw = assert_red_close(dw, dw64, f"cfg{index} dw")
    e_db = assert_red_close(db, db64, f"cfg{index} db")
    print(f"[parity] cfg{index} T={wl.T} C={wl.C} K={wl.K} S={wl.S} {wl.dtype}: max-abs y {e_y:.3e} dx {e_dx:.3e} "
          f"dw {e_dw:.3e} (max|dw| {float(dw64.abs().max()):.1f}) db {e_db:.3e}", flush=True)
    record_parity(f"cfg{index}", {"workload": wl.name, "T": wl.T, "C": wl.C, "K": wl.K, "S": wl.S,
                                  "y": error_stats(y, y64, wl.dtype), "dx": error_stats(dx, dx64, wl.dtype),
                                  "dw": error_stats(dw, dw64), "db": error_stats(db, db64)})
    # run-to-run determinism: bit-identical outputs, reductions included
    y2, dx2, dw2, db2 = _run_all(d)
    assert torch.equal(y, y2) and torch.equal(dx, dx2) and torch.equal(dw, dw2) and torch.equal(db, db2)


@pytest.mark.parametrize("K", [11, 21])
def test_headline_size_with_a_kernel_size_served_by_the_next_built_size(K):
    """Configuration 3's tokens, lengths and width (T=131072, C=1024, bf16) with K = 11 (runs as 15) and K = 21 (runs as
    31, the role-split kernels: every block walks 16 forward and 32 backward tiles) against the C oracle, and run twice."""
    print(f"[case] configuration 3 with K={K}", flush=True)
    wl = make_workload(3, with_dy=True)
    g = torch.Generator().manual_seed(K)
    w = (torch.randn(wl.C, K, generator=g) * K ** -0.5).bfloat16()
    y64 = O.c_oracle_fwd(wl.x, wl.cu_seqlens, w, wl.bias)
    dx64, dw64, db64 = O.c_oracle_bwd(wl.x, wl.dy, wl.cu_seqlens, w)
    xd, dyd, cud, wd, bd = (t.to(DEV) for t in (wl.x, wl.dy, wl.cu_seqlens, w, wl.bias))
    y = npa.varlen_dwconv_fwd(xd, cud, wd, bd)
    dx, dw, db = npa.varlen_dwconv_bwd(xd, dyd, cud, wd)
    assert dw.shape == (wl.C, K)
    assert_act_close(y, y64, wl.dtype, f"K={K} y")
    assert_act_close(dx, dx64, wl.dtype, f"K={K} dx")
    assert_red_close(dw, dw64, f"K={K} dw")
    assert_red_close(db, db64, f"K={K} db")
    dx2, dw2, db2 = npa.varlen_dwconv_bwd(xd, dyd, cud, wd)
    assert torch.equal(y, npa.varlen_dwconv_fwd(xd, cud, wd, bd)) and torch.equal(dx, dx2) and torch.equal(dw, dw2) and torch.equal(db, db2)


def test_configuration_1_against_the_fp32_reference_path():
    """Configuration 1 is defined against the fp32 per-sequence conv1d path itself."""
    wl = make_workload(1)
    y_ref = O.ref_dwconv_varlen(wl.x, wl.cu_seqlens, wl.weight, wl.bias, torch.float32)
    d = wl.to(DEV)
    y = npa.varlen_dwconv_fwd(d.x, d.cu_seqlens, d.weight, d.bias).cpu()
    rel = float((y - y_ref).abs().max() / y_ref.abs().max())
    assert rel <= 1e-5, rel


def _elementwise_rel(got, ref64, floor=1e-3):
    """Largest |got - ref| / |ref| over the elements with |ref| > floor (below it the quotient measures cancellation
    among the K products of size ~1, not the implementation)."""
    err = (got.detach().cpu().double() - ref64).abs()
    big = ref64.abs() > floor
    return float((err[big] / ref64[big].abs()).max()) if big.any() else 0.0


@pytest.mark.parametrize("name,index,kw", [("cfg1", 1, {}), ("cfg3_fp32_T8192_C1024", 3, dict(T=8192, C=1024))])
def test_fp32_elementwise_error_is_that_of_the_fp32_reference_path(name, index, kw):
    """"1e-5 relative" for fp32 is met norm-wise (max error / max |ref|, see gpu_util.assert_act_close). Element by
    element no fp32 evaluation meets it where the taps cancel; the reference path itself (per-sequence torch conv1d +
    autograd in fp32, oracle/dwconv_ref.py) does not. The bar here: against the same float64 oracle, the kernels' largest
    element-wise relative error is at most twice the fp32 reference path's own (plus 1e-6), for every output."""
    wl = make_workload(index, with_dy=True, **kw)
    x, w, b, dy, cu = wl.x.float(), wl.weight.float(), wl.bias.float(), wl.dy.float(), wl.cu_seqlens
    y64 = O.c_oracle_fwd(x, cu, w, b)
    dx64, dw64, db64 = O.c_oracle_bwd(x, dy, cu, w)
    ref = O.ref_dwconv_varlen_grads(x, cu, w, b, dy, torch.float32)
    xd, wd, bd, dyd, cud = (t.to(DEV) for t in (x, w, b, dy, cu))
    y = npa.varlen_dwconv_fwd(xd, cud, wd, bd)
    dx, dw, db = npa.varlen_dwconv_bwd(xd, dyd, cud, wd)
    stats = {}
    for what, got, r32, r64 in (("y", y, ref[0], y64), ("dx", dx, ref[1], dx64), ("dw", dw, ref[2], dw64), ("db", db, ref[3], db64)):
        k_rel, r_rel = _elementwise_rel(got, r64), _elementwise_rel(r32, r64)
        k_norm = float((got.cpu().double() - r64).abs().max() / r64.abs().max())
        r_norm = float((r32.double() - r64).abs().max() / r64.abs().max())
        stats[what] = {"kernel_max_rel": k_rel, "fp32_reference_path_max_rel": r_rel, "kernel_normwise": k_norm,
                       "fp32_reference_path_normwise": r_norm}
        print(f"[parity] {name} fp32 {what}: element-wise max-rel kernel {k_rel:.3e}, fp32 reference path {r_rel:.3e}; "
              f"norm-wise kernel {k_norm:.3e}, reference path {r_norm:.3e}", flush=True)
        assert k_rel <= 2.0 * r_rel + 1e-6, f"{name} {what}: kernel {k_rel:.3e} vs fp32 reference path {r_rel:.3e}"
        assert k_norm <= 1e-5
    record_parity(f"fp32_elementwise_{name}", {"workload": wl.name, "T": wl.T, "C": wl.C, "K": wl.K, **stats})


@pytest.mark.parametrize("C,K,dt", [(1024, 7, torch.bfloat16), (2048, 31, torch.bfloat16), (256, 5, torch.bfloat16),
                                     (100, 11, torch.float32), (768, 15, torch.bfloat16)])
def test_parameter_gradients_straight_in_bf16(C, K, dt):
    """NPLM_DWCONV_GRADS_BF16: the reduction kernel stores dw and db as bf16, rounding its fp32 totals once; that is bit
    for bit the cast of the fp32 outputs (every kernel family ends in the same reduction kernel). dx is unaffected."""
    x, cu, w, b, dy = _random_case([33, 1, 200, 2, 90, 64, 63, 7], C, K, dt, torch.bfloat16, seed=C * K)
    xd, cud, wd, dyd = (t.to(DEV) for t in (x, cu, w, dy))
    dx, dw, db = npa.varlen_dwconv_bwd(xd, dyd, cud, wd)
    dx2, dw2, db2 = npa.varlen_dwconv_bwd(xd, dyd, cud, wd, grads_bf16=True)
    assert dw2.dtype == torch.bfloat16 and db2.dtype == torch.bfloat16
    assert torch.equal(dx, dx2) and torch.equal(dw.bfloat16(), dw2) and torch.equal(db.bfloat16(), db2)
    # a request for dw/db alone may take another kernel family (other summation order): against its own fp32 result
    _, dw3, db3 = npa.varlen_dwconv_bwd(xd, dyd, cud, wd, need_dx=False, grads_bf16=True, residual=True)
    _, dw4, db4 = npa.varlen_dwconv_bwd(xd, dyd, cud, wd, need_dx=False, residual=True)
    assert torch.equal(dw3, dw4.bfloat16()) and torch.equal(db3, db4.bfloat16())
    # empty batch: zero-filled in bf16
    e = torch.empty((0, C), dtype=dt, device=DEV)
    _, dw0, db0 = npa.varlen_dwconv_bwd(e, e, torch.zeros(1, dtype=torch.int32, device=DEV), wd, grads_bf16=True)
    assert dw0.dtype == torch.bfloat16 and float(dw0.float().abs().max()) == 0.0 and float(db0.float().abs().max()) == 0.0


# ---- golden vectors -------------------------------------------------------------------------------
@pytest.mark.parametrize("name", ["cfg1_fp32_C64_K3", "boundary_fp32_C16_K7", "stress_bf16_C32_K7"])
def test_golden_vectors(name, golden_dir):
    z = np.load(f"{golden_dir}/{name}.npz", allow_pickle=False)
    dt = torch.bfloat16 if str(z["act_dtype"]) == "bfloat16" else torch.float32
    x, w, b, dy = (torch.from_numpy(z[k]).to(dt).to(DEV) for k in ("x", "w", "b", "dy"))
    cu = torch.from_numpy(z["cu_seqlens"]).to(DEV)
    y = npa.varlen_dwconv_fwd(x, cu, w, b)
    dx, dw, db = npa.varlen_dwconv_bwd(x, dy, cu, w)
    assert_act_close(y, torch.from_numpy(z["y"]).double(), dt, name + " y")
    assert_act_close(dx, torch.from_numpy(z["dx"]).double(), dt, name + " dx")
    assert_red_close(dw, torch.from_numpy(z["dw"]), name + " dw")
    assert_red_close(db, torch.from_numpy(z["db"]), name + " db")


# ---- shapes, kernel sizes, dtypes -------------------------------------------------------------------
def _random_case(lens, C, K, dt, wdt, seed=0, bias=True):
    g = torch.Generator().manual_seed(seed)
    lens = torch.tensor(lens)
    T = int(lens.sum())
    x = torch.randn(T, C, generator=g).to(dt)
    w = (torch.randn(C, K, generator=g) * K ** -0.5).to(wdt)
    b = (torch.randn(C, generator=g) * 0.02).to(wdt) if bias else None
    dy = torch.randn(T, C, generator=g).to(dt)
    return x, cu_from_lengths(lens), w, b, dy


def _check_case(x, cu, w, b, dy, what):
    y64 = O.c_oracle_fwd(x, cu, w, b)
    dx64, dw64, db64 = O.c_oracle_bwd(x, dy, cu, w)
    xd, cud, wd, dyd = x.to(DEV), cu.to(DEV), w.to(DEV), dy.to(DEV)
    bd = None if b is None else b.to(DEV)
    y = npa.varlen_dwconv_fwd(xd, cud, wd, bd)
    dx, dw, db = npa.varlen_dwconv_bwd(xd, dyd, cud, wd)
    assert_act_close(y, y64, x.dtype, what + " y")
    assert_act_close(dx, dx64, x.dtype, what + " dx")
    assert_red_close(dw, dw64, what + " dw")
    assert_red_close(db, db64, what + " db")


LENS_MIX = [1, 2, 3, 8, 0, 1, 150, 0, 5, 7, 6, 1, 64, 63, 65, 2, 300, 4]


@pytest.mark.parametrize("K", [1, 3, 5, 7, 9, 11, 13, 15, 17, 21, 29, 31, 33])
@pytest.mark.parametrize("dt", [torch.bfloat16, torch.float32])
def test_kernel_sizes(K, dt):
    print(f"[case] K={K} {dt}", flush=True)
    _check_case(*_random_case(LENS_MIX, 256, K, dt, dt, seed=K), f"K={K} {dt}")


@pytest.mark.parametrize("K,Kx,C,dt,wdt", [(11, 15, 1024, torch.bfloat16, torch.bfloat16), (13, 15, 264, torch.bfloat16, torch.float32),
                                           (1, 3, 512, torch.bfloat16, torch.bfloat16), (17, 31, 2048, torch.bfloat16, torch.bfloat16),
                                           (29, 31, 388, torch.float32, torch.float32), (21, 31, 128, torch.float32, torch.bfloat16)])
def test_kernel_sizes_without_kernels_of_their_own_run_as_the_next_size_with_zero_taps(K, Kx, C, dt, wdt):
    """An odd K <= 31 other than 3, 5, 7, 9, 15, 31 is served by the kernels of the next of 3, 15, 31: the caller's [C, K]
    taps sit in the middle of that kernel's taps and the outer ones are zero. Every output must equal, bit for bit, the
    call with explicitly zero-padded [C, Kx] taps (dw: its inner K columns), in every kernel family that size has, with
    and without the fused residual and with gradients stored in bf16; dw / db alone and dx alone take other kernels."""
    print(f"[case] K={K} as {Kx} C={C} {dt} w {wdt}", flush=True)
    x, cu, w, b, dy = _random_case(LENS_SPLIT, C, K, dt, wdt, seed=C + K)
    off = (Kx - K) // 2
    wx = torch.zeros(C, Kx, dtype=wdt)
    wx[:, off:off + K] = w
    xd, cud, wd, wxd, bd, dyd = (t.to(DEV) for t in (x, cu, w, wx, b, dy))
    _check_case(x, cu, w, b, dy, f"K={K}")
    algos = [None, 1] + ([2] if Kx == 3 else []) + ([3] if Kx in (15, 31) and (C * (2 if dt == torch.bfloat16 else 4)) % 16 == 0 else [])
    for algo in algos:
        tn = None if algo is None else _lib.Tuning(algo=algo)
        for res in (False, True):
            assert torch.equal(npa.varlen_dwconv_fwd(xd, cud, wd, bd, residual=res, tuning=tn),
                               npa.varlen_dwconv_fwd(xd, cud, wxd, bd, residual=res, tuning=tn)), (algo, res)
            dx, dw, db = npa.varlen_dwconv_bwd(xd, dyd, cud, wd, residual=res, tuning=tn)
            dxx, dwx, dbx = npa.varlen_dwconv_bwd(xd, dyd, cud, wxd, residual=res, tuning=tn)
            assert dw.shape == (C, K)
            assert torch.equal(dx, dxx) and torch.equal(dw, dwx[:, off:off + K]) and torch.equal(db, dbx), (algo, res)
        _, dwb, dbb = npa.varlen_dwconv_bwd(xd, dyd, cud, wd, grads_bf16=True, tuning=tn)
        assert torch.equal(dwb, dw.bfloat16()) and torch.equal(dbb, db.bfloat16())
    only_dx = npa.varlen_dwconv_bwd(xd, dyd, cud, wd, need_dw=False)[0]
    assert torch.equal(only_dx, npa.varlen_dwconv_bwd(xd, dyd, cud, wxd, need_dw=False)[0])
    _, dw1, db1 = npa.varlen_dwconv_bwd(xd, dyd, cud, wd, need_dx=False)
    _, dw1x, db1x = npa.varlen_dwconv_bwd(xd, dyd, cud, wxd, need_dx=False)
    assert torch.equal(dw1, dw1x[:, off:off + K]) and torch.equal(db1, db1x)


@pytest.mark.parametrize("C", [1, 7, 8, 24, 64, 72, 100, 128, 130, 384, 520, 576, 640, 768, 1000, 1024, 1152, 1280, 2048,
                               2560, 4104])
def test_channel_counts(C):
    """Every lane-slice width (8/4/2/1 channels per lane), partial wave-columns, odd channel counts, and the row
    widths that take 768- and 1280-byte column blocks in the LDS-staged kernels."""
    print(f"[case] C={C}", flush=True)
    _check_case(*_random_case([5, 1, 40, 2, 90, 3], C, 7, torch.bfloat16, torch.bfloat16, seed=C), f"C={C}")
    _check_case(*_random_case([5, 1, 40, 2, 90, 3], C, 3, torch.float32, torch.float32, seed=C), f"C={C} fp32")


@pytest.mark.parametrize("dt,wdt", [(torch.bfloat16, torch.float32), (torch.float32, torch.bfloat16)])
def test_mixed_activation_and_weight_dtypes(dt, wdt):
    _check_case(*_random_case(LENS_MIX, 512, 7, dt, wdt, seed=11), f"{dt}/{wdt}")


def test_no_bias():
    _check_case(*_random_case(LENS_MIX, 256, 7, torch.bfloat16, torch.bfloat16, seed=2, bias=False), "no bias")


@pytest.mark.parametrize("T", [1, 2, 7, 63, 64, 65, 127, 129, 1000])
def test_single_sequence_lengths_around_tile_edges(T):
    _check_case(*_random_case([T], 256, 7, torch.bfloat16, torch.bfloat16, seed=T), f"T={T}")


def test_empty_batch():
    x = torch.empty((0, 64), dtype=torch.bfloat16, device=DEV)
    cu = torch.zeros(1, dtype=torch.int32, device=DEV)
    w = torch.randn(64, 7, device=DEV).bfloat16()
    y = npa.varlen_dwconv_fwd(x, cu, w, None)
    dx, dw, db = npa.varlen_dwconv_bwd(x, x.clone(), cu, w)
    torch.cuda.synchronize()
    assert y.shape == (0, 64) and dx.shape == (0, 64)
    assert float(dw.abs().max()) == 0.0 and float(db.abs().max()) == 0.0


def test_unaligned_views_take_a_narrower_lane_slice():
    """Row slices that start 2 bytes off a 16-byte boundary must still be computed correctly."""
    x, cu, w, b, dy = _random_case([33, 90, 5], 264, 7, torch.bfloat16, torch.bfloat16, seed=4)
    y64 = O.c_oracle_fwd(x, cu, w, b)
    dx64, dw64, db64 = O.c_oracle_bwd(x, dy, cu, w)
    T, C = x.shape
    for off in (1, 2, 4):
        bx = torch.zeros(T * C + 8, dtype=torch.bfloat16, device=DEV)
        bg = torch.zeros(T * C + 8, dtype=torch.bfloat16, device=DEV)
        xv = bx[off:off + T * C].view(T, C)
        gv = bg[off:off + T * C].view(T, C)
        xv.copy_(x)
        gv.copy_(dy)
        assert xv.data_ptr() % 16 == 2 * off
        y = npa.varlen_dwconv_fwd(xv, cu.to(DEV), w.to(DEV), b.to(DEV))
        dx, dw, db = npa.varlen_dwconv_bwd(xv, gv, cu.to(DEV), w.to(DEV))
        assert_act_close(y, y64, x.dtype, f"offset {off} y")
        assert_act_close(dx, dx64, x.dtype, f"offset {off} dx")
        assert_red_close(dw, dw64, f"offset {off} dw")
        assert_red_close(db, db64, f"offset {off} db")


# ---- boundaries -----------------------------------------------------------------------------------
def test_nothing_leaks_across_sequences_even_nan_and_inf():
    x, cu, w, b, dy = _random_case([5, 3, 1, 12, 2, 200, 1, 1, 30], 256, 7, torch.bfloat16, torch.bfloat16, seed=9)
    cul = cu.tolist()
    xd, cud, wd, bd, dyd = (t.to(DEV) for t in (x, cu, w, b, dy))
    y0 = npa.varlen_dwconv_fwd(xd, cud, wd, bd)
    dx0, _, _ = npa.varlen_dwconv_bwd(xd, dyd, cud, wd)
    for seq in (3, 5, 6):
        s, e = cul[seq], cul[seq + 1]
        x2, dy2 = xd.clone(), dyd.clone()
        x2[s:e] = float("nan")
        dy2[s:e] = float("inf")
        y2 = npa.varlen_dwconv_fwd(x2, cud, wd, bd)
        dx2, _, _ = npa.varlen_dwconv_bwd(x2, dy2, cud, wd)
        keep = torch.ones(x.shape[0], dtype=torch.bool, device=DEV)
        keep[s:e] = False
        assert torch.equal(y0[keep], y2[keep]), f"forward leaked out of sequence {seq}"
        assert torch.equal(dx0[keep], dx2[keep]), f"dx leaked out of sequence {seq}"
        assert bool(torch.isnan(y2[s:e]).all())


# lengths with sequences of one and two rows in the middle of tiles, next to tile edges and at the very end (the last
# tile is partial, so its waves also hold copies of the last row)
POISON_LENS = [40, 1, 2, 50, 1, 300, 2, 30, 7, 1, 213, 2, 64, 1, 33, 700, 2, 1]


def _poison_rows(cul, lens, which):
    """Rows of the sequences picked by ``which`` = [(index into lens, ...)] -> (slice list, set of |k - P| reached)."""
    rows, reach = [], 0
    for i in which:
        rows.append((cul[i], cul[i + 1]))
        reach = max(reach, lens[i] - 1)
    return rows, reach


@pytest.mark.parametrize("C,K,dt", [(1024, 7, torch.bfloat16), (1024, 7, torch.float32), (256, 7, torch.bfloat16),
                                     (768, 9, torch.bfloat16), (2048, 31, torch.bfloat16), (1024, 15, torch.bfloat16),
                                     (512, 31, torch.float32), (104, 11, torch.bfloat16), (1024, 3, torch.bfloat16)])
def test_nonfinite_rows_reach_only_the_taps_their_products_belong_to(C, K, dt):
    """dw[c, k] sums x[t + k - P] * dy[t] over the pairs of rows that lie in one sequence. A sequence of L rows
    therefore contributes to the taps with |k - P| < L only: an Inf or NaN in it makes those taps non-finite and must
    leave every other tap of dw (and db, when only x is poisoned) exactly as it is without the poison, on the
    boundary paths of every kernel family (LDS-staged, sliding-window, role-split, runtime-K). Checked against the
    clean run (bit-equal on the untouched taps) and against the oracle (same finite set, same values there)."""
    print(f"[case] non-finite rows and dw: C={C} K={K} {dt}", flush=True)
    P = (K - 1) // 2
    x, cu, w, b, dy = _random_case(POISON_LENS, C, K, dt, dt, seed=C + K)
    cul = cu.tolist()
    xd, cud, wd, dyd = (t.to(DEV) for t in (x, cu, w, dy))
    _, dw0, db0 = npa.varlen_dwconv_bwd(xd, dyd, cud, wd)
    ones = [i for i, n in enumerate(POISON_LENS) if n == 1]
    twos = [i for i, n in enumerate(POISON_LENS) if n == 2]
    cases = [("x: Inf in every one-row sequence", ones, float("inf"), True),
             ("x: NaN in every two-row sequence", twos, float("nan"), True),
             ("x: Inf in the last row of the batch", [len(POISON_LENS) - 1], float("-inf"), True),
             ("dy: Inf in every one-row sequence", ones, float("inf"), False),
             ("dy: NaN in a two-row sequence", twos[1:2], float("nan"), False)]
    for what, which, val, in_x in cases:
        rows, reach = _poison_rows(cul, POISON_LENS, which)
        x2, dy2 = x.clone(), dy.clone()
        for s, e in rows:
            (x2 if in_x else dy2)[s:e] = val
        _, dw, db = npa.varlen_dwconv_bwd(x2.to(DEV), dy2.to(DEV), cud, wd)
        dw64, db64 = O.c_oracle_bwd(x2, dy2, cu, w)[1:]
        touched = torch.tensor([abs(k - P) <= reach for k in range(K)])
        assert bool((~torch.isfinite(dw[:, touched])).all()), f"{what}: a tap the rows feed stayed finite"
        assert torch.equal(dw[:, ~touched], dw0[:, ~touched]), f"{what}: a tap the rows do not feed changed"
        assert torch.equal(torch.isfinite(dw).cpu(), torch.isfinite(dw64)), f"{what}: finite set differs from the oracle's"
        if (~touched).any():
            assert_red_close(dw[:, ~touched], dw64[:, ~touched], f"{what}: dw")
        if in_x:
            assert torch.equal(db, db0), f"{what}: db changed"
        else:
            assert bool((~torch.isfinite(db)).all()) and bool((~torch.isfinite(db64)).all())


def test_static_packed_cu_seqlens():
    """cu_seqlens padded to a fixed length as the static-shape collator emits it (collator.py:430-450):
    pad pseudo-sequences after the real ones, then zero-length entries equal to F."""
    g = torch.Generator().manual_seed(5)
    lens = torch.randint(20, 129, (37,), generator=g)
    real_cu = cu_from_lengths(lens)
    T_real = int(real_cu[-1])
    F, W = 4096, 128
    assert T_real < F
    cu = static_packed_cu(real_cu, F, W, cu_len=96)
    assert int(cu[-1]) == F and int((cu[1:] == cu[:-1]).sum()) > 5
    x = torch.randn(F, 256, generator=g).bfloat16()
    dy = torch.randn(F, 256, generator=g).bfloat16()
    w = (torch.randn(256, 7, generator=g) * 7 ** -0.5).bfloat16()
    b = (torch.randn(256, generator=g) * 0.02).bfloat16()
    _check_case(x, cu, w, b, dy, "static-packed cu")
    npa.check_cu_seqlens(cu.to(DEV), F)


def test_check_cu_seqlens_reports_malformed_input():
    with pytest.raises(RuntimeError, match="cu_seqlens"):
        npa.check_cu_seqlens(torch.tensor([0, 5, 3, 9], dtype=torch.int32, device=DEV), 9)
    with pytest.raises(RuntimeError, match="cu_seqlens"):
        npa.check_cu_seqlens(torch.tensor([0, 5, 9], dtype=torch.int32, device=DEV), 10)
    npa.check_cu_seqlens(torch.tensor([0, 5, 5, 9], dtype=torch.int32, device=DEV), 9)


def test_malformed_cu_seqlens_cannot_fault():
    """cu is used only to mask taps: decreasing / out-of-range entries give garbage values, not faults."""
    x = torch.randn(300, 256, device=DEV).bfloat16()
    w = torch.randn(256, 7, device=DEV).bfloat16()
    for bad in ([0, 500, 20, 10 ** 9, -5, 300], [7, 100], [0], [0, 100]):
        cu = torch.tensor(bad, dtype=torch.int32, device=DEV)
        y = npa.varlen_dwconv_fwd(x, cu, w, None)
        dx, dw, db = npa.varlen_dwconv_bwd(x, x, cu, w)
        torch.cuda.synchronize()
        assert y.shape == x.shape and dx.shape == x.shape


# ---- launch geometry --------------------------------------------------------------------------------
SLIDING = [dict(algo=1, tile_rows=8, bt=1, nbt=1), dict(algo=1, tile_rows=16, bt=2, nbt=3),
           dict(algo=1, tile_rows=64, bt=4, nbt=8, xcd_remap=1), dict(algo=1, tile_rows=128, bt=2, nbt=16, xcd_remap=1),
           dict(algo=1, tile_rows=40, bt=1, nbt=64), dict(algo=1, tile_rows=256, bt=4, nbt=200), dict(algo=1)]
LDS = [dict(algo=2), dict(algo=2, nbt=1), dict(algo=2, nbt=7), dict(algo=2, nbt=100000), dict(algo=2, nbt=33)]


@pytest.mark.parametrize("tune", SLIDING + LDS, ids=lambda d: "-".join(f"{k}{v}" for k, v in d.items()))
def test_results_do_not_depend_on_launch_geometry(tune):
    """y and dx are bit-identical for either kernel family and any tiling; dw/db differ only by
    summation order."""
    wl, y64, dx64, dw64, db64 = workload_with_oracle(5, 9000, 1024)
    d = wl.to(DEV)
    y0, dx0, dw0, db0 = _run_all(d)
    tf = _lib.Tuning(**tune)
    y = npa.varlen_dwconv_fwd(d.x, d.cu_seqlens, d.weight, d.bias, tuning=tf)
    dx, dw, db = npa.varlen_dwconv_bwd(d.x, d.dy, d.cu_seqlens, d.weight, tuning=tf)
    assert torch.equal(y, y0) and torch.equal(dx, dx0)
    assert_red_close(dw, dw64, "dw")
    assert_red_close(db, db64, "db")
    torch.testing.assert_close(dw, dw0, rtol=1e-5, atol=1e-3)


@pytest.mark.parametrize("algo", [1, 2])
@pytest.mark.parametrize("index,T,C", [(5, 20000, 1024), (2, 9000, 2048), (2, 5000, 520)])
def test_both_kernel_families_match_the_oracle(algo, index, T, C):
    wl, y64, dx64, dw64, db64 = workload_with_oracle(index, T, C)
    d = wl.to(DEV)
    tf = _lib.Tuning(algo=algo)
    y = npa.varlen_dwconv_fwd(d.x, d.cu_seqlens, d.weight, d.bias, tuning=tf)
    dx, dw, db = npa.varlen_dwconv_bwd(d.x, d.dy, d.cu_seqlens, d.weight, tuning=tf)
    assert_act_close(y, y64, wl.dtype, "y")
    assert_act_close(dx, dx64, wl.dtype, "dx")
    assert_red_close(dw, dw64, "dw")
    assert_red_close(db, db64, "db")


def test_backward_outputs_can_be_requested_separately():
    wl, y64, dx64, dw64, db64 = workload_with_oracle(5, 9000, 1024)
    d = wl.to(DEV)
    _, dx0, dw0, db0 = _run_all(d)
    dx, dw, db = npa.varlen_dwconv_bwd(d.x, d.dy, d.cu_seqlens, d.weight, need_dw=False)
    assert dw is None and db is None and torch.equal(dx, dx0)
    dx, dw, db = npa.varlen_dwconv_bwd(d.x, d.dy, d.cu_seqlens, d.weight, need_dx=False)
    assert dx is None and torch.equal(dw, dw0) and torch.equal(db, db0)


def test_workspace_contents_do_not_matter():
    wl, *_ = workload_with_oracle(5, 9000, 1024)
    d = wl.to(DEV)
    _, _, dw0, db0 = _run_all(d)
    n = npa.bwd_workspace_bytes(wl.T, wl.C, wl.K, wl.dtype)
    ws = torch.full((n,), 0xFF, dtype=torch.uint8, device=DEV)   # NaN bit patterns everywhere
    _, dw, db = npa.varlen_dwconv_bwd(d.x, d.dy, d.cu_seqlens, d.weight, workspace=ws)
    assert torch.equal(dw, dw0) and torch.equal(db, db0)
    with pytest.raises(RuntimeError, match="workspace"):
        npa.varlen_dwconv_bwd(d.x, d.dy, d.cu_seqlens, d.weight, workspace=ws[: n // 2])


# ---- size-independent properties at the headline size -------------------------------------------------
def test_linearity_and_adjoint_identity_at_full_size():
    wl = make_workload(3).to(DEV)
    x, cu, w, dy = wl.x, wl.cu_seqlens, wl.weight, wl.dy
    y = npa.varlen_dwconv_fwd(x, cu, w, None)
    dx, dw, db = npa.varlen_dwconv_bwd(x, dy, cu, w)
    # <conv(x), dy> = <x, dx> = <w, dw>, each side accumulated in fp64 on the device. y and dx carry
    # one bf16 rounding per element (relative 2^-9, random sign), so the sums agree to ~1e-4 relative.
    lhs = (y.double() * dy.double()).sum()
    mid = (x.double() * dx.double()).sum()
    rhs = (w.double() * dw.double()).sum()
    scale = float((y.double().abs() * dy.double().abs()).sum())
    assert abs(float(lhs - mid)) <= 1e-4 * scale and abs(float(lhs - rhs)) <= 1e-4 * scale
    torch.testing.assert_close(db.double(), dy.double().sum(0), rtol=1e-6, atol=1e-3)
    # scaling x by 2 (exact in bf16) scales y and dw exactly by 2
    y2 = npa.varlen_dwconv_fwd(x * 2, cu, w, None)
    assert torch.equal(y2, y * 2)
    _, dw2, _ = npa.varlen_dwconv_bwd(x * 2, dy, cu, w, need_dx=False)
    assert torch.equal(dw2, dw * 2)


def test_rows_beyond_2_and_4_gib_offsets():
    """Maximum-size edge: 2.2 M rows x 2 KiB = 4.5 GB per tensor, so row offsets cross both 2^31 and 2^32
    bytes. Size-independent property: a run of whole sequences cut out of the big batch and processed
    alone (re-based cu_seqlens) gives bit-identical y and dx; dw/db agree between the two kernel families."""
    T, C, K = 2_200_000, 1024, 7
    g = torch.Generator().manual_seed(77)
    lens = torch.randint(20, 513, (T // 200,), generator=g)
    lens = lens[torch.cumsum(lens, 0) <= T]
    lens = torch.cat([lens, torch.tensor([T - int(lens.sum())])])
    cu = cu_from_lengths(lens).to(DEV)
    x = torch.randn(T, C, device=DEV, dtype=torch.bfloat16)
    dy = torch.randn(T, C, device=DEV, dtype=torch.bfloat16)
    w = (torch.randn(C, K, device=DEV) * K ** -0.5).bfloat16()
    b = (torch.randn(C, device=DEV) * 0.02).bfloat16()
    y = npa.varlen_dwconv_fwd(x, cu, w, b)
    dx, dw, db = npa.varlen_dwconv_bwd(x, dy, cu, w)
    cul = cu.tolist()
    S = len(cul) - 1
    for first, count in ((0, 40), (S // 2 - 20, 40), (S - 40, 40)):     # start, around 2-4 GiB, end
        s, e = cul[first], cul[first + count]
        sub = (cu[first:first + count + 1] - s).contiguous()
        ys = npa.varlen_dwconv_fwd(x[s:e], sub, w, b)
        dxs, _, _ = npa.varlen_dwconv_bwd(x[s:e], dy[s:e], sub, w)
        assert torch.equal(y[s:e], ys) and torch.equal(dx[s:e], dxs), f"rows {s}..{e}"
    assert (S // 2) > 0 and cul[S // 2] * C * 2 > 2 ** 31 and cul[S - 40] * C * 2 > 2 ** 32
    _, dw1, db1 = npa.varlen_dwconv_bwd(x, dy, cu, w, need_dx=False, tuning=_lib.Tuning(algo=1))
    torch.testing.assert_close(dw, dw1, rtol=2e-5, atol=0.05)
    torch.testing.assert_close(db, db1, rtol=2e-5, atol=0.05)
    torch.testing.assert_close(db, dy.float().sum(0), rtol=2e-5, atol=0.05)


@pytest.mark.parametrize("K,C,dt", [(7, 1024, torch.bfloat16), (7, 512, torch.float32), (31, 1024, torch.bfloat16),
                                    (9, 1024, torch.bfloat16), (7, 768, torch.bfloat16), (9, 1152, torch.bfloat16),
                                    (9, 1280, torch.bfloat16), (5, 576, torch.float32), (3, 320, torch.float32),
                                    (15, 1024, torch.bfloat16)])
@pytest.mark.parametrize("seq_len,nbt", [(64, 0), (96, 24), (17, 10), (512, 7)])
def test_equal_length_sequences_on_rotating_tile_slots(K, C, dt, seq_len, nbt):
    """Equal-length sequences put boundaries at a fixed period of tiles; the LDS kernels rotate the tile slots
    from round to round, and in the last round some blocks have no tile (2700 rows is not a whole number of
    rounds for any of these grids). Both kernel families must agree bit for bit on y and dx."""
    print(f"[case] K={K} C={C} {dt} seq_len={seq_len} nbt={nbt}", flush=True)
    T = 2700
    lens = [seq_len] * (T // seq_len) + ([T % seq_len] if T % seq_len else [])
    x, cu, w, b, dy = _random_case(lens, C, K, dt, dt, seed=K + seq_len)
    _check_case(x, cu, w, b, dy, f"K={K} seq_len={seq_len}")
    xd, cud, wd, bd, dyd = x.to(DEV), cu.to(DEV), w.to(DEV), b.to(DEV), dy.to(DEV)
    outs = []
    for algo in (1, 2):
        tf = _lib.Tuning(algo=algo, nbt=nbt)
        y = npa.varlen_dwconv_fwd(xd, cud, wd, bd, tuning=tf)
        try:
            dx, dw, db = npa.varlen_dwconv_bwd(xd, dyd, cud, wd, tuning=tf)
        except RuntimeError:         # no single-role LDS-staged backward at K = 15, 31
            assert algo == 2 and K in (15, 31)
            dx = None
        outs.append((y, dx))
    assert torch.equal(outs[0][0], outs[1][0])
    if outs[1][1] is not None:
        assert torch.equal(outs[0][1], outs[1][1])
    if K in (15, 31):                # the role-split LDS-staged kernels rotate their tile slots the same way
        tf = _lib.Tuning(algo=3, nbt=nbt)
        assert torch.equal(npa.varlen_dwconv_fwd(xd, cud, wd, bd, tuning=tf), outs[0][0])
        dx, dw, db = npa.varlen_dwconv_bwd(xd, dyd, cud, wd, tuning=tf)
        assert torch.equal(dx, outs[0][1])


# ---- role-split LDS-staged kernels (K = 31, 15) -------------------------------------------------------
LENS_SPLIT = [1, 2, 3, 8, 0, 1, 150, 0, 5, 7, 6, 1, 64, 63, 65, 2, 300, 4, 15, 16, 17, 30, 31, 32, 33, 700, 1, 1, 1,
              29, 0, 0, 45, 1200, 14]


@pytest.mark.parametrize("K,C,dt,nbt", [(31, 256, torch.bfloat16, 1), (31, 256, torch.bfloat16, 2), (15, 512, torch.bfloat16, 1),
                                        (31, 128, torch.float32, 1), (15, 128, torch.float32, 3)])
def test_role_split_blocks_that_walk_more_than_64_tiles(K, C, dt, nbt):
    """A block looks up the sequence of its next tile in a table it fills for its first 64 rounds and by a binary search
    after that; with at least 16 sequences (fewer: always the search). One to three blocks over 11388 rows walk 178, 89
    and 60 backward tiles of 64 rows and 89, 45 and 30 forward tiles of 128 rows each: both sides of that switch, in both
    passes. y and dx equal the sliding-window kernels' bit for bit, everything the oracle's."""
    print(f"[case] K={K} C={C} {dt} nbt={nbt}", flush=True)
    x, cu, w, b, dy = _random_case(LENS_SPLIT * 4, C, K, dt, dt, seed=C + nbt + K)
    assert x.shape[0] == 11388 and cu.numel() - 1 >= 16
    xd, cud, wd, dyd, bd = x.to(DEV), cu.to(DEV), w.to(DEV), dy.to(DEV), b.to(DEV)
    y1 = npa.varlen_dwconv_fwd(xd, cud, wd, bd, tuning=_lib.Tuning(algo=1))
    y3 = npa.varlen_dwconv_fwd(xd, cud, wd, bd, tuning=_lib.Tuning(algo=3, nbt=nbt))
    assert torch.equal(y3, y1)
    assert_act_close(y3, O.c_oracle_fwd(x, cu, w, b), dt, "y")
    dx64, dw64, db64 = O.c_oracle_bwd(x, dy, cu, w)
    dx1, dw1, db1 = npa.varlen_dwconv_bwd(xd, dyd, cud, wd, tuning=_lib.Tuning(algo=1))
    dx3, dw3, db3 = npa.varlen_dwconv_bwd(xd, dyd, cud, wd, tuning=_lib.Tuning(algo=3, nbt=nbt))
    assert torch.equal(dx3, dx1)
    assert_act_close(dx3, dx64, dt, "dx")
    assert_red_close(dw3, dw64, "dw")
    assert_red_close(db3, db64, "db")
    # the same rows as fewer than 16 sequences (the search in every round): neighbours merged, same total
    lens = torch.tensor(LENS_SPLIT * 4).view(-1, 14).sum(1).tolist()
    cu2 = cu_from_lengths(torch.tensor(lens))
    assert cu2.numel() - 1 == 10 and int(cu2[-1]) == x.shape[0]
    dx64b, dw64b, db64b = O.c_oracle_bwd(x, dy, cu2, w)
    dxb, dwb, dbb = npa.varlen_dwconv_bwd(xd, dyd, cu2.to(DEV), wd, tuning=_lib.Tuning(algo=3, nbt=nbt))
    assert torch.equal(dxb, npa.varlen_dwconv_bwd(xd, dyd, cu2.to(DEV), wd, tuning=_lib.Tuning(algo=1))[0])
    assert_act_close(dxb, dx64b, dt, "dx, 10 sequences")
    assert_red_close(dwb, dw64b, "dw, 10 sequences")
    assert_red_close(dbb, db64b, "db, 10 sequences")


@pytest.mark.parametrize("C,dt", [(256, torch.bfloat16), (264, torch.bfloat16), (1024, torch.bfloat16),
                                  (1152, torch.bfloat16), (2048, torch.bfloat16), (2056, torch.bfloat16),
                                  (128, torch.float32), (388, torch.float32), (1024, torch.float32)])
@pytest.mark.parametrize("nbt", [0, 1, 5])
@pytest.mark.parametrize("K", [31, 15])
def test_role_split_kernels_match_the_sliding_window_kernels_and_the_oracle(K, C, dt, nbt):
    """A fused K = 31 or 15 backward is served by a kernel whose waves are split into a dx role and a dw/db role over
    the same LDS tiles, the K = 31 forward by the dx role alone (at K = 15 on request). Sequences shorter than the
    halo, tile-edge lengths, empty sequences, partial column blocks and one or a few blocks walking every tile: y
    and dx must equal the sliding-window kernels' bit for bit, and dw/db the oracle's to the reduction tolerance."""
    print(f"[case] K={K} C={C} {dt} nbt={nbt}", flush=True)
    x, cu, w, b, dy = _random_case(LENS_SPLIT, C, K, dt, dt, seed=C + nbt + K)
    y64 = O.c_oracle_fwd(x, cu, w, b)
    dx64, dw64, db64 = O.c_oracle_bwd(x, dy, cu, w)
    xd, cud, wd, dyd, bd = x.to(DEV), cu.to(DEV), w.to(DEV), dy.to(DEV), b.to(DEV)
    for bias, res in ((bd, False), (None, False), (bd, True)):
        y1 = npa.varlen_dwconv_fwd(xd, cud, wd, bias, residual=res, tuning=_lib.Tuning(algo=1))
        y3 = npa.varlen_dwconv_fwd(xd, cud, wd, bias, residual=res, tuning=_lib.Tuning(algo=3, nbt=nbt))
        assert torch.equal(y3, y1)
        if nbt == 0:                                                             # (K = 15: the LDS-staged forward)
            assert torch.equal(npa.varlen_dwconv_fwd(xd, cud, wd, bias, residual=res), y3)
        if bias is not None and not res:
            assert_act_close(y3, y64, dt, "y")
    dx1, dw1, db1 = npa.varlen_dwconv_bwd(xd, dyd, cud, wd, tuning=_lib.Tuning(algo=1))
    dx3, dw3, db3 = npa.varlen_dwconv_bwd(xd, dyd, cud, wd, tuning=_lib.Tuning(algo=3, nbt=nbt))
    assert torch.equal(dx3, dx1)
    assert_act_close(dx3, dx64, dt, "dx")
    assert_red_close(dw3, dw64, "dw")
    assert_red_close(db3, db64, "db")
    torch.testing.assert_close(dw3, dw1, rtol=1e-5, atol=1e-3)
    again = npa.varlen_dwconv_bwd(xd, dyd, cud, wd, tuning=_lib.Tuning(algo=3, nbt=nbt))
    assert all(torch.equal(a, b_) for a, b_ in zip(again, (dx3, dw3, db3)))      # fixed summation order
    if nbt == 0:                                                                 # and it is the library's choice
        assert all(torch.equal(a, b_) for a, b_ in zip(npa.varlen_dwconv_bwd(xd, dyd, cud, wd), (dx3, dw3, db3)))


def test_role_split_kernels_serve_only_what_they_are_built_for():
    x, cu, w, b, dy = _random_case(LENS_SPLIT, 512, 31, torch.bfloat16, torch.bfloat16, seed=3)
    xd, cud, wd, dyd = x.to(DEV), cu.to(DEV), w.to(DEV), dy.to(DEV)
    dx0, dw0, db0 = npa.varlen_dwconv_bwd(xd, dyd, cud, wd)
    dx1, dw1, db1 = npa.varlen_dwconv_bwd(xd, dyd, cud, wd, tuning=_lib.Tuning(algo=1))
    dx, dw, db = npa.varlen_dwconv_bwd(xd, dyd, cud, wd, need_dw=False)           # partial requests: sliding-window
    assert dw is None and db is None and torch.equal(dx, dx0)
    dx, dw, db = npa.varlen_dwconv_bwd(xd, dyd, cud, wd, need_dx=False)
    assert dx is None and torch.equal(dw, dw1) and torch.equal(db, db1)
    assert_red_close(dw0, dw1.double().cpu(), "dw")
    with pytest.raises(RuntimeError):
        npa.varlen_dwconv_bwd(xd, dyd, cud, wd, need_dx=False, tuning=_lib.Tuning(algo=3))
    x, cu, w, b, dy = _random_case(LENS_SPLIT, 512, 9, torch.bfloat16, torch.bfloat16, seed=4)
    with pytest.raises(RuntimeError):                                             # K = 9 has no role-split kernel
        npa.varlen_dwconv_bwd(x.to(DEV), dy.to(DEV), cu.to(DEV), w.to(DEV), tuning=_lib.Tuning(algo=3))
    with pytest.raises(RuntimeError):
        npa.varlen_dwconv_fwd(x.to(DEV), cu.to(DEV), w.to(DEV), None, tuning=_lib.Tuning(algo=3))
    x, cu, w, b, dy = _random_case([40, 3], 64, 31, torch.bfloat16, torch.bfloat16, seed=5)   # rows too narrow
    with pytest.raises(RuntimeError):
        npa.varlen_dwconv_bwd(x.to(DEV), dy.to(DEV), cu.to(DEV), w.to(DEV), tuning=_lib.Tuning(algo=3))
    with pytest.raises(RuntimeError):
        npa.varlen_dwconv_fwd(x.to(DEV), cu.to(DEV), w.to(DEV), None, tuning=_lib.Tuning(algo=3))
    _check_case(x, cu, w, b, dy, "narrow rows K=31")
