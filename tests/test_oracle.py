"""Pins the CPU oracles (oracle/) before anything is checked against them.

The reference holds no convolution and no vectors for one, so the oracle is pinned by
 (i)   the library routine: torch.nn.functional.conv1d per sequence (and its autograd), fp64;
 (ii)  a C restatement from the definition and a pure-Python brute force with a different loop
       structure (scatter form for the gradients);
 (iii) closed forms a dropped term / wrong sign / off-by-one padding / flipped kernel would fail;
 (iv)  identities: adjoint <conv(x), dy> = <x, dx>, bilinear <conv(x; w), dy> = <w, dw>, no leakage,
       finite differences;
 (v)   the committed golden vectors.
"""
import numpy as np
import pytest
import torch

from nanoplm_amd.workloads import cu_from_lengths, make_workload
from oracle import dwconv_ref as O

torch.manual_seed(0)


def _case(lens, C, K, seed=0, bias=True):
    g = torch.Generator().manual_seed(seed)
    lens = torch.tensor(lens)
    T = int(lens.sum())
    x = torch.randn(T, C, generator=g, dtype=torch.float64).float()
    w = torch.randn(C, K, generator=g, dtype=torch.float64).float()
    b = torch.randn(C, generator=g, dtype=torch.float64).float() if bias else None
    dy = torch.randn(T, C, generator=g, dtype=torch.float64).float()
    return x, cu_from_lengths(lens), w, b, dy


CASES = [
    ([5], 3, 3),
    ([1, 1, 1], 2, 3),
    ([1, 2, 3, 8, 0, 1, 30, 0, 5], 4, 7),
    ([10, 20, 3], 5, 5),
    ([40, 2], 3, 31),
    ([7, 7, 7], 6, 1),
    ([0, 0, 4, 0], 2, 9),
]


@pytest.mark.parametrize("lens,C,K", CASES)
def test_three_statements_agree(lens, C, K):
    x, cu, w, b, dy = _case(lens, C, K)
    y_t, dx_t, dw_t, db_t = O.ref_dwconv_varlen_grads(x, cu, w, b, dy, torch.float64)
    y_c = O.c_oracle_fwd(x, cu, w, b)
    dx_c, dw_c, db_c = O.c_oracle_bwd(x, dy, cu, w)
    y_b, dx_b, dw_b, db_b = O.brute_force(x, cu, w, b, dy)
    for a, c, d in ((y_t, y_c, y_b), (dx_t, dx_c, dx_b), (dw_t, dw_c, dw_b), (db_t, db_c, db_b)):
        torch.testing.assert_close(a, c, rtol=1e-12, atol=1e-12)
        torch.testing.assert_close(a, d, rtol=1e-12, atol=1e-12)


def test_no_bias_path():
    x, cu, w, _, dy = _case([6, 9, 2], 3, 5, bias=False)
    y_t = O.ref_dwconv_varlen(x, cu, w, None, torch.float64)
    torch.testing.assert_close(y_t, O.c_oracle_fwd(x, cu, w, None), rtol=1e-12, atol=1e-12)
    torch.testing.assert_close(y_t, O.brute_force(x, cu, w, None), rtol=1e-12, atol=1e-12)


# ---- closed forms --------------------------------------------------------------------------
def test_k1_is_scale_and_shift():
    x, cu, w, b, _ = _case([4, 9, 1], 5, 1)
    want = x.double() * w.double()[:, 0] + b.double()
    torch.testing.assert_close(O.c_oracle_fwd(x, cu, w, b), want, rtol=0, atol=1e-14)
    torch.testing.assert_close(O.ref_dwconv_varlen(x, cu, w, b, torch.float64), want, rtol=0, atol=1e-14)


@pytest.mark.parametrize("K", [3, 7, 31])
def test_centre_delta_is_identity(K):
    x, cu, _, b, _ = _case([3, 50, 1, 12], 4, K)
    w = torch.zeros(4, K)
    w[:, (K - 1) // 2] = 1.0
    want = x.double() + b.double()
    torch.testing.assert_close(O.c_oracle_fwd(x, cu, w, b), want, rtol=0, atol=0)
    torch.testing.assert_close(O.ref_dwconv_varlen(x, cu, w, b, torch.float64), want, rtol=0, atol=1e-15)


@pytest.mark.parametrize("K,shift", [(3, -1), (3, 1), (7, -3), (7, 2)])
def test_off_centre_delta_shifts_without_flip(K, shift):
    """w = delta at tap P+shift  =>  y[t] = x[t+shift] inside the sequence, 0 past its ends.
    A flipped kernel (true convolution) would give x[t-shift]."""
    lens = [9, 4, 1, 15]
    x, cu, _, _, _ = _case(lens, 2, K)
    w = torch.zeros(2, K)
    w[:, (K - 1) // 2 + shift] = 1.0
    want = torch.zeros_like(x, dtype=torch.float64)
    cul = cu.tolist()
    for s, e in zip(cul[:-1], cul[1:]):
        for t in range(s, e):
            if s <= t + shift < e:
                want[t] = x[t + shift].double()
    torch.testing.assert_close(O.c_oracle_fwd(x, cu, w, None), want, rtol=0, atol=0)
    torch.testing.assert_close(O.ref_dwconv_varlen(x, cu, w, None, torch.float64), want, rtol=0, atol=0)


@pytest.mark.parametrize("K", [3, 7, 31])
def test_all_ones_kernel_is_clipped_window_sum(K):
    """w = 1, b = 0  =>  y[t] = prefix(min(e, t+P+1)) - prefix(max(s, t-P)) within the sequence."""
    lens = [1, 2, 40, 5, 3, 64]
    x, cu, _, _, _ = _case(lens, 3, K)
    w = torch.ones(3, K)
    P = (K - 1) // 2
    pre = torch.cat([torch.zeros(1, 3, dtype=torch.float64), torch.cumsum(x.double(), 0)])
    want = torch.empty_like(x, dtype=torch.float64)
    cul = cu.tolist()
    for s, e in zip(cul[:-1], cul[1:]):
        for t in range(s, e):
            want[t] = pre[min(e, t + P + 1)] - pre[max(s, t - P)]
    torch.testing.assert_close(O.c_oracle_fwd(x, cu, w, None), want, rtol=1e-12, atol=1e-12)
    torch.testing.assert_close(O.ref_dwconv_varlen(x, cu, w, None, torch.float64), want, rtol=1e-12, atol=1e-12)


def test_length_one_sequences_see_only_the_centre_tap():
    x, cu, w, b, dy = _case([1] * 9, 4, 7)
    want = x.double() * w.double()[:, 3] + b.double()
    torch.testing.assert_close(O.c_oracle_fwd(x, cu, w, b), want, rtol=0, atol=1e-14)
    dx, dw, db = O.c_oracle_bwd(x, dy, cu, w)
    torch.testing.assert_close(dx, dy.double() * w.double()[:, 3], rtol=0, atol=1e-14)
    want_dw = torch.zeros(4, 7, dtype=torch.float64)
    want_dw[:, 3] = (dy.double() * x.double()).sum(0)
    torch.testing.assert_close(dw, want_dw, rtol=1e-13, atol=1e-13)
    torch.testing.assert_close(db, dy.double().sum(0), rtol=1e-13, atol=1e-13)


# ---- identities ------------------------------------------------------------------------------
@pytest.mark.parametrize("lens,C,K", CASES)
def test_adjoint_and_bilinear_identities(lens, C, K):
    x, cu, w, _, dy = _case(lens, C, K, seed=3)
    y0 = O.c_oracle_fwd(x, cu, w, None)
    dx, dw, db = O.c_oracle_bwd(x, dy, cu, w)
    lhs = (y0 * dy.double()).sum()
    torch.testing.assert_close(lhs, (x.double() * dx).sum(), rtol=1e-11, atol=1e-11)
    torch.testing.assert_close(lhs, (w.double() * dw).sum(), rtol=1e-11, atol=1e-11)
    torch.testing.assert_close(db, dy.double().sum(0), rtol=1e-12, atol=1e-12)


def test_no_leak_between_sequences():
    x, cu, w, b, dy = _case([5, 3, 1, 12, 2], 3, 7)
    y = O.c_oracle_fwd(x, cu, w, b)
    dx, _, _ = O.c_oracle_bwd(x, dy, cu, w)
    x2, dy2 = x.clone(), dy.clone()
    x2[9:21] = 1e6      # sequence 3 = rows [9, 21)
    dy2[9:21] = -1e6
    y2 = O.c_oracle_fwd(x2, cu, w, b)
    dx2, _, _ = O.c_oracle_bwd(x2, dy2, cu, w)
    keep = torch.ones(x.shape[0], dtype=torch.bool)
    keep[9:21] = False
    assert torch.equal(y[keep], y2[keep])
    assert torch.equal(dx[keep], dx2[keep])
    y2t = O.ref_dwconv_varlen(x2, cu, w, b, torch.float64)
    assert torch.equal(O.ref_dwconv_varlen(x, cu, w, b, torch.float64)[keep], y2t[keep])


def test_finite_differences_of_the_c_oracle():
    x, cu, w, b, dy = _case([4, 1, 6], 2, 5, seed=5)
    dx, dw, db = O.c_oracle_bwd(x, dy, cu, w)

    def loss(xx, ww, bb):
        return float((O.c_oracle_fwd(xx, cu, ww, bb) * dy.double()).sum())

    # the operator is bilinear, so a central difference is exact up to rounding; use exactly
    # representable steps
    h = 2.0 ** -6
    for (t, c) in [(0, 0), (3, 1), (4, 0), (10, 1)]:
        xp, xm = x.clone(), x.clone()
        xp[t, c] += h
        xm[t, c] -= h
        assert abs((loss(xp, w, b) - loss(xm, w, b)) / (2 * h) - float(dx[t, c])) < 1e-9
    for (c, k) in [(0, 0), (1, 2), (0, 4)]:
        wp, wm = w.clone(), w.clone()
        wp[c, k] += h
        wm[c, k] -= h
        assert abs((loss(x, wp, b) - loss(x, wm, b)) / (2 * h) - float(dw[c, k])) < 1e-9
    bp, bm = b.clone(), b.clone()
    bp[1] += h
    bm[1] -= h
    assert abs((loss(x, w, bp) - loss(x, w, bm)) / (2 * h) - float(db[1])) < 1e-9


def test_gradcheck_of_the_reference_path():
    x, cu, w, b, _ = _case([3, 1, 5], 2, 3, seed=7)
    xd = x.double().requires_grad_(True)
    wd = w.double().requires_grad_(True)
    bd = b.double().requires_grad_(True)
    assert torch.autograd.gradcheck(lambda a, c, d: O.ref_dwconv_varlen(a, cu, c, d, torch.float64), (xd, wd, bd))


def test_sequence_permutation_equivariance():
    lens = [4, 9, 1, 6]
    x, cu, w, b, _ = _case(lens, 3, 5)
    y = O.c_oracle_fwd(x, cu, w, b)
    order = [2, 0, 3, 1]
    cul = cu.tolist()
    xs = [x[cul[i]:cul[i + 1]] for i in range(4)]
    ys = [y[cul[i]:cul[i + 1]] for i in range(4)]
    x2 = torch.cat([xs[i] for i in order])
    cu2 = cu_from_lengths(torch.tensor([lens[i] for i in order]))
    assert torch.equal(O.c_oracle_fwd(x2, cu2, w, b), torch.cat([ys[i] for i in order]))


def test_c_oracle_rejects_malformed_inputs():
    x, cu, w, b, _ = _case([4, 4], 2, 3)
    bad = cu.clone()
    bad[-1] = 7
    with pytest.raises(ValueError):
        O.c_oracle_fwd(x, bad, w, b)
    bad = torch.tensor([0, 5, 3, 8], dtype=torch.int32)
    with pytest.raises(ValueError):
        O.c_oracle_fwd(x, bad, w, b)
    with pytest.raises(ValueError):
        O.c_oracle_fwd(x, cu, torch.randn(2, 4), b)


# ---- medium size: library routine vs C restatement on benchmark-style inputs -------------------
@pytest.mark.parametrize("index,T,C", [(1, None, None), (2, 3000, 96), (4, 5000, 40), (5, 6000, 64)])
def test_reference_path_vs_c_oracle_on_config_mixes(index, T, C):
    wl = make_workload(index, T=T, C=C, with_dy=True)
    y_t, dx_t, dw_t, db_t = O.ref_dwconv_varlen_grads(wl.x, wl.cu_seqlens, wl.weight, wl.bias, wl.dy, torch.float64)
    y_c = O.c_oracle_fwd(wl.x, wl.cu_seqlens, wl.weight, wl.bias)
    dx_c, dw_c, db_c = O.c_oracle_bwd(wl.x, wl.dy, wl.cu_seqlens, wl.weight)
    torch.testing.assert_close(y_t, y_c, rtol=1e-11, atol=1e-11)
    torch.testing.assert_close(dx_t, dx_c, rtol=1e-11, atol=1e-11)
    torch.testing.assert_close(dw_t, dw_c, rtol=1e-11, atol=1e-10)
    torch.testing.assert_close(db_t, db_c, rtol=1e-11, atol=1e-10)


def test_fp32_reference_path_meets_the_fp32_tolerance_against_fp64():
    """The fp32 tolerance for the kernels (1e-5 relative) must be meaningful for configuration 1."""
    wl = make_workload(1)
    y32 = O.ref_dwconv_varlen(wl.x, wl.cu_seqlens, wl.weight, wl.bias, torch.float32).double()
    y64 = O.c_oracle_fwd(wl.x, wl.cu_seqlens, wl.weight, wl.bias)
    assert float((y32 - y64).abs().max() / y64.abs().max()) < 1e-6


# ---- golden vectors -----------------------------------------------------------------------------
GOLDEN = ["cfg1_fp32_C64_K3", "boundary_fp32_C16_K7", "stress_bf16_C32_K7"]


@pytest.mark.parametrize("name", GOLDEN)
def test_oracles_reproduce_golden_vectors(name, golden_dir):
    z = np.load(f"{golden_dir}/{name}.npz", allow_pickle=False)
    x, w, b, dy = (torch.from_numpy(z[k]) for k in ("x", "w", "b", "dy"))
    cu = torch.from_numpy(z["cu_seqlens"])
    y_c = O.c_oracle_fwd(x, cu, w, b)
    dx_c, dw_c, db_c = O.c_oracle_bwd(x, dy, cu, w)
    # y/dx are stored rounded to float32
    torch.testing.assert_close(y_c.float(), torch.from_numpy(z["y"]), rtol=0, atol=0)
    torch.testing.assert_close(dx_c.float(), torch.from_numpy(z["dx"]), rtol=0, atol=0)
    torch.testing.assert_close(dw_c, torch.from_numpy(z["dw"]), rtol=1e-12, atol=1e-12)
    torch.testing.assert_close(db_c, torch.from_numpy(z["db"]), rtol=1e-12, atol=1e-12)
    if name.startswith("stress_bf16"):
        # inputs really are bf16-representable
        assert torch.equal(x, x.bfloat16().float()) and torch.equal(dy, dy.bfloat16().float())


def test_golden_cfg1_is_configuration_1(golden_dir):
    z = np.load(f"{golden_dir}/cfg1_fp32_C64_K3.npz", allow_pickle=False)
    wl = make_workload(1)
    assert np.array_equal(z["x"], wl.x.numpy()) and np.array_equal(z["cu_seqlens"], wl.cu_seqlens.numpy())
    assert z["x"].shape[1] == 64 and z["w"].shape == (64, 3) and len(z["cu_seqlens"]) == 9
    lens = np.diff(z["cu_seqlens"])
    assert lens.min() >= 20 and lens.max() <= 128


# ---- residual connection (x + conv(x)) ---------------------------------------------------------------
def test_residual_oracles_agree_and_reduce_to_the_centre_weight_identity():
    """x + conv(x; w) = conv(x; w + delta_centre) because the centre tap is valid for every row; the
    three statements of the operator agree on it, and the gradients are dy + conv^T(dy), dw, db."""
    g = torch.Generator().manual_seed(77)
    lens = torch.tensor([1, 2, 9, 0, 3, 30, 1])
    cu = torch.zeros(len(lens) + 1, dtype=torch.int32)
    cu[1:] = torch.cumsum(lens, 0)
    T, C, K = int(lens.sum()), 6, 5
    x = torch.randn(T, C, generator=g, dtype=torch.float64)
    w = torch.randn(C, K, generator=g, dtype=torch.float64)
    b = torch.randn(C, generator=g, dtype=torch.float64)
    dy = torch.randn(T, C, generator=g, dtype=torch.float64)
    w1 = w.clone()
    w1[:, (K - 1) // 2] += 1.0
    y_res, dx_res, dw_res, db_res = O.ref_dwconv_varlen_grads(x, cu, w, b, dy, torch.float64, residual=True)
    y_id, dx_id, dw_id, db_id = O.ref_dwconv_varlen_grads(x, cu, w1, b, dy, torch.float64)
    torch.testing.assert_close(y_res, y_id, rtol=0, atol=1e-12)
    torch.testing.assert_close(dx_res, dx_id, rtol=0, atol=1e-12)
    torch.testing.assert_close(dw_res, dw_id, rtol=0, atol=1e-12)      # dw does not see the identity
    torch.testing.assert_close(db_res, db_id, rtol=0, atol=1e-12)
    yb, dxb, dwb, dbb = O.brute_force(x, cu, w1, b, dy)
    torch.testing.assert_close(y_res, yb, rtol=0, atol=1e-12)
    torch.testing.assert_close(dx_res, dxb, rtol=0, atol=1e-12)
    yc = O.c_oracle_fwd(x.float(), cu, w.float(), b.float(), residual=True)
    dxc, dwc, dbc = O.c_oracle_bwd(x.float(), dy.float(), cu, w.float(), residual=True)
    y32, dx32, dw32, db32 = O.ref_dwconv_varlen_grads(x.float(), cu, w.float(), b.float(), dy.float(), torch.float64,
                                                      residual=True)
    torch.testing.assert_close(yc, y32, rtol=0, atol=1e-12)
    torch.testing.assert_close(dxc, dx32, rtol=0, atol=1e-12)
    torch.testing.assert_close(dwc, dw32, rtol=0, atol=1e-12)
    # w = 0, b = 0: the identity
    y0 = O.ref_dwconv_varlen(x, cu, torch.zeros_like(w), None, torch.float64, residual=True)
    assert torch.equal(y0, x)


# ---- gated input (x_proj * silu(gate)) -------------------------------------------------------------------
def test_gated_oracle_against_closed_forms_and_finite_differences():
    """h = x_proj * gate / (1 + exp(-gate)) written out with numpy; gate = 0 silences the input (y = b);
    a large gate passes gate * x_proj through; dz against central differences in float64."""
    import numpy as np
    g = torch.Generator().manual_seed(5)
    lens = torch.tensor([4, 1, 9, 2])
    cu = torch.zeros(len(lens) + 1, dtype=torch.int32)
    cu[1:] = torch.cumsum(lens, 0)
    T, C, K = int(lens.sum()), 3, 5
    z = torch.randn(T, 2 * C, generator=g, dtype=torch.float64)
    w = torch.randn(C, K, generator=g, dtype=torch.float64)
    b = torch.randn(C, generator=g, dtype=torch.float64)
    dy = torch.randn(T, C, generator=g, dtype=torch.float64)
    y, dz, dw, db = O.ref_gated_dwconv_grads(z, cu, w, b, dy)
    zn = z.numpy()
    h = torch.from_numpy(zn[:, :C] * zn[:, C:] / (1.0 + np.exp(-zn[:, C:])))
    yb, dhb, dwb, dbb = O.brute_force(h, cu, w, b, dy)
    torch.testing.assert_close(y, yb, rtol=0, atol=1e-12)
    torch.testing.assert_close(dw, dwb, rtol=0, atol=1e-12)
    torch.testing.assert_close(db, dbb, rtol=0, atol=1e-12)
    # chain rule by hand: d x_proj = dh * silu(g), d gate = dh * x_proj * sig * (1 + g (1 - sig))
    sig = 1.0 / (1.0 + np.exp(-zn[:, C:]))
    dzb = np.concatenate([dhb.numpy() * zn[:, C:] * sig, dhb.numpy() * zn[:, :C] * sig * (1 + zn[:, C:] * (1 - sig))], 1)
    torch.testing.assert_close(dz, torch.from_numpy(dzb), rtol=0, atol=1e-12)
    # central differences on a few entries of z
    eps = 1e-6
    for (t, c) in [(0, 0), (5, 4), (13, 2), (15, 5)]:
        zp, zm = z.clone(), z.clone()
        zp[t, c] += eps
        zm[t, c] -= eps
        fd = ((O.ref_gated_dwconv_grads(zp, cu, w, b, None) - O.ref_gated_dwconv_grads(zm, cu, w, b, None)) * dy).sum() / (2 * eps)
        assert abs(float(fd) - float(dz[t, c])) < 1e-6
    # gate = 0 -> h = 0 -> y = bias;  gate = 40 -> silu(gate) = gate to 1e-16
    z0 = z.clone()
    z0[:, C:] = 0
    assert torch.equal(O.ref_gated_dwconv_grads(z0, cu, w, b, None), b.expand(T, C))
    z1 = z.clone()
    z1[:, C:] = 40.0
    torch.testing.assert_close(O.ref_gated_dwconv_grads(z1, cu, w, b, None), O.ref_dwconv_varlen(40.0 * z[:, :C], cu, w, b, torch.float64),
                               rtol=1e-14, atol=1e-12)


def test_layernorm_conv_oracle_against_the_written_out_formula_and_finite_differences():
    """ref_ln_dwconv_grads (F.layer_norm, then the conv loop, by autograd) against the formula written out -
    n = (x - mean) / sqrt(var + eps) * gamma + beta with the biased variance of a row, fed to the C restatement -
    and its gradients against central differences of that forward."""
    g = torch.Generator().manual_seed(11)
    lens = [1, 2, 5, 0, 9, 3]
    T, C, K, eps = sum(lens), 24, 5, 1e-5
    x = torch.randn(T, C, generator=g, dtype=torch.float64) * 2 + 0.5
    gam = torch.randn(C, generator=g, dtype=torch.float64)
    bet = torch.randn(C, generator=g, dtype=torch.float64)
    w = torch.randn(C, K, generator=g, dtype=torch.float64)
    b = torch.randn(C, generator=g, dtype=torch.float64)
    dy = torch.randn(T, C, generator=g, dtype=torch.float64)
    cu = cu_from_lengths(torch.tensor(lens))
    for residual in (False, True):
        y, dx, dgam, dbet, dw, db = O.ref_ln_dwconv_grads(x, cu, gam, bet, w, b, dy, eps, torch.float64, residual)
        mean = x.mean(1, keepdim=True)
        var = ((x - mean) ** 2).mean(1, keepdim=True)
        n = (x - mean) / torch.sqrt(var + eps) * gam + bet
        y2 = O.brute_force(n, cu, w, b) + (x if residual else 0)
        torch.testing.assert_close(y, y2, rtol=1e-12, atol=1e-12)

        def loss(xx, gg, hh):
            return float((O.ref_ln_dwconv_grads(xx, cu, gg, hh, w, b, None, eps, torch.float64, residual) * dy).sum())
        h = 1e-6
        for (t, c) in ((0, 0), (4, 7), (T - 1, C - 1), (9, 3)):
            e = torch.zeros_like(x); e[t, c] = h
            fd = (loss(x + e, gam, bet) - loss(x - e, gam, bet)) / (2 * h)
            assert abs(fd - float(dx[t, c])) < 1e-6 * max(1.0, abs(fd))
        for c in (0, 5, C - 1):
            e = torch.zeros_like(gam); e[c] = h
            fd = (loss(x, gam + e, bet) - loss(x, gam - e, bet)) / (2 * h)
            assert abs(fd - float(dgam[c])) < 1e-6 * max(1.0, abs(fd))
            fd = (loss(x, gam, bet + e) - loss(x, gam, bet - e)) / (2 * h)
            assert abs(fd - float(dbet[c])) < 1e-6 * max(1.0, abs(fd))
    # without a LayerNorm bias
    y = O.ref_ln_dwconv_grads(x, cu, gam, None, w, b, None, eps)
    torch.testing.assert_close(y, O.brute_force((x - mean) / torch.sqrt(var + eps) * gam, cu, w, b), rtol=1e-12, atol=1e-12)
