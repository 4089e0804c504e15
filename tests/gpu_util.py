"""Shared helpers of the GPU parity tests: tolerances of the specification and oracle caching."""
import functools

import torch

from nanoplm_amd.workloads import make_workload
from oracle import dwconv_ref as O

# bf16 activations: max-abs <= 2e-2 against the fp32/fp64 oracle (fp32 accumulation, one rounding).
BF16_ATOL = 2e-2
# fp32: <= 1e-5 relative.
F32_RTOL = 1e-5
# dw/db: the kernels' fp32 outputs against the double-accumulated oracle, max-abs <= 2e-2.
DWDB_ATOL = 2e-2


def assert_act_close(got, ref64, dtype, what):
    """y / dx against the float64 oracle, to the tolerance stated for ``dtype``."""
    got = got.detach().cpu().double()
    err = (got - ref64).abs()
    assert torch.isfinite(got).all(), f"{what}: non-finite values"
    if dtype == torch.bfloat16:
        # 2e-2 max-abs is below bf16's half-ulp (3.1e-2) once |v| >= 8; there one rounding is the bar
        small = ref64.abs() < 8.0
        worst = float(err[small].max()) if small.any() else 0.0
        assert worst <= BF16_ATOL, f"{what}: max-abs error {worst:.3e} > {BF16_ATOL}"
        if (~small).any():
            rel = float((err[~small] / ref64[~small].abs()).max())
            assert rel <= 2.0 ** -8, f"{what}: relative error {rel:.3e} above one bf16 rounding"
        # and never more than one bf16 rounding of the exact value (+ fp32 accumulation noise)
        bound = ref64.abs() * 2.0 ** -8 + 1e-5
        assert bool((err <= bound).all()), f"{what}: more than one bf16 rounding away from the oracle"
    else:
        scale = float(ref64.abs().max())
        rel = float(err.max()) / max(scale, 1e-30)
        assert rel <= F32_RTOL, f"{what}: max error / max|ref| = {rel:.3e} > {F32_RTOL}"
        big = ref64.abs() > 1e-2      # below that, cancellation among K terms of size ~1 dominates
        if big.any():
            relel = float((err[big] / ref64[big].abs()).max())
            assert relel <= 2e-4, f"{what}: element-wise relative error {relel:.3e}"
    return float(err.max())


def assert_red_close(got, ref64, what, atol=DWDB_ATOL):
    """dw / db (fp32 from the kernels) against the double-accumulated oracle."""
    assert got.dtype == torch.float32, f"{what} must be produced in fp32"
    got = got.detach().cpu().double()
    assert torch.isfinite(got).all(), f"{what}: non-finite values"
    err = float((got - ref64).abs().max())
    assert err <= atol, f"{what}: max-abs error {err:.3e} > {atol}"
    rel = err / max(float(ref64.abs().max()), 1e-30)
    assert rel <= 1e-5, f"{what}: max error / max|ref| = {rel:.3e}"
    return err


def error_stats(got, ref64, dtype=None):
    """What the parity tables report for one tensor: max-abs and max-rel error (rel over |ref| > 1e-3), and for
    bf16 how many elements have |ref| >= 8 (where one bf16 rounding exceeds 2e-2) with their max-abs error."""
    got = got.detach().cpu().double()
    err = (got - ref64).abs()
    big = ref64.abs() > 1e-3
    out = {"max_abs": float(err.max()), "max_rel": float((err[big] / ref64[big].abs()).max()) if big.any() else 0.0,
           "max_ref": float(ref64.abs().max())}
    if dtype == torch.bfloat16:
        large = ref64.abs() >= 8.0
        out["n_ref_ge_8"] = int(large.sum())
        out["max_abs_ref_ge_8"] = float(err[large].max()) if large.any() else 0.0
        out["max_abs_ref_lt_8"] = float(err[~large].max()) if (~large).any() else 0.0
    return out


def record_parity(name, stats):
    """Keep the parity magnitudes of a run as parity_<name>.json in the run's output folder (best effort: the figures are
    also printed)."""
    import json
    import os
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    try:
        os.makedirs(os.path.join(root, "gpurun_out"), exist_ok=True)
        with open(os.path.join(root, "gpurun_out", f"parity_{name}.json"), "w") as f:
            json.dump(stats, f, indent=1)
    except OSError:
        pass


@functools.lru_cache(maxsize=2)
def workload_with_oracle(index, T=None, C=None):
    """(workload on CPU, y64, dx64, dw64, db64) with the C oracle; dy is always generated."""
    wl = make_workload(index, T=T, C=C, with_dy=True)
    y = O.c_oracle_fwd(wl.x, wl.cu_seqlens, wl.weight, wl.bias)
    dx, dw, db = O.c_oracle_bwd(wl.x, wl.dy, wl.cu_seqlens, wl.weight)
    return wl, y, dx, dw, db
