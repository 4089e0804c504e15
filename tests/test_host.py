"""Host-side checks that need no GPU: the C-ABI library loads and exports what include/nplm_dwconv.h
declares, argument errors are reported before anything is launched, the workspace arithmetic, the
boundary cursor (run on the host over a host copy of cu_seqlens), the Python surface's validation,
and the workload generators."""
import ctypes
import os
import re

import numpy as np
import pytest
import torch

import nanoplm_amd
from nanoplm_amd import _lib
from nanoplm_amd.dwconv import exec_kernel_size
from nanoplm_amd.workloads import cu_from_lengths, make_workload, static_packed_cu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_library_exports_every_declared_symbol():
    header = open(os.path.join(ROOT, "include", "nplm_dwconv.h")).read()
    declared = set(re.findall(r"\b(nplm_dwconv_[a-z_]+)\s*\(", header))
    assert declared == set(_lib.PUBLIC_SYMBOLS)
    lib = ctypes.CDLL(_lib.LIB_PATH)
    for name in declared:
        assert hasattr(lib, name), name


def test_header_is_plain_c_and_a_c_program_links_and_calls_the_library(tmp_path):
    """include/nplm_dwconv.h compiles as strict C11 (no C++ left in it), every function it declares links from C against
    the shared object, and a C caller gets the version, the error strings, the workspace size and the argument errors
    (reported before anything is launched, so no GPU is needed)."""
    import shutil
    import subprocess
    if shutil.which("gcc") is None:
        pytest.skip("no C compiler")
    header = open(os.path.join(ROOT, "include", "nplm_dwconv.h")).read()
    names = sorted(set(re.findall(r"\b(nplm_dwconv_[a-z_]+)\s*\(", header)))
    src = tmp_path / "abi.c"
    src.write_text(
        "#include <stdio.h>\n#include <string.h>\n#include \"nplm_dwconv.h\"\n"
        "typedef void (*fn)(void);\n"
        "int main(void) {\n"
        "    fn all[] = {" + ", ".join(f"(fn){n}" for n in names) + "};\n"
        "    char fake[64];\n"
        "    void* a = (void*)(((size_t)fake + 15) & ~(size_t)15);   /* aligned, never dereferenced */\n"
        "    if (sizeof(all) / sizeof(all[0]) != " + str(len(names)) + ") return 10;\n"
        "    if (nplm_dwconv_version() < 100) return 11;\n"
        "    if (strcmp(nplm_dwconv_strerror(0), \"success\") != 0) return 12;\n"
        "    if (!strstr(nplm_dwconv_strerror(-NPLM_DWCONV_EKSIZE), \"odd\")) return 13;\n"
        "    if (nplm_dwconv_fwd(NULL, a, a, a, a, 128, 64, 3, 1, NPLM_DWCONV_BF16, NPLM_DWCONV_BF16, NULL) != -NPLM_DWCONV_ENULL) return 14;\n"
        "    if (nplm_dwconv_fwd(a, a, a, a, a, 128, 64, 4, 1, NPLM_DWCONV_BF16, NPLM_DWCONV_BF16, NULL) != -NPLM_DWCONV_EKSIZE) return 15;\n"
        "    if (nplm_dwconv_bwd(a, a, a, a, a, a, a, NULL, 0, 128, 64, 3, 1, NPLM_DWCONV_F32, NPLM_DWCONV_F32, NULL) != -NPLM_DWCONV_EWORKSPACE) return 16;\n"
        "    if (nplm_dwconv_fwd(NULL, NULL, NULL, NULL, NULL, 0, 64, 3, 0, NPLM_DWCONV_F32, NPLM_DWCONV_F32, NULL) != 0) return 17;   /* empty batch */\n"
        "    printf(\"%zu %zu\\n\", nplm_dwconv_bwd_workspace_bytes(131072, 1024, 7, NPLM_DWCONV_BF16), nplm_dwconv_bwd_workspace_bytes(131072, 1024, 11, NPLM_DWCONV_BF16));\n"
        "    return 0;\n}\n")
    exe = tmp_path / "abi"
    libdir = os.path.dirname(_lib.LIB_PATH)
    cc = subprocess.run(["gcc", "-std=c11", "-Wall", "-Wextra", "-Werror", "-pedantic", "-I", os.path.join(ROOT, "include"),
                         str(src), "-o", str(exe), "-L", libdir, "-l:" + os.path.basename(_lib.LIB_PATH), "-Wl,-rpath," + libdir,
                         "-Wl,-rpath-link,/opt/rocm/lib"], capture_output=True, text=True)
    assert cc.returncode == 0, cc.stderr
    run = subprocess.run([str(exe)], capture_output=True, text=True, timeout=120)
    assert run.returncode == 0, (run.returncode, run.stderr)
    lib = _lib.load()
    want = f"{lib.nplm_dwconv_bwd_workspace_bytes(131072, 1024, 7, 1)} {lib.nplm_dwconv_bwd_workspace_bytes(131072, 1024, 11, 1)}"
    assert run.stdout.strip() == want


def test_version_and_strerror():
    lib = _lib.load()
    assert lib.nplm_dwconv_version() >= 100
    assert _lib.strerror(0) == "success"
    for code in range(-8, 0):
        assert "nplm_dwconv" in _lib.strerror(code)


A = 0x10000   # a fake, well-aligned, never dereferenced device address


def _fwd(x=A, cu=A, w=A, b=A, y=A, T=128, C=64, K=3, S=1, act=1, wd=1):
    return _lib.load().nplm_dwconv_fwd(x, cu, w, b, y, T, C, K, S, act, wd, None)


def _bwd(x=A, dy=A, cu=A, w=A, dx=A, dw=A, db=A, ws=A, wsb=0, T=128, C=64, K=3, S=1, act=1, wd=1):
    return _lib.load().nplm_dwconv_bwd(x, dy, cu, w, dx, dw, db, ws, wsb, T, C, K, S, act, wd, None)


def test_argument_errors_are_reported_before_any_launch():
    assert _fwd(x=None) == -1 and _fwd(y=None) == -1 and _fwd(cu=None) == -1 and _fwd(w=None) == -1
    assert _fwd(T=-1) == -2 and _fwd(C=0) == -2 and _fwd(S=-1) == -2 and _fwd(T=2 ** 31) == -2
    assert _fwd(K=4) == -3 and _fwd(K=0) == -3 and _fwd(K=257) == -3
    assert _fwd(act=2) == -4 and _fwd(wd=7) == -4
    assert _fwd(x=A + 1) == -5 and _fwd(act=0, y=A + 2) == -5 and _fwd(wd=0, w=A + 2) == -5
    assert _fwd(T=0, x=None, y=None) == 0            # empty batch: nothing to do
    assert _bwd(dy=None) == -1 and _bwd(x=None) == -1 and _bwd(w=None) == -1
    assert _bwd(K=2) == -3 and _bwd(act=5) == -4 and _bwd(dx=A + 1) == -5
    assert _bwd(ws=None) == -6 and _bwd(ws=A + 64, wsb=1 << 30) == -6 and _bwd(wsb=16) == -6
    assert _bwd(dx=None, dw=None, db=None) == 0      # nothing requested


def test_workspace_bytes_arithmetic():
    lib = _lib.load()
    for (T, C, K, act) in [(131072, 1024, 7, 1), (131072, 2048, 31, 1), (65536, 1024, 7, 1), (776, 64, 3, 0),
                           (1, 8, 1, 1), (1000, 1000, 11, 0)]:
        n = lib.nplm_dwconv_bwd_workspace_bytes(T, C, K, act)
        slabs = lib.nplm_dwconv_bwd_slabs(T, C, K, act, None)
        assert slabs >= 1
        # enough for the library's default kernel and for the sliding-window kernel that a request for dx alone or
        # dw/db alone may take instead (K = 31), and no more than the larger of the two
        most = max(slabs, lib.nplm_dwconv_bwd_slabs(T, C, K, act, _lib.Tuning(algo=1)))
        Kx = exec_kernel_size(K)        # K = 1 runs as 3 taps and K = 11 as 15, with slabs of that many rows
        assert Kx == {7: 7, 31: 31, 3: 3, 1: 3, 11: 15}[K]
        assert n % 256 == 0 and n >= most * (Kx + 1) * C * 4 > n - 256
        assert n <= (16 << 20) + (Kx + 1) * C * 4       # partials are capped (one slab minimum)
    assert lib.nplm_dwconv_bwd_workspace_bytes(0, 64, 3, 1) == 0
    assert lib.nplm_dwconv_bwd_workspace_bytes(100, 64, 4, 1) == 0


def test_column_block_width_follows_the_row_width():
    """The LDS-staged backward deals one token block per CU and column block, so its slab count (256 / column
    blocks per row) shows which column-block width the planner picked: 1 KiB by default, 768 bytes for rows that
    are a multiple of that (C = 768, 1152 in bf16; 576 in fp32), 1280 bytes for rows of 1280 and 2560 bytes."""
    lib = _lib.load()
    lds = _lib.Tuning(algo=2)
    for (C, act, slabs) in [(1024, 1, 128), (2048, 1, 64), (512, 1, 256), (896, 1, 128), (768, 1, 128),
                            (1152, 1, 85), (640, 1, 256), (1280, 1, 128), (576, 0, 85), (512, 0, 128)]:
        assert lib.nplm_dwconv_bwd_slabs(131072, C, 7, act, lds) == slabs, (C, act)


# ---- boundary cursor ---------------------------------------------------------------------------
def _intervals(cu, T, start=0, step=1, relocate_every=0):
    cu = np.ascontiguousarray(np.asarray(cu, dtype=np.int32))
    n = max(0, (T - start + step - 1) // step)
    cs = np.full(n, -7, dtype=np.int32)
    ce = np.full(n, -7, dtype=np.int32)
    got = _lib.load().nplm_dwconv_debug_intervals(cu.ctypes.data, len(cu) - 1, T, start, step, relocate_every,
                                                  cs.ctypes.data, ce.ctypes.data)
    assert got == n
    return cs, ce


def _expected_intervals(cu, T):
    cs = np.empty(T, dtype=np.int32)
    ce = np.empty(T, dtype=np.int32)
    for s, e in zip(cu[:-1], cu[1:]):
        cs[s:e] = s
        ce[s:e] = e
    return cs, ce


def test_cursor_reproduces_the_reference_position_id_example():
    # src/nanoplm/pretraining/models/modern_bert/modeling.py:204: cu=[0,3,5,9] -> pos=[0,1,2,0,1,0,1,2,3]
    cs, ce = _intervals([0, 3, 5, 9], 9)
    assert (np.arange(9) - cs).tolist() == [0, 1, 2, 0, 1, 0, 1, 2, 3]
    assert ce.tolist() == [3, 3, 3, 5, 5, 9, 9, 9, 9]


@pytest.mark.parametrize("relocate_every", [0, 1, 5, 64])
@pytest.mark.parametrize("step", [1, 3, 8])
def test_cursor_on_random_cu_with_empty_sequences(step, relocate_every):
    rng = np.random.default_rng(1)
    for _ in range(20):
        lens = rng.integers(0, 12, size=rng.integers(1, 40))
        lens[rng.random(len(lens)) < 0.3] = 0
        if lens.sum() == 0:
            lens[0] = 3
        cu = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
        T = int(cu[-1])
        want_cs, want_ce = _expected_intervals(cu, T)
        for start in (0, 1, T // 2):
            cs, ce = _intervals(cu, T, start, step, relocate_every)
            assert np.array_equal(cs, want_cs[start::step]) and np.array_equal(ce, want_ce[start::step])


def test_cursor_on_static_packed_cu():
    """Fixed-length cu_seqlens of the static-shape collator (collator.py:430-450): pad pseudo-sequences
    after the real ones and trailing zero-length entries equal to F."""
    real = cu_from_lengths(torch.tensor([30, 17, 64, 5]))
    F, W = 256, 64
    cu = static_packed_cu(real, F, W, cu_len=12).numpy()
    assert cu.tolist() == [0, 30, 47, 111, 116, 180, 244, 256, 256, 256, 256, 256]
    want_cs, want_ce = _expected_intervals(cu, F)
    for relocate_every in (0, 16):
        cs, ce = _intervals(cu, F, 0, 1, relocate_every)
        assert np.array_equal(cs, want_cs) and np.array_equal(ce, want_ce)


def test_cursor_never_leaves_the_array_on_malformed_cu():
    # rows before cu[0] and after cu[S] form pseudo-sequences; decreasing entries cannot loop forever
    cs, ce = _intervals([4, 6, 9], 12)
    assert cs.tolist() == [0] * 4 + [4, 4] + [6, 6, 6] + [9] * 3
    assert ce.tolist() == [4] * 4 + [6, 6] + [9, 9, 9] + [12] * 3
    cs, ce = _intervals([0], 5)              # S = 0: one pseudo-sequence [0, T)
    assert cs.tolist() == [0] * 5 and ce.tolist() == [5] * 5
    _intervals([0, 9, 3, 7, 2, 12], 12)      # decreasing: only termination is asserted
    _intervals([0, 50, 100], 12)             # entries beyond T


# ---- Python surface -----------------------------------------------------------------------------
def test_cpu_tensors_are_refused():
    x = torch.randn(10, 8)
    cu = torch.tensor([0, 10], dtype=torch.int32)
    w = torch.randn(8, 3)
    with pytest.raises(RuntimeError, match="no CPU implementation"):
        nanoplm_amd.varlen_dwconv_fwd(x, cu, w)
    with pytest.raises(RuntimeError, match="no CPU implementation"):
        nanoplm_amd.VarlenDWConv1d(8, 3)(x, cu)
    with pytest.raises(RuntimeError, match="no CPU implementation"):
        nanoplm_amd.VarlenDWConv1dFunction.apply(x, cu, w, None)


def test_python_validation():
    cu = torch.tensor([0, 10], dtype=torch.int32)
    w = torch.randn(8, 3)
    from nanoplm_amd.dwconv import _validate
    with pytest.raises(ValueError):
        _validate(torch.randn(10), cu, w, None)
    with pytest.raises(TypeError):
        _validate(torch.randn(10, 8).half(), cu, w, None)
    with pytest.raises(ValueError):
        nanoplm_amd.VarlenDWConv1d(8, 4)
    m = nanoplm_amd.VarlenDWConv1d(16, 7)
    assert m.weight.shape == (16, 7) and m.bias.shape == (16,)
    assert nanoplm_amd.VarlenDWConv1d(16, 7, bias=False).bias is None


def test_missing_library_fails_loudly(monkeypatch):
    monkeypatch.setattr(_lib, "_lib", None)
    monkeypatch.setattr(_lib, "LIB_PATH", "/nonexistent/libnplm_dwconv.so")
    with pytest.raises(RuntimeError, match="is missing"):
        _lib.load()


def test_product_does_not_import_the_oracle():
    pkg = os.path.join(ROOT, "nanoplm_amd")
    for dirpath, _, files in os.walk(pkg):
        for f in files:
            if f.endswith((".py", ".h", ".hip", ".inc")):
                text = open(os.path.join(dirpath, f)).read()
                assert "oracle" not in text.lower() or f == "workloads.py", f


# ---- workloads ----------------------------------------------------------------------------------
def test_workload_generators_follow_the_config_definitions():
    w1 = make_workload(1)
    assert w1.S == 8 and w1.C == 64 and w1.K == 3 and w1.dtype == torch.float32 and w1.dy is None
    assert 20 <= int(w1.lengths.min()) and int(w1.lengths.max()) <= 128
    w2 = make_workload(2, C=16)
    assert w2.T == 32768 and w2.K == 7 and w2.dtype == torch.bfloat16 and w2.passes == "fwd"
    assert int(w2.lengths[:-1].min()) >= 20 and int(w2.lengths.max()) <= 512
    w5 = make_workload(5, C=8)
    assert w5.T == 65536 and w5.passes == "fwd+bwd" and w5.dy is not None
    ln = w5.lengths[:-1]
    short = ln <= 8
    assert bool(((ln >= 1) & (ln <= 8) | (ln >= 400) & (ln <= 512)).all())
    assert 0.5 < float(short.float().mean()) < 0.7
    w4 = make_workload(4, T=20000, C=8)
    assert w4.K == 31 and 20 <= int(w4.lengths[:-1].min()) and int(w4.lengths.max()) <= 1024
    for w in (w1, w2, w5, w4):
        cu = w.cu_seqlens
        assert cu.dtype == torch.int32 and int(cu[0]) == 0 and int(cu[-1]) == w.T and cu.numel() == w.S + 1
        assert bool((cu[1:] >= cu[:-1]).all())
    again = make_workload(2, C=16)
    assert torch.equal(again.x, w2.x) and torch.equal(again.cu_seqlens, w2.cu_seqlens)


def test_algorithmic_bytes_of_the_headline_config():
    w3 = make_workload(3, C=8)   # C shrunk for speed; the formula is checked at the real C by hand
    T, C, K, S, e = w3.T, w3.C, w3.K, w3.S, 2
    assert w3.algorithmic_bytes("fwd") == 2 * T * C * e + C * (K + 1) * e + 4 * (S + 1)
    assert w3.algorithmic_bytes("bwd") == 3 * T * C * e + C * K * e + 4 * C * (K + 1) + 4 * (S + 1)
    # at C=1024: 5*T*C*e = 1 342 177 280
    assert 5 * 131072 * 1024 * 2 == 1342177280


# ---- torch.library registration (traceability; no kernel is run) ------------------------------------
def test_custom_ops_trace_with_fake_tensors():
    """Schemas and fake (shape/dtype) implementations of the registered ops, without a GPU. The autograd
    formula needs a device context and is exercised by the GPU tests."""
    from torch._subclasses.fake_tensor import FakeTensorMode
    from torch.fx.experimental.proxy_tensor import make_fx

    assert str(torch.ops.nanoplm_amd.varlen_dwconv_fwd.default._schema) == (
        "nanoplm_amd::varlen_dwconv_fwd(Tensor x, Tensor cu_seqlens, Tensor weight, Tensor? bias, bool residual=False) -> Tensor")
    assert str(torch.ops.nanoplm_amd.varlen_dwconv_bwd.default._schema) == (
        "nanoplm_amd::varlen_dwconv_bwd(Tensor x, Tensor dy, Tensor cu_seqlens, Tensor weight, bool residual=False, bool grads_bf16=False) -> "
        "(Tensor, Tensor, Tensor)")
    with FakeTensorMode():
        x = torch.empty(100, 64, dtype=torch.bfloat16, device="cuda")
        cu = torch.empty(5, dtype=torch.int32, device="cuda")
        w = torch.empty(64, 7, dtype=torch.float32, device="cuda")
        b = torch.empty(64, dtype=torch.float32, device="cuda")
        y = nanoplm_amd.varlen_dwconv_compilable(x, cu, w, b)
        assert y.shape == x.shape and y.dtype == torch.bfloat16 and y.device.type == "cuda"
        dx, dw, db = nanoplm_amd.varlen_dwconv_bwd_op(x, y, cu, w)
        assert dx.shape == x.shape and dx.dtype == torch.bfloat16
        assert dw.shape == (64, 7) and dw.dtype == torch.float32 and db.shape == (64,) and db.dtype == torch.float32

    def f(x, cu, w):
        y = nanoplm_amd.varlen_dwconv_compilable(x, cu, w, None)
        return nanoplm_amd.varlen_dwconv_bwd_op(x, y, cu, w)

    with FakeTensorMode(allow_non_fake_inputs=True):
        args = (torch.empty(32, 16, device="cuda"), torch.empty(3, dtype=torch.int32, device="cuda"),
                torch.empty(16, 3, device="cuda"))
        gm = make_fx(f, tracing_mode="fake")(*args)
    targets = {str(n.target) for n in gm.graph.nodes if n.op == "call_function"}
    assert "nanoplm_amd.varlen_dwconv_fwd.default" in targets and "nanoplm_amd.varlen_dwconv_bwd.default" in targets
