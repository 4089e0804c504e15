"""nplm_dwconv_bwd_static: the backward entry point that allocates nothing (its dw/db partial sums live in
a static device array of the library) against nplm_dwconv_bwd_ex with a caller-owned workspace.

Both run the same kernels on the same launch geometry, so every output must be bit-identical. Calls are
made through the C ABI (ctypes), two in a row on the same GPU with the second one smaller, so that
whatever the first call left in the shared array is there when the second one runs.
"""
import ctypes

import pytest
import torch

from nanoplm_amd import _lib
from nanoplm_amd.workloads import cu_from_lengths, make_workload

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


_hip = None


def _device_free_bytes():
    """Free device memory as the HIP runtime counts it (hipMemGetInfo through ctypes)."""
    global _hip
    if _hip is None:
        _hip = ctypes.CDLL("libamdhip64.so")
        _hip.hipMemGetInfo.argtypes = [ctypes.POINTER(ctypes.c_size_t), ctypes.POINTER(ctypes.c_size_t)]
    free, total = ctypes.c_size_t(), ctypes.c_size_t()
    rc = _hip.hipMemGetInfo(ctypes.byref(free), ctypes.byref(total))
    assert rc == 0, f"hipMemGetInfo failed: {rc}"
    return free.value


def _inputs(lens, C, K, dt, seed):
    g = torch.Generator().manual_seed(seed)
    lens = torch.tensor(lens)
    T = int(lens.sum())
    x = torch.randn(T, C, generator=g).to(dt).to(DEV)
    dy = torch.randn(T, C, generator=g).to(dt).to(DEV)
    w = (torch.randn(C, K, generator=g) * K ** -0.5).to(dt).to(DEV)
    return x, dy, cu_from_lengths(lens).to(DEV), w


def _bwd_pair(x, dy, cu, w, flags=0, want_dx=True, want_red=True):
    """(outputs of nplm_dwconv_bwd_ex, outputs of nplm_dwconv_bwd_static) for the same inputs."""
    lib = _lib.load()
    T, C = x.shape
    K = w.shape[1]
    S = cu.numel() - 1
    act = _lib.BF16 if x.dtype == torch.bfloat16 else _lib.F32
    wdt = _lib.BF16 if w.dtype == torch.bfloat16 else _lib.F32
    stream = torch.cuda.current_stream().cuda_stream

    def outs():
        dx = torch.full_like(x, float("nan")) if want_dx else None
        dw = torch.full((C, K), float("nan"), dtype=torch.float32, device=DEV) if want_red else None
        db = torch.full((C,), float("nan"), dtype=torch.float32, device=DEV) if want_red else None
        return dx, dw, db

    def p(t):
        return None if t is None else t.data_ptr()

    ref = outs()
    nbytes = int(lib.nplm_dwconv_bwd_workspace_bytes(T, C, K, act))
    ws = torch.empty((max(nbytes, 256),), dtype=torch.uint8, device=DEV)
    _lib.check(lib.nplm_dwconv_bwd_ex(p(x), p(dy), p(cu), p(w), p(ref[0]), p(ref[1]), p(ref[2]), p(ws), ws.numel(),
                                      T, C, K, S, act, wdt, flags, stream), "nplm_dwconv_bwd_ex")
    def static(o):
        _lib.check(lib.nplm_dwconv_bwd_static(p(x), p(dy), p(cu), p(w), p(o[0]), p(o[1]), p(o[2]),
                                              T, C, K, S, act, wdt, flags, stream), "nplm_dwconv_bwd_static")

    # first call on this shape: may look up the scratch address and raise a kernel's LDS limit (no allocation either,
    # but the runtime may load a code object); the call that is bracketed below is a warm one
    static(outs())
    got = outs()
    torch.cuda.synchronize()
    before = torch.cuda.memory_allocated()
    free_before = _device_free_bytes()
    static(got)
    # the device's own count of free memory (hipMemGetInfo) sees a hipMalloc/hipFree inside the library, which torch's
    # caching allocator cannot; read it again while the call's kernels may still be running and after they have ended
    assert _device_free_bytes() == free_before, "nplm_dwconv_bwd_static changed the device's free memory"
    assert torch.cuda.memory_allocated() == before
    torch.cuda.synchronize()
    assert _device_free_bytes() == free_before, "nplm_dwconv_bwd_static changed the device's free memory"
    return ref, got


def _assert_same(ref, got, what):
    for name, a, b in zip(("dx", "dw", "db"), ref, got):
        if a is None:
            assert b is None
            continue
        assert torch.isfinite(b.float()).all(), f"{what}: {name} holds values the call did not write"
        assert torch.equal(a, b), f"{what}: {name} differs from nplm_dwconv_bwd_ex"


def test_headline_shape_then_a_smaller_call():
    """Two calls in a row through the static entry point: configuration 3 at full size, then a short ragged batch."""
    print("[case] static backward: cfg3 full size", flush=True)
    d = make_workload(3, with_dy=True).to(DEV)
    _assert_same(*_bwd_pair(d.x, d.dy, d.cu_seqlens, d.weight), "cfg3")
    print("[case] static backward: 700 rows after it", flush=True)
    small = _inputs([5, 1, 300, 2, 90, 3, 299], 1024, 7, torch.bfloat16, 1)
    _assert_same(*_bwd_pair(*small), "small after cfg3")
    # and the large one again, now after the small one
    _assert_same(*_bwd_pair(d.x, d.dy, d.cu_seqlens, d.weight), "cfg3 again")


@pytest.mark.parametrize("C,K,dt", [(2048, 31, torch.bfloat16), (256, 7, torch.float32), (1152, 5, torch.bfloat16),
                                     (100, 11, torch.bfloat16), (768, 15, torch.float32)])
def test_every_kernel_family_shares_the_scratch(C, K, dt):
    """LDS-staged, sliding-window and runtime-K backward kernels, each followed by a smaller call."""
    print(f"[case] static backward C={C} K={K} {dt}", flush=True)
    big = _inputs([400, 1, 37, 512, 64, 63, 2, 900, 20, 333], C, K, dt, C + K)
    _assert_same(*_bwd_pair(*big), f"C={C} K={K}")
    small = _inputs([7, 1, 40], C, K, dt, C + K + 1)
    _assert_same(*_bwd_pair(*small), f"C={C} K={K} small")


def test_flags_and_partial_outputs():
    x, dy, cu, w = _inputs([33, 200, 1, 90], 1024, 7, torch.bfloat16, 5)
    _assert_same(*_bwd_pair(x, dy, cu, w, flags=_lib.RESIDUAL), "residual")
    _assert_same(*_bwd_pair(x, dy, cu, w, want_dx=False), "dw/db only")
    _assert_same(*_bwd_pair(x, dy, cu, w, want_red=False), "dx only")


def test_shapes_beyond_the_scratch_are_refused():
    """C*(K+1) fp32 partial sums above 16 MiB: a clear error and nothing launched; the workspace entry point takes it."""
    lib = _lib.load()
    C, K, T = 140000, 31, 4
    assert (K + 1) * C * 4 > _lib.STATIC_SCRATCH_BYTES
    x, dy, cu, w = _inputs([T], C, K, torch.bfloat16, 3)
    dx = torch.zeros_like(x)
    dw = torch.zeros((C, K), dtype=torch.float32, device=DEV)
    db = torch.zeros((C,), dtype=torch.float32, device=DEV)
    stream = torch.cuda.current_stream().cuda_stream
    rc = lib.nplm_dwconv_bwd_static(x.data_ptr(), dy.data_ptr(), cu.data_ptr(), w.data_ptr(), dx.data_ptr(),
                                    dw.data_ptr(), db.data_ptr(), T, C, K, 1, _lib.BF16, _lib.BF16, 0, stream)
    assert rc == -_lib.ESCRATCH
    assert "scratch" in _lib.strerror(rc)
    torch.cuda.synchronize()
    assert float(dx.abs().max()) == 0.0 and float(dw.abs().max()) == 0.0     # nothing ran
    # dx alone needs no partial sums, so it is served
    rc = lib.nplm_dwconv_bwd_static(x.data_ptr(), dy.data_ptr(), cu.data_ptr(), w.data_ptr(), dx.data_ptr(),
                                    None, None, T, C, K, 1, _lib.BF16, _lib.BF16, 0, stream)
    assert rc == 0
    ref, _ = _bwd_pair(x, dy, cu, w, want_red=False)
    assert torch.equal(ref[0], dx)


def test_empty_batch_zero_fills():
    lib = _lib.load()
    C, K = 64, 7
    dw = torch.full((C, K), 3.0, dtype=torch.float32, device=DEV)
    db = torch.full((C,), 3.0, dtype=torch.float32, device=DEV)
    rc = lib.nplm_dwconv_bwd_static(None, None, None, None, None, dw.data_ptr(), db.data_ptr(), 0, C, K, 0,
                                    _lib.BF16, _lib.BF16, 0, torch.cuda.current_stream().cuda_stream)
    assert rc == 0
    torch.cuda.synchronize()
    assert float(dw.abs().max()) == 0.0 and float(db.abs().max()) == 0.0


def test_static_backward_is_captured_and_replayed_by_a_hip_graph():
    """The callers the entry point is for: a HIP graph capture, under which an allocation inside the call would fail
    the capture. Captured once (after a warm call outside the capture), replayed with new contents in the static input
    buffers, with eager work and synchronisation between the replays; every replay equals nplm_dwconv_bwd_ex."""
    lib = _lib.load()
    x, dy, cu, w = _inputs([100, 3, 512, 1, 408, 2, 2, 77], 1024, 7, torch.bfloat16, 11)
    T, C = x.shape
    K, S = w.shape[1], cu.numel() - 1
    dx = torch.empty_like(x)
    dw = torch.empty((C, K), dtype=torch.float32, device=DEV)
    db = torch.empty((C,), dtype=torch.float32, device=DEV)

    def call():
        _lib.check(lib.nplm_dwconv_bwd_static(x.data_ptr(), dy.data_ptr(), cu.data_ptr(), w.data_ptr(), dx.data_ptr(),
                                              dw.data_ptr(), db.data_ptr(), T, C, K, S, _lib.BF16, _lib.BF16, 0,
                                              torch.cuda.current_stream().cuda_stream), "nplm_dwconv_bwd_static")

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        call()                                         # warm-up outside the capture
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        call()
    for it in range(3):
        nx, ndy, _, _ = _inputs([100, 3, 512, 1, 408, 2, 2, 77], 1024, 7, torch.bfloat16, 20 + it)
        x.copy_(nx)
        dy.copy_(ndy)
        dx.fill_(float("nan"))
        dw.fill_(float("nan"))
        db.fill_(float("nan"))
        graph.replay()
        torch.cuda.synchronize()
        ref, _ = _bwd_pair(nx, ndy, cu, w)
        assert torch.equal(dx, ref[0]) and torch.equal(dw, ref[1]) and torch.equal(db, ref[2]), f"replay {it}"
