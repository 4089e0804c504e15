"""GPU tests of the autograd Function / nn.Module surface against the reference path on the CPU."""
import pytest
import torch

import nanoplm_amd as npa
from nanoplm_amd.workloads import make_workload
from oracle import dwconv_ref as O

from gpu_util import assert_act_close, assert_red_close

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def test_function_backward_matches_reference_autograd_fp32():
    wl = make_workload(1, with_dy=True)
    y_r, dx_r, dw_r, db_r = O.ref_dwconv_varlen_grads(wl.x, wl.cu_seqlens, wl.weight, wl.bias, wl.dy, torch.float64)
    x = wl.x.to(DEV).requires_grad_(True)
    w = wl.weight.to(DEV).requires_grad_(True)
    b = wl.bias.to(DEV).requires_grad_(True)
    y = npa.VarlenDWConv1dFunction.apply(x, wl.cu_seqlens.to(DEV), w, b)
    y.backward(wl.dy.to(DEV))
    assert_act_close(y, y_r, torch.float32, "y")
    assert_act_close(x.grad, dx_r, torch.float32, "dx")
    assert_red_close(w.grad, dw_r, "dw")
    assert_red_close(b.grad, db_r, "db")


def test_module_under_autocast_with_fp32_parameters():
    """bf16 activations with fp32 master parameters, as under torch.autocast in the training loop
    (src/nanoplm/pretraining/pure_pipeline.py:717-722); gradients come back in the parameters' dtype."""
    wl = make_workload(5, T=5000, C=512)
    conv = npa.VarlenDWConv1d(512, 7).to(DEV)
    with torch.no_grad():
        conv.weight.copy_(wl.weight.float())
        conv.bias.copy_(wl.bias.float())
    x = wl.x.to(DEV).requires_grad_(True)
    with torch.autocast("cuda", dtype=torch.bfloat16):
        y = conv(x, wl.cu_seqlens.to(DEV))
    assert y.dtype == torch.bfloat16
    y.backward(wl.dy.to(DEV))
    assert conv.weight.grad.dtype == torch.float32 and x.grad.dtype == torch.bfloat16
    y_r, dx_r, dw_r, db_r = O.ref_dwconv_varlen_grads(wl.x, wl.cu_seqlens, wl.weight, wl.bias, wl.dy, torch.float64)
    assert_act_close(y, y_r, torch.bfloat16, "y")
    assert_act_close(x.grad, dx_r, torch.bfloat16, "dx")
    assert_red_close(conv.weight.grad, dw_r, "dw")
    assert_red_close(conv.bias.grad, db_r, "db")


def test_bf16_parameters_get_bf16_gradients_and_frozen_inputs_get_none():
    wl = make_workload(5, T=3000, C=256)
    x = wl.x.to(DEV)                                   # no grad wanted for x
    w = wl.weight.to(DEV).requires_grad_(True)
    b = wl.bias.to(DEV).requires_grad_(True)
    y = npa.varlen_dwconv(x, wl.cu_seqlens.to(DEV), w, b)
    y.backward(wl.dy.to(DEV))
    assert w.grad.dtype == torch.bfloat16 and b.grad.dtype == torch.bfloat16
    _, _, dw_r, db_r = O.ref_dwconv_varlen_grads(wl.x, wl.cu_seqlens, wl.weight, wl.bias, wl.dy, torch.float64)
    # one bf16 rounding of the fp32 result
    assert bool(((w.grad.double().cpu() - dw_r).abs() <= dw_r.abs() * 2.0 ** -8 + 1e-3).all())
    assert bool(((b.grad.double().cpu() - db_r).abs() <= db_r.abs() * 2.0 ** -8 + 1e-3).all())
    # only dx requested
    x2 = wl.x.to(DEV).requires_grad_(True)
    y2 = npa.varlen_dwconv(x2, wl.cu_seqlens.to(DEV), w.detach(), b.detach())
    y2.backward(wl.dy.to(DEV))
    assert x2.grad is not None


def test_non_contiguous_inputs_are_accepted():
    wl = make_workload(5, T=2000, C=256)
    xt = wl.x.to(DEV).t().contiguous().t()             # [T, C] view with transposed strides
    assert not xt.is_contiguous()
    y = npa.varlen_dwconv_fwd(xt, wl.cu_seqlens.to(DEV), wl.weight.to(DEV), wl.bias.to(DEV))
    y0 = npa.varlen_dwconv_fwd(wl.x.to(DEV), wl.cu_seqlens.to(DEV), wl.weight.to(DEV), wl.bias.to(DEV))
    assert torch.equal(y, y0)


def test_runs_on_a_side_stream():
    wl = make_workload(5, T=4000, C=256).to(DEV)
    y0 = npa.varlen_dwconv_fwd(wl.x, wl.cu_seqlens, wl.weight, wl.bias)
    s = torch.cuda.Stream()
    s.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(s):
        y1 = npa.varlen_dwconv_fwd(wl.x, wl.cu_seqlens, wl.weight, wl.bias)
        dx1, dw1, db1 = npa.varlen_dwconv_bwd(wl.x, wl.dy, wl.cu_seqlens, wl.weight)
    s.synchronize()
    dx0, dw0, db0 = npa.varlen_dwconv_bwd(wl.x, wl.dy, wl.cu_seqlens, wl.weight)
    torch.cuda.synchronize()
    assert torch.equal(y0, y1) and torch.equal(dx0, dx1) and torch.equal(dw0, dw1) and torch.equal(db0, db1)


def test_registered_custom_ops_pass_opcheck_and_compile_without_graph_breaks():
    """torch.compile(dynamic=False) is how the reference runs its model
    (src/nanoplm/pretraining/pure_pipeline.py:519-524); the conv must trace as one opaque op and accept
    the static collator's fixed-length cu_seqlens (collator.py:430-450)."""
    from nanoplm_amd.workloads import static_packed_cu

    wl = make_workload(2, T=3000, C=256, with_dy=True)
    F, W = 4096, 512
    cu = static_packed_cu(wl.cu_seqlens, F, W, cu_len=64).to(DEV)
    g = torch.Generator().manual_seed(3)
    x = torch.randn(F, 256, generator=g).bfloat16().to(DEV)
    dy = torch.randn(F, 256, generator=g).bfloat16().to(DEV)
    torch.library.opcheck(npa.varlen_dwconv_fwd_op, (x, cu, wl.weight.to(DEV), wl.bias.to(DEV)),
                          test_utils=("test_schema", "test_faketensor"))
    torch.library.opcheck(npa.varlen_dwconv_bwd_op, (x, dy, cu, wl.weight.to(DEV)),
                          test_utils=("test_schema", "test_faketensor"))

    conv = npa.VarlenDWConv1d(256, 7).to(DEV).to(torch.bfloat16)
    with torch.no_grad():
        conv.weight.copy_(wl.weight.to(DEV))
        conv.bias.copy_(wl.bias.to(DEV))

    def run(mod):
        xin = x.clone().requires_grad_(True)
        for p in conv.parameters():
            p.grad = None
        y = mod(xin, cu)
        (y.float() * dy.float()).sum().backward()
        return y.detach(), xin.grad, conv.weight.grad.clone(), conv.bias.grad.clone()

    y0, dx0, dw0, db0 = run(conv)
    compiled = torch.compile(conv, backend="aot_eager", fullgraph=True, dynamic=False)
    y1, dx1, dw1, db1 = run(compiled)
    assert torch.equal(y0, y1) and torch.equal(dx0, dx1) and torch.equal(dw0, dw1) and torch.equal(db0, db1)
    # and against the oracle on the real (unpadded) part
    T = wl.T
    cu_host = cu.cpu()
    y64 = O.c_oracle_fwd(x.cpu(), cu_host, wl.weight, wl.bias)
    assert_act_close(y1, y64, torch.bfloat16, "compiled y")
    assert T < F


def test_forward_and_backward_replay_correctly_from_a_hip_graph():
    """The op allocates nothing, reads cu_seqlens on the device and never synchronises, so a training
    step that contains it can be captured (reference: torch.compile + static shapes,
    pure_pipeline.py:519-529). Replay several times with new contents in the static buffers, with eager
    work and synchronisation between replays, and compare every replay with the eager result."""
    torch.manual_seed(1)
    lens = torch.tensor([100, 3, 512, 1, 408])
    cu = torch.zeros(6, dtype=torch.int32)
    cu[1:] = torch.cumsum(lens, 0)
    cu = cu.to(DEV)
    T, C, K = int(lens.sum()), 1024, 7
    w = (torch.randn(C, K, device=DEV) * K ** -0.5).bfloat16()
    b = (torch.randn(C, device=DEV) * 0.02).bfloat16()
    sx = torch.zeros(T, C, device=DEV, dtype=torch.bfloat16)
    sdy = torch.zeros_like(sx)
    ws = torch.empty(npa.bwd_workspace_bytes(T, C, K, torch.bfloat16), dtype=torch.uint8, device=DEV)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):                      # warm-up outside capture
        npa.varlen_dwconv_fwd(sx, cu, w, b, residual=True)
        npa.varlen_dwconv_bwd(sx, sdy, cu, w, residual=True, workspace=ws)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        gy = npa.varlen_dwconv_fwd(sx, cu, w, b, residual=True)
        gdx, gdw, gdb = npa.varlen_dwconv_bwd(sx, sdy, cu, w, residual=True, workspace=ws)
    for it in range(4):
        x = torch.randn(T, C, device=DEV).bfloat16()
        dy = torch.randn(T, C, device=DEV).bfloat16()
        sx.copy_(x)
        sdy.copy_(dy)
        graph.replay()
        torch.cuda.synchronize()
        ey = npa.varlen_dwconv_fwd(x, cu, w, b, residual=True)
        edx, edw, edb = npa.varlen_dwconv_bwd(x, dy, cu, w, residual=True)
        torch.cuda.synchronize()
        assert torch.equal(gy, ey) and torch.equal(gdx, edx), f"replay {it}"
        assert torch.equal(gdw, edw) and torch.equal(gdb, edb), f"replay {it}"


def test_the_integration_guides_ctypes_binding_runs_as_written():
    """The reference-side binding a maintainer would paste (the first Python block of the integration guide: a ctypes
    load of the shared object and an autograd Function over the two plain entry points) is executed as it stands, with
    only the library's file name replaced by its path, and gives this package's own results bit for bit."""
    import os
    import re
    from nanoplm_amd import _lib
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    guide = open(os.path.join(root, "INTEGRATION.md")).read()
    block = re.search(r"```python\n(import ctypes, torch\n.*?)```", guide, re.S).group(1)
    assert 'ctypes.CDLL("libnplm_dwconv.so")' in block
    ns = {}
    exec(block.replace('"libnplm_dwconv.so"', repr(_lib.LIB_PATH)), ns)
    fn = ns["VarlenDWConv1dFunction"]
    for cfg, kw in ((1, {}), (5, dict(T=5000, C=512))):
        wl = make_workload(cfg, with_dy=True, **kw)
        d = wl.to(DEV)
        x = d.x.clone().requires_grad_(True)
        w = d.weight.clone().requires_grad_(True)
        b = d.bias.clone().requires_grad_(True)
        y = fn.apply(x, d.cu_seqlens, w, b)
        y.backward(d.dy)
        assert torch.equal(y, npa.varlen_dwconv_fwd(d.x, d.cu_seqlens, d.weight, d.bias))
        dx, dw, db = npa.varlen_dwconv_bwd(d.x, d.dy, d.cu_seqlens, d.weight)
        assert torch.equal(x.grad, dx) and torch.equal(w.grad, dw.to(w.dtype)) and torch.equal(b.grad, db.to(b.dtype))
