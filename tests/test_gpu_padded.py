"""Padded-batch door of the op ([B, L, C] + attention mask, the reference's SDPA-path layout,
modeling.py:505-544) and the flat_weight parameterisation, on the GPU against the oracle."""
import pytest
import torch

import nanoplm_amd as npa
from oracle import dwconv_ref as O
from tests.gpu_util import assert_act_close, assert_red_close

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _padded_case(lens, L, C, K, dt, seed):
    g = torch.Generator().manual_seed(seed)
    B = len(lens)
    x = torch.randn(B, L, C, generator=g).to(dt)
    mask = torch.zeros(B, L, dtype=torch.bool)
    for b, n in enumerate(lens):
        mask[b, :n] = True
    w = (torch.randn(C, K, generator=g) * K ** -0.5).to(dt)
    bias = (torch.randn(C, generator=g) * 0.02).to(dt)
    return x, mask, w, bias


def _oracle_on_real_rows(x, mask, w, bias, residual=False):
    idx, cu, _ = npa.unpad_input(mask)
    B, L, C = x.shape
    return idx, O.c_oracle_fwd(x.reshape(B * L, C)[idx], cu, w, bias, residual=residual)


@pytest.mark.parametrize("residual", [False, True])
def test_right_padded_batch_in_place(residual):
    lens = [37, 128, 0, 1, 90, 128, 5]
    x, mask, w, bias = _padded_case(lens, 128, 1024, 7, torch.bfloat16, seed=1)
    idx, y64 = _oracle_on_real_rows(x, mask, w, bias, residual)
    xd, md, wd, bd = x.to(DEV), mask.to(DEV), w.to(DEV), bias.to(DEV)
    y = npa.padded_dwconv(xd, md, wd, bd, residual=residual)
    assert y.shape == x.shape
    assert_act_close(y.reshape(-1, 1024)[idx.to(DEV)], y64, x.dtype, "padded y (real rows)")
    assert torch.isfinite(y.float()).all()
    # padding positions depend on pad rows only: change every real token, pads stay bit-identical
    x2 = xd.clone()
    x2[md] = 7.0
    y2 = npa.padded_dwconv(x2, md, wd, bd, residual=residual)
    assert torch.equal(y[~md], y2[~md])


def test_arbitrary_mask_goes_through_gather_and_scatter():
    g = torch.Generator().manual_seed(2)
    B, L, C = 5, 64, 256
    x = torch.randn(B, L, C, generator=g)
    mask = torch.rand(B, L, generator=g) > 0.3          # holes anywhere (left padding included)
    mask[2] = False
    w = torch.randn(C, 5, generator=g) * 5 ** -0.5
    bias = torch.randn(C, generator=g) * 0.02
    idx, y64 = _oracle_on_real_rows(x, mask, w, bias)
    y = npa.padded_dwconv(x.to(DEV), mask.to(DEV), w.to(DEV), bias.to(DEV), assume_right_padded=False)
    assert_act_close(y.reshape(-1, C)[idx.to(DEV)], y64, x.dtype, "gathered y")
    assert float(y[~mask.to(DEV)].abs().sum()) == 0.0


def test_padded_module_gradients_match_the_packed_op():
    """Loss on real tokens only (what masked-LM labels give): dw/db/dx of the in-place padded route
    equal those of the packed route on the gathered rows."""
    lens = [50, 128, 3, 77]
    x, mask, w, bias = _padded_case(lens, 128, 256, 7, torch.float32, seed=3)
    idx, cu, _ = npa.unpad_input(mask)
    conv = npa.VarlenDWConv1d(256, 7, device=DEV)
    with torch.no_grad():
        conv.weight.copy_(w)
        conv.bias.copy_(bias)
    xd = x.to(DEV).requires_grad_(True)
    md = mask.to(DEV)
    gy = torch.randn(int(mask.sum()), 256, device=DEV)
    y = conv.forward_padded(xd, md)
    (y[md] * gy).sum().backward()
    dw_p, db_p, dx_p = conv.weight.grad.clone(), conv.bias.grad.clone(), xd.grad.clone()
    conv.zero_grad()
    xr = x.reshape(-1, 256)[idx].to(DEV).requires_grad_(True)
    (conv(xr, cu.to(DEV)) * gy).sum().backward()
    torch.testing.assert_close(dw_p, conv.weight.grad, rtol=1e-5, atol=1e-4)
    torch.testing.assert_close(db_p, conv.bias.grad, rtol=1e-5, atol=1e-4)
    torch.testing.assert_close(dx_p[md], xr.grad, rtol=1e-5, atol=1e-5)
    assert float(dx_p[~md].abs().sum()) == 0.0


def test_flat_weight_module_trains_like_the_2d_one():
    torch.manual_seed(4)
    lens = torch.tensor([30, 2, 200, 24])
    cu = torch.zeros(5, dtype=torch.int32)
    cu[1:] = torch.cumsum(lens, 0)
    cu = cu.to(DEV)
    a = npa.VarlenDWConv1d(128, 7, residual=True, device=DEV)
    b = npa.VarlenDWConv1d(128, 7, residual=True, flat_weight=True, device=DEV)
    with torch.no_grad():
        b.weight_flat.copy_(a.weight.reshape(-1))
        b.bias.copy_(a.bias)
    x = torch.randn(256, 128, device=DEV)
    gy = torch.randn(256, 128, device=DEV)
    a(x, cu).backward(gy)
    b(x, cu).backward(gy)
    assert torch.equal(b.weight_flat.grad.view(128, 7), a.weight.grad)
    assert torch.equal(b.bias.grad, a.bias.grad)
    # zero-initialised residual block is the identity
    z = npa.VarlenDWConv1d(128, 7, residual=True, init="zero", device=DEV)
    assert torch.equal(z(x, cu), x)


def test_padded_door_compiles_without_graph_breaks():
    """forward_padded inside a compiled model (torch.compile(dynamic=False), pure_pipeline.py:519-524): the call
    reaches the registered custom ops, so fullgraph=True holds, forward and backward."""
    lens = [37, 128, 0, 1, 90, 128, 5]
    x, mask, w, bias = _padded_case(lens, 128, 1024, 7, torch.bfloat16, seed=3)
    conv = npa.VarlenDWConv1d(1024, 7, residual=True, device=DEV, dtype=torch.bfloat16)
    with torch.no_grad():
        conv.weight.copy_(w.to(DEV))
        conv.bias.copy_(bias.to(DEV))
    xd, md = x.to(DEV), mask.to(DEV)

    class Door(torch.nn.Module):
        def __init__(self):
            super().__init__()
            self.conv = conv

        def forward(self, xx, mm):
            return self.conv.forward_padded(xx, mm)

    def run(mod):
        conv.zero_grad()
        xin = xd.clone().requires_grad_(True)
        y = mod(xin, md)
        y.float().square().sum().backward()
        return y.detach(), xin.grad, conv.weight.grad.clone(), conv.bias.grad.clone()

    door = Door()
    eager = run(door)
    torch._dynamo.reset()
    compiled = run(torch.compile(door, backend="aot_eager", fullgraph=True, dynamic=False))
    for a, b in zip(eager, compiled):
        assert torch.equal(a, b)
