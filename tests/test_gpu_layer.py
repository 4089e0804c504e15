"""The conv called the way an encoder layer would call it.

A test-only stand-in with the shape of the reference's layer
(src/nanoplm/pretraining/models/modern_bert/modeling.py:404-439: ``x = x + f(norm(x))`` twice) and of its
SwiGLU MLP (:286-302: ``Wi`` -> gate product -> ``Wo``): a pre-norm feeds ``VarlenDWConv1d(residual=True)``,
whose output is projected back into the residual stream; a second pre-norm feeds ``Wi``, the gated conv runs
between ``Wi`` and ``Wo``. ``cu_seqlens`` is the static collator's fixed-length tensor (collator.py:430-450)
and is passed down to both convs. Run as the reference runs its model: fp32 parameters under
``torch.autocast(bfloat16)`` (pure_pipeline.py:717-722), eager and ``torch.compile(dynamic=False)``
(:519-524), forward + backward.

Checked against the same composition evaluated in float64 on the CPU with the oracle's per-sequence conv1d
loop, and against a GPU twin under the same autocast whose convs are plain torch ops rounding where autocast
makes conv1d round (so the matmuls round identically on both sides and only the conv differs).
"""
import pytest
import torch
import torch.nn.functional as F
from torch import nn

import nanoplm_amd as npa
from nanoplm_amd.workloads import cu_from_lengths, static_packed_cu
from oracle import dwconv_ref as O

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def shifted_conv(x, cu, w, b, residual, dt):
    """The per-sequence conv as K masked, shifted products in plain torch ops (differentiable, no conv library on
    the GPU), rounding where ``torch.autocast`` makes ``F.conv1d`` round: inputs cast to ``dt``, fp32
    accumulation, result in ``dt``; the residual is the caller-side add ``x + conv(x)``."""
    T, K = x.shape[0], w.shape[1]
    P = (K - 1) // 2
    pos = torch.arange(T, device=x.device)
    seg = torch.searchsorted(cu[1:].long().contiguous(), pos, right=True)       # sequence index of every row
    acc_dt = torch.float64 if dt == torch.float64 else torch.float32
    xq, wq = x.to(dt).to(acc_dt), w.to(dt).to(acc_dt)
    acc = torch.zeros_like(xq) if b is None else b.to(dt).to(acc_dt).expand_as(xq)
    for k in range(K):
        src = pos + (k - P)
        inside = (src >= 0) & (src < T)
        src = src.clamp(0, T - 1)
        inside = inside & (seg[src] == seg)
        acc = acc + torch.where(inside[:, None], xq[src], 0.0) * wq[:, k]
    y = acc.to(dt)
    return x + y if residual else y


class ConvLayer(nn.Module):
    """conv='hip': this library's module; conv='ref': the oracle's per-sequence conv1d loop in ``ref_dtype``;
    conv='shift': ``shifted_conv`` rounding to ``ref_dtype``."""

    def __init__(self, hidden, inter, K, conv="hip", ref_dtype=None, fuse_norm=False):
        super().__init__()
        self.conv_kind, self.ref_dtype, self.fuse_norm = conv, ref_dtype, fuse_norm
        self.attn_norm = nn.LayerNorm(hidden, eps=1e-5, bias=False)
        self.mix_conv = npa.VarlenDWConv1d(hidden, K, residual=True)
        self.mix_out = nn.Linear(hidden, hidden, bias=False)
        self.mlp_norm = nn.LayerNorm(hidden, eps=1e-5, bias=False)
        self.Wi = nn.Linear(hidden, 2 * inter, bias=False)
        self.mlp_conv = npa.VarlenDWConv1d(inter, K)
        self.Wo = nn.Linear(inter, hidden, bias=False)
        self.seen = {}

    def _conv(self, mod, x, cu, residual):
        if self.conv_kind == "shift":
            return shifted_conv(x, cu, mod.weight, mod.bias, residual, self.ref_dtype)
        return O.ref_dwconv_varlen(x, cu, mod.weight, mod.bias, self.ref_dtype, residual=residual)

    def forward(self, x, cu_seqlens):
        if self.fuse_norm:      # the mixer is conv(norm(x)): the norm runs inside the conv's kernels
            if self.conv_kind == "hip":
                h = npa.ln_varlen_dwconv_compilable(x, cu_seqlens, self.attn_norm.weight, self.attn_norm.bias, self.mix_conv.weight,
                                                    self.mix_conv.bias, eps=self.attn_norm.eps)
            else:
                h = self._conv(self.mix_conv, self.attn_norm(x), cu_seqlens, False)
            return self._mlp(x + self.mix_out(h), cu_seqlens)
        h = self.attn_norm(x)
        if not torch.compiler.is_compiling():
            self.seen["mix_conv_in"] = h.dtype
        if self.conv_kind == "hip":
            h = self.mix_conv(h, cu_seqlens)                     # h + conv(h), one pass
        else:
            h = self._conv(self.mix_conv, h, cu_seqlens, True)
        return self._mlp(x + self.mix_out(h), cu_seqlens)

    def _mlp(self, x, cu_seqlens):
        z = self.Wi(self.mlp_norm(x))
        if not torch.compiler.is_compiling():
            self.seen["mlp_conv_in"] = z.dtype
        if self.conv_kind == "hip":
            g = self.mlp_conv.forward_gated(z, cu_seqlens)       # conv(x_proj * silu(gate))
        else:
            x_proj, gate = z.chunk(2, dim=-1)
            g = self._conv(self.mlp_conv, F.silu(gate) * x_proj, cu_seqlens, False)
        return x + self.Wo(g)


def _inputs(hidden, F_rows, seed):
    g = torch.Generator().manual_seed(seed)
    lens = torch.randint(20, 513, (64,), generator=g)
    real = cu_from_lengths(lens)
    n = int((real <= F_rows - 40).sum())                  # leave a pad run at the end
    cu = static_packed_cu(real[:n], F_rows, 512, cu_len=48)
    assert int(cu[-1]) == F_rows and int((cu[1:] == cu[:-1]).sum()) > 0
    x = torch.randn(F_rows, hidden, generator=g)
    dy = torch.randn(F_rows, hidden, generator=g)
    return x, dy, cu


def _make(hidden, inter, K, seed, fuse_norm=False):
    torch.manual_seed(seed)
    layer = ConvLayer(hidden, inter, K, fuse_norm=fuse_norm)
    with torch.no_grad():       # convs that do something: taps ~ N(0, 1/K)
        for c in (layer.mix_conv, layer.mlp_conv):
            c.weight.normal_(0, K ** -0.5)
            c.bias.normal_(0, 0.02)
    return layer


def _run(layer, x, dy, cu, autocast):
    for p in layer.parameters():
        p.grad = None
    xin = x.clone().requires_grad_(True)
    dev = xin.device.type
    with torch.autocast(device_type=dev, dtype=torch.bfloat16, enabled=autocast):
        y = layer(xin, cu)
    y.backward(dy.to(y.dtype))
    grads = {n.replace("_orig_mod.", ""): p.grad.detach().clone() for n, p in layer.named_parameters()}
    grads["x"] = xin.grad.detach().clone()
    return y.detach(), grads


def _twin(layer, conv, ref_dtype=None, device=DEV, dtype=None):
    t = ConvLayer(layer.mix_conv.channels, layer.mlp_conv.channels, layer.mix_conv.kernel_size, conv, ref_dtype, layer.fuse_norm)
    t.load_state_dict(layer.state_dict())
    t = t.to(device)
    return t.to(dtype) if dtype is not None else t


def _rel(a, b):
    b = b.to(a.device, torch.float64)
    return float((a.double() - b).abs().max() / b.abs().max().clamp_min(1e-30))


SHAPES = [(1024, 2048), (768, 1152)]      # hidden / intermediate: the pretraining preset and the model defaults


@pytest.mark.parametrize("hidden,inter", SHAPES)
def test_layer_in_fp32_matches_the_float64_composition(hidden, inter):
    """No autocast: every kernel runs in fp32; all outputs within 1e-4 of max |reference| (the fp32 matmuls' share)."""
    print(f"[case] layer fp32 hidden={hidden} inter={inter}", flush=True)
    x, dy, cu = _inputs(hidden, 2048, 1)
    layer = _make(hidden, inter, 7, 2)
    y64, g64 = _run(_twin(layer, "ref", torch.float64, "cpu", torch.float64), x.double(), dy.double(), cu, False)
    torch.backends.cuda.matmul.allow_tf32 = False
    y, g = _run(layer.to(DEV), x.to(DEV), dy.to(DEV), cu.to(DEV), False)
    assert y.dtype == torch.float32
    assert _rel(y, y64) <= 1e-4, _rel(y, y64)
    for name in g64:
        assert _rel(g[name], g64[name]) <= 1e-4, (name, _rel(g[name], g64[name]))


@pytest.mark.parametrize("hidden,inter", SHAPES)
def test_layer_under_bf16_autocast(hidden, inter):
    print(f"[case] layer autocast hidden={hidden} inter={inter}", flush=True)
    x, dy, cu = _inputs(hidden, 2048, 3)
    layer = _make(hidden, inter, 7, 4)
    y64, g64 = _run(_twin(layer, "ref", torch.float64, "cpu", torch.float64), x.double(), dy.double(), cu, False)
    xd, dyd, cud = x.to(DEV), dy.to(DEV), cu.to(DEV)
    ref = _twin(layer, "shift", torch.bfloat16)
    hip = layer.to(DEV)
    y, g = _run(hip, xd, dyd, cud, True)
    # what reaches each door under autocast with fp32 parameters: LayerNorm hands the residual-stream conv
    # fp32, the Linear hands the gated conv bf16
    assert hip.seen == {"mix_conv_in": torch.float32, "mlp_conv_in": torch.bfloat16}
    assert y.dtype == torch.float32 and all(v.dtype == torch.float32 for v in g.values())

    # (1) against float64: the bf16 matmuls and activations set the error, 2^-7 of the largest value is generous
    worst = {"y": _rel(y, y64), **{n: _rel(g[n], g64[n]) for n in g64}}
    print("[parity] layer autocast vs float64, max error / max |ref|: " +
          ", ".join(f"{k} {v:.2e}" for k, v in worst.items()), flush=True)
    assert max(worst.values()) <= 2.0 ** -7, worst

    # (2) against the same layer with plain-torch convs under the same autocast: the matmuls round the same way
    # on both sides, so what is left is the conv's own rounding (autocast would run conv1d in bf16; the kernels
    # keep the fp32 stream in fp32 and never round h): no further from float64 than that twin is
    yr, gr = _run(ref, xd, dyd, cud, True)
    assert _rel(y, y64) <= _rel(yr, y64) * 2 + 1e-4
    for n in g64:
        assert _rel(g[n], g64[n]) <= _rel(gr[n], g64[n]) * 2 + 1e-4, n


@pytest.mark.parametrize("backend", ["aot_eager", "inductor"])
@pytest.mark.parametrize("hidden,inter", SHAPES)
def test_layer_compiled_like_the_reference_compiles_its_model(hidden, inter, backend):
    """torch.compile(model, dynamic=False) (pure_pipeline.py:519-524; Inductor is its default backend): one graph,
    forward and backward, under autocast. aot_eager must reproduce eager bit for bit; Inductor fuses the
    elementwise ops around the opaque convs and may round those differently, so it is held to the float64 bar."""
    print(f"[case] layer compiled {backend} hidden={hidden} inter={inter}", flush=True)
    x, dy, cu = _inputs(hidden, 2048, 5)
    layer = _make(hidden, inter, 7, 6)
    y64, g64 = _run(_twin(layer, "ref", torch.float64, "cpu", torch.float64), x.double(), dy.double(), cu, False)
    xd, dyd, cud = x.to(DEV), dy.to(DEV), cu.to(DEV)
    hip = layer.to(DEV)
    y, g = _run(hip, xd, dyd, cud, True)
    torch._dynamo.reset()
    compiled = torch.compile(hip, backend=backend, fullgraph=True, dynamic=False)
    try:
        yc, gc = _run(compiled, xd, dyd, cud, True)
    except Exception as e:
        if backend == "inductor" and "nanoplm_amd" not in str(e):
            pytest.skip(f"Inductor cannot build on this box: {type(e).__name__}: {str(e)[:300]}")
        raise
    if backend == "aot_eager":
        assert torch.equal(yc, y)
        for n in g:
            assert torch.equal(gc[n], g[n]), n
    else:
        assert _rel(yc, y64) <= 2.0 ** -7
        for n in g64:
            assert _rel(gc[n], g64[n]) <= 2.0 ** -7, n


@pytest.mark.parametrize("backend", ["eager", "aot_eager", "inductor"])
@pytest.mark.parametrize("hidden,inter", SHAPES)
def test_layer_with_the_norm_fused_into_the_conv(hidden, inter, backend):
    """The mixer as conv(norm(x)) with the LayerNorm inside the conv's kernels (modeling.py:404-438: every sub-module
    takes a pre-norm of the residual stream). Under autocast with fp32 parameters the stream is fp32: rows of 3 and
    4 KiB, the statistics kernel + the normalising conv forward, and the fused backward. Against the float64
    composition and against the unfused layer under the same autocast (torch's LayerNorm, then the HIP conv)."""
    print(f"[case] layer fused norm {backend} hidden={hidden} inter={inter}", flush=True)
    x, dy, cu = _inputs(hidden, 2048, 7)
    layer = _make(hidden, inter, 7, 8, fuse_norm=True)
    y64, g64 = _run(_twin(layer, "ref", torch.float64, "cpu", torch.float64), x.double(), dy.double(), cu, False)
    xd, dyd, cud = x.to(DEV), dy.to(DEV), cu.to(DEV)
    ref = _twin(layer, "shift", torch.bfloat16)
    hip = layer.to(DEV)
    assert npa.ln_supported(xd, hip.mix_conv.weight)
    mod = hip
    if backend != "eager":
        torch._dynamo.reset()
        mod = torch.compile(hip, backend=backend, fullgraph=True, dynamic=False)
    try:
        y, g = _run(mod, xd, dyd, cud, True)
    except Exception as e:
        if backend == "inductor" and "nanoplm_amd" not in str(e):
            pytest.skip(f"Inductor cannot build on this box: {type(e).__name__}: {str(e)[:300]}")
        raise
    worst = {"y": _rel(y, y64), **{n: _rel(g[n], g64[n]) for n in g64}}
    print("[parity] layer with fused norm vs float64, max error / max |ref|: " +
          ", ".join(f"{k} {v:.2e}" for k, v in worst.items()), flush=True)
    assert max(worst.values()) <= 2.0 ** -7, worst
    yr, gr = _run(ref, xd, dyd, cud, True)
    assert _rel(y, y64) <= _rel(yr, y64) * 2 + 1e-4
    for n in g64:
        assert _rel(g[n], g64[n]) <= _rel(gr[n], g64[n]) * 2 + 1e-4, n
    if backend == "aot_eager":
        ye, ge = _run(hip, xd, dyd, cud, True)
        assert torch.equal(ye, y)
        for n in g:
            assert torch.equal(ge[n], g[n]), n
