"""Host-side logic around the op (no GPU): padded-batch boundaries, un/pad helpers, and how the
module's parameters are seen by the reference's optimizer grouping rules."""
import torch
from torch import nn

import nanoplm_amd as npa


# ---- padded batches -----------------------------------------------------------------------------------
def test_right_padded_cu_seqlens_lists_real_and_pad_runs():
    mask = torch.tensor([[1, 1, 1, 0, 0], [1, 1, 1, 1, 1], [0, 0, 0, 0, 0], [1, 0, 0, 0, 0]])
    cu = npa.right_padded_cu_seqlens(mask)
    assert cu.dtype == torch.int32
    assert cu.tolist() == [0, 3, 5, 10, 10, 10, 15, 16, 20]
    assert bool(npa.is_right_padded(mask))
    assert not bool(npa.is_right_padded(torch.tensor([[0, 1, 1], [1, 1, 0]])))
    # fixed length 2B+1 whatever the lengths are (static shapes for torch.compile(dynamic=False))
    assert npa.right_padded_cu_seqlens(torch.ones(7, 9, dtype=torch.bool)).numel() == 15


def test_unpad_and_pad_follow_the_reference_contracts():
    """indices / int32 cu_seqlens / 0-D max_seqlen as modeling.py:164-178; scatter back with zeros
    at padding as modeling.py:181-194. Worked example of modeling.py:204: lengths 3, 2, 4."""
    mask = torch.tensor([[1, 1, 1, 0], [0, 1, 1, 0], [1, 1, 1, 1]])
    idx, cu, mx = npa.unpad_input(mask)
    assert idx.tolist() == [0, 1, 2, 5, 6, 8, 9, 10, 11]
    assert cu.dtype == torch.int32 and cu.tolist() == [0, 3, 5, 9]
    assert mx.dim() == 0 and int(mx) == 4
    h = torch.arange(9.0)[:, None].repeat(1, 2) + 1
    out = npa.pad_output(h, idx, 3, 4)
    assert out.shape == (3, 4, 2)
    assert torch.equal(out.reshape(12, 2)[idx], h)
    assert float(out.reshape(12, 2)[[3, 4, 7]].abs().sum()) == 0.0


# ---- the reference's grouping rules, restated -----------------------------------------------------------
def _ref_routes_to_muon(name, p):
    """src/nanoplm/pretraining/optim.py:43-53 (embedding names never match a conv parameter)."""
    if p.ndim == 1:
        return False
    return p.ndim == 2


def _ref_use_weight_decay(name, p):
    """src/nanoplm/pretraining/pure_pipeline.py:68-76."""
    lname = name.lower()
    if not p.requires_grad or p.ndim < 2:
        return False
    return not ("bias" in lname or "norm" in lname)


class _Layer(nn.Module):
    def __init__(self, **kw):
        super().__init__()
        self.Wo = nn.Linear(16, 16, bias=False)
        self.conv = npa.VarlenDWConv1d(16, 7, **kw)


def test_default_tap_table_would_be_sent_to_muon_and_decayed():
    named = dict(_Layer().named_parameters())
    assert _ref_routes_to_muon("conv.weight", named["conv.weight"])
    assert _ref_use_weight_decay("conv.weight", named["conv.weight"])
    assert not _ref_use_weight_decay("conv.bias", named["conv.bias"])


def test_flat_weight_lands_in_adamw_without_decay_under_the_reference_rules():
    m = _Layer(flat_weight=True)
    named = dict(m.named_parameters())
    assert "conv.weight_flat" in named and "conv.weight" not in named
    p = named["conv.weight_flat"]
    assert p.ndim == 1 and p.numel() == 16 * 7
    assert not _ref_routes_to_muon("conv.weight_flat", p)
    assert not _ref_use_weight_decay("conv.weight_flat", p)
    # the [C, K] view is what the kernels get, and gradients reach the flat parameter through it
    w = m.conv.weight
    assert w.shape == (16, 7) and w.data_ptr() == p.data_ptr()
    w.sum().backward()
    assert torch.equal(p.grad, torch.ones_like(p))
    assert list(m.conv.state_dict()) == ["weight_flat", "bias"]


def test_split_conv_parameters_takes_exactly_the_conv_parameters_out():
    m = nn.Sequential(_Layer(), _Layer(flat_weight=True))
    conv, rest = npa.split_conv_parameters(m)
    assert len(conv) == 4 and sorted(rest) == ["0.Wo.weight", "1.Wo.weight"]
    names = [n for n, _ in npa.conv_parameters(m)]
    assert names == ["0.conv.weight", "0.conv.bias", "1.conv.weight_flat", "1.conv.bias"]
    # the optimizer a caller would build from it
    opt = torch.optim.AdamW([{"params": conv, "weight_decay": 0.0}, {"params": list(rest.values())}])
    assert sum(len(g["params"]) for g in opt.param_groups) == 6


def test_init_options():
    torch.manual_seed(0)
    z = npa.VarlenDWConv1d(32, 7, residual=True, init="zero")
    assert float(z.weight.detach().abs().sum()) == 0.0 and float(z.bias.detach().abs().sum()) == 0.0
    i = npa.VarlenDWConv1d(32, 7, init="identity", flat_weight=True)
    w = i.weight.detach()
    assert torch.equal(w[:, 3], torch.ones(32)) and float(w.abs().sum()) == 32.0
    n = npa.VarlenDWConv1d(4096, 7)
    assert abs(float(n.weight.detach().std()) - 7 ** -0.5) < 0.01 and abs(float(n.bias.detach().std()) - 0.02) < 0.002
    try:
        npa.VarlenDWConv1d(8, 3, init="kaiming")
    except ValueError as e:
        assert "init" in str(e)
    else:
        raise AssertionError("unknown init accepted")
