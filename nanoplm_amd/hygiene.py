"""Optimizer routing helpers for models that contain :class:`VarlenDWConv1d`.

The reference builds its parameter groups from names and shapes alone
(src/nanoplm/pretraining/optim.py:36-53: 1-D -> AdamW, embeddings -> AdamW, every other ``ndim == 2``
-> Muon; src/nanoplm/pretraining/pure_pipeline.py:68-76: weight decay for ``ndim >= 2`` unless the
name contains "bias" or "norm"). A ``[C, K]`` tap table is 2-D, so it would be orthogonalised by Muon
and decayed. Two ways out:

* construct the module with ``flat_weight=True`` (the parameter is then 1-D and both rules send it to
  AdamW without decay, no change on the reference side), or
* keep ``[C, K]`` and take the conv parameters out before the reference's grouping with the helpers
  below.
"""
from __future__ import annotations

from typing import Dict, Iterator, List, Tuple

import torch
from torch import nn

from .dwconv import VarlenDWConv1d


def conv_parameters(model: nn.Module) -> Iterator[Tuple[str, nn.Parameter]]:
    """(qualified name, parameter) of every parameter owned by a VarlenDWConv1d inside ``model``."""
    for mod_name, mod in model.named_modules():
        if isinstance(mod, VarlenDWConv1d):
            for p_name, p in mod.named_parameters(recurse=False):
                yield (f"{mod_name}.{p_name}" if mod_name else p_name), p


def split_conv_parameters(model: nn.Module) -> Tuple[List[nn.Parameter], Dict[str, nn.Parameter]]:
    """(conv parameters, every other named parameter). The first list belongs in an AdamW group with
    ``weight_decay=0``; the second dict is what the reference's grouping rules should see."""
    conv = dict(conv_parameters(model))
    ids = {id(p) for p in conv.values()}
    rest = {n: p for n, p in model.named_parameters() if id(p) not in ids}
    return list(conv.values()), rest
