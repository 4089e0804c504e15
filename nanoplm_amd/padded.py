"""Padded-batch front end of the varlen depthwise conv.

The reference model has two paths: packed ``[total_tokens, hidden]`` + ``cu_seqlens`` (flash-attn
varlen) and padded ``[batch, seq_len, hidden]`` + attention mask (SDPA fallback,
src/nanoplm/pretraining/models/modern_bert/modeling.py:505-544); it moves between them with
``_unpad_input`` / ``_pad_output`` (modeling.py:164-194). This module gives the conv the same two
doors without any host synchronisation:

* ``right_padded_cu_seqlens(attention_mask)`` -- for masks of the form 1..1 0..0 per row (right
  padding, what the reference's collators emit) the padded tensor viewed as ``[B*L, C]`` already IS a
  packed tensor: row block b holds a real sequence of ``len_b`` rows followed by a pad run. The
  returned ``cu_seqlens`` (2B+1 entries, fixed length) lists both, so the kernels run in place with
  no gather/scatter; pad runs become pseudo-sequences whose outputs depend only on pad rows.
* ``unpad_input`` / ``pad_output`` -- the general route for arbitrary masks, same contracts as the
  reference helpers (indices, int32 cu_seqlens, 0-D max_seqlen).
"""
from __future__ import annotations

from typing import Optional, Tuple

import torch
import torch.nn.functional as F

from .dwconv import varlen_dwconv


def right_padded_cu_seqlens(attention_mask: torch.Tensor) -> torch.Tensor:
    """int32 ``[2B+1]`` boundaries of a right-padded ``[B, L]`` mask over the flat ``[B*L]`` row axis:
    ``[0, len_0, L, L+len_1, 2L, ..., B*L]``. Zero-length entries (full or empty rows) are legal for the
    kernels. No host synchronisation; the length is fixed, so it is ``torch.compile(dynamic=False)``
    friendly like the static collator's ``cu_seqlens`` (collator.py:430-450)."""
    if attention_mask.dim() != 2:
        raise ValueError("attention_mask must be [batch, seq_len]")
    B, L = attention_mask.shape
    seqlens = attention_mask.sum(dim=-1, dtype=torch.int32)
    starts = torch.arange(B, device=attention_mask.device, dtype=torch.int32) * L
    inner = torch.stack((starts, starts + seqlens), dim=1).flatten()
    end = torch.full((1,), B * L, device=attention_mask.device, dtype=torch.int32)
    return torch.cat((inner, end))


def is_right_padded(attention_mask: torch.Tensor) -> torch.Tensor:
    """0-D bool tensor: every row of the mask is a run of ones followed by a run of zeros.
    (A debugging aid; reading it on the host synchronises.)"""
    m = attention_mask.to(torch.int32)
    return (m[:, 1:] <= m[:, :-1]).all()


def unpad_input(attention_mask: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    """(indices, cu_seqlens, max_seqlen) of the non-padding positions of a ``[B, L]`` mask; the same
    contract as the reference's ``_unpad_input`` (modeling.py:164-178)."""
    seqlens = attention_mask.sum(dim=-1, dtype=torch.int32)
    indices = torch.nonzero(attention_mask.flatten(), as_tuple=False).flatten()
    cu_seqlens = F.pad(torch.cumsum(seqlens, dim=0, dtype=torch.int32), (1, 0))
    return indices, cu_seqlens, seqlens.max()


def pad_output(hidden: torch.Tensor, indices: torch.Tensor, batch: int, seqlen: int) -> torch.Tensor:
    """Scatter flat ``[total_tokens, ...]`` rows back to ``[batch, seqlen, ...]`` (zeros at padding);
    same contract as the reference's ``_pad_output`` (modeling.py:181-194)."""
    out = torch.zeros((batch * seqlen, *hidden.shape[1:]), device=hidden.device, dtype=hidden.dtype)
    out[indices] = hidden
    return out.view(batch, seqlen, *hidden.shape[1:])


def padded_dwconv(x: torch.Tensor, attention_mask: torch.Tensor, weight: torch.Tensor,
                  bias: Optional[torch.Tensor] = None, residual: bool = False,
                  assume_right_padded: bool = True) -> torch.Tensor:
    """Depthwise conv over a padded batch ``x:[B, L, C]`` with ``attention_mask:[B, L]``.

    Real positions get exactly what the packed op gives their sequence. With
    ``assume_right_padded`` (default) nothing is copied: padding positions hold the conv of the pad
    run they belong to (finite, and independent of every real token), as in the reference's padded
    path where layers also compute on pad rows. Otherwise the rows are gathered, convolved and
    scattered back, and padding positions are zero."""
    if x.dim() != 3 or attention_mask.shape != x.shape[:2]:
        raise ValueError("x must be [B, L, C] and attention_mask [B, L]")
    B, L, C = x.shape
    if assume_right_padded:
        cu = right_padded_cu_seqlens(attention_mask)
        y = varlen_dwconv(x.reshape(B * L, C), cu, weight, bias, residual)
        return y.view(B, L, C)
    indices, cu, _ = unpad_input(attention_mask)
    y = varlen_dwconv(x.reshape(B * L, C)[indices], cu, weight, bias, residual)
    return pad_output(y, indices, B, L)
