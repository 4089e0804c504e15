"""Seeded synthetic inputs for the five benchmark/parity configurations of the varlen depthwise conv.

Everything is drawn on the CPU from ``torch.Generator().manual_seed(20260000 + index)`` in fp32, in
the fixed order lengths -> x -> weight -> bias -> dy, then cast once to the configuration's dtype,
so the GPU kernels and the CPU oracle see bit-identical inputs on any machine.

Sequence-length mixes follow the packed-batch regime of the reference
(src/nanoplm/pretraining/collator.py:250-327: many sequences of 20..512 residues packed back to
back, ``cu_seqlens`` = int32 cumulative lengths starting at 0).
"""
from __future__ import annotations

import dataclasses
from typing import Optional

import torch


@dataclasses.dataclass
class Workload:
    index: int
    name: str
    passes: str            # "fwd" or "fwd+bwd"
    dtype: torch.dtype
    T: int
    C: int
    K: int
    lengths: torch.Tensor  # int64 [S]
    cu_seqlens: torch.Tensor  # int32 [S+1]
    x: torch.Tensor
    weight: torch.Tensor
    bias: torch.Tensor
    dy: Optional[torch.Tensor]

    @property
    def S(self) -> int:
        return int(self.lengths.numel())

    def to(self, device) -> "Workload":
        def mv(t):
            return None if t is None else t.to(device)
        return dataclasses.replace(self, cu_seqlens=mv(self.cu_seqlens), x=mv(self.x), weight=mv(self.weight),
                                   bias=mv(self.bias), dy=mv(self.dy))

    def algorithmic_bytes(self, passes: Optional[str] = None) -> int:
        """Bytes one launch must move: fwd = 2TCe + C(K+1)e_w + 4(S+1); bwd = 3TCe + CKe_w + 4C(K+1) + 4(S+1)."""
        e = self.x.element_size()
        ew = self.weight.element_size()
        T, C, K, S = self.T, self.C, self.K, self.S
        fwd = 2 * T * C * e + C * (K + 1) * ew + 4 * (S + 1)
        bwd = 3 * T * C * e + C * K * ew + 4 * C * (K + 1) + 4 * (S + 1)
        passes = passes or self.passes
        return {"fwd": fwd, "bwd": bwd, "fwd+bwd": fwd + bwd}[passes]

    def algorithmic_flops(self, passes: Optional[str] = None) -> int:
        """Floating-point operations one launch must do: fwd = 2KTC; bwd = 4KTC (dx and dw) + TC (db)."""
        T, C, K = self.T, self.C, self.K
        fwd = 2 * K * T * C
        bwd = 4 * K * T * C + T * C
        passes = passes or self.passes
        return {"fwd": fwd, "bwd": bwd, "fwd+bwd": fwd + bwd}[passes]


_SPECS = {
    1: dict(name="cfg1_fp32_fwd_8seq_C64_K3", passes="fwd", dtype=torch.float32, T=None, C=64, K=3, mix="n8_u20_128"),
    2: dict(name="cfg2_bf16_fwd_T32768_C1024_K7", passes="fwd", dtype=torch.bfloat16, T=32768, C=1024, K=7,
            mix="u20_512"),
    3: dict(name="cfg3_bf16_fwdbwd_T131072_C1024_K7", passes="fwd+bwd", dtype=torch.bfloat16, T=131072, C=1024, K=7,
            mix="u20_512"),
    4: dict(name="cfg4_bf16_fwdbwd_T131072_C2048_K31_lognormal", passes="fwd+bwd", dtype=torch.bfloat16, T=131072,
            C=2048, K=31, mix="lognormal"),
    5: dict(name="cfg5_bf16_fwdbwd_T65536_C1024_K7_boundary_stress", passes="fwd+bwd", dtype=torch.bfloat16,
            T=65536, C=1024, K=7, mix="stress"),
}


def _draw_lengths(mix: str, n: int, g: torch.Generator) -> torch.Tensor:
    if mix == "n8_u20_128":
        return torch.randint(20, 129, (n,), generator=g)
    if mix == "u20_512":
        return torch.randint(20, 513, (n,), generator=g)
    if mix == "lognormal":
        z = torch.randn(n, generator=g) * 0.8 + 5.5
        return torch.clamp(torch.round(torch.exp(z)), 20, 1024).to(torch.int64)
    if mix == "stress":
        short = torch.rand(n, generator=g) < 0.6
        a = torch.randint(1, 9, (n,), generator=g)
        b = torch.randint(400, 513, (n,), generator=g)
        return torch.where(short, a, b)
    raise ValueError(mix)


def draw_lengths(mix: str, T: Optional[int], g: torch.Generator) -> torch.Tensor:
    """Lengths of the given mix; with T, appended until the total reaches T and the last one is truncated."""
    if T is None:
        return _draw_lengths(mix, 8, g)
    chunks, total = [], 0
    while total < T:
        c = _draw_lengths(mix, 1024, g)
        chunks.append(c)
        total += int(c.sum())
    lens = torch.cat(chunks)
    csum = torch.cumsum(lens, 0)
    n = int(torch.searchsorted(csum, torch.tensor(T)).item()) + 1   # first n lengths reach T
    lens = lens[:n].clone()
    lens[-1] -= int(csum[n - 1]) - T
    assert int(lens.sum()) == T and int(lens.min()) >= 1
    return lens


def cu_from_lengths(lengths: torch.Tensor) -> torch.Tensor:
    cu = torch.zeros(lengths.numel() + 1, dtype=torch.int32)
    cu[1:] = torch.cumsum(lengths, 0).to(torch.int32)
    return cu


def make_workload(index: int, *, T: Optional[int] = None, C: Optional[int] = None,
                  with_dy: Optional[bool] = None) -> Workload:
    """Configuration ``index`` (1..5) on the CPU. ``T`` / ``C`` shrink it for quick tests (same seed, same mix)."""
    spec = dict(_SPECS[index])
    if T is not None and spec["T"] is not None:
        spec["T"] = T
    if C is not None:
        spec["C"] = C
    g = torch.Generator().manual_seed(20260000 + index)
    lengths = draw_lengths(spec["mix"], spec["T"], g)
    T_ = int(lengths.sum())
    C_, K = spec["C"], spec["K"]
    dt = spec["dtype"]
    x = torch.randn(T_, C_, generator=g).to(dt)
    w = (torch.randn(C_, K, generator=g) * (K ** -0.5)).to(dt)
    b = (torch.randn(C_, generator=g) * 0.02).to(dt)
    want_dy = (spec["passes"] == "fwd+bwd") if with_dy is None else with_dy
    dy = torch.randn(T_, C_, generator=g).to(dt) if want_dy else None
    return Workload(index=index, name=spec["name"], passes=spec["passes"], dtype=dt, T=T_, C=C_, K=K,
                    lengths=lengths, cu_seqlens=cu_from_lengths(lengths), x=x, weight=w, bias=b, dy=dy)


def static_packed_cu(cu_seqlens: torch.Tensor, F: int, max_seq_len: int, cu_len: int) -> torch.Tensor:
    """Fixed-length cu_seqlens as the reference's static-shape collator builds it
    (src/nanoplm/pretraining/collator.py:430-450): the real boundaries, then pad pseudo-sequences of
    at most ``max_seq_len`` rows covering [T, F), then zero-length entries equal to F."""
    T = int(cu_seqlens[-1])
    out = torch.full((cu_len,), F, dtype=torch.int32)
    n = cu_seqlens.numel()
    out[:n] = cu_seqlens
    pos, idx, pad = T, n, F - T
    while pad > 0 and idx < cu_len:
        chunk = min(max_seq_len, pad)
        pos += chunk
        out[idx] = pos
        pad -= chunk
        idx += 1
    return out
