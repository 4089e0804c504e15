#!/usr/bin/env python3
"""Writes the golden fixtures under tests/golden/ from the CPU oracle (run once, in this repo).

The reference snapshot holds no convolution and no vectors for one, so these are produced by the
repo's own reference path -- the per-sequence ``torch.nn.functional.conv1d`` loop and its autograd
in float64 (oracle/dwconv_ref.py) -- and are valid only together with tests/test_oracle.py, which
pins that path against the C restatement, brute force and closed forms before trusting it.

    python tests/golden/make_golden.py

Each .npz holds inputs (x, w, b, dy as float32 -- for bf16 cases the bf16 values upcast, which is
exact -- and int32 cu_seqlens) and outputs computed in float64 (y, dx stored rounded to float32 to
keep the files small; dw, db stored as float64). Loaded with numpy.load(allow_pickle=False).
"""
import os
import sys

import numpy as np
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)

from nanoplm_amd.workloads import cu_from_lengths, make_workload  # noqa: E402
from oracle.dwconv_ref import ref_dwconv_varlen_grads  # noqa: E402

OUT = os.path.dirname(os.path.abspath(__file__))


def save(name, x, cu, w, b, dy, act_dtype):
    y, dx, dw, db = ref_dwconv_varlen_grads(x.float(), cu, w.float(), b.float(), dy.float(), torch.float64)
    np.savez_compressed(
        os.path.join(OUT, name + ".npz"),
        x=x.float().numpy(), w=w.float().numpy(), b=b.float().numpy(), dy=dy.float().numpy(),
        cu_seqlens=cu.numpy().astype(np.int32), y=y.float().numpy(), dx=dx.float().numpy(), dw=dw.numpy(),
        db=db.numpy(),
        act_dtype=np.array(act_dtype))
    print(name, tuple(x.shape), "K =", w.shape[1], "S =", cu.numel() - 1)


def main():
    # configuration 1 complete (fp32, 8 sequences of 20..128 rows, C=64, K=3), plus a dy for the backward
    wl = make_workload(1, with_dy=True)
    save("cfg1_fp32_C64_K3", wl.x, wl.cu_seqlens, wl.weight, wl.bias, wl.dy, "float32")

    # boundary micro-case: sequences shorter than the K=7 radius next to long ones, and empty ones
    g = torch.Generator().manual_seed(20260101)
    lens = torch.tensor([1, 2, 3, 8, 0, 1, 450, 0, 5, 7, 6, 1])
    T, C, K = int(lens.sum()), 16, 7
    x = torch.randn(T, C, generator=g)
    w = torch.randn(C, K, generator=g) * K ** -0.5
    b = torch.randn(C, generator=g) * 0.02
    dy = torch.randn(T, C, generator=g)
    save("boundary_fp32_C16_K7", x, cu_from_lengths(lens), w, b, dy, "float32")

    # bf16 inputs (stored upcast): 60 sequences, 60% of them 1..8 rows (shorter than the K=7 radius),
    # the rest 20..60 rows, shuffled; C=32, K=7
    g = torch.Generator().manual_seed(20260102)
    n = 60
    short = torch.rand(n, generator=g) < 0.6
    lens = torch.where(short, torch.randint(1, 9, (n,), generator=g), torch.randint(20, 61, (n,), generator=g))
    T, C, K = int(lens.sum()), 32, 7
    x = torch.randn(T, C, generator=g).bfloat16()
    w = (torch.randn(C, K, generator=g) * K ** -0.5).bfloat16()
    b = (torch.randn(C, generator=g) * 0.02).bfloat16()
    dy = torch.randn(T, C, generator=g).bfloat16()
    save("stress_bf16_C32_K7", x, cu_from_lengths(lens), w, b, dy, "bfloat16")


if __name__ == "__main__":
    main()
