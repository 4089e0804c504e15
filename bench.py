#!/usr/bin/env python3
"""Benchmark of the varlen depthwise conv hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--config 3] [--no-cpu-baseline]

A step is one forward plus one backward (dx, dweight, dbias) of the configured workload through the
C ABI of libnplm_dwconv.so, with every input already resident in HBM. The default workload is
configuration 3 of nanoplm_amd.workloads (T=131072 packed tokens, C=1024, K=7, bf16), the one the
headline metric is quoted on. Four input/output sets (> 256 MB each) are rotated, and the backward of a
step works on the set two places away from the forward's, so that no kernel reads a tensor that an
earlier kernel left in the 256 MB Infinity Cache: at least two other kernels (>= 1.3 GB of traffic) run
between two touches of the same tensor, as in a training step, where a layer's backward runs long
after its forward. (ms_per_step_same_tensors is the same loop with forward and backward on one set, where
the backward finds part of x still cached; informational.)

Order of one run: an untimed pre-warm (the same forward + backward launches for --prewarm-ms, so that
the GPU has reached its steady clocks and every buffer has been touched before anything is timed),
W warm-up steps, then the loop of K steps timed --reps times in a row, each repetition bracketed by
a stream synchronisation on both sides.

One JSON line is printed:
  value         tokens/s of the median repetition of the K timed steps (wall clock); ms_per_step_min
                and ms_per_step_reps give the fastest repetition and all of them
  roofline      the dominant kernel (the fused backward): algorithmic bytes per launch divided by its
                median duration over at least 50 launches, measured with HIP events recorded on the
                launch stream (median_us, min_us and the mean avg_us are all printed)
  roofline_fwd  the same for the forward kernel (informational)
  back_to_back_us  span of 30 consecutive launches of one pass divided by 30 (informational: an event
                record ends a kernel with a cache write-back that consecutive launches overlap)
  cpu_baseline  the reference path (per-sequence torch conv1d + autograd, oracle/dwconv_ref.py) timed
                on this box's host cores on a bounded sample of the same workload
"""
from __future__ import annotations

import argparse
import ctypes
import json
import os
import statistics
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBPS = 8000.0   # MI355X HBM3E
VALU_PEAK_TFLOPS = 157.3  # MI355X fp32 vector ALU (256 CUs x 4 SIMDs x 32 FMA lanes x 2 flop x 2.4 GHz)

# HBM bytes per launch measured with rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE on this benchmark and
# scaled by what the same counters read for nplm_dwconv_debug_copy of known size (see
# profiles/bench_cfg3_hbm_traffic.md and profiles/bench_cfg2_cfg4_cfg5_hbm_traffic.md): keyed by
# (workload name, kernel[, variant]). Counters cannot be read from inside this process, so a workload or variant
# without an entry (configuration 1, --residual, other widths) reports traffic = null and says why.
MEASURED_TRAFFIC = {
    ("cfg2_bf16_fwd_T32768_C1024_K7", "forward"): 136261404,                       # 1.015 x algorithmic
    ("cfg3_bf16_fwdbwd_T131072_C1024_K7", "forward"): 544057555,                   # 1.013 x
    ("cfg3_bf16_fwdbwd_T131072_C1024_K7", "backward"): 816871634,                  # 1.014 x
    ("cfg4_bf16_fwdbwd_T131072_C2048_K31_lognormal", "forward"): 1075682217,       # 1.002 x
    ("cfg4_bf16_fwdbwd_T131072_C2048_K31_lognormal", "backward"): 1619868128,      # 1.005 x
    ("cfg5_bf16_fwdbwd_T65536_C1024_K7_boundary_stress", "forward"): 272198320,    # 1.014 x
    ("cfg5_bf16_fwdbwd_T65536_C1024_K7_boundary_stress", "backward"): 410672393,   # 1.020 x
    # --gated --config 4 (profiles/bench_cfg4_gated_hbm_traffic.md)
    ("cfg4_bf16_fwdbwd_T131072_C2048_K31_lognormal", "forward", "gated"): 1637482695,    # 1.016 x
    ("cfg4_bf16_fwdbwd_T131072_C2048_K31_lognormal", "backward", "gated"): 2693567122,   # 1.003 x
    # --ln and --fp32 --ln (profiles/bench_cfg3_layernorm_fused_hbm_traffic.md); the backward figure is the fused kernel's alone
    ("cfg3_bf16_fwdbwd_T131072_C1024_K7", "forward", "ln"): 551613338,             # 1.027 x
    ("cfg3_bf16_fwdbwd_T131072_C1024_K7", "backward", "ln"): 830305929,            # 1.031 x
    ("cfg3_fp32_fwdbwd_T131072_C1024_K7", "forward", "ln"): 1092201837,            # 1.017 x
    ("cfg3_fp32_fwdbwd_T131072_C1024_K7", "backward", "ln"): 1641691951,           # 1.019 x
}
MIN_EVENT_LAUNCHES = 50   # per-kernel event samples, whatever --steps says


def _hip():
    lib = ctypes.CDLL("libamdhip64.so")
    lib.hipEventCreate.argtypes = [ctypes.POINTER(ctypes.c_void_p)]
    lib.hipEventRecord.argtypes = [ctypes.c_void_p, ctypes.c_void_p]
    lib.hipEventSynchronize.argtypes = [ctypes.c_void_p]
    lib.hipEventElapsedTime.argtypes = [ctypes.POINTER(ctypes.c_float), ctypes.c_void_p, ctypes.c_void_p]
    return lib


class HipEvents:
    """Raw HIP events on a given stream (torch.cuda.Event only sees torch's current stream)."""

    def __init__(self, n):
        self.hip = _hip()
        self.ev = []
        for _ in range(n):
            e = ctypes.c_void_p()
            rc = self.hip.hipEventCreate(ctypes.byref(e))
            if rc:
                raise RuntimeError(f"hipEventCreate failed: {rc}")
            self.ev.append(e)

    @staticmethod
    def record_raw(event, stream):
        rc = _hip().hipEventRecord(ctypes.c_void_p(event), ctypes.c_void_p(stream))
        if rc:
            raise RuntimeError(f"hipEventRecord failed: {rc}")

    def record(self, i, stream):
        rc = self.hip.hipEventRecord(self.ev[i], ctypes.c_void_p(stream))
        if rc:
            raise RuntimeError(f"hipEventRecord failed: {rc}")

    def elapsed_us(self, i, j):
        self.hip.hipEventSynchronize(self.ev[j])
        ms = ctypes.c_float()
        rc = self.hip.hipEventElapsedTime(ctypes.byref(ms), self.ev[i], self.ev[j])
        if rc:
            raise RuntimeError(f"hipEventElapsedTime failed: {rc}")
        return ms.value * 1e3


def cpu_baseline(wl, sample_tokens):
    """Reference path on the host cores, on the first sequences of the workload (about sample_tokens rows)."""
    import torch
    from oracle.dwconv_ref import ref_dwconv_varlen_grads

    cu = wl.cu_seqlens
    n = int(torch.searchsorted(cu, torch.tensor(sample_tokens, dtype=cu.dtype)).item())
    n = max(1, min(n, cu.numel() - 1))
    Ts = int(cu[n])
    x, dy, cus = wl.x[:Ts], wl.dy[:Ts], cu[: n + 1]
    # every host core the box gives this process (BASELINE: torch.set_num_threads(os.cpu_count())); both counts are reported
    threads_default = torch.get_num_threads()
    host_cores = os.cpu_count() or threads_default
    torch.set_num_threads(host_cores)
    threads = torch.get_num_threads()

    def run(dtype):
        ref_dwconv_varlen_grads(x, cus, wl.weight, wl.bias, dy, dtype)      # warm-up
        ts = []
        for _ in range(3):
            t = time.perf_counter()
            ref_dwconv_varlen_grads(x, cus, wl.weight, wl.bias, dy, dtype)
            ts.append(time.perf_counter() - t)
        return statistics.median(ts)

    t_bf16 = run(wl.dtype)
    t_f32 = run(torch.float32)
    return {
        "value": Ts / t_bf16, "unit": "tokens/s", "cores": threads, "kind": "port",
        "sample": f"first {n} sequences ({Ts} of {wl.T} tokens) of {wl.name}, fwd+bwd via per-sequence "
                  f"torch conv1d + autograd in {str(wl.dtype).replace('torch.', '')}, median of 3 after 1 warm-up",
        "seconds_per_pass": t_bf16,
        "fp32_tokens_per_s": Ts / t_f32,
        "os_cpu_count": host_cores, "torch_default_threads": threads_default,
    }


def device_loop_baseline(d, passes, reps=3):
    """The path the reference would take for this op on the same GPU without this library: one
    ``torch.nn.functional.conv1d(groups=C)`` per sequence over the packed rows, concatenated, gradients by autograd
    (whatever convolution library torch dispatches to). Informational: a whole step per repetition, wall clock."""
    import torch
    import torch.nn.functional as F

    cu = d.cu_seqlens.cpu().tolist()
    C, K = d.weight.shape
    x = d.x.detach().clone().requires_grad_(passes == "fwd+bwd")
    w = d.weight.detach().clone().requires_grad_(passes == "fwd+bwd")
    b = d.bias.detach().clone().requires_grad_(passes == "fwd+bwd")

    def step():
        x.grad = w.grad = b.grad = None
        ys = [F.conv1d(x[s:e].t().unsqueeze(0), w.to(x.dtype).unsqueeze(1), b.to(x.dtype), padding=K // 2, groups=C)[0].t()
              for s, e in zip(cu[:-1], cu[1:]) if e > s]
        y = torch.cat(ys, 0)
        if passes == "fwd+bwd":
            y.backward(d.dy)

    t0 = time.perf_counter()
    step()                      # first pass: the convolution library picks (and may build) its kernels per length
    torch.cuda.synchronize()
    first_s = time.perf_counter() - t0
    ts = []
    for _ in range(reps):
        torch.cuda.synchronize()
        t = time.perf_counter()
        step()
        torch.cuda.synchronize()
        ts.append(time.perf_counter() - t)
    med = statistics.median(ts)
    return {"ms_per_step": med * 1e3, "tokens_per_s": d.x.shape[0] / med, "first_step_s": first_s, "reps": reps,
            "sequences": len(cu) - 1, "what": f"per-sequence torch conv1d loop + autograd on the GPU, {passes}"}


def autograd_step_times(npa, d, xs, gs, args, nset):
    """The step as a model pays for it: ``VarlenDWConv1d`` forward + ``y.backward(dy)`` (the call site a conv module
    has in the reference: src/nanoplm/pretraining/models/modern_bert/modeling.py:421-439, backward driven by
    src/nanoplm/pretraining/pure_pipeline.py:739-742), on the same rotating tensor sets and in the same order as the
    raw loop: the backward of a step runs two forwards after its own forward. One block = nset steps
    (F0 F1 F2 B0 F3 B1 B2 B3). Timed eagerly (host work of the wrappers included; it overlaps the GPU as long as it is
    shorter) and replayed from one captured HIP graph of a block. Gradients are set to None before every block, as
    ``optimizer.zero_grad(set_to_none=True)`` does, so nothing is accumulated into an old gradient."""
    import torch

    wl_dtype = d.x.dtype
    T, C = d.x.shape
    K = d.weight.shape[1]
    dev = d.x.device
    conv = npa.VarlenDWConv1d(C, K, residual=bool(args.residual or args.ln)).to(dev).to(d.weight.dtype)
    with torch.no_grad():
        conv.weight.copy_(d.weight)
        conv.bias.copy_(d.bias)
    norm = None
    if args.ln:
        norm = torch.nn.LayerNorm(C, eps=1e-5).to(dev).to(d.weight.dtype)
    cu = d.cu_seqlens
    leaves = [x.detach().requires_grad_(True) for x in xs]
    params = list(conv.parameters()) + (list(norm.parameters()) if norm is not None else [])

    def forward(j):
        if args.ln:
            return conv.forward_prenorm(leaves[j], cu, norm)
        if args.gated:
            return conv.forward_gated(leaves[j], cu)
        return conv(leaves[j], cu)

    def block():
        for t in leaves + params:
            t.grad = None
        ys = []
        for j in range(nset):
            ys.append(forward(j))
            if j >= 2:
                ys[j - 2].backward(gs[j - 2])
        for j in range(nset - 2, nset):
            ys[j].backward(gs[j])

    def timed(fn, nblocks, reps):
        out = []
        for _ in range(reps):
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            for _ in range(nblocks):
                fn()
            torch.cuda.synchronize()
            out.append((time.perf_counter() - t0) * 1e3 / (nblocks * nset))
        return out

    nblocks = max(1, (args.steps + nset - 1) // nset)
    for _ in range(max(2, args.warmup // nset)):
        block()
    eager = timed(block, nblocks, max(1, args.reps))
    res = {"ms_per_step_autograd": statistics.median(eager), "ms_per_step_autograd_min": min(eager),
           "autograd_what": f"VarlenDWConv1d{'.forward_prenorm' if args.ln else '.forward_gated' if args.gated else ''} + "
                            f"y.backward(dy), blocks of {nset} steps on the rotating sets, eager"}
    try:
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            for _ in range(3):
                block()
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        for t in leaves + params:
            t.grad = None
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            block()
        graph.replay()
        torch.cuda.synchronize()
        rep = timed(graph.replay, nblocks, max(1, args.reps))
        res["ms_per_step_autograd_graph"] = statistics.median(rep)
        res["ms_per_step_autograd_graph_min"] = min(rep)
        del graph
    except Exception as exc:      # a capture that fails must not lose the rest of the line
        res["ms_per_step_autograd_graph"] = None
        res["autograd_graph_error"] = f"{type(exc).__name__}: {exc}"[:300]
    for t in leaves + params:
        t.grad = None
    return res


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--config", type=int, default=3, choices=[1, 2, 3, 4, 5])
    ap.add_argument("--residual", action="store_true",
                    help="fused residual variant: y = x + conv(x), dx = dy + conv^T(dy) (same traffic)")
    ap.add_argument("--gated", action="store_true",
                    help="gated variant: input z = [x_proj | gate] of width 2C, conv over x_proj * silu(gate) "
                         "(informational; per-kernel figures then bracket backward + finalize together)")
    ap.add_argument("--ln", action="store_true",
                    help="LayerNorm-fused variant: y = x + conv(layer_norm(x)) in one forward kernel; the backward (conv "
                         "backward over the re-normalised x, then the LayerNorm input gradient) is bracketed as one "
                         "figure like --gated (configurations whose rows fit 2 KiB: 2, 3, 5)")
    ap.add_argument("--fp32", action="store_true",
                    help="the configuration's tensors in fp32: what a conv on the residual stream receives under "
                         "torch.autocast with fp32 parameters (informational; twice the activation bytes)")
    ap.add_argument("--channels", type=int, default=None,
                    help="the configuration's lengths and kernel size at another width, e.g. 768, the reference's default "
                         "hidden size (informational)")
    ap.add_argument("--reps", type=int, default=15, help="repetitions of the timed K-step loop (median reported)")
    ap.add_argument("--prewarm-ms", type=float, default=6000.0,
                    help="untimed steps run for this long before the warm-up steps")
    ap.add_argument("--device-loop", action="store_true",
                    help="also time the per-sequence torch conv1d loop (the reference's way to this op) on the GPU; "
                         "its first pass can take minutes while the convolution library prepares kernels per length")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-autograd", action="store_true",
                    help="skip the module-level figures (ms_per_step_autograd, ms_per_step_autograd_graph)")
    ap.add_argument("--cpu-sample-tokens", type=int, default=65536)
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py measures one GPU: this build has no multi-GPU path (run with --gpus 1); "
                 "the op shards at sequence boundaries or along channels without communication.")

    import torch
    import nanoplm_amd as npa
    from nanoplm_amd import _lib
    from nanoplm_amd.workloads import make_workload

    if not torch.cuda.is_available():
        sys.exit("bench.py needs a ROCm GPU")
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    lib = _lib.load()

    wl = make_workload(args.config, with_dy=True)
    if args.channels and args.channels != wl.C:
        import dataclasses
        base_c = wl.C
        wl = make_workload(args.config, C=args.channels, with_dy=True)
        wl = dataclasses.replace(wl, name=wl.name.replace(f"_C{base_c}_", f"_C{args.channels}_"))
    if args.fp32 and wl.dtype != torch.float32:
        import dataclasses
        wl = dataclasses.replace(wl, name=wl.name.replace("bf16", "fp32"), dtype=torch.float32, x=wl.x.float(),
                                 weight=wl.weight.float(), bias=wl.bias.float(), dy=None if wl.dy is None else wl.dy.float())
    d = wl.to(dev)
    T, C, K, S = wl.T, wl.C, wl.K, wl.S
    fwd_bwd = wl.passes == "fwd+bwd"
    if args.ln and (args.gated or C * d.x.element_size() > 8192 or K > 9):
        sys.exit("--ln needs rows of at most 8 KiB and K <= 9 (configurations 2, 3, 5) and excludes --gated")
    NSET = 4
    BWD_SHIFT = 2          # the backward of step i uses set (i + BWD_SHIFT) % NSET
    if args.gated and not fwd_bwd:
        sys.exit("--gated needs a forward+backward configuration (3, 4 or 5)")
    xs = [d.x] + [torch.randn(T, C, device=dev).to(wl.dtype) for _ in range(NSET - 1)]
    if args.gated:       # z = [x_proj | gate]; dz has the same shape
        xs = [torch.randn(T, 2 * C, device=dev).to(wl.dtype) for _ in range(NSET)]
    gs = [d.dy] + [torch.randn(T, C, device=dev).to(wl.dtype) for _ in range(NSET - 1)]
    ys = [torch.empty_like(d.x) for _ in range(NSET)]
    dxs = [torch.empty_like(xs[0]) for _ in range(NSET)]
    dw = torch.empty((C, K), dtype=torch.float32, device=dev)
    db = torch.empty((C,), dtype=torch.float32, device=dev)
    act = _lib.BF16 if wl.dtype == torch.bfloat16 else _lib.F32
    ws_bytes = int((lib.nplm_dwconv_gated_bwd_workspace_bytes if args.gated else lib.nplm_dwconv_ln_bwd_workspace_bytes if args.ln
                    else lib.nplm_dwconv_bwd_workspace_bytes)(T, C, K, act))
    if args.gated and ws_bytes == 0:
        sys.exit("the fused gated kernels are not built for this configuration")
    ws = torch.empty((max(ws_bytes, 256),), dtype=torch.uint8, device=dev)
    stream = torch.cuda.current_stream().cuda_stream
    cu, w, b = d.cu_seqlens, d.weight, d.bias
    flags = _lib.RESIDUAL if (args.residual or args.ln) else 0
    if args.ln:
        ln_w = (1 + 0.1 * torch.randn(C, device=dev)).to(w.dtype)
        ln_b = (0.1 * torch.randn(C, device=dev)).to(w.dtype)
        stats = [torch.empty((T, 2), dtype=torch.float32, device=dev) for _ in range(NSET)]
        dln = torch.empty((2, C), dtype=torch.float32, device=dev)
    def fwd(i):
        j = i % NSET
        if args.ln:
            _lib.check(lib.nplm_dwconv_ln_fwd(xs[j].data_ptr(), cu.data_ptr(), ln_w.data_ptr(), ln_b.data_ptr(), 1e-5,
                                              w.data_ptr(), b.data_ptr(), ys[j].data_ptr(), stats[j].data_ptr(), T, C, K, S,
                                              act, act, flags, stream), "nplm_dwconv_ln_fwd")
            return
        if args.gated:
            _lib.check(lib.nplm_dwconv_gated_fwd(xs[j].data_ptr(), cu.data_ptr(), w.data_ptr(), b.data_ptr(),
                                                 ys[j].data_ptr(), T, C, K, S, act, act, flags, stream), "nplm_dwconv_gated_fwd")
            return
        _lib.check(lib.nplm_dwconv_fwd_ex(xs[j].data_ptr(), cu.data_ptr(), w.data_ptr(), b.data_ptr(),
                                          ys[j].data_ptr(), T, C, K, S, act, act, flags, stream), "nplm_dwconv_fwd_ex")

    def bwd(i, t=None, shift=BWD_SHIFT):
        j = (i + shift) % NSET
        args_ = (xs[j].data_ptr(), gs[j].data_ptr(), cu.data_ptr(), w.data_ptr(), dxs[j].data_ptr(), dw.data_ptr(),
                 db.data_ptr(), ws.data_ptr(), ws.numel(), T, C, K, S, act, act)
        if args.ln:
            rc = lib.nplm_dwconv_ln_bwd(xs[j].data_ptr(), gs[j].data_ptr(), cu.data_ptr(), stats[j].data_ptr(), ln_w.data_ptr(),
                                        ln_b.data_ptr(), w.data_ptr(), dxs[j].data_ptr(), dw.data_ptr(), db.data_ptr(),
                                        dln[0].data_ptr(), dln[1].data_ptr(), ws.data_ptr(), ws.numel(), T, C, K, S, act, act,
                                        flags, stream)
            if t is not None and t.mid_event:      # no mid-call event on this entry point: mark the end instead
                HipEvents.record_raw(t.mid_event, stream)
        elif args.gated:
            rc = lib.nplm_dwconv_gated_bwd(*args_, flags, stream)
            if t is not None and t.mid_event:      # no mid-call event on this entry point: mark the end instead
                HipEvents.record_raw(t.mid_event, stream)
        else:
            rc = lib.nplm_dwconv_bwd_ex(*args_, flags, stream) if t is None else lib.nplm_dwconv_bwd_tuned(*args_, stream, t)
        _lib.check(rc, "nplm_dwconv_bwd")

    def step(i):
        fwd(i)
        if fwd_bwd:
            bwd(i)

    # ---- untimed pre-warm: the same launches until the clocks have settled --------------------------
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    prewarm_steps = 0
    while (time.perf_counter() - t0) * 1e3 < args.prewarm_ms:
        for i in range(50):
            step(prewarm_steps + i)
        prewarm_steps += 50
        torch.cuda.synchronize()
    prewarm_ms = (time.perf_counter() - t0) * 1e3

    # ---- whole-step throughput: W warm-up steps, then K timed steps, repeated ------------------------
    for i in range(args.warmup):
        step(i)
    rep_ms = []
    for _ in range(max(1, args.reps)):
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for i in range(args.steps):
            step(i)
        torch.cuda.synchronize()
        rep_ms.append((time.perf_counter() - t0) * 1e3 / args.steps)
    ms_per_step = statistics.median(rep_ms)
    tokens_per_s = T / (ms_per_step / 1e3)
    same_ms = []
    if fwd_bwd:      # informational: forward and backward of a step on the same tensors
        for _ in range(5):
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            for i in range(args.steps):
                fwd(i)
                bwd(i, shift=0)
            torch.cuda.synchronize()
            same_ms.append((time.perf_counter() - t0) * 1e3 / args.steps)

    # ---- the same step through the module and autograd (the surface a model calls), eagerly and from a HIP graph ----
    autograd = None
    if fwd_bwd and not args.no_autograd:
        autograd = autograd_step_times(npa, d, xs, gs, args, NSET)

    # ---- per-kernel durations with HIP events on the launch stream ---------------------------------
    # The same step sequence as the timed loop above, launched back to back without host
    # synchronisation, with one pair of events per step around the kernel being measured; one pass
    # over the steps per kernel, so that a step never carries more than two event records (every
    # record ends the kernel before it with a cache write-back, which the kernel after it pays for).
    n_ev = min(max(args.steps, MIN_EVENT_LAUNCHES), 100)
    evs = [HipEvents(4) for _ in range(n_ev)]

    def event_pass(which):
        for i in range(n_ev):
            e = evs[i]
            if which == "fwd":
                e.record(0, stream)
                fwd(i)
                e.record(1, stream)
                if fwd_bwd:
                    bwd(i)
            elif which == "bwd":        # event 2 is recorded inside the call, between the fused kernel and finalize
                fwd(i)
                e.record(1, stream)
                t = _lib.Tuning(flags=flags)
                t.mid_event = e.ev[2]
                bwd(i, t)
            else:                       # finalize: from the library's mid-call event to the end of the call
                fwd(i)
                t = _lib.Tuning(flags=flags)
                t.mid_event = e.ev[2]
                bwd(i, t)
                e.record(3, stream)
        torch.cuda.synchronize()

    event_pass("fwd")
    fwd_us = [e.elapsed_us(0, 1) for e in evs]
    bwd_us, fin_us = [], []
    if fwd_bwd:
        event_pass("bwd")
        bwd_us = [e.elapsed_us(1, 2) for e in evs]
        event_pass("fin")
        fin_us = [e.elapsed_us(2, 3) for e in evs]
    ev = evs[0]
    fwd_bytes = wl.algorithmic_bytes("fwd")
    bwd_bytes = wl.algorithmic_bytes("bwd") if fwd_bwd else 0
    if args.gated:       # z is read once more per pass and dz is twice as wide as dx
        tce = T * C * d.x.element_size()
        fwd_bytes += tce
        bwd_bytes += 2 * tce
    step_bytes = fwd_bytes + bwd_bytes

    def roof(nbytes, samples_us, kernel):
        """Roofline of one kernel against both ceilings it can meet: HBM on its algorithmic bytes and the fp32 vector
        ALU on its algorithmic flops (forward 2KTC, backward 4KTC + TC; no MFMA in this op). `bound` names the ceiling
        that takes longer at its peak, i.e. the one that binds; achieved/peak/unit/frac are that ceiling's, and both
        ceilings' figures are kept under "hbm" and "valu"."""
        med = statistics.median(samples_us)
        gbps = nbytes / med / 1e3
        flops = wl.algorithmic_flops("fwd" if kernel == "forward" else "bwd")
        tflops = flops / med / 1e6
        traffic = (MEASURED_TRAFFIC.get((wl.name, kernel, "ln")) if args.ln else
                   MEASURED_TRAFFIC.get((wl.name, kernel, "gated")) if args.gated else
                   None if args.residual else MEASURED_TRAFFIC.get((wl.name, kernel)))
        hbm = {"achieved": gbps, "peak": HBM_PEAK_GBPS, "unit": "GB/s", "frac": gbps / HBM_PEAK_GBPS,
               "algorithmic_bytes": nbytes, "us_at_peak": nbytes / HBM_PEAK_GBPS / 1e3}
        valu = {"achieved": tflops, "peak": VALU_PEAK_TFLOPS, "unit": "TFLOP/s", "frac": tflops / VALU_PEAK_TFLOPS,
                "algorithmic_flops": flops, "us_at_peak": flops / VALU_PEAK_TFLOPS / 1e6}
        valu_bound = valu["us_at_peak"] >= hbm["us_at_peak"] and not (args.gated or args.ln)
        top = valu if valu_bound else hbm
        r = {"bound": "valu" if valu_bound else "hbm", "achieved": top["achieved"], "peak": top["peak"], "unit": top["unit"],
             "frac": top["frac"], "flops_per_byte": flops / nbytes, "ridge_flops_per_byte": VALU_PEAK_TFLOPS * 1e3 / HBM_PEAK_GBPS,
             "hbm": hbm, "valu": valu,
             "traffic": traffic, "kernel": kernel, "median_us": med, "min_us": min(samples_us),
             "avg_us": statistics.fmean(samples_us), "launches": len(samples_us), "algorithmic_bytes": nbytes}
        if traffic is None:
            r["traffic_note"] = ("no rocprofv3 FETCH_SIZE/WRITE_SIZE measurement is kept for this workload/variant; "
                                 "the counters are read by the profiler, not by this process")
        return r

    out = {
        "metric": "varlen dwconv fwd+bwd tokens/s and HBM GB/s (% peak), T=131072 C=1024 K=7 bf16"
                  if args.config == 3 and not args.gated and not args.ln and not args.fp32 and not args.channels else
                  f"varlen {'gated ' if args.gated else 'layernorm-fused ' if args.ln else ''}dwconv "
                  f"{wl.passes} tokens/s ({wl.name})",
        "value": tokens_per_s, "unit": "tokens/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": ms_per_step, "ms_per_step_min": min(rep_ms), "reps": len(rep_ms),
        "ms_per_step_reps": [round(v, 5) for v in rep_ms], "prewarm_ms": prewarm_ms, "prewarm_steps": prewarm_steps,
        "ms_per_step_same_tensors": statistics.median(same_ms) if same_ms else None,
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": str(wl.dtype).replace("torch.", "").replace("bfloat16", "bf16").replace("float32", "f32"),
        "data": "synthetic (seeded: lengths, x, weight, bias, dy drawn on the CPU, see nanoplm_amd/workloads.py)",
        "config": {"workload": wl.name, "T": T, "C": C, "K": K, "S": S, "passes": wl.passes,
                   "rotating_sets": NSET, "backward_set_shift": BWD_SHIFT if fwd_bwd else None, "residual": bool(args.residual or args.ln), "gated": bool(args.gated), "layernorm": bool(args.ln)},
        "step_algorithmic_bytes": step_bytes,
        "step_GBps": step_bytes / (ms_per_step * 1e-3) / 1e9,
        "step_frac_of_hbm_peak": step_bytes / (ms_per_step * 1e-3) / 1e9 / HBM_PEAK_GBPS,
        "step_algorithmic_flops": wl.algorithmic_flops(),
        "step_TFLOPps": wl.algorithmic_flops() / (ms_per_step * 1e-3) / 1e12,
        "step_frac_of_valu_peak": wl.algorithmic_flops() / (ms_per_step * 1e-3) / 1e12 / VALU_PEAK_TFLOPS,
    }
    if autograd:
        out.update(autograd)
        out["autograd_over_raw"] = autograd["ms_per_step_autograd"] / ms_per_step
        out["autograd_graph_over_raw"] = (autograd["ms_per_step_autograd_graph"] / ms_per_step
                                          if autograd.get("ms_per_step_autograd_graph") else None)
    if fwd_bwd:
        out["roofline"] = roof(bwd_bytes, bwd_us, "backward")
        out["roofline_fwd"] = roof(fwd_bytes, fwd_us, "forward")
        out["finalize_median_us"] = statistics.median(fin_us)
    else:
        out["roofline"] = roof(fwd_bytes, fwd_us, "forward")

    # ---- the same launches back to back (no event between them): each figure is the span of N launches
    # divided by N, so it holds a launch gap but no end-of-kernel cache write-back forced by an event --
    def span_us(fn, n=30):
        for i in range(3):
            fn(i)
        ev.record(0, stream)
        for i in range(n):
            fn(i)
        ev.record(1, stream)
        torch.cuda.synchronize()
        return ev.elapsed_us(0, 1) / n

    out["back_to_back_us"] = {"forward": span_us(fwd)}
    if fwd_bwd:
        out["back_to_back_us"]["backward_plus_finalize"] = span_us(bwd)

    # ---- what a plain copy reaches on this box (context for the roofline fraction) ----------------
    cp_us = []
    for i in range(20):
        ev.record(0, stream)
        _lib.check(lib.nplm_dwconv_debug_copy(xs[i % NSET].data_ptr(), ys[i % NSET].data_ptr(),
                                              T * C * d.x.element_size(), stream), "nplm_dwconv_debug_copy")
        ev.record(1, stream)
        torch.cuda.synchronize()
        cp_us.append(ev.elapsed_us(0, 1))
    out["plain_copy_GBps"] = 2 * T * C * d.x.element_size() / statistics.median(cp_us[2:]) / 1e3

    if args.device_loop and not (args.gated or args.ln):
        out["reference_loop_on_gpu"] = device_loop_baseline(d, wl.passes)
    if not args.no_cpu_baseline:
        out["cpu_baseline"] = cpu_baseline(wl, args.cpu_sample_tokens)
    print(json.dumps(out))


if __name__ == "__main__":
    main()
