#!/usr/bin/env python3
"""Benchmark of the streaming-attention hot path on one MI355X.

A step is one forward + backward of the operator through its public API on one batch of
synthetic inputs already resident in HBM.  The headline workload is
B=4, H=16, T=16384, D=128, bf16, chunk 256, 8 back chunks, lens ~ U{T/2..T}.

Prints one JSON line:
  value      effective TFLOP/s = 14*D*H*P / step time, P = unmasked (query, key) pairs
             (value_block_granular counts whole chunk x chunk blocks that hold any allowed pair)
  roofline   the dominant kernel (longest average launch) timed on its own with HIP events on the
             launch stream.  The bound is chosen per workload from the step's arithmetic intensity
             (algorithmic flop / algorithmic HBM bytes against the machine balance): matrix-pipe
             bound workloads report TFLOP/s against the MFMA peak of their element type, HBM-bound
             ones GB/s against 8 TB/s.  `traffic` (HBM bytes per launch) comes from rocprofv3
             counter runs of this script, quoted from the committed summaries under profiles/.
  measured_ceilings  what a bare MFMA stream (constant and random bf16 operands) and a plain copy
             reach on this GPU in this run (libsa_probe.so), beside the published peaks
  cpu_baseline  the CPU oracle forward+backward in fp32 on the host cores, on a bounded sample
             of the same workload (one batch element, all heads), and the reference's dense-mask
             SDPA formulation on the reference's CPU-sized configuration
"""
from __future__ import annotations

import argparse
import json
import math
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.join(ROOT, "kernels_amd"))
sys.path.insert(0, ROOT)

PEAK_BF16_TFLOPS = 2500.0   # MI355X dense bf16 / fp16 MFMA, published
PEAK_F32_TFLOPS = 157.3     # MI355X dense fp32 MFMA, published
PEAK_HBM_GBS = 8000.0       # MI355X HBM3E, published

WORKLOADS = {
    # name: (B, H, T, D, dtype, C, R, lens mode, q/k/v scale)
    "cpu_ref_fp32": (2, 4, 512, 64, "float32", 64, 2, "uniform_256_512", 1.0),
    "bf16_T4096_D64": (8, 16, 4096, 64, "bfloat16", 128, 4, "full", None),
    "headline_bf16_T16384_D128": (4, 16, 16384, 128, "bfloat16", 256, 8, "uniform_half_full", 1.0),
    "ragged_fp16_T2048_D128": (16, 8, 2048, 128, "float16", 64, 1, "loguniform_64_T", 1.0),
    "long_bf16_T65536_D128": (1, 32, 65536, 128, "bfloat16", 512, 16, "full", 1.0),
    # the largest shapes of the reference's own benchmark grid (benchmark/benchmark_streaming_attention.py:43-111), for profiling
    "refgrid_fp16_T3000_D64_C10": (128, 12, 3000, 64, "float16", 10, 9, "full", 1.0),
    "refgrid_fp16_T3000_D64_C32": (128, 12, 3000, 64, "float16", 32, 2, "full", 1.0),
}
DEFAULT = "headline_bf16_T16384_D128"


def unmasked_pairs(T, C, R, lens_list):
    """Allowed (query, key) pairs per head, summed over the batch (closed form per chunk)."""
    total = 0
    for L in lens_list:
        L = min(int(L), T)
        c = 0
        while c * C < L:
            rows = min((c + 1) * C, L) - c * C
            keys = min((c + 1) * C, L) - max(0, c - R) * C
            total += rows * keys
            c += 1
    return total


def unmasked_block_pairs(T, C, R, lens_list):
    """Pairs in chunk x chunk blocks that hold at least one allowed pair (the figure a
    block-skipping kernel cannot go below), per head, summed over the batch."""
    total = 0
    for L in lens_list:
        L = min(int(L), T)
        n = -(-L // C)                      # chunks that hold a valid position
        for c in range(n):
            total += C * C * (min(c, R) + 1)
    return total


def make_inputs(name, device, zeros=False):
    import torch

    B, H, T, D, dtype_name, C, R, lens_mode, qkv_scale = WORKLOADS[name]
    dtype = getattr(torch, dtype_name)
    g = torch.Generator().manual_seed(20)
    if lens_mode == "full":
        lens = None
        lens_list = [T] * B
    elif lens_mode == "uniform_half_full":
        lens = torch.randint(T // 2, T + 1, (B,), generator=g, dtype=torch.int32)
    elif lens_mode == "uniform_256_512":
        lens = torch.randint(256, 513, (B,), generator=g, dtype=torch.int32)
    elif lens_mode == "loguniform_64_T":
        u = torch.rand(B, generator=g, dtype=torch.float64)
        lens = torch.exp(math.log(64.0) + u * (math.log(T) - math.log(64.0))).round().to(torch.int32)
    else:
        raise ValueError(lens_mode)
    if lens is not None:
        lens_list = lens.tolist()
    dg = torch.Generator(device=device).manual_seed(20)
    scale = D ** -0.5 if qkv_scale is None else qkv_scale
    q, k, v = [(torch.randn(B, H, T, D, generator=dg, device=device, dtype=torch.float32) * scale).to(dtype)
               for _ in range(3)]
    d_o = torch.randn(B, H, T, D, generator=dg, device=device, dtype=torch.float32).to(dtype)
    if zeros:   # same launches on operands that never toggle a multiplier input
        q, k, v, d_o = (torch.zeros_like(t) for t in (q, k, v, d_o))
    return dict(q=q, k=k, v=v, d_o=d_o, lens=lens.to(device) if lens is not None else None,
                lens_list=lens_list, B=B, H=H, T=T, D=D, C=C, R=R, dtype=dtype_name)


def time_kernels(w, iters, only=None):
    """Average duration of each kernel (or of those named in `only`) launched on its own through the C ABI, in ms."""
    import torch
    from streaming_attention import _lib

    lib = _lib.load()
    q, k, v, d_o, lens = w["q"], w["k"], w["v"], w["d_o"], w["lens"]
    B, H, T, D, C, R = w["B"], w["H"], w["T"], w["D"], w["C"], w["R"]
    dt = _lib.DTYPE_IDS["torch." + w["dtype"]]
    scale = D ** -0.5
    o = torch.empty_like(q)
    lse = torch.empty(B, H, T, dtype=torch.float32, device=q.device)
    delta = torch.empty_like(lse)
    dq, dk, dv = torch.empty_like(q), torch.empty_like(q), torch.empty_like(q)
    lp, ls = (lens.data_ptr(), lens.stride(0)) if lens is not None else (None, 0)
    st = torch.cuda.current_stream().cuda_stream
    s4 = _lib.strides4

    def fwd():
        return lib.sa_forward(q.data_ptr(), k.data_ptr(), v.data_ptr(), lp, ls, o.data_ptr(), lse.data_ptr(),
                              s4(q), s4(k), s4(v), B, H, T, D, C, R, scale, dt, st)

    def dlt():
        return lib.sa_bwd_delta(o.data_ptr(), d_o.data_ptr(), delta.data_ptr(), s4(o), s4(d_o), B, H, T, D, dt, st)

    def dqf():
        return lib.sa_bwd_dq(q.data_ptr(), k.data_ptr(), v.data_ptr(), lp, ls, d_o.data_ptr(), lse.data_ptr(),
                             delta.data_ptr(), dq.data_ptr(), s4(q), s4(k), s4(v), s4(d_o),
                             B, H, T, D, C, R, scale, dt, st)

    def dkv():
        return lib.sa_bwd_dkdv(q.data_ptr(), k.data_ptr(), v.data_ptr(), lp, ls, d_o.data_ptr(), lse.data_ptr(),
                               delta.data_ptr(), dk.data_ptr(), dv.data_ptr(), s4(q), s4(k), s4(v), s4(d_o),
                               B, H, T, D, C, R, scale, dt, st)

    out = {}
    for name, fn in (("fwd", fwd), ("delta", dlt), ("dq", dqf), ("dkdv", dkv)):
        if only is not None and name not in only:
            continue
        _lib.check(fn(), name)
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()   # events and launches share torch's current stream `st`
        for _ in range(iters):
            fn()
        e1.record()
        e1.synchronize()
        out[name] = e0.elapsed_time(e1) / iters
    return out


def cpu_baseline(w, name, budget_s=12.0):
    """The CPU restatement of the algorithm timed on the host cores, on a bounded sample of the
    benchmarked workload: batch element 0 (all heads) through the chunk-by-chunk fp32 oracle,
    forward + backward, repeated for about `budget_s` seconds.  The reference's own dense-mask
    SDPA formulation cannot hold a T x T mask at these sizes; it is timed beside it on the
    reference's CPU-sized configuration (B=2, H=4, T=512, D=64)."""
    import torch
    from oracle import sa_oracle

    H, T, D, C, R = w["H"], w["T"], w["D"], w["C"], w["R"]
    q, k, v, d_o = (w[n][:1].detach().float().cpu() for n in ("q", "k", "v", "d_o"))
    lens = w["lens"][:1].cpu() if w["lens"] is not None else None
    L0 = w["lens_list"][0]
    flops = 14.0 * D * H * unmasked_pairs(T, C, R, [L0])
    sa_oracle.windowed(q, k, v, lens, C, R, d_out=d_o)          # warm-up
    n, t0 = 0, time.perf_counter()
    while n < 2 or time.perf_counter() - t0 < budget_s:
        sa_oracle.windowed(q, k, v, lens, C, R, d_out=d_o)
        n += 1
    dt = (time.perf_counter() - t0) / n

    Bs, Hs, Ts, Ds, _, Cs, Rs, _, _ = WORKLOADS["cpu_ref_fp32"]
    g = torch.Generator().manual_seed(20)
    qs, ks, vs, gs = [torch.randn(Bs, Hs, Ts, Ds, generator=g) for _ in range(4)]
    ls = torch.randint(256, 513, (Bs,), generator=g, dtype=torch.int32)
    fl_s = 14.0 * Ds * Hs * unmasked_pairs(Ts, Cs, Rs, ls.tolist())
    for _ in range(3):
        sa_oracle.sdpa_fwd_bwd(qs, ks, vs, ls, Cs, Rs, gs)
    m, t1 = 0, time.perf_counter()
    while m < 10 or time.perf_counter() - t1 < 2.0:
        sa_oracle.sdpa_fwd_bwd(qs, ks, vs, ls, Cs, Rs, gs)
        m += 1
    dt_s = (time.perf_counter() - t1) / m
    return {
        "value": flops / dt / 1e12, "unit": "TFLOP/s", "cores": torch.get_num_threads(), "kind": "port",
        "sample": f"batch element 0 of {name} (len {L0}, H={H}, T={T}, D={D}, chunk={C}, back={R}) in fp32 "
                  f"through the chunk-by-chunk oracle, {n} fwd+bwd iterations of {dt:.2f} s each; "
                  f"host has {os.cpu_count()} logical cpus",
        "dense_mask_sdpa_config1": {
            "value": fl_s / dt_s / 1e12, "unit": "TFLOP/s",
            "sample": f"B={Bs} H={Hs} T={Ts} D={Ds} fp32 chunk={Cs} back={Rs} lens~U[256,512], {m} fwd+bwd "
                      f"iterations of the dense-mask SDPA oracle, {dt_s * 1e3:.2f} ms each"},
    }


# HBM bytes per launch from rocprofv3 FETCH_SIZE / WRITE_SIZE (separate --pmc runs of this script, scaled by
# what the same counters read for the 1 GiB copy of --calibrate-copy).  Counter runs cannot be made from
# inside a timed run, so the figures of the committed counter runs are quoted: profiles/hbm_traffic.json
# holds them (the per-workload summaries under profiles/ show the same numbers with their commands;
# tests/test_boundary.py checks that the two agree).  A workload or kernel without a counter run reports null.
TRAFFIC_FILE = os.path.join(ROOT, "profiles", "hbm_traffic.json")
TRAFFIC_SOURCE = "quoted from profiles/hbm_traffic.json (rocprofv3 FETCH_SIZE/WRITE_SIZE runs; not measured in this run)"


def hbm_bytes_per_launch():
    """{workload: {kernel: HBM bytes per launch}} from the committed counter runs ({} if the file is missing)."""
    try:
        with open(TRAFFIC_FILE) as f:
            return json.load(f)["hbm_bytes_per_launch"]
    except (OSError, KeyError, ValueError):
        return {}


def measured_ceilings():
    """Bare MFMA stream and plain copy on this GPU, through libsa_probe.so (bench support code)."""
    import ctypes

    path = os.path.join(ROOT, "kernels_amd", "streaming_attention", "libsa_probe.so")
    if not os.path.exists(path):
        return {"error": f"{path} not built (make -C kernels_amd/csrc)"}
    lib = ctypes.CDLL(path)
    lib.sa_probe_mfma_bf16.argtypes = [ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.POINTER(ctypes.c_double)]
    lib.sa_probe_copy.argtypes = [ctypes.c_size_t, ctypes.c_int, ctypes.POINTER(ctypes.c_double)]
    out = {}
    v = ctypes.c_double()
    for name, rnd in (("bf16_mfma_constant_operands_tflops", 0), ("bf16_mfma_random_operands_tflops", 1)):
        rc = lib.sa_probe_mfma_bf16(rnd, 4000, 2, ctypes.byref(v))
        out[name] = v.value if rc == 0 else f"hip error {rc}"
    rc = lib.sa_probe_copy(1 << 30, 5, ctypes.byref(v))
    out["copy_read_plus_write_gbs"] = v.value if rc == 0 else f"hip error {rc}"
    out["note"] = ("v_mfma_f32_32x32x16_bf16 only, 2 waves per SIMD, 8 accumulator chains per wave; copy of 1 GiB "
                   "with 16-byte accesses, bytes read + bytes written")
    return out


def reference_sweep(device, iters=20):
    """The reference's own benchmark grid (benchmark/benchmark_streaming_attention.py:113-292):
    fp16, B=128, H=12, D=64, (context, back) in {(10, 9), (32, 2)}, six lengths from 257 to 3000,
    lens = None; forward under inference mode and forward+backward, HIP-event means, and the
    reference's flop count 4*T*W*H*D*B with W = context*(1+back) (x3.5 for forward+backward), which
    counts the full band, not the unmasked pairs."""
    import torch
    from streaming_attention import streaming_attention

    B, H, D = 128, 12, 64
    rows = []
    for C, R in ((10, 9), (32, 2)):
        for T in [int(round(257 + i * (3000 - 257) / 5)) for i in range(6)]:
            g = torch.Generator(device=device).manual_seed(20)
            q, k, v = [torch.randn(B, H, T, D, generator=g, device=device, dtype=torch.float16) for _ in range(3)]
            d_o = torch.randn(B, H, T, D, generator=g, device=device, dtype=torch.float16)

            def timed(fn):
                for _ in range(3):
                    fn()
                torch.cuda.synchronize()
                e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                e0.record()
                for _ in range(iters):
                    fn()
                e1.record()
                e1.synchronize()
                return e0.elapsed_time(e1) / iters

            def fwd():
                with torch.inference_mode():
                    streaming_attention(q, k, v, None, C, R)

            qg, kg, vg = (t.clone().requires_grad_() for t in (q, k, v))

            def fwd_bwd():
                qg.grad = kg.grad = vg.grad = None
                streaming_attention(qg, kg, vg, None, C, R).backward(d_o)

            t_f, t_fb = timed(fwd), timed(fwd_bwd)
            band = 4.0 * T * C * (1 + R) * H * D * B
            rows.append({"context_size": C, "back_contexts": R, "T": T, "fwd_ms": t_f, "fwd_bwd_ms": t_fb,
                         "fwd_band_tflops": band / (t_f * 1e-3) / 1e12,
                         "fwd_bwd_band_tflops": 3.5 * band / (t_fb * 1e-3) / 1e12,
                         "unmasked_pairs_per_head": unmasked_pairs(T, C, R, [T] * B)})
            del q, k, v, d_o, qg, kg, vg
    return rows


def tune_sweep(device, iters=10):
    """Every variant of the 16-bit forward, dQ and dK/dV kernels (include/streaming_attention.h,
    sa_tune_override) timed on a grid of head dimension x context_size x back_contexts, B=4, H=16,
    T=16384 (K and V together exceed the 256 MiB last-level cache), lens drawn uniformly from [T/2, T]
    as in the headline workload.  The first cell is timed twice and its first reading dropped (the
    first launches after start-up run at lower clocks).  The fastest variant per
    (D, context_size class, window class) is what the library's launch-configuration table holds
    (kernels_amd/csrc/gen_tune_table.py turns this output into the table); the reference reaches its
    choice by autotuning at run time (src/streaming_attention/kernel.py:1154-1193)."""
    import torch
    from streaming_attention import _lib

    lib = _lib.load()
    B, H, T = 4, 16, 16384
    names = {"fwd": ["narrow", "pipelined"], "dq": ["narrow", "pipelined"], "dkdv": ["blockskip", "pipelined", "split"]}
    rows = []
    try:
        for dtype_name in ("bfloat16", "float16"):
            for D in (64, 128):
                for C in (16, 32, 64, 128, 256, 512, 1024):
                    seen = set()
                    for window in (128, 512, 2048, 8192):   # one per window class of the table
                        R = max(0, window // C - 1)
                        if R in seen or (dtype_name == "float16" and window != 2048):
                            continue   # same problem again / the second type only confirms the first
                        seen.add(R)
                        g = torch.Generator(device=device).manual_seed(20)
                        dt = getattr(torch, dtype_name)
                        q, k, v, d_o = [torch.randn(B, H, T, D, generator=g, device=device, dtype=torch.float32).to(dt)
                                        for _ in range(4)]
                        lens = torch.randint(T // 2, T + 1, (B,), generator=torch.Generator().manual_seed(20),
                                             dtype=torch.int32).to(device)
                        w = dict(q=q, k=k, v=v, d_o=d_o, lens=lens, B=B, H=H, T=T, D=D, C=C, R=R, dtype=dtype_name)
                        if not rows:
                            time_kernels(w, iters)   # warm-up, discarded
                        row = {"dtype": dtype_name, "D": D, "context_size": C, "back_contexts": R,
                               "table": {kn: names[kn][lib.sa_launch_choice(D, C, R, ki)]
                                         for ki, kn in enumerate(("fwd", "dq", "dkdv"))}}
                        for ki, kn in enumerate(("fwd", "dq", "dkdv")):
                            for vi, vn in enumerate(names[kn]):
                                if vn == "pipelined" and D != 128:
                                    continue
                                _lib.check(lib.sa_tune_override(ki, vi), "sa_tune_override")
                                row[f"{kn}_{vn}_ms"] = time_kernels(w, iters)[kn]
                            _lib.check(lib.sa_tune_override(ki, -1), "sa_tune_override")
                        for kn in names:
                            cand = {vn: row[f"{kn}_{vn}_ms"] for vn in names[kn] if f"{kn}_{vn}_ms" in row}
                            row[f"{kn}_best"] = min(cand, key=cand.get)
                        rows.append(row)
                        del q, k, v, d_o
    finally:
        for ki in range(3):
            lib.sa_tune_override(ki, -1)
    return rows



def path_sweep(device, iters=10):
    """Per-kernel times of every (dtype, head dimension) family the library serves, on one shape
    (B=4, H=16, T=4096, context_size=128, back_contexts=4, lens=None): the 16-bit D in {64, 128, 256}
    kernels next to the first-generation kernels that serve float32 and D in {16, 32}
    (the reference covers the same range from one tuned kernel, src/streaming_attention/kernel.py:196-203,
    1288-1290).  Rates are executed flop (S and dP are computed by both backward kernels) and
    algorithmic HBM bytes."""
    import torch

    B, H, T, C, R = 4, 16, 4096, 128, 4
    P = unmasked_pairs(T, C, R, [T] * B)
    rows = []
    for dtype_name in ("float32", "float16", "bfloat16"):
        for D in (16, 32, 64, 128, 256):
            dt = getattr(torch, dtype_name)
            g = torch.Generator(device=device).manual_seed(20)
            q, k, v, d_o = [(torch.randn(B, H, T, D, generator=g, device=device, dtype=torch.float32) * D ** -0.25).to(dt)
                            for _ in range(4)]
            w = dict(q=q, k=k, v=v, d_o=d_o, lens=None, B=B, H=H, T=T, D=D, C=C, R=R, dtype=dtype_name)
            kt = time_kernels(w, iters)
            es = 4 if dtype_name == "float32" else 2
            tensor, stat = float(B * H * T) * D * es, 4.0 * B * H * T
            fl = {"fwd": 4.0 * D * H * P, "dq": 6.0 * D * H * P, "dkdv": 8.0 * D * H * P}
            by = {"fwd": 4 * tensor + stat, "delta": 2 * tensor + stat, "dq": 5 * tensor + 2 * stat,
                  "dkdv": 6 * tensor + 2 * stat}
            rows.append({"dtype": dtype_name, "D": D, "kernel_ms": kt,
                         "kernel_tflops": {n: fl[n] / (kt[n] * 1e-3) / 1e12 for n in fl},
                         "kernel_gbs": {n: by[n] / (kt[n] * 1e-3) / 1e9 for n in by},
                         "fwd_bwd_effective_tflops": 14.0 * D * H * P / (sum(kt.values()) * 1e-3) / 1e12})
            del q, k, v, d_o
    return rows



VARIANT_NAMES = {"fwd": ["narrow", "pipelined"], "dq": ["narrow", "pipelined"], "dkdv": ["blockskip", "pipelined", "split"]}


def measure_workload(name, dev, steps, warmup, kernel_iters, zeros=False, compiled=False):
    """One workload: `steps` forward+backward steps through the public API between two synchronisations
    (ms_per_step, value), the same step bracketed by events for the median (at least 50 of them), each
    kernel on its own through the C ABI, and the roofline entry of the slowest kernel."""
    import torch
    from streaming_attention import _lib, compiled_wrapper, streaming_attention

    w = make_inputs(name, dev, zeros=zeros)
    B, H, T, D, C, R = w["B"], w["H"], w["T"], w["D"], w["C"], w["R"]
    P = unmasked_pairs(T, C, R, w["lens_list"])
    flops_step = 14.0 * D * H * P
    q, k, v = (w[n].requires_grad_() for n in ("q", "k", "v"))

    def step():
        q.grad = k.grad = v.grad = None
        out = streaming_attention(q, k, v, w["lens"], C, R)
        out.backward(w["d_o"])

    for _ in range(warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        step()
    torch.cuda.synchronize()
    ms_per_step = (time.perf_counter() - t0) * 1e3 / steps
    value = flops_step / (ms_per_step * 1e-3) / 1e12

    # the same steps once more, each bracketed by events on the stream they run on, for the median
    n_med = max(steps, 50)
    evs = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(n_med)]
    for e0, e1 in evs:
        e0.record()
        step()
        e1.record()
    torch.cuda.synchronize()
    per_step = sorted(e0.elapsed_time(e1) for e0, e1 in evs)
    median_ms = per_step[len(per_step) // 2] if len(per_step) % 2 else \
        0.5 * (per_step[len(per_step) // 2 - 1] + per_step[len(per_step) // 2])

    # the same step captured once into a HIP graph and replayed: what a caller pays who takes the Python and
    # dispatcher work out of the loop (the library records nothing but its kernels into the graph)
    graph_ms = None
    try:
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            for _ in range(3):
                step()
        torch.cuda.current_stream().wait_stream(side)
        graph = torch.cuda.CUDAGraph()
        q.grad = k.grad = v.grad = None
        with torch.cuda.graph(graph):
            out = streaming_attention(q, k, v, w["lens"], C, R)
            out.backward(w["d_o"])
        for _ in range(warmup):
            graph.replay()
        torch.cuda.synchronize()
        t2 = time.perf_counter()
        for _ in range(steps):
            graph.replay()
        torch.cuda.synchronize()
        graph_ms = (time.perf_counter() - t2) * 1e3 / steps
        del graph
    except Exception as e:      # reported, never fatal for the headline figures
        print(f"graph replay of {name} not measured: {e!r}", file=sys.stderr)

    compiled_ms = None
    if compiled:
        # the same step through the torch.compile'd wrapper that the reference puts around the op
        with compiled_wrapper():
            for _ in range(warmup):
                step()
            torch.cuda.synchronize()
            t1 = time.perf_counter()
            for _ in range(steps):
                step()
            torch.cuda.synchronize()
            compiled_ms = (time.perf_counter() - t1) * 1e3 / steps

    kt = time_kernels(w, kernel_iters)
    lib = _lib.load()
    variants = {kn: (VARIANT_NAMES[kn][lib.sa_launch_choice(D, C, R, ki)] if w["dtype"] != "float32" and D >= 64
                     else "first generation")
                for ki, kn in enumerate(("fwd", "dq", "dkdv"))}
    # GEMMs each kernel performs per unmasked pair: fwd S,PV; dq S,dP,dQ; dkdv S,dP,dV,dK
    kernel_flops = {"fwd": 4.0 * D * H * P, "dq": 6.0 * D * H * P, "dkdv": 8.0 * D * H * P}
    es = 4 if w["dtype"] == "float32" else 2
    N = B * H * T
    tensor = float(N) * D * es
    # Algorithmic HBM bytes per launch: every operand read once, every result written once.  Positions
    # t >= lens[b] of the inputs are never read, the outputs are written in full (zeros there); delta
    # reads all rows of O and dO.
    valid = sum(min(int(L), T) for L in w["lens_list"]) / float(B * T)
    rd, rows = tensor * valid, 4.0 * N
    kernel_bytes = {"fwd": 3.0 * rd + tensor + rows, "delta": 2.0 * tensor + rows,
                    "dq": 4.0 * rd + 2.0 * rows * valid + tensor, "dkdv": 4.0 * rd + 2.0 * rows * valid + 2.0 * tensor}
    # per step every tensor once: forward reads q, k, v and writes O; backward reads q, k, v, O, dO and
    # writes dQ, dK, dV; lse and delta are written and read once each
    step_bytes = 8.0 * rd + 4.0 * tensor + 4.0 * rows
    peak_tflops = PEAK_F32_TFLOPS if w["dtype"] == "float32" else PEAK_BF16_TFLOPS
    balance = peak_tflops * 1e12 / (PEAK_HBM_GBS * 1e9)            # flop per byte at which the two roofs meet
    intensity = flops_step / step_bytes
    bound = "mfma" if intensity >= balance else "hbm"
    dom = max(kernel_flops, key=lambda n: kt[n])
    traffic = hbm_bytes_per_launch().get(name, {}).get(dom)
    if bound == "mfma":
        achieved = kernel_flops[dom] / (kt[dom] * 1e-3) / 1e12
        roofline = {"kernel": dom, "bound": "mfma", "achieved": achieved, "peak": peak_tflops, "unit": "TFLOP/s",
                    "frac": achieved / peak_tflops}
    else:
        achieved = kernel_bytes[dom] / (kt[dom] * 1e-3) / 1e9
        roofline = {"kernel": dom, "bound": "hbm", "achieved": achieved, "peak": PEAK_HBM_GBS, "unit": "GB/s",
                    "frac": achieved / PEAK_HBM_GBS}
    roofline.update({"traffic": traffic, "traffic_source": TRAFFIC_SOURCE if traffic is not None else None,
                     "algorithmic_bytes": kernel_bytes[dom], "algorithmic_flops": kernel_flops[dom],
                     "arithmetic_intensity_flop_per_byte": intensity, "machine_balance_flop_per_byte": balance})
    q.grad = k.grad = v.grad = None
    return {"inputs": w, "pairs": P, "flops_step": flops_step, "step_bytes": step_bytes, "ms_per_step": ms_per_step,
            "value": value, "median_ms": median_ms, "median_steps": n_med, "compiled_wrapper_ms_per_step": compiled_ms,
            "graph_replay_ms_per_step": graph_ms, "kernel_ms": kt, "kernel_variants": variants,
            "kernel_tflops": {n: kernel_flops[n] / (kt[n] * 1e-3) / 1e12 for n in kernel_flops},
            "kernel_gbs": {n: kernel_bytes[n] / (kt[n] * 1e-3) / 1e9 for n in kernel_bytes}, "roofline": roofline}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=100)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--workload", default=DEFAULT, choices=sorted(WORKLOADS))
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-ceilings", action="store_true", help="skip the MFMA / copy ceiling measurement")
    ap.add_argument("--no-other-workloads", action="store_true",
                    help="with the default workload: do not time the other GPU configurations after it")
    ap.add_argument("--kernel-iters", type=int, default=10)
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="only run a 1 GiB device-to-device copy (known traffic) for scaling HBM counters")
    ap.add_argument("--zero-inputs", action="store_true",
                    help="all-zero q, k, v, dO: the same kernels and launch shapes without data-dependent "
                         "switching power (a diagnostic; the result line is marked and is not the metric)")
    ap.add_argument("--path-sweep", action="store_true",
                    help="time the kernels of every (dtype, head dimension) family on one shape and print the rows as JSON")
    ap.add_argument("--tune-sweep", action="store_true",
                    help="time every kernel variant on a (D, context_size, window) grid and print the rows as JSON")
    ap.add_argument("--reference-sweep", action="store_true",
                    help="time the grid of the reference's own benchmark script instead of a workload")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build runs on one GPU only (no collectives, no sharding); use --gpus 1")

    import torch

    assert torch.cuda.is_available(), "bench.py needs a GPU"
    dev = torch.device("cuda:0")
    if args.calibrate_copy:
        src = torch.ones(1 << 28, dtype=torch.float32, device=dev)   # 1 GiB read + 1 GiB written per copy
        dst = torch.empty_like(src)
        for _ in range(3):
            dst.copy_(src)
        torch.cuda.synchronize()
        print(json.dumps({"calibration": "3 copies of 1 GiB (2^28 fp32): 1048576 KiB read and written each"}))
        return
    if args.reference_sweep:
        print(json.dumps({"sweep": "reference benchmark grid, fp16 B=128 H=12 D=64", "n_gpus": 1,
                          "rows": reference_sweep(dev)}))
        return
    if args.path_sweep:
        print(json.dumps({"sweep": "dtype x head dimension, B=4 H=16 T=4096 context_size=128 back_contexts=4", "n_gpus": 1,
                          "rows": path_sweep(dev)}))
        return
    if args.tune_sweep:
        print(json.dumps({"sweep": "kernel variants, B=4 H=16 T=16384, lens ~ U[T/2, T]", "n_gpus": 1,
                          "rows": tune_sweep(dev)}))
        return
    m = measure_workload(args.workload, dev, args.steps, args.warmup, args.kernel_iters, zeros=args.zero_inputs,
                         compiled=True)
    w, kt = m["inputs"], m["kernel_ms"]
    B, H, T, D, C, R = w["B"], w["H"], w["T"], w["D"], w["C"], w["R"]
    P_blocks = unmasked_block_pairs(T, C, R, w["lens_list"])
    result = {
        "metric": "effective TFLOP/s fwd+bwd (unmasked blocks) at 1 GPU; % of bf16 MFMA peak",
        "value": m["value"], "unit": "TFLOP/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": m["ms_per_step"], "median_ms": m["median_ms"], "median_steps": m["median_steps"],
        "compiled_wrapper_ms_per_step": m["compiled_wrapper_ms_per_step"],
        "graph_replay_ms_per_step": m["graph_replay_ms_per_step"],
        "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None,
        "dtype": {"bfloat16": "bf16", "float16": "f16", "float32": "f32"}[w["dtype"]],
        "data": "synthetic, all zeros (diagnostic run)" if args.zero_inputs else "synthetic",
        "config": {"workload": args.workload, "B": B, "H": H, "T": T, "D": D, "context_size": C,
                   "back_contexts": R, "lens": w["lens_list"], "unmasked_pairs_per_head": m["pairs"],
                   "flops_per_step": m["flops_step"], "algorithmic_bytes_per_step": m["step_bytes"]},
        "pct_of_bf16_mfma_peak": 100.0 * m["value"] / PEAK_BF16_TFLOPS,
        "value_block_granular": 14.0 * D * H * P_blocks / (m["ms_per_step"] * 1e-3) / 1e12,
        "step_hbm_gbs": m["step_bytes"] / (m["ms_per_step"] * 1e-3) / 1e9,
        "peaks_used": {"bf16_mfma_tflops": PEAK_BF16_TFLOPS, "f32_mfma_tflops": PEAK_F32_TFLOPS,
                       "hbm_gbs": PEAK_HBM_GBS},
        "kernel_ms": kt,
        "kernel_variants": m["kernel_variants"],
        "kernel_ms_note": ("each kernel launched on its own through the C ABI; for this dtype and head dimension the step's "
                           "backward forms delta inside the dQ kernel and does not launch the delta pass timed here"
                           if w["dtype"] != "float32" and D >= 64 else "each kernel launched on its own through the C ABI"),
        "kernel_tflops": m["kernel_tflops"],
        "kernel_gbs": m["kernel_gbs"],
        "roofline": m["roofline"],
    }
    del w, m
    torch.cuda.empty_cache()
    if args.workload == DEFAULT and not args.zero_inputs and not args.no_other_workloads:
        # the other GPU configurations of the baseline, timed after the headline (which stays `value`):
        # fewer steps where a step is long, more where the host would otherwise dominate
        others = {}
        for name, steps in (("bf16_T4096_D64", 200), ("ragged_fp16_T2048_D128", 300), ("long_bf16_T65536_D128", 10)):
            o = measure_workload(name, dev, steps, 5, args.kernel_iters if "long" not in name else 3)
            dom = o["roofline"]["kernel"]
            others[name] = {
                "ms_per_step": o["ms_per_step"], "median_ms": o["median_ms"], "steps": steps,
                "graph_replay_ms_per_step": o["graph_replay_ms_per_step"],
                "effective_tflops": o["value"], "pct_of_bf16_mfma_peak": 100.0 * o["value"] / PEAK_BF16_TFLOPS,
                "step_hbm_gbs": o["step_bytes"] / (o["ms_per_step"] * 1e-3) / 1e9,
                "kernel_ms": o["kernel_ms"], "kernel_variants": o["kernel_variants"], "dominant_kernel": dom,
                "roofline": {k: o["roofline"][k] for k in ("kernel", "bound", "achieved", "peak", "unit", "frac", "traffic")},
                "config": {"B": o["inputs"]["B"], "H": o["inputs"]["H"], "T": o["inputs"]["T"], "D": o["inputs"]["D"],
                           "dtype": o["inputs"]["dtype"], "context_size": o["inputs"]["C"],
                           "back_contexts": o["inputs"]["R"], "lens": o["inputs"]["lens_list"]},
            }
            del o
            torch.cuda.empty_cache()
        result["other_workloads"] = others
    if not args.no_ceilings:
        result["measured_ceilings"] = measured_ceilings()
    if not args.no_cpu_baseline:
        result["cpu_baseline"] = cpu_baseline(make_inputs(args.workload, dev, zeros=args.zero_inputs), args.workload)
    print(json.dumps(result))


if __name__ == "__main__":
    main()
