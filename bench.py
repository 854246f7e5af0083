#!/usr/bin/env python3
"""Benchmark of the GPT-2 fp32 forward pass on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

A step is one gpt2_forward over one batch of synthetic token ids (GPT-2 124M,
B=8, T=1024, seeded random weights; ids already resident in HBM).  Prints ONE
JSON line on stdout: whole-forward tokens/s, the roofline position of the
dominant kernel (the FP32-MFMA GEMM) measured with HIP events around every
launch of a second, identical set of K steps, the per-launch breakdown, the
stand-alone kernel figures at the BASELINE shapes, and the CPU oracle timed on
the host cores on a bounded sample of the same workload.
"""
from __future__ import annotations

import argparse
import importlib
import json
import math
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

PEAK_FP32_MFMA_TFLOPS = 157.3   # MI355X dense FP32 matrix
PEAK_HBM_GBS = 8000.0           # MI355X HBM3E


def dominant_traffic_bytes():
    """HBM bytes per launch of the dominant GEMM kernel (mean of the qkv, attproj and fcproj
    shapes at M = 8192, the two projections with the residual add in their epilogue as the
    driver runs them), as recorded in profiles/kernels_baseline_shapes_pmc.txt from two
    `rocprofv3 --pmc` runs of `bench.py --pmc-probe`: FETCH_SIZE (scaled x2.0: a 256 MiB copy
    reads 131 101 KiB on that counter) and WRITE_SIZE (scale 1.0).  None if the summary is
    missing or does not hold the line."""
    import re
    try:
        text = open(os.path.join(ROOT, "profiles", "kernels_baseline_shapes_pmc.txt")).read()
    except OSError:
        return None
    m = re.search(r"dominant kernel of bench\.py.*?:\s*(\d+) bytes of HBM-side traffic per launch", text)
    return int(m.group(1)) if m else None


def log(*a):
    print(*a, file=sys.stderr, flush=True)


def init_params_on_device(model, syn, cfg, seed):
    """GPT-2 initialisation written straight into the device parameter buffer."""
    import torch
    flat = model.params_tensor()
    g = torch.Generator(device="cuda")
    g.manual_seed(seed)
    L = cfg["num_layers"]
    off = 0
    for name, shape in syn.param_shapes(**cfg).items():
        n = int(math.prod(shape))
        seg = flat[off:off + n]
        if name in ("wte", "qkvw", "fcw"):
            seg.normal_(0.0, 0.02, generator=g)
        elif name in ("attprojw", "fcprojw"):
            seg.normal_(0.0, 0.02 / math.sqrt(2 * L), generator=g)
        elif name == "wpe":
            seg.normal_(0.0, 0.01, generator=g)
        elif name in ("ln1w", "ln2w", "lnfw"):
            seg.fill_(1.0)
        else:
            seg.zero_()
        off += n
    assert off == flat.numel()


def forward_flops(cfg, B, T):
    C, L, V, NH = cfg["channels"], cfg["num_layers"], cfg["vocab_size"], cfg["num_heads"]
    M = B * T
    mm = {"matmul_qkv": 2 * M * C * 3 * C, "matmul_attproj": 2 * M * C * C,
          "matmul_fc_gelu": 2 * M * C * 4 * C, "matmul_fcproj": 2 * M * 4 * C * C}
    per_forward = {k: v * L for k, v in mm.items()}
    per_forward["matmul_lmhead"] = 2 * M * C * V
    per_forward["attention"] = L * 4 * B * NH * (C // NH) * T * (T + 1) // 2
    return per_forward


def forward_bytes(cfg, B, T, sums_in_matmul):
    """Algorithmic bytes per forward of the memory-bound launches.  Where the driver forms the
    residual sums in the projections' epilogues, the normalisation that follows reads the sum
    and writes its normalisation (8 bytes per entry) instead of reading two rows and writing
    two (16)."""
    C, L = cfg["channels"], cfg["num_layers"]
    M = B * T
    return {"encoder": 4 * M + 8 * M * C + 4 * T * C,
            "layernorm": 8 * M * C + 8 * C,
            "fused_residual_layernorm": 2 * L * ((8 if sums_in_matmul else 16) * M * C + 8 * C)}


LAUNCHES = {"encoder": 1, "layernorm": 1, "matmul_lmhead": 1}


def time_launch(g2, fn, iters=30, warmup=10, groups=5):
    """HIP events on the null stream around `iters` back-to-back launches, `groups` times; the
    median group's average per launch (one group in five catches a clock or host hiccup)."""
    import torch
    for i in range(warmup):
        fn(i)
    torch.cuda.synchronize()
    per_launch = []
    n = warmup
    for _ in range(groups):
        t = g2.Timer()
        t.start()
        for i in range(iters):
            fn(n + i)
        per_launch.append(t.stop_ms() / iters)
        n += iters
    return sorted(per_launch)[len(per_launch) // 2]


def marker_overhead_ms(g2):
    """What one event between two launches adds to the interval it closes.  The profiled
    forward records an event after every launch and charges a launch the time between its two
    events: the launch-to-launch time PLUS the event marker's own trip through the command
    processor.  The library measures it the way it records those events, on launches that do
    next to nothing (median of five runs of 64 launches)."""
    L = g2.lib()
    us = sorted(L.gpt2hip_profile_marker_overhead_us(64) for _ in range(5))
    if us[0] < 0:
        raise RuntimeError("gpt2hip_profile_marker_overhead_us failed")
    return us[2] / 1e3


def library_ms(g2, fn, **kw):
    """The same-node vendor-library column of a stand-alone row: `fn` (a torch call, rocBLAS /
    hipBLASLt / MIOpen / AOTriton underneath) timed with the same events on the same buffers.
    Outside the product and outside every timed region of the forward pass; a routine that
    is not available on the box is reported as such."""
    import torch
    try:
        with torch.no_grad():
            fn(0)
            torch.cuda.synchronize()
            return {"library_ms": time_launch(g2, fn, **kw)}
    except Exception as e:  # noqa: BLE001 - whatever the library raises is the row's note
        torch.cuda.synchronize()
        return {"library_ms": None, "library_note": f"unavailable here: {type(e).__name__}: {str(e)[:160]}"}


def standalone(g2):
    """Per-kernel figures at the BASELINE shapes (configs 1-3).

    Launches go straight through the ctypes entry points with pre-extracted device
    pointers: the Python wrappers' argument checks cost more host time than the
    shortest of these kernels runs, which would otherwise be what gets timed.
    """
    import torch
    import torch.nn.functional as F
    torch.backends.cuda.matmul.allow_tf32 = False   # the library column is fp32 like ours
    L = g2.lib()
    out = []
    M = 8192
    dev = "cuda"
    P = lambda t: t.data_ptr()
    # fused residual+layernorm: rotate over 8 buffer sets (> 256 MiB Infinity Cache)
    for C in (768, 1024):
        sets = 8
        x = torch.randn(sets, M, C, device=dev)
        r = torch.randn(sets, M, C, device=dev)
        o = torch.empty(sets, M, C, device=dev)
        s = torch.empty(sets, M, C, device=dev)
        mean = torch.empty(M, device=dev)
        rstd = torch.empty(M, device=dev)
        w = torch.randn(C, device=dev) * 0.1 + 1
        b = torch.randn(C, device=dev) * 0.1
        args = [(P(s[k]), P(o[k]), P(mean), P(rstd), P(x[k]), P(r[k]), P(w), P(b), 8, 1024, C)
                for k in range(sets)]
        ms = time_launch(g2, lambda i: L.fused_residual_layernorm_forward(*args[i % sets]),
                         iters=96, warmup=16)
        nbytes = 16 * M * C + 8 * C + 8 * M
        gbs = nbytes / ms / 1e6
        row = {"kernel": "fused_residual_layernorm", "shape": f"N={M},C={C}", "ms": ms,
               "GB/s": gbs, "frac_hbm": gbs / PEAK_HBM_GBS,
               "note": f"rotating {sets} buffer sets, {sets * 4 * M * C * 4 >> 20} MiB"}

        def torch_ln(i, x=x, r=r, s=s, o=o, w=w, b=b, C=C, sets=sets):
            k = i % sets
            torch.add(x[k], r[k], out=s[k])
            o[k].copy_(F.layer_norm(s[k], (C,), w, b, 1e-5))
        row.update(library_ms(g2, torch_ln, iters=96, warmup=16))
        row["library"] = "torch.add + F.layer_norm (+ copy into the output buffer), fp32"
        out.append(row)
        del x, r, o, s
    # matmul at the GPT-2 124M linear shapes
    for (C, OC, bias) in ((768, 2304, True), (768, 768, True), (768, 3072, True), (3072, 768, True),
                          (768, 50257, False)):
        x = torch.randn(M, C, device=dev)
        w = torch.randn(OC, C, device=dev) * 0.02
        bb = torch.randn(OC, device=dev) * 0.02 if bias else None
        o = torch.empty(M, OC, device=dev)
        a = (P(o), P(x), P(w), P(bb) if bias else None, 8, 1024, C, OC)
        ms = time_launch(g2, lambda i: L.matmul_forward(*a), iters=10 if OC > 10000 else 40)
        tf = 2.0 * M * C * OC / ms / 1e9
        row = {"kernel": "matmul_forward", "shape": f"M={M},C={C},OC={OC}", "ms": ms,
               "TFLOP/s": tf, "frac_fp32_mfma": tf / PEAK_FP32_MFMA_TFLOPS}
        lib_fn = ((lambda i: torch.addmm(bb, x, w.t(), out=o)) if bias
                  else (lambda i: torch.mm(x, w.t(), out=o)))
        row.update(library_ms(g2, lib_fn, iters=10 if OC > 10000 else 40))
        row["library"] = ("torch.addmm(bias, x, w^T, out=)" if bias else "torch.mm(x, w^T, out=)") + \
            " fp32, TF32 off (rocBLAS / hipBLASLt underneath)"
        if row.get("library_ms"):
            row["library_frac_fp32_mfma"] = 2.0 * M * C * OC / row["library_ms"] / 1e9 / PEAK_FP32_MFMA_TFLOPS
        out.append(row)
        del x, w, o
    # K split between workgroups (a lent workspace) where a problem has too few tiles: the
    # 3072 -> 768 projection at B*T below the benchmark's
    ws = g2.matmul_forward_splitk_workspace()
    for Ms in (256, 1024, 3072):
        C, OC = 3072, 768
        x = torch.randn(Ms, C, device=dev)
        w = torch.randn(OC, C, device=dev) * 0.02
        bb = torch.randn(OC, device=dev) * 0.02
        o = torch.empty(Ms, OC, device=dev)
        a = (P(o), P(x), P(w), P(bb), 1, Ms, C, OC)
        a_ws = a + (0, P(ws), ws.numel())
        ms_plain = time_launch(g2, lambda i: L.matmul_forward(*a), iters=40)
        ms = time_launch(g2, lambda i: L.matmul_forward_splitk_status(*a_ws), iters=40)
        tf = 2.0 * Ms * C * OC / ms / 1e9
        plan = g2.matmul_forward_splitk_plan(1, Ms, C, OC, ws.numel())
        out.append({"kernel": "matmul_forward_splitk", "shape": f"M={Ms},C={C},OC={OC}", "ms": ms,
                    "TFLOP/s": tf, "frac_fp32_mfma": tf / PEAK_FP32_MFMA_TFLOPS,
                    "note": f"tile {plan[0]}x{plan[1]}, K split {plan[2]} ways; matmul_forward "
                            f"(no workspace): {ms_plain:.4f} ms"})
        del x, w, o
    # the two projections with the block's residual add in their epilogue, as the driver runs
    # them at this size (out = resid + product), beside the plain product of the same shape
    for (C, OC) in ((768, 768), (3072, 768)):
        x = torch.randn(M, C, device=dev)
        w = torch.randn(OC, C, device=dev) * 0.02
        bb = torch.randn(OC, device=dev) * 0.02
        r = torch.randn(M, OC, device=dev)
        o = torch.empty(M, OC, device=dev)
        a = (P(o), P(x), P(w), P(bb), P(r), 8, 1024, C, OC, P(ws), ws.numel())
        ms = time_launch(g2, lambda i: L.matmul_forward_residual_status(*a), iters=40)
        ms_plain = time_launch(g2, lambda i: L.matmul_forward(*a[:4], *a[5:9]), iters=40)
        tf = 2.0 * M * C * OC / ms / 1e9
        out.append({"kernel": "matmul_forward_residual", "shape": f"M={M},C={C},OC={OC}", "ms": ms,
                    "TFLOP/s": tf, "frac_fp32_mfma": tf / PEAK_FP32_MFMA_TFLOPS,
                    "note": f"matmul_forward of the same shape in the same loop: {ms_plain:.4f} ms; the "
                            "add saves the normalisation kernel behind it half its traffic "
                            "(layernorm_forward against fused_residual_layernorm below)"})
        del x, w, o, r
    # causal attention
    for (B, T, NH) in ((8, 1024, 12), (8, 256, 12), (8, 1024, 16), (8, 256, 16)):
        C = NH * 64
        qkv = torch.randn(B, T, 3 * C, device=dev)
        o = torch.empty(B, T, C, device=dev)
        a = (P(o), None, None, P(qkv), B, T, C, NH)
        ms = time_launch(g2, lambda i: L.attention_forward(*a), iters=40)
        tf = 4.0 * B * NH * 64 * T * (T + 1) / 2 / ms / 1e9
        row = {"kernel": "attention_forward", "shape": f"B={B},T={T},NH={NH},HS=64", "ms": ms,
               "TFLOP/s": tf, "frac_fp32_mfma": tf / PEAK_FP32_MFMA_TFLOPS}
        q5 = qkv.view(B, T, 3, NH, 64)
        qh, kh, vh = (q5[:, :, j].transpose(1, 2) for j in range(3))     # (B, NH, T, 64) views of packed qkv
        row.update(library_ms(g2, lambda i: F.scaled_dot_product_attention(qh, kh, vh, is_causal=True),
                              iters=20, warmup=3, groups=3))
        row["library"] = "torch scaled_dot_product_attention(is_causal=True) fp32 on views of the packed qkv"
        if row.get("library_ms"):
            row["library_frac_fp32_mfma"] = (4.0 * B * NH * 64 * T * (T + 1) / 2 / row["library_ms"] / 1e9
                                            / PEAK_FP32_MFMA_TFLOPS)
        out.append(row)
        del qkv, o, q5, qh, kh, vh
    # the other bandwidth kernels at the 124M B=8 T=1024 sizes, rotating buffers
    N = M * 3072
    a4 = torch.randn(4, N, device=dev)
    o4 = torch.empty(4, N, device=dev)
    args = [(P(o4[k]), P(a4[k]), N) for k in range(4)]
    ms = time_launch(g2, lambda i: L.gelu_forward(*args[i % 4]), iters=40)
    out.append({"kernel": "gelu_forward", "shape": f"N={N}", "ms": ms, "GB/s": 8 * N / ms / 1e6,
                "frac_hbm": 8 * N / ms / 1e6 / PEAK_HBM_GBS})
    N = M * 768
    args = [(P(o4[k]), P(a4[k]), P(a4[(k + 1) % 4]), N) for k in range(4)]
    ms = time_launch(g2, lambda i: L.residual_forward(*args[i % 4]), iters=96, warmup=16)
    out.append({"kernel": "residual_forward", "shape": f"N={N}", "ms": ms, "GB/s": 12 * N / ms / 1e6,
                "frac_hbm": 12 * N / ms / 1e6 / PEAK_HBM_GBS,
                "note": "operands 100 MiB apart in 4 rotating sets"})
    del a4, o4
    C = 768
    x = torch.randn(16, M, C, device=dev)
    o = torch.empty(16, M, C, device=dev)
    w = torch.ones(C, device=dev)
    b = torch.zeros(C, device=dev)
    args = [(P(o[k]), None, None, P(x[k]), P(w), P(b), 8, 1024, C) for k in range(16)]
    ms = time_launch(g2, lambda i: L.layernorm_forward(*args[i % 16]), iters=96, warmup=16)
    nb = 8 * M * C + 8 * C
    out.append({"kernel": "layernorm_forward", "shape": f"N={M},C={C}", "ms": ms,
                "GB/s": nb / ms / 1e6, "frac_hbm": nb / ms / 1e6 / PEAK_HBM_GBS,
                "note": "rotating 16 buffer sets, 768 MiB"})
    # encoder gather and argmax at the forward's sizes
    V = 50257
    wte = torch.randn(V, C, device=dev) * 0.02
    wpe = torch.randn(1024, C, device=dev) * 0.01
    ids = torch.randint(0, V, (8, 1024), dtype=torch.int32, device=dev)
    args = [(P(o[k]), P(ids), P(wte), P(wpe), 8, 1024, C) for k in range(16)]
    ms = time_launch(g2, lambda i: L.encoder_forward(*args[i % 16]), iters=96, warmup=16)
    nb = 4 * M + 8 * M * C + 4 * 1024 * C
    out.append({"kernel": "encoder_forward", "shape": f"B=8,T=1024,C={C}", "ms": ms,
                "GB/s": nb / ms / 1e6, "frac_hbm": nb / ms / 1e6 / PEAK_HBM_GBS})
    del x, o, wte
    logits = torch.randn(M, V, device=dev)
    am = torch.empty(M, dtype=torch.int32, device=dev)
    a = (P(am), P(logits), M, V)
    ms = time_launch(g2, lambda i: L.argmax_forward(*a), iters=10, warmup=3)
    nb = 4 * M * V + 4 * M
    out.append({"kernel": "argmax_forward", "shape": f"N={M},V={V}", "ms": ms,
                "GB/s": nb / ms / 1e6, "frac_hbm": nb / ms / 1e6 / PEAK_HBM_GBS,
                "note": "1.65 GB of logits: larger than the Infinity Cache"})
    # lm-head + argmax: two launches through the logits buffer against the fused launcher
    x = torch.randn(M, C, device=dev)
    wte = torch.randn(V, C, device=dev) * 0.02
    a_mm = (P(logits), P(x), P(wte), None, 8, 1024, C, V)
    def unfused(i):
        L.matmul_forward(*a_mm)
        L.argmax_forward(*a)
    ms_unfused = time_launch(g2, unfused, iters=8, warmup=2)
    need = L.matmul_forward_argmax_workspace(8, 1024, V)
    ws = torch.empty(need, dtype=torch.uint8, device=dev)
    a_f = (P(am), P(ws), need, P(x), P(wte), None, 8, 1024, C, V)
    ms_fused = time_launch(g2, lambda i: L.matmul_forward_argmax_status(*a_f), iters=8, warmup=2)
    tf = 2.0 * M * C * V / ms_fused / 1e9
    out.append({"kernel": "matmul_forward_argmax", "shape": f"M={M},C={C},OC={V}", "ms": ms_fused,
                "TFLOP/s": tf, "frac_fp32_mfma": tf / PEAK_FP32_MFMA_TFLOPS,
                "note": f"matmul_forward + argmax_forward through 1.65 GB of logits: {ms_unfused:.3f} ms"})
    return out


def pmc_probe(g2):
    """One launch of every kernel at its BASELINE shape plus a plain copy of known size,
    for `rocprofv3 --pmc` runs: the copy calibrates FETCH_SIZE / WRITE_SIZE."""
    import torch
    dev = "cuda"
    M = 8192
    src = torch.randn(64 << 20, device=dev)          # 256 MiB
    dst = torch.empty_like(src)
    for _ in range(2):
        dst.copy_(src)                                # plain copy: reads 256 MiB, writes 256 MiB
    for (C, OC) in ((768, 2304), (768, 768), (768, 3072), (3072, 768), (768, 50257)):
        x = torch.randn(M, C, device=dev)
        w = torch.randn(OC, C, device=dev) * 0.02
        o = torch.empty(M, OC, device=dev)
        for _ in range(2):
            g2.matmul_forward(o, x, w, None, 8, 1024, C, OC)
        del x, w, o
    for C in (768, 1024):
        x = torch.randn(M, C, device=dev)
        r = torch.randn(M, C, device=dev)
        o = torch.empty(M, C, device=dev)
        s2 = torch.empty(M, C, device=dev)
        w = torch.ones(C, device=dev)
        b = torch.zeros(C, device=dev)
        dst.copy_(src)                                # push the operands out of the caches
        g2.fused_residual_layernorm_forward(s2, o, None, None, x, r, w, b, 8, 1024, C)
    qkv = torch.randn(8, 1024, 3 * 768, device=dev)
    o = torch.empty(8, 1024, 768, device=dev)
    for _ in range(2):
        g2.attention_forward(o, None, None, qkv, 8, 1024, 768, 12)
    del qkv, o
    # the two projections as the driver runs them at this size (residual add in the epilogue),
    # and the normalisation of the sum that follows them
    for (C, OC) in ((768, 768), (3072, 768)):
        x = torch.randn(M, C, device=dev)
        w = torch.randn(OC, C, device=dev) * 0.02
        r = torch.randn(M, OC, device=dev)
        o = torch.empty(M, OC, device=dev)
        for _ in range(2):
            g2.matmul_forward_residual(o, x, w, None, r, 8, 1024, C, OC)
        del x, w, o, r
    x = torch.randn(M, 768, device=dev)
    o = torch.empty(M, 768, device=dev)
    dst.copy_(src)                                    # push the operands out of the caches
    g2.layernorm_forward(o, None, None, x, torch.ones(768, device=dev), torch.zeros(768, device=dev), 8, 1024, 768)
    torch.cuda.synchronize()
    print(json.dumps({"pmc_probe": "done", "copy_bytes_each_way": src.numel() * 4}))


def clock_probe(g2):
    """Shader clocks per K slab and sustained clock frequency inside the GEMM kernel,
    with zero and with N(0,1) operands (same instructions, different switching power)."""
    import numpy as np
    import torch
    M = 8192
    rows = []
    for (C, OC) in ((768, 2304), (768, 768), (768, 3072), (3072, 768), (768, 50257)):
        for data in ("zeros", "normal"):
            x = torch.zeros(M, C, device="cuda") if data == "zeros" else torch.randn(M, C, device="cuda")
            w = (torch.zeros(OC, C, device="cuda") if data == "zeros"
                 else torch.randn(OC, C, device="cuda") * 0.02)
            o = torch.empty(M, OC, device="cuda")
            for _ in range(10):                       # bring the chip to its sustained state
                g2.matmul_forward(o, x, w, None, 8, 1024, C, OC)
            p = g2.matmul_forward_probe(o, x, w, None, 8, 1024, C, OC).astype(np.float64)
            ns = (p[:, 1] - p[:, 0]) * 10.0
            clk = p[:, 3] - p[:, 2]
            nslab = C // 32
            waves_per_simd = 2                        # both wave layouts put 2 waves on a SIMD
            mfma_cycles = 64 * (128 * 192 // (32 * 32)) * 16 / 4   # per slab and SIMD: 6144
            rows.append({"shape": f"M={M},C={C},OC={OC}", "operands": data,
                         "workgroups": int(len(p)), "loop_us": float(ns.mean() / 1e3),
                         "shader_clocks_per_slab": float(clk.mean() / nslab),
                         "sustained_MHz": float(clk.sum() / ns.sum() * 1e3),
                         "mfma_cycles_per_slab_one_workgroup": mfma_cycles})
            log("  clock_probe", json.dumps(rows[-1]))
            del x, w, o
    print(json.dumps({"clock_probe": rows}))


def decode_bench(model, cfg, B, T0, steps):
    """Incremental inference: a prompt of T0 tokens per sequence, then `steps` single-token
    steps against the key/value cache, once with one launch per operation and once with the
    persistent decode-step kernel.  A step is bound by streaming the weights (and the cache
    rows read by attention) from HBM once: that is the roofline the GB/s figure is set against."""
    import torch
    V, C, L = cfg["vocab_size"], cfg["channels"], cfg["num_layers"]
    ids = torch.randint(0, V, (B, T0), dtype=torch.int32, device="cuda")
    nxt = torch.randint(0, V, (steps + 4, B), dtype=torch.int32, device="cuda")
    pos = T0 + steps / 2
    weight_bytes = 4 * (L * (12 * C * C + 13 * C) + V * C + 2 * C)
    cache_bytes = 2 * L * B * pos * C * 4
    out = {"decode": f"B={B}, prompt T0={T0}, {steps} steps", "bytes_per_step": weight_bytes + cache_bytes}
    for name, persistent in (("launch_per_operation", False), ("persistent_kernel", True)):
        model.decode_options(persistent=persistent)
        model.prefill(ids)
        for i in range(4):
            model.decode(nxt[i])
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        model.prefill(ids)
        torch.cuda.synchronize()
        out["prefill_ms"] = (time.perf_counter() - t0) * 1e3
        # three runs of `steps` steps from the same prompt, the median one reported: the first run
        # after the cache has been (re)allocated for another batch size is now and then much slower
        runs = []
        for _ in range(3):
            t0 = time.perf_counter()
            for i in range(steps):
                model.decode(nxt[4 + i])
            torch.cuda.synchronize()
            runs.append((time.perf_counter() - t0) / steps * 1e3)
            model.prefill(ids)
            torch.cuda.synchronize()
        ms = sorted(runs)[1]
        gbs = (weight_bytes + cache_bytes) / ms / 1e6
        out[name] = {"ms_per_step": ms, "tokens_per_s": B / ms * 1e3, "GB/s": gbs,
                     "frac_hbm": gbs / PEAK_HBM_GBS,
                     "finite": bool(torch.isfinite(model.step_logits()).all())}
    if model.decode_probe_size() == 0:
        out["persistent_kernel"]["note"] = ("the persistent kernel does not take this model or batch: "
                                            "both rows are one launch per operation")
    else:
        # one more step with the persistent kernel's clock probe: per phase kind, the mean time
        # a workgroup works and the mean time from its arrival to everybody's arrival
        clk = model.decode_probe(nxt[0]).cpu().numpy().astype("float64") * 10.0  # ns
        names = ("qkv", "attention", "attproj", "fc_gelu", "fcproj")
        done, passed = clk[:, 0, :], clk[:, 1, :]
        work = {n: [] for n in names}
        wait = {n: [] for n in names}
        for p in range(5 * L):
            if p:
                work[names[p % 5]].append(float((done[p] - passed[p - 1]).mean()))
            wait[names[p % 5]].append(float((passed[p] - done[p]).mean()))
        out["persistent_kernel"]["probe_us"] = {
            "kernel": float((done[5 * L].max() - clk[0, 0, :].min()) / 1e3),
            "lm_head": float((done[5 * L] - passed[5 * L - 1]).mean() / 1e3),
            "work": {n: float(sum(v) / max(len(v), 1) / 1e3) for n, v in work.items()},
            "barrier": {n: float(sum(v) / max(len(v), 1) / 1e3) for n, v in wait.items()}}
    log("  decode", json.dumps(out))
    return out


def cpu_baseline(model, cfg, B, T):
    """The CPU oracle on the host cores: one forward of the whole benchmark batch
    (a few seconds on 16 cores), after one untimed pass at B=1 to warm the threads."""
    import numpy as np
    import oracle
    params = model.params_tensor().cpu().numpy()
    ids = np.random.default_rng(0).integers(0, cfg["vocab_size"], (B, T), dtype=np.int32)
    kw = dict(maxT=cfg["max_seq_len"], V=cfg["vocab_size"], L=cfg["num_layers"],
              NH=cfg["num_heads"], C=cfg["channels"])
    oracle.gpt2_forward(params, ids[:1], **kw)
    t0 = time.monotonic()
    oracle.gpt2_forward(params, ids, **kw)
    dt = time.monotonic() - t0
    return {"value": B * T / dt, "unit": "tokens/s", "cores": oracle.num_threads(),
            "nproc": os.cpu_count(), "cpus_allowed": len(os.sched_getaffinity(0)), "kind": "port",
            "sample": f"one forward of the same workload, B={B}, T={T} ({dt:.2f} s wall); "
                      "plain-C/OpenMP restatement of llm.c's CPU gpt2_forward"}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--model", choices=("124M", "350M", "774M", "1558M"), default="124M",
                    help="124M is the benchmark's model; the others are the wider GPT-2 sizes (with --batch)")
    ap.add_argument("--batch", type=int, default=None)
    ap.add_argument("--seq-len", type=int, default=1024)
    ap.add_argument("--no-standalone", action="store_true")
    ap.add_argument("--no-cpu", action="store_true")
    ap.add_argument("--decode", type=int, default=0, metavar="STEPS",
                    help="time prefill + STEPS single-token decode steps (key/value cache) instead")
    ap.add_argument("--graph", action="store_true",
                    help="also time the forward pass replayed from a HIP graph")
    ap.add_argument("--clock-probe", action="store_true",
                    help="in-kernel wall/shader clock probe of the GEMM, zero vs normal operands")
    ap.add_argument("--pmc-probe", action="store_true",
                    help="launch each kernel once plus a calibration copy (for rocprofv3 --pmc)")
    args = ap.parse_args()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print("bench.py: this build runs on ONE GPU (the forward pass shards over the batch with "
              "no exchange, so N GPUs would be N independent copies of this run); use --gpus 1",
              file=sys.stderr)
        sys.exit(2)

    import torch
    g2 = importlib.import_module("cuda-gpt2-inference_amd")
    syn = importlib.import_module("cuda-gpt2-inference_amd.synthetic")
    if not os.path.exists(g2.LIB_PATH):  # load what is built; build only if nothing is
        import __graft_entry__
        __graft_entry__.build()
    if not torch.cuda.is_available():
        print("bench.py: no GPU", file=sys.stderr)
        sys.exit(2)
    torch.cuda.set_device(0)

    if args.pmc_probe:
        pmc_probe(g2)
        return
    if args.clock_probe:
        clock_probe(g2)
        return
    cfg = dict({"124M": g2.GPT2_124M, "350M": g2.GPT2_350M, "774M": g2.GPT2_774M, "1558M": g2.GPT2_1558M}[args.model])
    B = args.batch or (8 if args.model == "124M" else 4)
    T = args.seq_len
    model = g2.GPT2(**cfg)
    init_params_on_device(model, syn, cfg, seed=1337)
    ids = torch.randint(0, cfg["vocab_size"], (B, T), dtype=torch.int32, device="cuda")
    model.reserve(B, T)
    if args.decode:
        print(json.dumps({"decode": [decode_bench(model, cfg, B, T, args.decode)]}))
        model.close()
        return

    for _ in range(args.warmup):
        model.forward(ids)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        model.forward(ids)
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    ms_per_step = dt / args.steps * 1e3
    tokens_per_s = B * T * args.steps / dt
    finite = bool(torch.isfinite(model.logits()[0, :4]).all())
    log(f"forward {args.model} B={B} T={T}: {ms_per_step:.3f} ms/step, {tokens_per_s:,.0f} tok/s"
        f" (logits finite: {finite})")

    # the llm.c signature: token ids handed over in host memory (32 KiB per step here), copied
    # in stream order and waited for before the launches are issued; not the reported value
    host_ids = ids.cpu().numpy()
    model.forward(host_ids)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        model.forward(host_ids)
    torch.cuda.synchronize()
    host_ids_ms = (time.perf_counter() - t0) / args.steps * 1e3
    log(f"  with host token ids (gpt2_forward): {host_ids_ms:.3f} ms/step")

    graph_ms = None
    if args.graph:
        for _ in range(max(args.warmup, 2)):          # the first call captures
            model.forward_graph(ids)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(args.steps):
            model.forward_graph(ids)
        torch.cuda.synchronize()
        graph_ms = (time.perf_counter() - t0) / args.steps * 1e3
        log(f"  replayed from a HIP graph: {graph_ms:.3f} ms/step")

    # the same K steps again with a HIP event around every launch
    prof = {k: 0.0 for k in g2.PROF_CATEGORIES}
    for _ in range(args.steps):
        for k, v in model.forward_profiled(ids).items():
            prof[k] += v
    prof = {k: v / args.steps for k, v in prof.items()}   # ms per forward per category
    flops = forward_flops(cfg, B, T)
    sums_in_matmul = g2.forward_sums_in_matmul(cfg, B, T)
    nbytes = forward_bytes(cfg, B, T, sums_in_matmul)
    L = cfg["num_layers"]
    marker_ms = marker_overhead_ms(g2)
    log(f"  event marker between two launches: +{marker_ms * 1e3:.2f} us per interval")
    kernels = []
    for k in g2.PROF_CATEGORIES:
        launches = LAUNCHES.get(k, 2 * L if k == "fused_residual_layernorm" else L)
        row = {"launch": k, "launches_per_forward": launches, "ms_per_forward": prof[k],
               "ms_per_launch": prof[k] / launches}
        # the same figure with the event marker's own cost taken out of every interval: what a
        # launch takes from the end of its predecessor to its own end, as in an unprofiled pass
        net = max(prof[k] - launches * marker_ms, 1e-9)
        if k in flops:
            tf = flops[k] / prof[k] / 1e9
            row.update({"TFLOP/s": tf, "frac_fp32_mfma": tf / PEAK_FP32_MFMA_TFLOPS,
                        "frac_fp32_mfma_net_of_marker": flops[k] / net / 1e9 / PEAK_FP32_MFMA_TFLOPS})
        else:
            gbs = nbytes[k] / prof[k] / 1e6
            row.update({"GB/s": gbs, "frac_hbm": gbs / PEAK_HBM_GBS,
                        "frac_hbm_net_of_marker": nbytes[k] / net / 1e6 / PEAK_HBM_GBS,
                        "note": "inside the forward pass, operands may be served by the 256 MiB "
                                "Infinity Cache"})
        if sums_in_matmul and k == "fused_residual_layernorm":
            row["note"] = ("at this size the driver adds the residual stream in the epilogues of the two "
                           "projections (matmul_forward_residual_status) and these launches are "
                           "layernorm_forward on the sum: 8 bytes per entry instead of 16; " + row["note"])
        if sums_in_matmul and k in ("matmul_attproj", "matmul_fcproj"):
            row["note"] = "out = residual + product: the block's residual add is in this launch's epilogue"
        if k == "encoder":
            row["note"] = ("the pass's first launch: its interval also holds the opening event's own trip and "
                           "the host's launch latency (the device finishes the untimed launches in front of it "
                           "before the host has queued the next one); the kernel by itself is the "
                           "encoder_forward row of standalone[]")
        kernels.append(row)
        log(f"  {k:26s} {prof[k]:8.3f} ms/fwd  " + (f"{row.get('TFLOP/s', 0):7.1f} TFLOP/s"
            if k in flops else f"{row.get('GB/s', 0):7.0f} GB/s"))
    # Dominant kernel: matmul_dma_kernel<128,192,4,2,false>, which runs the qkv, attention-
    # projection and fc-projection GEMMs (3 per layer; at sizes where the driver adds the residual
    # stream in the projections' epilogues those two launches are the instantiation of the same
    # kernel that fetches its tile of the residual during the slab loop; the fc GEMM with its
    # GELU epilogue and the lm-head are other instantiations of the same source).
    dom = ("matmul_qkv", "matmul_attproj", "matmul_fcproj")
    dom_launches = 3 * L
    dom_flops = sum(flops[k] for k in dom) / dom_launches
    dom_ms = sum(prof[k] for k in dom) / dom_launches
    achieved = dom_flops / dom_ms / 1e9
    roofline = {"bound": "mfma", "achieved": achieved, "peak": PEAK_FP32_MFMA_TFLOPS,
                "unit": "TFLOP/s", "frac": achieved / PEAK_FP32_MFMA_TFLOPS,
                "traffic": (dominant_traffic_bytes()
                            if (args.model == "124M" and B == 8 and T == 1024) else None),
                "traffic_source": "recorded from two rocprofv3 --pmc runs of bench.py --pmc-probe "
                                  "(profiles/kernels_baseline_shapes_pmc.txt), not counted in this run",
                "kernel": ("matmul_dma_kernel<128,192,4,2,false> (qkv: plain epilogue; attproj, fcproj: "
                           "residual add in the epilogue)" if B * T == 8192 else
                           "matmul_forward, qkv / attproj / fcproj launches (tile shape by size)"),
                "avg_launch_ms": dom_ms, "flops_per_launch": dom_flops,
                "launches_per_forward": dom_launches}

    result = {
        "metric": "GPT-2 124M fp32 fwd tokens/s (B=8,T=1024); matmul % FP32 MFMA peak",
        "value": tokens_per_s, "unit": "tokens/s", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": ms_per_step, "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": "f32", "data": "synthetic",
        "config": {"workload": f"GPT-2 {args.model} fp32 forward, B={B}, T={T}, seeded random "
                               "weights, uniform random token ids resident in HBM",
                   "global_batch": B, "seq_len": T},
        "roofline": roofline,
        "forward_frac_fp32_mfma": (sum(flops.values()) / (ms_per_step * 1e9)) / PEAK_FP32_MFMA_TFLOPS,
        "kernels": kernels,
    }
    result["host_ids_ms_per_step"] = host_ids_ms
    result["profile_marker_overhead_us"] = marker_ms * 1e3
    result["profile_note"] = ("kernels[].ms_per_launch is the time between the events recorded before "
                              "and after a launch, which includes the closing event's own "
                              "profile_marker_overhead_us; the *_net_of_marker fractions take that out")
    if graph_ms is not None:
        result["graph_replay_ms_per_step"] = graph_ms
    if not args.no_standalone:
        result["standalone"] = standalone(g2)
        for r in result["standalone"]:
            log("  standalone", json.dumps(r))
        # the path's next caller: incremental decoding against a key/value cache
        # (a row per batch size: up to 16 sequences one persistent kernel per step, beyond that
        # one launch per operation either way)
        result["decode"] = [decode_bench(model, cfg, b, 128, 64) for b in (1, 8, 16, 32, 64)]
    if not args.no_cpu:
        result["cpu_baseline"] = cpu_baseline(model, cfg, B, T)
        log("  cpu_baseline", json.dumps(result["cpu_baseline"]))
    if not args.no_standalone and args.model == "124M" and B == 8 and T == 1024:
        # the second end-to-end workload: GPT-2 350M, B=4, T=1024
        model.close()
        cfg2 = dict(g2.GPT2_350M)
        model = g2.GPT2(**cfg2)
        init_params_on_device(model, syn, cfg2, seed=1338)
        ids2 = torch.randint(0, cfg2["vocab_size"], (4, 1024), dtype=torch.int32, device="cuda")
        for _ in range(args.warmup):
            model.forward(ids2)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(args.steps):
            model.forward(ids2)
        torch.cuda.synchronize()
        ms2 = (time.perf_counter() - t0) / args.steps * 1e3
        fl2 = sum(forward_flops(cfg2, 4, 1024).values())
        result["gpt2_350M_B4_T1024"] = {
            "ms_per_step": ms2, "tokens_per_s": 4 * 1024 / ms2 * 1e3,
            "forward_frac_fp32_mfma": fl2 / (ms2 * 1e9) / PEAK_FP32_MFMA_TFLOPS}
        log("  350M", json.dumps(result["gpt2_350M_B4_T1024"]))
    model.close()
    print(json.dumps(result), flush=True)


if __name__ == "__main__":
    main()
