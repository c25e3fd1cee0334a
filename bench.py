#!/usr/bin/env python3
"""Headline benchmark: train tokens/s of one full 104m step (forward + loss + backward + AdamW)
at B=32, T=1024 on one MI355X, bf16 storage with fp32 accumulation, synthetic seeded token ids
and random-init weights.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--loss cut|dense] [--dtype bf16|f16] [--no-cpu-baseline]

Prints ONE JSON line. Besides the contract fields it carries
  roofline     – the kernel that takes the most time in the step, on the launch it spends most
                 of it in (dX of the gate/up projection): algorithmic FLOPs of that launch / its average
                 duration inside the step (HIP events around every operator call of one eager
                 pass on the step's stream), against the 2.5 PFLOP/s dense bf16 MFMA peak; the
                 same launch timed 20 times back to back; the per-kind breakdown of the step;
                 `gemm_launches` (every contraction of the step by position: shape, microseconds, fraction) and
                 `kernels` (every backward operator alone at the configuration's shape, HIP events on the launch
                 stream, against its HBM or MFMA roofline);
  cpu_baseline – the float32 CPU restatement of the reference's operators (oracle/, "port")
                 timed on this host on bounded samples of the same workload: one full train step, the
                 reference's CPU-runnable configuration (forward + loss at B=1, T=256) and each backward
                 operator alone.
--dtype f16 --loss dense is the configuration of the reference's own published run (F16 storage, dense
cross-entropy over materialised logits: train/train.cpp:59, 436-440).
This run uses one GPU; --gpus above 1 exits with a message.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

import numpy as np

PEAK_BF16_TFLOPS = 2500.0
PEAK_HBM_GBS = 8000.0


def op_work(cfg, batch, seq, loss_mode):
    """Algorithmic FLOPs (MFMA-bound kinds) or HBM bytes (bandwidth-bound kinds) per step and kind."""
    N, H, I, V, L = batch * seq, cfg.hidden_size, cfg.intermediate_size, cfg.vocabulary_size, cfg.num_layers
    HQ, HKV, D = cfg.num_query_heads, cfg.num_kv_heads, cfg.head_dim
    QW, KW = HQ * D, HKV * D
    layer_weights = QW * H + 2 * KW * H + H * QW + 2 * I * H + H * I
    linear = 2.0 * N * layer_weights * L
    head = 2.0 * N * V * H
    attention = 2.0 * batch * HQ * seq * seq * D / 2  # one causal matmul
    e = 2  # bytes per 16-bit element
    work = {
        "gemm_fwd": ("mfma", linear + (head if loss_mode == "dense" else 0)),
        "gemm_dx": ("mfma", linear + (head if loss_mode == "dense" else 0)),
        "gemm_dw": ("mfma", linear + (head if loss_mode == "dense" else 0)),
        "cut_ce": ("mfma", 3 * head),
        "attn_fwd": ("mfma", 2 * attention * L),
        "attn_bwd": ("mfma", 5 * attention * L),
        "dense_ce": ("hbm", 2.0 * N * V * e),
        "rmsnorm_fwd": ("hbm", (2 * N * H * 2 + N * (QW + KW) * 2) * e * L + 2 * N * H * e),
        # the two hidden-wide norms of a block also read the residual gradient they are added to
        "rmsnorm_bwd": ("hbm", (2 * N * H * 4 + N * (QW + KW) * 3) * e * L + 3 * N * H * e),
        "rope_fwd": ("hbm", N * (QW + KW) * 2 * e * L),
        "rope_bwd": ("hbm", N * (QW + KW) * 2 * e * L),
        "swiglu_fwd": ("hbm", N * I * 3 * e * L),
        "swiglu_bwd": ("hbm", N * I * 5 * e * L),
        "embedding_fwd": ("hbm", N * H * 2 * e),
        "embedding_bwd": ("hbm", N * H * 3 * e),
    }
    return work


# The kernel that takes the largest share of a step is the 256x256-tile contraction with a k-contiguous
# A and an n-contiguous B (dX = dY W: every input gradient of a projection and of the classifier). Its
# roofline entry is measured on the launch it spends most time in: the input gradient of the fused
# gate/up projection, [N, 2I] x [2I, H].
PROBE_KERNEL = "gemm_mfma_kernel<bf16, 256, 256, A k-contiguous, B n-contiguous> (dX of the gate/up projection)"
TRAFFIC_FILE = os.path.join(os.path.dirname(os.path.abspath(__file__)), "profiles",
                            "gemm_dx_256x256_gate_projection_pmc.txt")


def kernel_probe(torch, cfg, batch, seq, stream, launches, seed, dtype=None, data="random"):
    """Average duration of one launch of the dominant kernel: HIP events on the launch stream. data = "zeros" runs the
    same launch on all-zero operands (same instructions, same memory traffic, no switching in the multipliers): the
    difference to random data is what the chip's power limit costs."""
    from cgpt_amd import ops

    dtype = dtype or torch.bfloat16
    rows, hidden, inter = batch * seq, cfg.hidden_size, 2 * cfg.intermediate_size  # [gate; up] as one weight
    generator = torch.Generator(device="cuda").manual_seed(seed)
    dy = torch.randn(rows, inter, device="cuda", generator=generator).to(dtype)
    x = torch.empty(rows, hidden, device="cuda", dtype=dtype)  # shape only: no weight gradient is asked for
    w = (torch.randn(inter, hidden, device="cuda", generator=generator) * 0.02).to(dtype)
    dx = torch.empty(rows, hidden, device="cuda", dtype=dtype)
    if data == "zeros":
        dy.zero_()
        w.zero_()
    start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    with torch.cuda.stream(stream):
        for _ in range(3):
            ops.linear_backward(dx, None, None, dy, x, w, None, stream)
        start.record(stream)
        for _ in range(launches):
            ops.linear_backward(dx, None, None, dy, x, w, None, stream)
        stop.record(stream)
    stop.synchronize()
    seconds = start.elapsed_time(stop) * 1e-3 / launches
    flops = 2.0 * rows * hidden * inter
    algorithmic_bytes = 2 * (rows * inter + inter * hidden + rows * hidden)
    return {"seconds": seconds, "flops": flops, "algorithmic_bytes": algorithmic_bytes, "launches": launches,
            "shape": f"[{rows}, {inter}] x [{inter}, {hidden}]"}


def gemm_shapes(cfg, batch, seq):
    """(M, N, K) of every contraction label of the step profile ("kind.position")."""
    N, H, I, V = batch * seq, cfg.hidden_size, cfg.intermediate_size, cfg.vocabulary_size
    QKV = (cfg.num_query_heads + 2 * cfg.num_kv_heads) * cfg.head_dim
    QW = cfg.num_query_heads * cfg.head_dim
    outs = {"qkv": (QKV, H), "o": (H, QW), "gate_up": (2 * I, H), "down": (H, I), "classifier": (V, H)}  # (out, in)
    shapes = {}
    for name, (o, i) in outs.items():
        shapes[f"gemm_fwd.{name}"] = (N, o, i)   # Y[N, out] = X[N, in] W^T
        shapes[f"gemm_dx.{name}"] = (N, i, o)    # dX[N, in] = dY[N, out] W
        shapes[f"gemm_dw.{name}"] = (o, i, N)    # dW[out, in] = dY^T X
    # The stacked weight gradients pair the q projection with the output projection (one shape) and leave [k; v].
    shapes["gemm_dw.q_o"] = (QW + H, H, N)
    shapes["gemm_dw.kv"] = (QKV - QW, H, N)
    return shapes


def timed(torch, stream, fn, launches=20, warm=3):
    """Average seconds per call of fn(), HIP events recorded on the stream the kernels are launched on."""
    start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    with torch.cuda.stream(stream):
        for _ in range(warm):
            fn()
        start.record(stream)
        for _ in range(launches):
            fn()
        stop.record(stream)
    stop.synchronize()
    return start.elapsed_time(stop) * 1e-3 / launches


def isolated_kernels(torch, cfg, batch, seq, dtype, stream, seed, only="", secondary=True):
    """Every backward operator alone at the configuration's shape: algorithmic bytes or FLOPs of one call /
    its average duration over 20 back-to-back calls. `only`: run just the sections whose name contains it (or one
    of several, separated by commas)."""
    from cgpt_amd import ops

    N, H, I, V = batch * seq, cfg.hidden_size, cfg.intermediate_size, cfg.vocabulary_size
    HQ, HKV, D = cfg.num_query_heads, cfg.num_kv_heads, cfg.head_dim
    e = 2
    gen = torch.Generator(device="cuda").manual_seed(seed)

    def rnd(*shape, scale=1.0):
        return (torch.randn(*shape, device="cuda", generator=gen) * scale).to(dtype)

    out = {}

    def want(section):
        return any(part in section for part in only.split(","))

    def record(name, bound, amount, seconds, shape):
        rate = amount / seconds / (1e12 if bound == "mfma" else 1e9)
        peak = PEAK_BF16_TFLOPS if bound == "mfma" else PEAK_HBM_GBS
        out[name] = {"shape": shape, "bound": bound, "us": round(seconds * 1e6, 1), "rate": round(rate, 1),
                     "unit": "TFLOP/s" if bound == "mfma" else "GB/s", "frac": round(rate / peak, 4)}

    for rows, hidden in ((N, H), (N * HQ, D), (N * HKV, D)) if want("rmsnorm") else ():
        x, dy, w = rnd(rows, hidden), rnd(rows, hidden), rnd(hidden)
        dx, dw = torch.empty_like(x), torch.empty_like(w)
        t = timed(torch, stream, lambda: ops.rmsnorm_backward(dx, dw, dy, x, w, 1e-5, stream))
        record(f"rmsnorm_backward[{rows},{hidden}]", "hbm", 3 * rows * hidden * e, t, f"x, dy read, dx written")
        del x, dy, dx
    if secondary and want("secondary"):
        # The 12 x 768 shape named beside the preset (12:4 heads of 64): norm, rotary, attention and cut cross-entropy.
        import dataclasses
        second = dataclasses.replace(cfg, hidden_size=768, num_query_heads=12, num_kv_heads=4, head_dim=64, rotary_dim=64)
        for section in ("rmsnorm", "rope", "attention", "cut_cross_entropy"):
            for name, entry in isolated_kernels(torch, second, batch, seq, dtype, stream, seed, section, False).items():
                out["secondary: " + name] = entry
    ids = torch.randint(0, V, (N,), device="cuda", generator=gen, dtype=torch.int32)
    if not (want("rope") or want("attention")):
        return _isolated_rest(torch, ops, want, record, rnd, timed, stream, out, N, H, I, V, e, ids)
    q, k = rnd(batch, seq, HQ, D), rnd(batch, seq, HKV, D)
    pos = torch.arange(seq, device="cuda", dtype=torch.float32)[:, None]
    theta = pos / torch.pow(torch.tensor(10000.0, device="cuda"), torch.arange(D // 2, device="cuda") * 2.0 / D)[None, :]
    cos, sin = torch.cos(theta).to(dtype), torch.sin(theta).to(dtype)
    gq, gk = torch.empty_like(q), torch.empty_like(k)
    if want("rope"):
        t = timed(torch, stream, lambda: ops.rope_backward(gq, gk, q, k, cos, sin, stream))
        record(f"rope_backward q[{batch},{seq},{HQ},{D}] k[..,{HKV},..]", "hbm", 2 * (q.numel() + k.numel()) * e, t, "read + write")
    if not want("attention"):
        return _isolated_rest(torch, ops, want, record, rnd, timed, stream, out, N, H, I, V, e, ids)
    v = rnd(batch, seq, HKV, D)
    o, lse = torch.empty_like(q), torch.empty(batch, seq, HQ, device="cuda")
    do = rnd(batch, seq, HQ, D)
    opt = ops.FlashAttentionOptions(HQ, HKV, D)
    causal_matmul = 2.0 * batch * HQ * seq * seq * D / 2
    t = timed(torch, stream, lambda: ops.flash_gqa_attention_forward_with_lse(o, lse, q, k, v, stream, opt))
    record("flash_gqa_attention_forward_with_lse", "mfma", 2 * causal_matmul, t, f"B={batch} T={seq} {HQ}:{HKV} heads D={D}, 2 causal matmuls")
    gv = torch.empty_like(k)
    t = timed(torch, stream, lambda: ops.flash_gqa_attention_backward_with_lse(gq, gk, gv, do, o, lse, q, k, v, stream, opt))
    record("flash_gqa_attention_backward_with_lse", "mfma", 5 * causal_matmul, t,
           f"B={batch} T={seq} {HQ}:{HKV} heads D={D}, 5 causal matmuls counted (7 executed)")
    del q, k, v, o, do, gq, gk, gv
    return _isolated_rest(torch, ops, want, record, rnd, timed, stream, out, N, H, I, V, e, ids)


def _isolated_rest(torch, ops, want, record, rnd, timed, stream, out, N, H, I, V, e, ids):
    dtype = rnd(1).dtype
    if want("swiglu"):
        gate_up, dy = rnd(N, 2 * I), rnd(N, I)
        g_gate_up = torch.empty_like(gate_up)
        t = timed(torch, stream, lambda: ops.swiglu_backward_packed(g_gate_up, dy, gate_up, stream))
        record(f"swiglu_backward[{N},{I}]", "hbm", 5 * N * I * e, t, "dy, gate, up read; dgate, dup written")
        del gate_up, dy, g_gate_up
    if want("embedding"):
        dy, table = rnd(N, H), torch.zeros(V, H, device="cuda", dtype=dtype)
        t = timed(torch, stream, lambda: ops.embedding_backward(table, dy, ids, N, stream, ops.EmbeddingBackwardOptions(accumulate_weight=True)))
        record(f"embedding_backward {N} tokens into [{V},{H}]", "hbm", 3 * N * H * e, t, "dy read, table rows read and written")
        del dy, table
    if want("cut_cross_entropy"):
        x, c = rnd(N, H), rnd(V, H, scale=0.02)
        dx, dc, loss = torch.empty_like(x), torch.empty_like(c), torch.zeros(1, device="cuda")
        t = timed(torch, stream, lambda: ops.cut_cross_entropy_forward_backward(loss, dx, dc, x, c, ids, N, stream, 1024.0), launches=5, warm=2)
        record(f"cut_cross_entropy_forward_backward [{N},{H}] x [{V},{H}]", "mfma", 3 * 2.0 * N * V * H, t,
               "3 vocabulary contractions executed (logits, dX, dC); 4 in a recompute formulation")
        del x, c, dx, dc
    if want("copy"):  # calibration of the profiler's FETCH_SIZE / WRITE_SIZE counters: reads and writes 1 GiB
        source = torch.empty(1 << 30, dtype=torch.uint8, device="cuda")
        target = torch.empty_like(source)
        t = timed(torch, torch.cuda.current_stream(), lambda: target.copy_(source), launches=5, warm=1)
        record("copy 1 GiB (torch)", "hbm", 2.0 * (1 << 30), t, "1 GiB read, 1 GiB written")
        del source, target
    if want("adamw"):
        # The preset's parameter list (2 + 11 per layer tensors): all of it in three launches.
        layers = 8
        QW, KW = H, H // 4
        shapes = [(V, H), (H,)] + layers * [(H,), (QW, H), (KW, H), (H // 8,), (H // 8,), (KW, H), (H, QW), (H,), (I, H), (I, H), (H, I)]
        entries = []
        for shape in shapes:
            parameter = rnd(*shape, scale=0.02)
            entries.append(ops.AdamWBatchEntry(parameter, rnd(*shape), ops.AdamWState.for_parameter(parameter)))
        count = sum(e.parameter.numel() for e in entries)
        workspace = ops.AdamWWorkspace()
        options = ops.AdamWOptions(learning_rate=3e-4, beta1=0.9, beta2=0.95, epsilon=1e-8, weight_decay=0.1,
                                   loss_scale=1024.0, max_grad_norm=1.0)
        t = timed(torch, stream, lambda: ops.adamw_step_many_async(entries, options, workspace, stream), launches=5, warm=1)
        record(f"adamw_step_many_async {count} parameters in {len(entries)} tensors", "hbm", 30.0 * count, t,
               "30 B/parameter: 16-bit gradient read twice (norm, update), fp32 master and both moments read and written, "
               "16-bit parameter written")
        del entries, workspace
    if want("dense_cross_entropy"):
        rows = N // 2
        logits = rnd(rows, V)
        grad, loss = torch.empty_like(logits), torch.zeros(1, device="cuda")
        t = timed(torch, stream, lambda: ops.cross_entropy_forward_backward(loss, grad, logits, ids[:rows], rows, stream, 1024.0), launches=10)
        record(f"cross_entropy_forward_backward[{rows},{V}]", "hbm", 2 * rows * V * e, t, "logits read once, gradient written once")
    return out


def published_kernel_shapes(torch, stream, seed):
    """The launches of the reference's own kernel table (kernel_profile.md:9-25: B = 1, T = 512, 32:8 heads, D = 128,
    hidden 4096, measured by its authors on a 192 GB/s GPU) on this GPU: average us over 50 back-to-back calls beside
    the published milliseconds. Context only (--kernels-only published): other hardware, not a configuration of the
    benchmark, and launches so small (2 to 100 MB) that they measure launch latency as much as rate."""
    from cgpt_amd import ops

    gen = torch.Generator(device="cuda").manual_seed(seed)

    def rnd(*shape, dtype=torch.float16):
        return torch.randn(*shape, device="cuda", generator=gen).to(dtype)

    out = {}

    def record(name, published_ms, seconds):
        out[name] = {"us": round(seconds * 1e6, 1), "published_ms_on_other_hardware": published_ms}

    for dtype, label, ms in ((torch.float16, "F16", 0.1228), (torch.bfloat16, "BF16", 0.1230)):
        x, dy, w = rnd(512, 4096, dtype=dtype), rnd(512, 4096, dtype=dtype), rnd(4096, dtype=dtype)
        dx, dw = torch.empty_like(x), torch.empty_like(w)
        record(f"rmsnorm_backward {label} [512,4096]", ms,
               timed(torch, stream, lambda: ops.rmsnorm_backward(dx, dw, dy, x, w, 1e-5, stream), launches=50))
    B, T, HQ, HKV, D = 1, 512, 32, 8, 128
    q, k, v, do = rnd(B, T, HQ, D), rnd(B, T, HKV, D), rnd(B, T, HKV, D), rnd(B, T, HQ, D)
    pos = torch.arange(T, device="cuda", dtype=torch.float32)[:, None]
    theta = pos / torch.pow(torch.tensor(10000.0, device="cuda"), torch.arange(D // 2, device="cuda") * 2.0 / D)[None, :]
    cos, sin = torch.cos(theta).to(torch.float16), torch.sin(theta).to(torch.float16)
    gq, gk, gv = torch.empty_like(q), torch.empty_like(k), torch.empty_like(k)
    record("rope_backward F16 q[1,512,32,128] k[1,512,8,128]", 0.0640,
           timed(torch, stream, lambda: ops.rope_backward(gq, gk, q, k, cos, sin, stream), launches=50))
    opt = ops.FlashAttentionOptions(HQ, HKV, D, causal=False)
    o, lse = torch.empty_like(q), torch.empty(B, T, HQ, device="cuda")
    ops.flash_gqa_attention_forward_with_lse(o, lse, q, k, v, stream, opt)
    record("flash_gqa_attention_backward F16 B=1 T=512 32:8 D=128 non-causal", 1.9464,
           timed(torch, stream, lambda: ops.flash_gqa_attention_backward(gq, gk, gv, do, q, k, v, stream, opt), launches=50))
    record("flash_gqa_attention_backward_with_lse, same shape", 1.6369,
           timed(torch, stream, lambda: ops.flash_gqa_attention_backward_with_lse(gq, gk, gv, do, o, lse, q, k, v, stream, opt),
                 launches=50))
    ids = torch.arange(512, device="cuda", dtype=torch.int32)  # embedding_test.cu:205-230: distinct ids, accumulating
    dy, table = rnd(512, 4096), torch.zeros(32000, 4096, device="cuda", dtype=torch.float16)
    accumulate = ops.EmbeddingBackwardOptions(accumulate_weight=True)
    record("embedding_backward F16 512 tokens into [32000,4096]", 0.0766,
           timed(torch, stream, lambda: ops.embedding_backward(table, dy, ids, 512, stream, accumulate), launches=50))
    del table
    logits = rnd(512, 50257, dtype=torch.float32)
    grad, loss = torch.empty_like(logits), torch.zeros(1, device="cuda")
    targets = torch.randint(0, 50257, (512,), device="cuda", generator=gen, dtype=torch.int32)
    record("cross_entropy_forward_backward F32 [512,50257]", 2.3196,
           timed(torch, stream, lambda: ops.cross_entropy_forward_backward(loss, grad, logits, targets, 512, stream), launches=50))
    return out


def source_digest(name):
    """sha256 of a kernel source file (the summaries under profiles/ record the one they were made with)."""
    import hashlib

    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "cgpt_amd", "csrc", name)
    with open(path, "rb") as handle:
        return hashlib.sha256(handle.read()).hexdigest()


def measured_traffic():
    """(HBM bytes per launch of the probe kernel from the committed counter summary or None, note). The summary
    names the sha256 of the kernel source it was measured with; when the source has changed since, the figure is
    reported with a warning (stderr and `traffic_note`) instead of silently."""
    value, recorded = None, None
    try:
        with open(TRAFFIC_FILE) as handle:
            for line in handle:
                if line.startswith("traffic_bytes_per_launch"):
                    value = float(line.split("=")[1].split()[0])
                if line.startswith("gemm_hip_sha256"):
                    recorded = line.split("=")[1].strip()
    except OSError:
        return None, "no counter summary found"
    if value is None:
        return None, "the counter summary holds no traffic figure"
    if recorded is None or recorded != source_digest("gemm.hip"):
        note = "STALE: cgpt_amd/csrc/gemm.hip has changed since profiles/gemm_dx_256x256_gate_projection_pmc.txt was measured"
        print("bench.py: warning: roofline.traffic is " + note, file=sys.stderr)
        return value, note
    return value, "measured with the current cgpt_amd/csrc/gemm.hip"


def cpu_model_name():
    try:
        with open("/proc/cpuinfo") as handle:
            for line in handle:
                if line.startswith("model name"):
                    return line.split(":", 1)[1].strip()
    except OSError:
        pass
    return "unknown"


def cpu_operator_samples(seed):
    """Each backward operator of the CPU port alone, at the largest shape of the configuration that stays within
    a few seconds on this host (seconds and the same algorithmic rate the GPU table uses)."""
    import torch

    from oracle import cpu_ops as c

    g = torch.Generator().manual_seed(seed)
    out = {}

    def sample(name, amount, unit, shape, fn):
        start = time.perf_counter()
        fn()
        seconds = time.perf_counter() - start
        out[name] = {"shape": shape, "seconds": round(seconds, 3), "rate": round(amount / seconds / 1e9, 2), "unit": unit}

    rows, hidden = 32768, 1024
    x, dy, w = torch.randn(rows, hidden, generator=g), torch.randn(rows, hidden, generator=g), torch.ones(hidden)
    dx, dw = torch.empty_like(x), torch.empty_like(w)
    sample("rmsnorm_backward", 3 * rows * hidden * 4, "GB/s", f"[{rows},{hidden}] fp32", lambda: c.rmsnorm_backward(dx, dw, dy, x, w, 1e-5))
    q, k = torch.randn(8, 1024, 8, 128, generator=g), torch.randn(8, 1024, 2, 128, generator=g)
    cos, sin = torch.rand(1024, 64, generator=g), torch.rand(1024, 64, generator=g)
    gq, gk = torch.empty_like(q), torch.empty_like(k)
    sample("rope_backward", 2 * (q.numel() + k.numel()) * 4, "GB/s", "q[8,1024,8,128] k[8,1024,2,128] fp32", lambda: c.rope_backward(gq, gk, q, k, cos, sin))
    gate, up, dyi = (torch.randn(8192, 2048, generator=g) for _ in range(3))
    dg, du = torch.empty_like(gate), torch.empty_like(up)
    sample("swiglu_backward", 5 * gate.numel() * 4, "GB/s", "[8192,2048] fp32", lambda: c.swiglu_backward(dg, du, dyi, gate, up))
    rows, fin, fout = 1024, 1024, 1024
    x, wt, dy = torch.randn(rows, fin, generator=g), torch.randn(fout, fin, generator=g), torch.randn(rows, fout, generator=g)
    gi, gw, gb = torch.empty_like(x), torch.empty_like(wt), torch.empty(fout)
    sample("linear_backward", 2 * 2.0 * rows * fin * fout, "GFLOP/s", f"rows {rows}, {fout}x{fin} fp32 (dX and dW)", lambda: c.linear_backward(gi, gw, gb, dy, x, wt))
    tokens = torch.randint(0, 32000, (32768,), generator=g, dtype=torch.int32)
    dy, table = torch.randn(32768, 1024, generator=g), torch.zeros(32000, 1024)
    sample("embedding_backward", 3 * dy.numel() * 4, "GB/s", "32768 tokens into [32000,1024] fp32", lambda: c.embedding_backward(table, dy, tokens, True, True))
    logits, targets = torch.randn(1024, 32000, generator=g), torch.randint(0, 32000, (1024,), generator=g, dtype=torch.int32)
    grad, loss = torch.empty_like(logits), torch.empty(1)
    sample("cross_entropy_forward_backward", 2 * logits.numel() * 4, "GB/s", "[1024,32000] fp32", lambda: c.cross_entropy_forward_backward(loss, grad, logits, targets, 1024.0))
    T = 64
    q, k, v = torch.randn(1, T, 8, 128, generator=g), torch.randn(1, T, 2, 128, generator=g), torch.randn(1, T, 2, 128, generator=g)
    do = torch.randn(1, T, 8, 128, generator=g)
    gq, gk, gv = torch.empty_like(q), torch.empty_like(k), torch.empty_like(v)
    sample("flash_gqa_attention_backward", 5 * 2.0 * 8 * T * T * 128 / 2, "GFLOP/s",
           f"B=1 T={T} 8:2 heads D=128 fp32; NOT extrapolable: the operator recomputes the softmax row per output element "
           "(cost grows with T^3)", lambda: c.attention_backward(gq, gk, gv, do, q, k, v, 8, 2, 128))
    n = 104_090_624
    p_, g_, m_, a_, b_ = torch.zeros(n), torch.full((n,), 1e-3), torch.zeros(n), torch.zeros(n), torch.zeros(n)
    sample("adamw", 30.0 * n, "GB/s", f"{n} parameters fp32 (rate on the 30 B/parameter the 16-bit GPU update moves)",
           lambda: c.adamw(p_, g_, m_, a_, b_, 1, 3e-4, 0.9, 0.95, 1e-8, 0.1, 1024.0, 1.0, parallel=True))
    return out


def cpu_baseline(seed):
    """The CPU port on this host: (1) `value`: one full step of the same 104m model (forward + loss + backward +
    AdamW) at B=1 and the longest sequence that keeps the sample near 10-30 s (T doubles from 16 while the last step
    took under 8 s and four times as long would still stay under 40 s); (2) the reference's CPU-runnable
    configuration: forward + cross-entropy loss at B=1, T=256, fp32, with its loss and logits checksum; (3) each
    backward operator alone."""
    from oracle import cpu_model, cpu_ops

    cfg = dict(vocab=32000, layers=8, hidden=1024, inter=2048, hq=8, hkv=2, d=128, eps=1e-5)
    batch, seq = 1, 16
    seconds, loss = cpu_model.timed_train_step(cfg, batch, seq, seed)
    while seconds < 8.0 and 4.0 * seconds < 40.0 and seq < 128:
        seq *= 2
        seconds, loss = cpu_model.timed_train_step(cfg, batch, seq, seed)
    forward_seconds, forward_loss, checksum = cpu_model.timed_forward_loss(cfg, 1, 256, seed)
    return {"value": batch * seq / seconds, "unit": "tokens/s", "cores": cpu_ops.max_threads(), "kind": "port",
            "cpu": cpu_model_name(),
            "sample": f"one full 104m train step (fwd+loss+bwd+AdamW, fp32) at B={batch}, T={seq}: "
                      f"{seconds:.1f} s, loss {loss:.3f}; the fixed AdamW pass over 104M parameters is part of "
                      "the sample, the contractions are unblocked loops",
            "configuration_1": {"workload": "forward + cross-entropy loss, 104m dims, fp32, B=1, T=256 "
                                            "(src/core/generation_cpu.cpp:323-379 order; linear_forward_cpu is "
                                            "serial for more than one row)",
                                "seconds": round(forward_seconds, 2), "tokens_per_s": round(256 / forward_seconds, 2),
                                "loss": forward_loss, "logits_checksum": checksum},
            "operators": cpu_operator_samples(seed)}


def main() -> int:
    parser = argparse.ArgumentParser()
    parser.add_argument("--gpus", type=int, default=1)
    parser.add_argument("--steps", type=int, default=10)
    parser.add_argument("--warmup", type=int, default=3)
    parser.add_argument("--batch", type=int, default=32)
    parser.add_argument("--seq", type=int, default=1024)
    parser.add_argument("--loss", choices=["cut", "dense"], default="cut")
    parser.add_argument("--dtype", choices=["bf16", "f16"], default="bf16")
    parser.add_argument("--shape", choices=["104m", "12x768"], default="104m",
                        help="104m = the reference's preset (8 layers, hidden 1024, 8:2 heads of 128); 12x768 = the "
                             "12-layer, 768-wide decoder with 12:4 heads of 64 (a parity shape, not the bench line)")
    parser.add_argument("--no-kernel-table", action="store_true", help="skip the isolated per-operator launches")
    parser.add_argument("--no-graph", action="store_true")
    parser.add_argument("--no-cpu-baseline", action="store_true")
    parser.add_argument("--seed", type=int, default=0)
    parser.add_argument("--kernels-only", metavar="NAME", default=None,
                        help="run only the isolated operator launches whose name contains NAME (rmsnorm, rope, "
                             "attention, swiglu, embedding, cut_cross_entropy, dense_cross_entropy, adamw, copy, secondary, published; several "
                             "separated by commas; '' = all) and print "
                             "their table: the target of per-kernel rocprofv3 runs")
    parser.add_argument("--probe-data", choices=["random", "zeros"], default="random",
                        help="operands of --probe-only: random bf16 values, or zeros (same launch without switching "
                             "activity in the multipliers, to show what the power limit costs)")
    parser.add_argument("--probe-launches", type=int, default=20, help="timed launches of --probe-only")
    parser.add_argument("--probe-only", action="store_true",
                        help="launch only the dominant kernel (20x) and a 1 GiB device copy: the target of the "
                             "rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE runs behind roofline.traffic")
    args = parser.parse_args()
    if args.gpus != 1:
        print(f"bench.py: this build runs on one GPU; --gpus {args.gpus} is not supported "
              "(no collectives are part of the measured path)", file=sys.stderr)
        return 2

    import torch

    import ctypes

    from cgpt_amd import capi
    from cgpt_amd.model import LOSS_CUT, LOSS_DENSE, Model, ModelConfig
    from cgpt_amd.ops import AdamWOptions

    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        return 3
    device = torch.device("cuda:0")
    dtype = torch.bfloat16 if args.dtype == "bf16" else torch.float16
    cfg = ModelConfig(dtype=dtype)  # the reference's 104m preset
    if args.shape == "12x768":
        cfg = ModelConfig(dtype=dtype, num_layers=12, hidden_size=768, num_query_heads=12, num_kv_heads=4, head_dim=64,
                          rotary_dim=64)
    if args.kernels_only is not None:
        stream = torch.cuda.Stream(device=device)
        shown = {"kernels": isolated_kernels(torch, cfg, args.batch, args.seq, dtype, stream, args.seed, args.kernels_only)}
        if "published" in args.kernels_only or args.kernels_only == "":
            shown["published_kernel_shapes"] = published_kernel_shapes(torch, stream, args.seed)
        print(json.dumps(shown))
        return 0
    if args.probe_only:
        stream = torch.cuda.Stream(device=device)
        probe = kernel_probe(torch, cfg, args.batch, args.seq, stream, args.probe_launches, args.seed, None, args.probe_data)
        source = torch.empty(1 << 30, dtype=torch.uint8, device=device)
        target = torch.empty_like(source)
        for _ in range(5):
            target.copy_(source)  # calibration: reads 1 GiB and writes 1 GiB per launch
        torch.cuda.synchronize()
        print(json.dumps({"probe": PROBE_KERNEL, "data": args.probe_data, **probe, "copy_bytes": 1 << 30}))
        return 0
    model = Model(cfg, args.batch, args.seq, seed=args.seed, device=device)
    rng = np.random.default_rng(args.seed)
    model.set_tokens(rng.integers(0, cfg.vocabulary_size, size=(args.batch, args.seq)),
                     rng.integers(0, cfg.vocabulary_size, size=(args.batch, args.seq)))
    options = AdamWOptions(learning_rate=3e-4, beta1=0.9, beta2=0.95, epsilon=1e-8, weight_decay=0.1,
                           loss_scale=1024.0, max_grad_norm=1.0)
    loss_mode = LOSS_CUT if args.loss == "cut" else LOSS_DENSE
    stream = torch.cuda.Stream(device=device)
    use_graph = not args.no_graph

    for _ in range(args.warmup):
        model.train_step(options, loss_mode, use_graph, stream)
    loss_after_warmup, finite, _ = model.status(stream)
    torch.cuda.synchronize()
    start = time.perf_counter()
    for _ in range(args.steps):
        model.train_step(options, loss_mode, use_graph, stream)
    stream.synchronize()
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - start
    last_loss, finite_after, steps_done = model.status(stream)
    tokens = args.batch * args.seq
    ms_per_step = elapsed / max(args.steps, 1) * 1e3

    probe = kernel_probe(torch, cfg, args.batch, args.seq, stream, 20, args.seed, dtype)
    labelled = model.profile(options.loss_scale, loss_mode, stream)
    # Labels are "kind" or "kind.part"; the parts of a kind add up in the breakdown.
    breakdown = {}
    for label, ms in labelled.items():
        kind = label.split(".")[0]
        breakdown[kind] = breakdown.get(kind, 0.0) + ms
    # The probe's launch inside the step: one per layer in the event-timed eager pass.
    in_step_seconds = labelled["gemm_dx.gate_up"] * 1e-3 / cfg.num_layers
    work = op_work(cfg, args.batch, args.seq, args.loss)
    # When the per-head norms carry the rotary embedding (one pass), its algorithmic bytes count with theirs.
    for rope, norm in (("rope_fwd", "rmsnorm_fwd"), ("rope_bwd", "rmsnorm_bwd")):
        if rope not in breakdown:
            work[norm] = (work[norm][0], work[norm][1] + work[rope][1])
    achieved = probe["flops"] / in_step_seconds / 1e12
    back_to_back = probe["flops"] / probe["seconds"] / 1e12
    per_kind = {}
    for kind, ms in sorted(breakdown.items(), key=lambda kv: -kv[1]):
        if kind not in work:
            continue
        b, amt = work[kind]
        rate = amt / (ms * 1e-3) / (1e12 if b == "mfma" else 1e9)
        per_kind[kind] = {"ms": round(ms, 3), "rate": round(rate, 1), "unit": "TFLOP/s" if b == "mfma" else "GB/s",
                          "frac": round(rate / (PEAK_BF16_TFLOPS if b == "mfma" else PEAK_HBM_GBS), 4)}
    # Every contraction of the step by position: one launch per layer (the classifier's: one per step).
    shapes = gemm_shapes(cfg, args.batch, args.seq)
    launches = {}
    for label, ms in labelled.items():
        if label in shapes:
            m_, n_, k_ = shapes[label]
            calls = 1 if label.endswith("classifier") else cfg.num_layers
            tflops = 2.0 * m_ * n_ * k_ * calls / (ms * 1e-3) / 1e12
            launches[label] = {"m": m_, "n": n_, "k": k_, "calls": calls, "us_per_call": round(ms * 1e3 / calls, 1),
                               "tflops": round(tflops, 1), "frac": round(tflops / PEAK_BF16_TFLOPS, 4)}
    family = {kind: per_kind[kind]["frac"] for kind in ("gemm_fwd", "gemm_dx", "gemm_dw") if kind in per_kind}
    # Launches that carry a SwiGLU operator in their epilogue (no separate swiglu time in the breakdown then): their
    # time also pays for that operator's traffic, so the families are given without them as well.
    carriers = (("gemm_fwd", "gemm_fwd.gate_up", "swiglu_fwd", "SwiGLU forward"),
                ("gemm_dx", "gemm_dx.down", "swiglu_bwd", "SwiGLU gradient"))
    for kind, label, operator, what in carriers:
        if operator in breakdown or label not in launches or kind not in breakdown or operator not in work:
            continue
        entry = launches[label]
        carried = work[operator][1] / cfg.num_layers
        entry["carries"] = (f"{what}: {carried / 1e6:.0f} MB of operator traffic per launch "
                            f"({carried / (PEAK_HBM_GBS * 1e9) * 1e6:.0f} us at {PEAK_HBM_GBS / 1e3:.0f} TB/s)")
        rest_ms = breakdown[kind] - labelled[label]
        rest_flops = work[kind][1] - 2.0 * entry["m"] * entry["n"] * entry["k"] * entry["calls"]
        if rest_ms > 0:
            family[f"{kind} without the launch that carries the {what}"] = round(rest_flops / (rest_ms * 1e-3) / 1e12 / PEAK_BF16_TFLOPS, 4)
    # All event-timed launches of the probe kernel's instantiation in the step (plain, unsegmented dX with 256 x 256
    # tiles: the gate/up and the output projection's input gradients, one each per layer), FLOPs over time.
    same_kernel = [launches[label] for label in ("gemm_dx.gate_up", "gemm_dx.o") if label in launches]
    weighted_flops = sum(2.0 * e["m"] * e["n"] * e["k"] * e["calls"] for e in same_kernel)
    weighted_seconds = sum(e["us_per_call"] * 1e-6 * e["calls"] for e in same_kernel)
    weighted_frac = weighted_flops / weighted_seconds / 1e12 / PEAK_BF16_TFLOPS if weighted_seconds > 0 else None
    traffic, traffic_note = measured_traffic()
    scratch_bytes = int(capi.lib().cgptx_scratch_bytes(ctypes.c_void_p(stream.cuda_stream)))
    kernels = {} if args.no_kernel_table else isolated_kernels(torch, cfg, args.batch, args.seq, dtype, stream, args.seed)
    # AdamW over the model's own parameters (3 launches for all tensors): 30 B/parameter with 16-bit gradients and
    # parameters. (--kernels-only adamw runs the same update on a parameter list of its own.)
    adamw_seconds = timed(torch, stream, lambda: model.optimizer_step(options, stream), launches=5, warm=1)
    adamw_bytes = 30.0 * model.num_parameters
    kernels["adamw_step_many_async"] = {
        "shape": f"{model.num_parameters} parameters in {2 + 11 * cfg.num_layers} tensors", "bound": "hbm", "us": round(adamw_seconds * 1e6, 1),
        "rate": round(adamw_bytes / adamw_seconds / 1e9, 1), "unit": "GB/s",
        "frac": round(adamw_bytes / adamw_seconds / 1e9 / PEAK_HBM_GBS, 4)}
    num_parameters = model.num_parameters
    model.close()
    del model
    capi.call("cgptx_release_scratch")
    torch.cuda.empty_cache()

    def secondary_step(batch, seq, step_dtype, step_loss):
        """ms per step of another configuration of the same model (3 warm-up, 10 timed steps, hipGraph)."""
        other = Model(ModelConfig(dtype=step_dtype), batch, seq, seed=args.seed, device=device)
        other.set_tokens(rng.integers(0, cfg.vocabulary_size, size=(batch, seq)), rng.integers(0, cfg.vocabulary_size, size=(batch, seq)))
        for _ in range(3):
            other.train_step(options, step_loss, True, stream)
        other.status(stream)
        torch.cuda.synchronize()
        begin = time.perf_counter()
        for _ in range(10):
            other.train_step(options, step_loss, True, stream)
        stream.synchronize()
        torch.cuda.synchronize()
        seconds = (time.perf_counter() - begin) / 10
        loss, finite, _ = other.status(stream)
        other.close()
        capi.call("cgptx_release_scratch")
        torch.cuda.empty_cache()
        return {"ms_per_step": round(seconds * 1e3, 3), "tokens_per_s": round(batch * seq / seconds, 1), "loss_last": loss,
                "all_finite": bool(finite)}

    secondary = {}
    if args.shape == "104m" and not args.no_kernel_table:
        secondary["bf16, B=8, T=4096, cut cross-entropy (the long-context variant of the configuration)"] = \
            secondary_step(8, 4096, torch.bfloat16, LOSS_CUT)
        secondary["f16, B=32, T=1024, dense cross-entropy (storage and loss of the reference's own published run)"] = \
            secondary_step(32, 1024, torch.float16, LOSS_DENSE)

    result = {
        "metric": f"train tokens/sec, {args.shape} fwd+bwd+AdamW B={args.batch} T={args.seq}",
        "value": tokens * args.steps / elapsed,
        "unit": "tokens/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": ms_per_step,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": args.dtype,
        "data": "synthetic",
        "config": {"workload": f"full {args.shape} train step (embedding, {cfg.num_layers} blocks, {args.loss} cross-entropy, backward, "
                               f"AdamW), B={args.batch}, T={args.seq}, hipGraph={'on' if use_graph else 'off'}",
                   "parameters": num_parameters, "global_batch": args.batch, "seq_len": args.seq,
                   "loss_scale": 1024.0},
        "scratch_bytes": scratch_bytes,
        "scratch_note": "device memory the operators of the step took beyond the caller's tensors (one arena per stream, sized "
                        "by the largest request): with the cut cross-entropy it is the logits chunk, rows x vocabulary in "
                        "the storage dtype",
        "secondary_steps": secondary,
        "loss_after_warmup": loss_after_warmup, "loss_last": last_loss, "all_finite": bool(finite and finite_after),
        "optimizer_steps": steps_done,
        "roofline": {"bound": "mfma", "achieved": achieved, "peak": PEAK_BF16_TFLOPS, "unit": "TFLOP/s",
                     "frac": achieved / PEAK_BF16_TFLOPS, "traffic": traffic, "traffic_note": traffic_note,
                     "frac_time_weighted": weighted_frac,
                     "kernel": PROBE_KERNEL, "launch_shape": probe["shape"],
                     "launch_us": in_step_seconds * 1e6, "launches_timed": cfg.num_layers,
                     "flops_per_launch": probe["flops"], "algorithmic_bytes_per_launch": probe["algorithmic_bytes"],
                     "back_to_back": {"launch_us": probe["seconds"] * 1e6, "launches_timed": probe["launches"],
                                      "achieved": back_to_back, "frac": back_to_back / PEAK_BF16_TFLOPS},
                     "note": "achieved = algorithmic FLOPs of one launch / average duration of that launch inside "
                             "the train step (HIP events on the step's stream around each of its calls, one per "
                             "layer, in one eager pass over the step); back_to_back = the same launch 20 times in a "
                             "row on random bf16 data, where the chip's power limit lowers the clock; traffic = "
                             "HBM bytes per launch from rocprofv3 --pmc FETCH_SIZE and WRITE_SIZE, calibrated on a "
                             "1 GiB copy; breakdown = per operator kind, algorithmic work of one step / summed "
                             "event-timed duration of its calls (the same eager pass); "
                             "family_step_wide = the contraction family's fractions over the whole step (from "
                             "breakdown), next to the best launch quoted as `frac`; gemm_launches = every contraction "
                             "by position in that pass (the projections' weight gradients run as one launch over "
                             "all layers when the model's shapes are tile-aligned: their us_per_call is that launch's "
                             "duration divided by the layers); kernels = each backward operator alone at the configuration's "
                             "shape, 20 back-to-back launches between HIP events on the launch stream; "
                             "frac_time_weighted = FLOPs over time of all event-timed launches of the probe kernel's "
                             "instantiation in the step (dX of the gate/up and of the output projection, every layer), "
                             "beside the best launch quoted as `frac`",
                     "family_step_wide": family,
                     "breakdown": per_kind, "gemm_launches": launches, "kernels": kernels},
    }
    if not args.no_cpu_baseline:
        result["cpu_baseline"] = cpu_baseline(args.seed)
    print(json.dumps(result))
    return 0


if __name__ == "__main__":
    sys.exit(main())
