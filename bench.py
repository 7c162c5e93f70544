#!/usr/bin/env python3
"""Benchmark of the MI355X operator backend on the headline workload.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--no-cpu-baseline] [--no-extras] [--no-decode | --decode] [--train LIST]

Workload (BASELINE.json configs[2], the one the fused-attention TFLOP/s metric is quoted on):
standalone causal fused attention in fp32, batch 8, heads 16, seq 2048, head_dim 64, Q/K/V/dOut
i.i.d. N(0,1) from a fixed seed, scale 1/sqrt(64).  One "step" = forward O plus backward dQ, dK, dV
(bf_hip_attention_forward + bf_hip_attention_backward through the C ABI), inputs resident in HBM.

Prints ONE JSON line.  `value` = algorithmic FLOPs of a step (14*hd*P with P = B*H*S(S+1)/2 causal
pairs: 4*hd*P forward, 10*hd*P backward, the FlashAttention convention; exp/softmax not counted)
divided by the measured time per step.  `roofline` describes the dominant kernel (the key-tile-owner
backward kernel that produces dK and dV and leaves dS in HBM for the dQ kernel), timed live with HIP events on the stream the kernels run on.
`cpu_baseline` times the CPU reference on a bounded sample of the same workload on this host.
Everything on one GPU: this build has no multi-GPU path.
"""
from __future__ import annotations

import argparse
import ctypes
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

PEAK_FP32_MFMA_TFLOPS = 157.3   # MI355X dense fp32 matrix peak
PEAK_BF16_MFMA_TFLOPS = 2500.0  # MI355X dense bf16 matrix peak
PEAK_HBM_GBS = 8000.0           # MI355X HBM3E peak

# HBM bytes per launch of the dominant kernel: rocprofv3 --pmc FETCH_SIZE and WRITE_SIZE runs of this workload,
# each scaled by what the same counter reads for a plain 256 MiB copy (x2.000 and x1.000): 979 MB read +
# 1224 MB written (1095 MB of that is the dS hand-over; the read side moves between 0.6 and 1.0 GB from run to run
# with what the L2s happen to keep).  profiles/attention_c3_kernel_trace.md holds the commands
# and the raw counter values.
MEASURED_TRAFFIC_BYTES = {"attnBackwardDkvPipedKernel": 1969678618}
# Share of cycles with the matrix pipe busy, same kernel, same workload, by counter (same profile file)
MEASURED_MFMA_BUSY = {"attnBackwardDkvPipedKernel": 0.44}


def attention_flops(batch, heads, seq, hd):
    pairs = batch * heads * seq * (seq + 1) // 2
    # dkv: S, dP, dV, dK; dq: dS*K alone when dS is handed over, S and dP again when it is recomputed
    return {"fwd": 4 * hd * pairs, "bwd": 10 * hd * pairs, "dkv": 8 * hd * pairs, "dq": 2 * hd * pairs,
            "dq_recompute": 6 * hd * pairs, "pairs": pairs}


def time_region(bf, stream, fn, steps, warmup):
    """Mean milliseconds per call of fn() over `steps` calls, HIP events on `stream`."""
    for _ in range(warmup):
        fn()
    stream.synchronize()
    start, stop = bf.Event(), bf.Event()
    start.record(stream)
    for _ in range(steps):
        fn()
    stop.record(stream)
    stop.synchronize()
    return start.elapsed_ms(stop) / steps


def bench_attention(bf, steps, warmup):
    D, call = bf.DeviceTensor, bf.capi.call
    batch, heads, seq, hd = 8, 16, 2048, 64
    dim, scale = heads * hd, 1.0 / np.sqrt(np.float32(hd))
    rng = np.random.default_rng(42)
    gen = lambda: D.fromHost(rng.standard_normal((batch, seq, dim), dtype=np.float32))
    q, k, v, go = gen(), gen(), gen(), gen()
    out, dq, dk, dv = D((batch, seq, dim)), D((batch, seq, dim)), D((batch, seq, dim)), D((batch, seq, dim))
    m, l = D((batch, heads, seq)), D((batch, heads, seq))
    lse2, dvec = D((batch, heads, seq)), D((batch, heads, seq))
    stream = bf.Stream()
    sh = stream.handle
    dims = (batch, heads, seq, seq, dim, ctypes.c_float(scale), 0, sh)

    fwd = lambda: call("bf_hip_attention_forward", q.ptr, k.ptr, v.ptr, out.ptr, m.ptr, l.ptr, *dims)
    bwd = lambda: call("bf_hip_attention_backward", go.ptr, q.ptr, k.ptr, v.ptr, out.ptr, m.ptr, l.ptr, dq.ptr, dk.ptr,
                       dv.ptr, *dims)
    prep = lambda: call("bf_hip_attention_backward_prepare", out.ptr, go.ptr, m.ptr, l.ptr, lse2.ptr, dvec.ptr, batch,
                        heads, seq, dim, sh)
    # the two kernels bf_hip_attention_backward launches after prepare: dK/dV leaving dS behind, dQ from that dS
    ds_bytes = ctypes.c_size_t(0)
    call("bf_hip_attention_ds_bytes", batch, heads, seq, seq, ctypes.byref(ds_bytes))
    ds = D((ds_bytes.value // 4,))
    dkv = lambda: call("bf_hip_attention_backward_dkv_ds", go.ptr, q.ptr, k.ptr, v.ptr, lse2.ptr, dvec.ptr, dk.ptr, dv.ptr,
                       ds.ptr, *dims)
    dqk = lambda: call("bf_hip_attention_backward_dq_from_ds", ds.ptr, k.ptr, dq.ptr, *dims)
    # the route taken when the dS buffer does not fit: both kernels recompute S and dP
    dkv_re = lambda: call("bf_hip_attention_backward_dkv", go.ptr, q.ptr, k.ptr, v.ptr, lse2.ptr, dvec.ptr, dk.ptr, dv.ptr,
                          *dims)
    dq_re = lambda: call("bf_hip_attention_backward_dq", go.ptr, q.ptr, k.ptr, v.ptr, lse2.ptr, dvec.ptr, dq.ptr, *dims)

    def step():
        fwd()
        bwd()

    # the timed region of the contract: exactly `steps` steps between two synchronisations
    for _ in range(warmup):
        step()
    stream.synchronize()
    bf.capi.call("bf_hip_synchronize")
    t0 = time.perf_counter()
    start, stop = bf.Event(), bf.Event()
    start.record(stream)
    for _ in range(steps):
        step()
    stop.record(stream)
    stop.synchronize()
    bf.capi.call("bf_hip_synchronize")
    wall_ms = (time.perf_counter() - t0) * 1e3 / steps
    ms_step = start.elapsed_ms(stop) / steps

    # per-kernel durations, live, same stream
    per = {name: time_region(bf, stream, fn, steps, 1) for name, fn in
           (("forward", fwd), ("prepare", prep), ("dkv", dkv), ("dq", dqk), ("dkv_recompute", dkv_re),
            ("dq_recompute", dq_re))}
    fl = attention_flops(batch, heads, seq, hd)
    # the same pass with every product on the fp32 MFMA (bf_hip_attention_set_route(0)); everything above ran on the
    # default route, whose forward and dK/dV kernels put each fp32 product on the bf16 matrix pipe as six MFMAs
    call("bf_hip_attention_set_route", 0)
    try:
        fp32 = {"forward_ms": time_region(bf, stream, fwd, steps, 2), "dkv_ms": time_region(bf, stream, dkv, steps, 1),
                "step_ms": time_region(bf, stream, step, steps, 1)}
    finally:
        call("bf_hip_attention_set_route", 7)
    return {"ms_per_step": ms_step, "wall_ms_per_step": wall_ms, "kernel_ms": per, "flops": fl, "fp32_mfma_route": fp32,
            "shape": {"batch": batch, "heads": heads, "seq": seq, "head_dim": hd}}


def cpu_baseline_attention(seconds_budget=20.0):
    """The CPU reference (oracle/_ref, else the restatement) on a sample of (batch, head) slices at full
    sequence length; slices are independent, so FLOP/s on the sample is FLOP/s on the workload."""
    from oracle import bfo
    impl = bfo.reference() or bfo.oracle()
    kind = "reference" if impl.is_reference else "port"
    seq, hd = 2048, 64
    rng = np.random.default_rng(7)
    mk = lambda: rng.standard_normal((1, seq, hd), dtype=np.float32)
    q, k, v, go = mk(), mk(), mk(), mk()
    flops_slice = 14 * hd * (seq * (seq + 1) // 2)
    done, t0 = 0, time.perf_counter()
    while True:
        impl.attentionCoreForward(q, k, v, 1, 0.125, 0)
        impl.attentionCoreBackward(go, q, k, v, 1, 0.125, 0)
        done += 1
        elapsed = time.perf_counter() - t0
        if elapsed + elapsed / done > seconds_budget or done >= 8:
            break
    return {"value": round(flops_slice * done / elapsed / 1e12, 6), "unit": "TFLOP/s", "cores": 1, "kind": kind,
            "sample": f"{done} of 128 (batch, head) slices of the workload at full seq 2048, head_dim 64, fwd+bwd, "
                      f"{elapsed:.1f} s on one host core (the reference CPU backend is single-threaded)"}


def bench_extras(bf, steps):
    """Secondary figures (not part of `value`): the bandwidth-bound kernels at the sizes of the GPT-small and
    long-context configurations, priced in algorithmic bytes (every distinct input read once, every output
    written once), and the bf16 projection GEMM on N(0,1) operands."""
    D, call = bf.DeviceTensor, bf.capi.call
    stream = bf.Stream()
    sh = stream.handle
    rng = np.random.default_rng(3)
    extras = {}

    def timed(fn, warm):
        ms = time_region(bf, stream, fn, steps, warm)
        if ms * steps < 0.5:   # a region of a few hundred microseconds is mostly the events' own latency: time 2 ms of calls
            ms = time_region(bf, stream, fn, min(2000, int(2.0 / max(ms, 1e-3)) + 1), 0)
        return ms

    def hbm(name, nbytes, fn):
        ms = timed(fn, 2)
        gbs = nbytes / ms / 1e6
        extras[name] = {"ms": round(ms, 4), "GB/s": round(gbs, 1), "frac_hbm": round(gbs / PEAK_HBM_GBS, 3)}

    def rand(*shape, scale=1.0):
        return D.fromHost(rng.standard_normal(shape, dtype=np.float32) * np.float32(scale))

    # long-context hidden activation [16384, 8192] (512 MiB) and model-width rows [16384, 2048]
    rows, hid, dm = 16384, 8192, 2048
    x, g, y = rand(rows, hid), rand(rows, hid), D((rows, hid))
    bias = rand(hid)
    n = rows * hid
    hbm("silu_16384x8192", 8 * n, lambda: call("bf_hip_act_forward", x.ptr, y.ptr, n, bf.capi.ACT_SILU, sh))
    hbm("gelu_backward_16384x8192", 12 * n, lambda: call("bf_hip_act_backward", x.ptr, g.ptr, y.ptr, n, bf.capi.ACT_GELU, sh))
    hbm("add_bias_silu_16384x8192", 8 * n, lambda: call("bf_hip_add_bias_act", x.ptr, bias.ptr, y.ptr, rows, hid, bf.capi.ACT_SILU, sh))
    hbm("add_16384x8192", 12 * n, lambda: call("bf_hip_add", x.ptr, g.ptr, y.ptr, n, sh))
    hbm("accumulate_16384x8192", 12 * n, lambda: call("bf_hip_accumulate", y.ptr, g.ptr, n, sh))
    dbias = D((hid,))
    hbm("bias_grad_16384x8192", 4 * n, lambda: call("bf_hip_bias_grad", g.ptr, dbias.ptr, rows, hid, sh))
    half = D((rows, hid // 2))
    hbm("cvt_f32_bf16_16384x8192", 6 * n, lambda: call("bf_hip_cvt_f32_bf16", x.ptr, half.ptr, n, sh))
    hbm("cvt_f32_bf16_transpose_16384x8192", 6 * n, lambda: call("bf_hip_cvt_f32_bf16_transpose", x.ptr, half.ptr, rows, hid, sh))
    nr = rows * dm * 4   # [65536, 2048]: four blocks' worth of rows, 512 MiB
    hbm("rmsnorm_65536x2048", 8 * nr, lambda: call("bf_hip_rmsnorm", x.ptr, y.ptr, nr // dm, dm, sh))
    hbm("rmsnorm_backward_65536x2048", 12 * nr, lambda: call("bf_hip_rmsnorm_backward", x.ptr, g.ptr, y.ptr, nr // dm, dm, sh))
    hbm("softmax_65536x2048", 8 * nr, lambda: call("bf_hip_softmax", x.ptr, y.ptr, nr // dm, dm, sh))
    del x, g, y, half

    # the row kernels at the sizes a GPT-small step runs them (24 and 12 launches a step): 8192 tokens x 768 features
    # (25 MB a tensor: the last-level cache holds all of it, so these read faster than HBM could deliver) and the
    # feed-forward block's backward pass over 8192 x 3072
    rows_s, dm_s, hid_s = 8192, 768, 3072
    xs, gs, ads, ys = rand(rows_s, dm_s), rand(rows_s, dm_s), rand(rows_s, dm_s), D((rows_s, dm_s))
    ims = D((rows_s, dm_s), itemsize=2)
    ns = rows_s * dm_s
    hbm("rmsnorm_to_image_8192x768", 6 * ns, lambda: call("bf_hip_rmsnorm_img", xs.ptr, None, ims.ptr, rows_s, dm_s, sh))
    hbm("rmsnorm_backward_add_with_image_8192x768", 18 * ns,
        lambda: call("bf_hip_rmsnorm_backward_add_img", xs.ptr, gs.ptr, ads.ptr, ys.ptr, ims.ptr, rows_s, dm_s, sh))
    zs, dhs, bs_ = rand(rows_s, hid_s), rand(rows_s, hid_s), rand(hid_s)
    dzs = D((rows_s, hid_s))
    dbs = D((hid_s,))
    nh = rows_s * hid_s
    hbm("add_bias_gelu_backward_8192x3072", 12 * nh,
        lambda: call("bf_hip_add_bias_act_backward", zs.ptr, bs_.ptr, dhs.ptr, dzs.ptr, dbs.ptr, rows_s, hid_s, bf.capi.ACT_GELU, sh))
    del xs, gs, ads, ys, ims, zs, dhs, dzs

    # GPT-small logits [8192, 32000] (0.98 GiB): sparse cross-entropy reads logits once and writes the gradient
    rows, vocab, dim = 8192, 32000, 768
    logits, grad = rand(rows, vocab), D((rows, vocab))
    target = D.fromHost(rng.integers(0, vocab, rows).astype(np.float32))
    loss = D.zeros((1,))
    hbm("cross_entropy_sparse_8192x32000", 8 * rows * vocab,
        lambda: call("bf_hip_cross_entropy_sparse", logits.ptr, target.ptr, grad.ptr, loss.ptr, rows, vocab, 0, sh))
    del logits, grad
    # long-context logits [16384, 50257] (3.07 GiB): rows of odd length, 16-byte accesses through a per-row shift
    rows_lc, vocab_lc = 16384, 50257
    logits, grad = rand(rows_lc, vocab_lc), D((rows_lc, vocab_lc))
    target_lc = D.fromHost(rng.integers(0, vocab_lc, rows_lc).astype(np.float32))
    hbm("cross_entropy_sparse_16384x50257", 8 * rows_lc * vocab_lc,
        lambda: call("bf_hip_cross_entropy_sparse", logits.ptr, target_lc.ptr, grad.ptr, loss.ptr, rows_lc, vocab_lc, 0, sh))
    del logits, grad

    # embedding table [32000, 768]: gather of 8192 tokens; scatter-add backward writes the whole table gradient
    table, dtable = rand(vocab, dim), D((vocab, dim))
    ids = D.fromHost(rng.integers(0, vocab, rows).astype(np.float32))
    out, gout = D((rows, dim)), rand(rows, dim)
    hbm("embedding_forward_8192x768", rows * dim * 8 + rows * 4,
        lambda: call("bf_hip_embedding_forward", ids.ptr, table.ptr, out.ptr, rows, vocab, dim, sh))
    hbm("embedding_backward_8192x768_into_32000x768", rows * dim * 4 + vocab * dim * 4,
        lambda: call("bf_hip_embedding_backward", ids.ptr, gout.ptr, dtable.ptr, rows, vocab, dim, sh))

    # AdamW over the GPT-small parameter set (134 951 168 values in 76 tensors): 28 bytes per parameter
    counts = [vocab * dim, 1024 * dim] + [dim * dim] * 48 + [dim * 3072, 3072, 3072 * dim, dim] * 12 + [dim * vocab, vocab]
    total = sum(counts)
    pool = [D.zeros((total,)) for _ in range(4)]   # params, grads, m, v as slices of four big buffers
    offs = np.concatenate([[0], np.cumsum(counts)[:-1]])
    arr = lambda t: (ctypes.c_void_p * len(counts))(*[t.ptr.value + int(o) * 4 if hasattr(t.ptr, "value") else t.ptr + int(o) * 4 for o in offs])
    ps, gs, ms_, vs = (arr(t) for t in pool)
    cn = (ctypes.c_size_t * len(counts))(*counts)
    hbm("adamw_134951168_params", 28 * total,
        lambda: call("bf_hip_adamw_multi", ps, gs, ms_, vs, cn, len(counts), 1, ctypes.c_float(1e-3), ctypes.c_float(0.9),
                     ctypes.c_float(0.999), ctypes.c_float(1e-8), ctypes.c_float(0.01), sh))
    hbm("zero_multi_134951168_params", 4 * total, lambda: call("bf_hip_zero_multi", gs, cn, len(counts), sh))
    del pool

    # what the matrix pipes deliver with nothing else running: the K loop of the 256 x 256 tile with its operand fragments
    # held in registers (random N(0,1) bf16 values), one workgroup of eight wavefronts per compute unit, for both bf16 MFMA
    # shapes; `implied_clock_ghz` is the clock at which 4096 flop per clock and compute unit give that rate
    cus = bf.capi.device_props(0).compute_units
    operands = D((32768,), itemsize=2)
    call("bf_hip_cvt_f32_bf16", rand(32768).ptr, operands.ptr, 32768, None)
    sink = D((cus * 512,))
    ceiling = {}
    k_steps = 2048   # 2048 steps of 2*256*256*64 flop per workgroup: ~3 ms a launch, as long as the largest product below
    for shape, name in ((0, "32x32x16"), (1, "16x16x32")):
        ms = timed(lambda: call("bf_hip_mfma_only_loop", operands.ptr, sink.ptr, shape, cus, k_steps, sh), 3)
        tf = 2 * 256 * 256 * 64 * k_steps * cus / ms / 1e9
        ceiling[name] = {"ms": round(ms, 4), "TFLOP/s": round(tf, 1), "frac_bf16_mfma": round(tf / PEAK_BF16_MFMA_TFLOPS, 3),
                         "implied_clock_ghz": round(tf * 1e12 / (4096 * cus) / 1e9, 3)}
    extras["mfma_only_ceiling"] = {"what": "K loop of the shipped 256x256x64 bf16 tile, operands in registers (no LDS, no global memory), "
                                           f"{cus} workgroups x 8 wavefronts, {k_steps} K steps a launch, N(0,1) operands", **ceiling}
    ceiling_tf = ceiling["32x32x16"]["TFLOP/s"]   # the instruction the shipped kernels issue

    # bf16 projection GEMM (C2 shape and a long-context shape), operands N(0,1) / N(0,1/64) rounded to bf16
    def gemm(m, n_, k):
        a, w = rand(m, k), rand(k, n_, scale=1 / 64)
        abf, wbf, c = D((m, k), itemsize=2), D((n_, k), itemsize=2), D((m, n_))
        call("bf_hip_cvt_f32_bf16", a.ptr, abf.ptr, m * k, None)
        call("bf_hip_cvt_f32_bf16_transpose", w.ptr, wbf.ptr, k, n_, None)
        ms = timed(lambda: call("bf_hip_gemm_bf16_nt", abf.ptr, wbf.ptr, c.ptr, m, n_, k, sh), 3)
        tf = 2 * m * n_ * k / ms / 1e9
        extras[f"gemm_bf16_{m}x{n_}x{k}"] = {"ms": round(ms, 4), "TFLOP/s": round(tf, 1), "frac_bf16_mfma": round(tf / PEAK_BF16_MFMA_TFLOPS, 3),
                                             "frac_of_measured_mfma_ceiling": round(tf / ceiling_tf, 3)}
        ms = timed(lambda: call("bf_hip_matmul_bf16", a.ptr, w.ptr, c.ptr, m, k, n_, 1, sh), 3)
        extras[f"matmul_bf16_fp32_io_{m}x{n_}x{k}"] = {"ms": round(ms, 4), "TFLOP/s": round(2 * m * n_ * k / ms / 1e9, 1)}
    # fused attention at the other shapes the library serves: the GPT-small and long-context layers, and head dims
    # above 128 (fp32-MFMA kernels padded to 192 or 256); forward, dK/dV with the dS hand-over, dQ from dS
    def attention(batch, heads, seq, hd):
        dim, scale = heads * hd, 1.0 / np.sqrt(np.float32(hd))
        q, k, v, go = (rand(batch, seq, dim) for _ in range(4))
        out, dq, dk, dv = (D((batch, seq, dim)) for _ in range(4))
        m, l, lse2, dvec = (D((batch, heads, seq)) for _ in range(4))
        dims = (batch, heads, seq, seq, dim, ctypes.c_float(scale), 0, sh)
        ds_bytes = ctypes.c_size_t(0)
        call("bf_hip_attention_ds_bytes", batch, heads, seq, seq, ctypes.byref(ds_bytes))
        ds = D((ds_bytes.value // 4,))
        fwd = lambda: call("bf_hip_attention_forward", q.ptr, k.ptr, v.ptr, out.ptr, m.ptr, l.ptr, *dims)
        fwd()
        call("bf_hip_attention_backward_prepare", out.ptr, go.ptr, m.ptr, l.ptr, lse2.ptr, dvec.ptr, batch, heads, seq, dim, sh)
        dkv = lambda: call("bf_hip_attention_backward_dkv_ds", go.ptr, q.ptr, k.ptr, v.ptr, lse2.ptr, dvec.ptr, dk.ptr, dv.ptr, ds.ptr, *dims)
        dqk = lambda: call("bf_hip_attention_backward_dq_from_ds", ds.ptr, k.ptr, dq.ptr, *dims)
        fl = attention_flops(batch, heads, seq, hd)
        t = {name: timed(fn, 5) for name, fn in (("forward", fwd), ("dkv", dkv), ("dq", dqk))}
        total = (fl["fwd"] + fl["dkv"] + fl["dq"]) / (t["forward"] + t["dkv"] + t["dq"]) / 1e9
        extras[f"attention_b{batch}_h{heads}_s{seq}_hd{hd}"] = {
            "ms": {name: round(ms, 4) for name, ms in t.items()},
            "TFLOP/s": {"forward": round(fl["fwd"] / t["forward"] / 1e9, 1), "dkv": round(fl["dkv"] / t["dkv"] / 1e9, 1),
                        "dq": round(fl["dq"] / t["dq"] / 1e9, 1), "forward_dkv_dq": round(total, 1)},
            "frac_fp32_mfma": round(total / PEAK_FP32_MFMA_TFLOPS, 3)}
    attention(8, 12, 1024, 64)
    attention(4, 16, 4096, 128)
    attention(4, 8, 2048, 192)
    attention(4, 8, 2048, 256)

    gemm(4096, 4096, 4096)
    gemm(16384, 8192, 2048)
    # GPT-small shapes: FFN up, FFN down / its input gradient (tall and narrow: 128-row tiles), FFN weight gradient (K slices)
    gemm(8192, 3072, 768)
    gemm(8192, 768, 3072)
    gemm(768, 3072, 8192)
    extras.update(vendor_gemm_reference([(4096, 4096, 4096), (16384, 8192, 2048), (8192, 3072, 768), (8192, 768, 3072), (768, 3072, 8192)]))
    return extras


_VENDOR_GEMM_CHILD = r"""
import json, sys, torch
shapes, peak = json.loads(sys.argv[1]), float(sys.argv[2])
out = {}
for m, n, k in shapes:
    a = torch.randn(m, k, device="cuda", dtype=torch.bfloat16)
    bt = (torch.randn(n, k, device="cuda", dtype=torch.bfloat16) / 64).t()   # the operand statistics of the kernels above
    run = lambda: torch.mm(a, bt, out_dtype=torch.float32)
    for _ in range(3):
        run()
    torch.cuda.synchronize()
    count = 10
    while True:   # as `timed` above: ten launches, or as many as make 2 ms
        start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        start.record()
        for _ in range(count):
            run()
        end.record()
        torch.cuda.synchronize()
        best = start.elapsed_time(end) / count
        if best * count >= 0.5 or count > 10:
            break
        count = max(11, int(2.0 / best))
    tf = 2 * m * n * k / best / 1e9
    out["vendor_library_gemm_bf16_%dx%dx%d" % (m, n, k)] = {"ms": round(best, 4), "TFLOP/s": round(tf, 1), "frac_bf16_mfma": round(tf / peak, 3)}
    del a, bt
print(json.dumps(out))
"""


def vendor_gemm_reference(shapes):
    """The same products (bf16 operands, second one stored transposed, fp32 result) through the vendor's GEMM library as
    PyTorch calls it (torch.mm -> hipBLASLt): what a library call delivers on this box, beside the hand-written kernels
    above.  In a child process (PyTorch brings a HIP runtime of its own, which cannot share a process with the one this
    library is linked to) while this one is idle, timed as the kernels above are.  Empty where that fails."""
    import signal
    import subprocess
    child = None
    try:
        # a session of its own, so that whatever helpers the child starts can be ended with it by process group
        child = subprocess.Popen([sys.executable, "-c", _VENDOR_GEMM_CHILD, json.dumps(shapes), str(PEAK_BF16_MFMA_TFLOPS)],
                                 stdout=subprocess.PIPE, stderr=subprocess.PIPE, text=True, start_new_session=True)
        out, _ = child.communicate(timeout=240)
        return json.loads(out.strip().splitlines()[-1])
    except Exception as err:   # no torch, an older torch without out_dtype, a time-out: no comparison
        return {"vendor_library_gemm_bf16": {"skipped": str(err)[:120]}}
    finally:
        if child is not None:
            try:
                os.killpg(child.pid, signal.SIGKILL)   # the group this function created: the child if it hangs, and anything it left
            except (ProcessLookupError, PermissionError):
                pass
            try:
                child.wait(timeout=10)
            except Exception:
                pass


def lm_layers(hl, vocab, dim, seq, heads, hidden, act, blocks):
    layers = [(hl.EMBEDDING, vocab, dim), (hl.POSITIONAL, seq)]
    for _ in range(blocks):
        layers += [(hl.ATTENTION, heads), (hl.FEEDFORWARD, hidden, act)]
    return layers + [(hl.LINEAR, vocab)]


TRAIN_CONFIGS = {
    # name: (vocab, d_model, heads, blocks, ffn, activation (0 silu / 1 gelu), seq, batch, bf16, optimizer)
    "tiny_lm": dict(vocab=256, dim=128, heads=4, blocks=1, ffn=512, act=1, seq=64, batch=8, bf16=False, adamw=True,
                    what="BASELINE.json configs[0]: tiny LM, fp32, full step with AdamW"),
    "gpt_small": dict(vocab=32000, dim=768, heads=12, blocks=12, ffn=3072, act=1, seq=1024, batch=8, bf16=True, adamw=True,
                      what="BASELINE.json configs[3]: GPT-small shape, bf16 projections + fp32 attention, full step with sparse CE and AdamW"),
    "long_context": dict(vocab=50257, dim=2048, heads=16, blocks=8, ffn=8192, act=0, seq=4096, batch=4, bf16=True, adamw=False,
                         what="BASELINE.json configs[4]: long-context LM, bf16 projections, forward + backward with sparse CE"),
}


MLP_CONFIG = dict(rows=4096, width=4096, what="BASELINE.json configs[1]: MLP [4096 tokens, 4096] -> linear(4096) -> silu -> "
                  "linear(4096), bf16 projections with fp32 accumulation, forward + backward against an MSE loss")


def bench_mlp(bf, steps, warmup):
    """The README MLP: forward, MSE loss and backward through the C++ operator layer's Model (no optimizer step)."""
    from blackforge_amd import hostlayer as hl
    rows, width = MLP_CONFIG["rows"], MLP_CONFIG["width"]
    model = hl.HostModel([(hl.LINEAR, width), (hl.SILU,), (hl.LINEAR, width)], input_features=width, use_bf16=True)
    rng = np.random.default_rng(42)
    for i, count in enumerate(model.counts):
        bias = model.names[i].endswith(".bias")
        model.set_value(i, np.zeros(count, np.float32) if bias else rng.standard_normal(count, dtype=np.float32) * np.float32(1 / 64))
    x = bf.DeviceTensor.fromHost(rng.standard_normal((rows, width), dtype=np.float32))
    y = bf.DeviceTensor.fromHost(rng.standard_normal((rows, width), dtype=np.float32))
    step = lambda: model.trainStep(x, y, hl.LOSS_MSE, 0, 0.0)
    for _ in range(warmup):
        step()
    bf.capi.call("bf_hip_synchronize")
    model.readLossSum()
    start, stop = bf.Event(), bf.Event()
    start.record(None)
    for _ in range(steps):
        step()
    stop.record(None)
    stop.synchronize()
    ms = start.elapsed_ms(stop) / steps
    # Five products are executed: two forward, the hidden tensor's gradient, two weight gradients.  The gradient with
    # respect to the model's INPUT (a sixth product, which the reference's Model::backward forms and drops) has no reader
    # and is not formed; the figures below count what runs.
    flops = 5 * 2 * rows * width * width
    # floor: the five products at the bf16 MFMA peak, plus the passes outside the GEMMs at the HBM peak (input image,
    # activation image, loss and its gradient with image, bias column sums, pre-activation gradient image: ~10 passes of
    # 4 bytes over [rows, width])
    floor_ms = flops / PEAK_BF16_MFMA_TFLOPS / 1e9 + 10 * rows * width * 4 / PEAK_HBM_GBS / 1e6
    return {"workload": MLP_CONFIG["what"], "tokens_per_s": round(rows / (ms * 1e-3), 1), "ms_per_step": round(ms, 3), "tokens": rows,
            "algorithmic_tflop_per_step": round(flops / 1e12, 4), "tflops": round(flops / (ms * 1e-3) / 1e12, 2),
            "products": "5 of 4096^3 executed (forward x2, hidden gradient, two weight gradients); the input gradient, a sixth product "
                        "nobody reads, is not formed, and is not counted",
            "mean_loss": round(model.readLossSum() / (steps * rows * width), 4),
            "roofline": {"bound": "mfma", "achieved": round(flops / ms / 1e9, 2), "peak": round(flops / floor_ms / 1e9, 2), "unit": "TFLOP/s",
                         "frac": round(floor_ms / ms, 4), "floor_ms": round(floor_ms, 3),
                         "note": "peak = executed FLOPs / (five products at the bf16 MFMA peak + 10 fp32-sized passes over [rows, width] at the HBM peak)"}}


def cpu_baseline_mlp():
    """The reference CPU backend on the MLP: cpu::Model linear -> silu -> linear with an MSE loss on a sample of rows
    (its cost is linear in the row count)."""
    from oracle import bfo
    impl = bfo.reference() or bfo.oracle()
    rows, width, sample = MLP_CONFIG["rows"], MLP_CONFIG["width"], 16
    rng = np.random.default_rng(5)
    model = impl.model([(bfo.LINEAR, width), (bfo.SILU,), (bfo.LINEAR, width)], input_features=width)
    for i, count in enumerate(model.counts):
        model.value(i)[:] = np.resize(rng.standard_normal(4099, dtype=np.float32) * np.float32(1 / 64), count)
    x = rng.standard_normal((sample, width), dtype=np.float32)
    y = rng.standard_normal((sample, width), dtype=np.float32)
    t0 = time.perf_counter()
    model.zeroGrad()
    out = model.forward(x, out_capacity=x.size)
    _, grad = impl.meanSquaredError(out.reshape(sample, width), y)
    model.backward(grad)
    elapsed = time.perf_counter() - t0
    return {"value": round(sample / elapsed, 3), "unit": "tokens/s", "cores": 1, "kind": "reference" if impl.is_reference else "port",
            "extrapolated": True,
            "sample": f"{sample} of {rows} rows through cpu::Model (forward, MSE, backward) in {elapsed:.2f} s on one host core; rows are independent"}


def train_step_flops(c):
    """Algorithmic FLOPs of one step: 6*tokens*(matmul weights) + 14*hd*P per attention layer."""
    tokens = c["batch"] * c["seq"]
    weights = c["blocks"] * (4 * c["dim"] ** 2 + 2 * c["dim"] * c["ffn"]) + c["dim"] * c["vocab"]
    pairs = c["batch"] * c["heads"] * c["seq"] * (c["seq"] + 1) // 2
    return 6 * tokens * weights + c["blocks"] * 14 * (c["dim"] // c["heads"]) * pairs


def train_step_roofline(c, ms):
    """The step against its matrix-pipe floor: bf16 MFMA peak for the projections, fp32 MFMA peak for the attention core
    (the elementwise and loss kernels are HBM-bound and add to the floor what their algorithmic bytes cost at HBM peak)."""
    tokens = c["batch"] * c["seq"]
    weights = c["blocks"] * (4 * c["dim"] ** 2 + 2 * c["dim"] * c["ffn"]) + c["dim"] * c["vocab"]
    pairs = c["batch"] * c["heads"] * c["seq"] * (c["seq"] + 1) // 2
    gemm_flops = 6 * tokens * weights
    attn_flops = c["blocks"] * 14 * (c["dim"] // c["heads"]) * pairs
    peak_gemm = PEAK_BF16_MFMA_TFLOPS if c["bf16"] else PEAK_FP32_MFMA_TFLOPS
    floor_ms = gemm_flops / peak_gemm / 1e9 + attn_flops / PEAK_FP32_MFMA_TFLOPS / 1e9
    # bandwidth part: cross-entropy 8 B per logit, AdamW 28 B per parameter, per block ~14 passes over [tokens, dim] and
    # ~5 over [tokens, ffn] in fp32 (normalisations, residuals, activations and the bf16 images the GEMMs read)
    params = weights + c["vocab"] * c["dim"] + c["seq"] * c["dim"]
    hbm_bytes = 8 * tokens * c["vocab"] + (28 * params if c["adamw"] else 4 * params) + \
        c["blocks"] * tokens * 4 * (14 * c["dim"] + 5 * c["ffn"])
    floor_ms += hbm_bytes / PEAK_HBM_GBS / 1e6
    return {"bound": "mfma", "achieved": round((gemm_flops + attn_flops) / ms / 1e9, 2),
            "peak": round((gemm_flops + attn_flops) / floor_ms / 1e9, 2), "unit": "TFLOP/s", "frac": round(floor_ms / ms, 4),
            "floor_ms": round(floor_ms, 3),
            "note": "peak = algorithmic FLOPs / (projection FLOPs at the bf16 MFMA peak + attention FLOPs at the fp32 MFMA peak "
                    "+ elementwise, loss and optimizer bytes at the HBM peak)"}


def cpu_baseline_train_step(name):
    """The reference CPU backend's training step, measured on a bounded sample and extrapolated (it would take an hour or
    more at full size): cpu::Model with ONE block + the LM head and with the LM head alone, batch 1, a short sequence at
    full widths and vocabulary (projection cost is linear in tokens), plus the attention core of one (batch, head) slice
    at a sequence length the host finishes in seconds (its cost is quadratic in the sequence length)."""
    from oracle import bfo
    impl = bfo.reference() or bfo.oracle()
    c = TRAIN_CONFIGS[name]
    rng = np.random.default_rng(11)
    s0 = {"tiny_lm": c["seq"], "gpt_small": 32, "long_context": 8}[name]

    def timed_model(blocks, batch=1, seq=None):
        seq = seq or s0
        # the reference's feed-forward block is SiLU only; where the configuration says GELU the real reference is timed
        # with SiLU (same projections, one transcendental per hidden element either way)
        act = 0 if impl.is_reference else c["act"]
        model = impl.model(lm_layers(bfo, c["vocab"], c["dim"], c["seq"], c["heads"], c["ffn"], act, blocks))
        for i, count in enumerate(model.counts):   # the loops' cost does not depend on the values: a cheap non-constant fill
            model.value(i)[:] = np.resize(rng.standard_normal(4099, dtype=np.float32) * np.float32(0.02), count)
        ids = rng.integers(0, c["vocab"], (batch, seq)).astype(np.float32)
        tgt = rng.integers(0, c["vocab"], batch * seq).astype(np.float32)
        t0 = time.perf_counter()
        model.zeroGrad()
        logits = model.forward(ids, out_capacity=batch * seq * c["vocab"])
        _, grad = impl.softmaxCrossEntropySparse(logits.reshape(batch * seq, c["vocab"]), tgt)
        model.backward(grad)
        if c["adamw"]:
            model.adamwStep()
        return time.perf_counter() - t0

    if name == "tiny_lm":   # small enough to run whole
        step_s = min(timed_model(c["blocks"], c["batch"], c["seq"]) for _ in range(3))
        return {"value": round(c["batch"] * c["seq"] / step_s, 1), "unit": "tokens/s", "cores": 1,
                "kind": "reference" if impl.is_reference else "port", "extrapolated": False,
                "sample": ("feed-forward activation SiLU in place of GELU (the reference block has no GELU); " if impl.is_reference else "") +
                          f"the whole step (zeroGrad, forward, sparse CE, backward, AdamW) through cpu::Model, best of 3, {step_s * 1e3:.1f} ms on one host core"}
    def timed_block():
        """One attention + feed-forward block alone on [1, s0, dim] features: forward, backward, optimizer."""
        act = 0 if impl.is_reference else c["act"]
        model = impl.model([(bfo.ATTENTION, c["heads"]), (bfo.FEEDFORWARD, c["ffn"], act)], input_features=c["dim"])
        for i, count in enumerate(model.counts):
            model.value(i)[:] = np.resize(rng.standard_normal(4099, dtype=np.float32) * np.float32(0.02), count)
        x = rng.standard_normal((1, s0, c["dim"]), dtype=np.float32)
        g = rng.standard_normal((1, s0, c["dim"]), dtype=np.float32)
        t0 = time.perf_counter()
        model.zeroGrad()
        model.forward(x, out_capacity=x.size)
        model.backward(g)
        if c["adamw"]:
            model.adamwStep()
        return time.perf_counter() - t0

    # embedding + head + loss at two token counts: a cost per step (zeroing and scatter-add over the whole embedding table,
    # the optimizer over the parameters) and a cost per token
    t_head, t_head2 = timed_model(0), timed_model(0, 1, 2 * s0)
    head_per_token = max(t_head2 - t_head, 0.0) / s0
    head_fixed = max(t_head - head_per_token * s0, 0.0)
    t_block = timed_block()
    hd = c["dim"] // c["heads"]
    s_attn = min(c["seq"], 1024)
    mk = lambda: rng.standard_normal((1, s_attn, hd), dtype=np.float32)
    q, k, v, go = mk(), mk(), mk(), mk()
    t0 = time.perf_counter()
    impl.attentionCoreForward(q, k, v, 1, hd ** -0.5, 0)
    impl.attentionCoreBackward(go, q, k, v, 1, hd ** -0.5, 0)
    t_core = (time.perf_counter() - t0) * (c["seq"] / s_attn) ** 2
    # per step: every token passes the head once and every block once; every (batch, head) slice runs the attention core
    tokens = c["batch"] * c["seq"]
    step_s = head_fixed + tokens * head_per_token + tokens / s0 * c["blocks"] * t_block + c["blocks"] * c["batch"] * c["heads"] * t_core
    return {"value": round(c["batch"] * c["seq"] / step_s, 3), "unit": "tokens/s", "cores": 1,
            "kind": "reference" if impl.is_reference else "port", "extrapolated": True,
            "sample": ("feed-forward activation SiLU in place of GELU (the reference block has no GELU); " if impl.is_reference and c["act"] == 1 else "") +
                      f"cpu::Model of one attention + feed-forward block, and of embedding + LM head + loss, each on batch 1 x {s0} tokens at full widths "
                      f"(head {head_fixed:.2f} s per step + {head_per_token * 1e3:.1f} ms per token from runs at {s0} and {2 * s0} tokens, block {t_block:.2f} s), "
                      f"scaled by tokens x {c['blocks']} blocks; attention core of one "
                      f"(batch, head) slice at seq {s_attn} ({t_core * (s_attn / c['seq']) ** 2:.2f} s) scaled quadratically to seq {c['seq']} "
                      f"and by {c['batch'] * c['heads']} slices x {c['blocks']} blocks; one host core, extrapolated step {step_s:.0f} s"}


def bench_train_step(bf, name, steps, warmup, with_graph=True):
    """One training step of the C++ operator layer's Model (hip::Model) through its C harness."""
    from blackforge_amd import hostlayer as hl
    c = TRAIN_CONFIGS[name]
    model = hl.HostModel(lm_layers(hl, c["vocab"], c["dim"], c["seq"], c["heads"], c["ffn"], c["act"], c["blocks"]), use_bf16=c["bf16"])
    rng = np.random.default_rng(42)
    n_params = 0
    for i, count in enumerate(model.counts):
        n_params += count
        is_bias = model.names[i].endswith((".bias", ".b1", ".b2"))
        model.set_value(i, np.zeros(count, np.float32) if is_bias else rng.standard_normal(count, dtype=np.float32) * np.float32(0.02))
    D = bf.DeviceTensor
    ids = D.fromHost(rng.integers(0, c["vocab"], (c["batch"], c["seq"])).astype(np.float32))
    tgt = D.fromHost(rng.integers(0, c["vocab"], c["batch"] * c["seq"]).astype(np.float32))
    opt = 1 if c["adamw"] else 0
    step = lambda: model.trainStep(ids, tgt, hl.LOSS_SPARSE_CE, opt, 1e-3)
    for _ in range(warmup):
        step()
    bf.capi.call("bf_hip_synchronize")
    model.readLossSum()
    start, stop = bf.Event(), bf.Event()
    t0 = time.perf_counter()
    start.record(None)
    for _ in range(steps):
        step()
    stop.record(None)
    stop.synchronize()
    bf.capi.call("bf_hip_synchronize")
    wall_ms = (time.perf_counter() - t0) * 1e3 / steps
    ms = start.elapsed_ms(stop) / steps
    loss = model.readLossSum() / (steps * c["batch"] * c["seq"])
    tokens = c["batch"] * c["seq"]
    flops = train_step_flops(c)
    out = {"workload": c["what"], "tokens_per_s": round(tokens / (ms * 1e-3), 1), "ms_per_step": round(ms, 3),
           "wall_ms_per_step": round(wall_ms, 3), "tokens": tokens, "parameters": n_params,
           "algorithmic_tflop_per_step": round(flops / 1e12, 4), "tflops": round(flops / (ms * 1e-3) / 1e12, 2),
           "mean_loss": round(float(loss), 4), "roofline": train_step_roofline(c, ms)}
    if name == "tiny_lm" and with_graph:
        # the same step recorded once as a HIP graph and replayed (hip::CapturedTrainStep): ~95 launches become one submission
        recorded = model.captureTrainStep(ids, tgt, hl.LOSS_SPARSE_CE, opt, 1e-3)
        replays = max(steps, 200)
        for _ in range(max(warmup, 10)):
            recorded.run(1e-3)
        bf.capi.call("bf_hip_synchronize")
        t0 = time.perf_counter()
        start.record(None)   # the default stream orders itself with the recording's stream
        for _ in range(replays):
            recorded.run(1e-3)
        stop.record(None)
        stop.synchronize()
        wall = (time.perf_counter() - t0) * 1e3 / replays
        rms = start.elapsed_ms(stop) / replays
        model.readLossSum()
        recorded.close()
        out["recorded_step"] = {"what": "the same step replayed from a HIP graph (bit-identical results)", "ms_per_step": round(rms, 4),
                                "wall_ms_per_step": round(wall, 4), "tokens_per_s": round(tokens / (rms * 1e-3), 1), "replays": replays}
    return out


def bench_decode(bf, tokens=32, prompt=1024):
    """Incremental decoding (Model::forwardIncremental, model.cu:385-424) of the GPT-small shape, one sequence: a prompt,
    then `tokens` single-token steps, timed.  A step reads every Linear weight once (bf16 images in bf16 mode, 2 bytes a
    parameter; fp32 otherwise) and the cached keys and values (fp32): that is the algorithmic traffic the rate is set against."""
    from blackforge_amd import hostlayer as hl
    c = TRAIN_CONFIGS["gpt_small"]
    out = {}
    for mode, bf16 in (("fp32", False), ("bf16", True)):
        model = hl.HostModel(lm_layers(hl, c["vocab"], c["dim"], 2 * prompt, c["heads"], c["ffn"], c["act"], c["blocks"]), use_bf16=bf16)
        rng = np.random.default_rng(42)
        for i, count in enumerate(model.counts):
            model.set_value(i, np.resize(rng.standard_normal(65537, dtype=np.float32) * np.float32(0.02), count))
        D = bf.DeviceTensor
        prompt_first = D.fromHost(rng.integers(0, c["vocab"], (1, prompt)).astype(np.float32))
        prompt_ms = 1e9
        for _ in range(4):   # the prompt's pass (the time to the first token), best of the runs after the first
            model.resetGenerationState()
            bf.capi.call("bf_hip_synchronize")
            t0 = time.perf_counter()
            model.forwardIncremental(prompt_first, read=False)
            bf.capi.call("bf_hip_synchronize")
            if _ > 0:
                prompt_ms = min(prompt_ms, (time.perf_counter() - t0) * 1e3)
        # greedy generation as the reference's `generate` runs it (main.cpp:594-617): the next token is the device-side
        # argmax of the last position's logits, one index read back per step
        def step():
            token = D.fromHost(np.array([[float(model.argmaxLast(c["vocab"]))]], np.float32))
            model.forwardIncremental(token, read=False)
        for _ in range(3):
            step()
        bf.capi.call("bf_hip_synchronize")
        t0 = time.perf_counter()
        for _ in range(tokens):
            step()
        bf.capi.call("bf_hip_synchronize")
        ms = (time.perf_counter() - t0) * 1e3 / tokens
        # the same generation with token and position kept on the device (Model::generateGreedy: no read-back inside the
        # loop); the prompt is inside the clock, so two lengths are timed and their difference is the cost of the extra tokens
        prompt_ids = D.fromHost(rng.integers(0, c["vocab"], (1, prompt)).astype(np.float32))
        model.generateGreedy(prompt_ids, 4)
        times = {}
        for n in (tokens, 9 * tokens):
            bf.capi.call("bf_hip_synchronize")
            t0 = time.perf_counter()
            model.generateGreedy(prompt_ids, n)
            times[n] = (time.perf_counter() - t0) * 1e3
        on_device_ms = (times[9 * tokens] - times[tokens]) / (8 * tokens)
        matrix_params = c["blocks"] * (4 * c["dim"] ** 2 + 2 * c["dim"] * c["ffn"]) + c["dim"] * c["vocab"]
        context = prompt + 3 + tokens // 2
        bytes_per_token = matrix_params * (2 if bf16 else 4) + c["blocks"] * 2 * context * c["dim"] * 4
        gbs = bytes_per_token / (ms * 1e-3) / 1e9
        on_device_context = prompt + 5 * tokens
        on_device_bytes = matrix_params * (2 if bf16 else 4) + c["blocks"] * 2 * on_device_context * c["dim"] * 4
        on_device_gbs = on_device_bytes / (on_device_ms * 1e-3) / 1e9
        out[mode] = {"ms_per_token": round(ms, 4), "tokens_per_s": round(1e3 / ms, 1), "context": context,
                     "prompt_ms": round(prompt_ms, 3), "prompt_tokens_per_s": round(prompt / (prompt_ms * 1e-3), 1),
                     "algorithmic_bytes_per_token": bytes_per_token,
                     "roofline": {"bound": "hbm", "achieved": round(gbs, 1), "peak": PEAK_HBM_GBS, "unit": "GB/s", "frac": round(gbs / PEAK_HBM_GBS, 4)},
                     "on_device_loop": {"what": "Model::generateGreedy: argmax, token and position stay on the device, the host launches ahead; "
                                               f"(time of {9 * tokens} tokens - time of {tokens}) / {8 * tokens}",
                                       "ms_per_token": round(on_device_ms, 4), "tokens_per_s": round(1e3 / on_device_ms, 1), "context": on_device_context,
                                       "algorithmic_bytes_per_token": on_device_bytes,
                                       "roofline": {"bound": "hbm", "achieved": round(on_device_gbs, 1), "peak": PEAK_HBM_GBS, "unit": "GB/s",
                                                    "frac": round(on_device_gbs / PEAK_HBM_GBS, 4)}}}
        del model
    out["workload"] = (f"GPT-small shape (BASELINE.json configs[3]), one sequence, prompt of {prompt} tokens, then {tokens} single-token steps "
                       "of greedy generation: device-side argmax of the last logits, then Model::forwardIncremental on that token (wall clock around "
                       "the steps: about a hundred launches a token, bounded by their latency)")
    return out


def cpu_baseline_decode(prompt=1024):
    """The reference CPU backend on one decoding step of the same model (fp32, one host core): ONE block's incremental
    attention over a cache of `prompt` positions and its feed-forward block, timed and multiplied by the twelve blocks,
    plus the head once (the embedding row and the positional add are negligible beside them)."""
    from oracle import bfo
    impl = bfo.reference() or bfo.oracle()
    c = TRAIN_CONFIGS["gpt_small"]
    rng = np.random.default_rng(12)
    dim, ffn, vocab = c["dim"], c["ffn"], c["vocab"]
    fill = lambda *shape: np.resize(rng.standard_normal(4099, dtype=np.float32) * np.float32(0.02), shape)
    x = rng.standard_normal((1, 1, dim), dtype=np.float32)
    wq, wk, wv, wo = (fill(dim, dim) for _ in range(4))
    kc, vc = rng.standard_normal((1, prompt, dim), dtype=np.float32), rng.standard_normal((1, prompt, dim), dtype=np.float32)
    w1, b1, w2, b2 = fill(dim, ffn), fill(ffn), fill(ffn, dim), fill(dim)
    head_w, head_b = fill(dim, vocab), fill(vocab)
    best_block, best_head = 1e30, 1e30
    for _ in range(3):
        t0 = time.perf_counter()
        y, _, _ = impl.selfAttentionIncremental(x, wq, wk, wv, wo, c["heads"], kc, vc)
        impl.feedForward(y, w1, b1, w2, b2, 0)
        t1 = time.perf_counter()
        impl.linear(y.reshape(1, dim), head_w, head_b)
        t2 = time.perf_counter()
        best_block, best_head = min(best_block, t1 - t0), min(best_head, t2 - t1)
    token_s = c["blocks"] * best_block + best_head
    return {"value": round(1.0 / token_s, 2), "unit": "tokens/s", "cores": 1, "kind": "reference" if impl.is_reference else "port",
            "extrapolated": True,
            "sample": f"one block (selfAttentionIncremental over {prompt} cached positions + feedForward, SiLU) {best_block * 1e3:.1f} ms x {c['blocks']} blocks + "
                      f"the head {best_head * 1e3:.1f} ms = {token_s * 1e3:.0f} ms a token on one host core, best of 3"}


def extras_summary(extras):
    """The north-star targets in three numbers: the bf16 projection at 4096^3 against the bf16 MFMA peak, and the worst and
    the median bandwidth kernel against the HBM peak."""
    hbm = sorted((v["frac_hbm"], k) for k, v in extras.items() if "frac_hbm" in v)
    gemms = {k: v["frac_bf16_mfma"] for k, v in extras.items() if "frac_bf16_mfma" in v and not k.startswith("vendor_")}
    vendor = {k[len("vendor_library_"):]: v["frac_bf16_mfma"] for k, v in extras.items() if "frac_bf16_mfma" in v and k.startswith("vendor_")}
    out = {"bf16_gemm_frac_of_peak": gemms}
    if vendor:
        out["vendor_library_frac_of_peak"] = vendor
    if hbm:
        out["hbm_min"] = {"kernel": hbm[0][1], "frac": hbm[0][0]}
        out["hbm_median"] = {"kernel": hbm[len(hbm) // 2][1], "frac": hbm[len(hbm) // 2][0]}
        out["hbm_below_0.70"] = [k for f, k in hbm if f < 0.70]
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=40)
    ap.add_argument("--warmup", type=int, default=20, help="untimed steps first; the chip needs some 30 ms of work to reach its "
                    "steady clocks (3 warm-up steps read 6 %% slower than 20)")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-extras", action="store_true", help="skip the bandwidth kernels and the bf16 GEMMs")
    ap.add_argument("--no-decode", action="store_true", help="skip the incremental-decoding leg (--no-extras skips it too)")
    ap.add_argument("--decode", action="store_true", help="run the incremental-decoding leg even with --no-extras")
    ap.add_argument("--no-graph", action="store_true", help="skip the recorded (HIP graph) variant of the tiny-LM step; for runs under a "
                    "profiler, whose kernel tracing does not survive a stream capture on this stack")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="also launch one plain 256 MiB copy (bf_hip_scale by 1.0) so that a counter run of this command "
                         "holds a kernel of known HBM traffic to scale FETCH_SIZE / WRITE_SIZE by")
    ap.add_argument("--train", default="gpt_small,long_context,mlp,tiny_lm", help="comma list of train-step workloads to add (tiny_lm, mlp, gpt_small, "
                    "long_context) or 'none'")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build runs on one GPU only (no collectives, no sharding); use --gpus 1")

    import blackforge_amd as bf
    bf.capi.load()
    if bf.capi.device_count() < 1:
        sys.exit("bench.py: no HIP device visible; the operator library has no CPU fallback")
    props = bf.capi.device_props(0)

    if args.calibrate_copy:
        n = 64 * 1024 * 1024   # 256 MiB read + 256 MiB written by flat4Kernel<ScaleOp>
        src, dst = bf.DeviceTensor.zeros((n,)), bf.DeviceTensor((n,))
        bf.capi.call("bf_hip_scale", src.ptr, ctypes.c_float(1.0), dst.ptr, n, None)
        bf.capi.call("bf_hip_synchronize")
        del src, dst
    res = bench_attention(bf, args.steps, args.warmup)
    fl = res["flops"]
    total_flops = fl["fwd"] + fl["bwd"]
    value = total_flops / (res["ms_per_step"] * 1e-3) / 1e12
    dkv_ms = res["kernel_ms"]["dkv"]
    achieved = fl["dkv"] / (dkv_ms * 1e-3) / 1e12
    line = {
        "metric": "fused-attn fwd+bwd TFLOP/s",
        "value": round(value, 3),
        "unit": "TFLOP/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(res["ms_per_step"], 4),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f32",
        "data": "synthetic",
        "config": {"workload": "causal fused attention fwd+bwd, fp32 in and out, batch 8, heads 16, seq 2048, head_dim 64 "
                               "(BASELINE.json configs[2])", **res["shape"],
                   "route": "default: every product (forward, dK/dV, dQ from the stored dS) as six bf16 MFMAs on operands split into "
                            "three bf16 terms (fp32 accuracy, fp32 accumulation)",
                   "precision": "fp32 inputs, outputs, statistics and accumulation; every product keeps all term products above 2^-24 "
                                "of it, and the parity tests hold this route to the same bounds against the CPU reference as the "
                                "fp32-MFMA route (fp32_mfma_route below: the same step with every product on v_mfma_f32_32x32x2_f32)"},
        # `achieved` counts the algorithm's fp32 flops (8 hd per visible pair), priced against the fp32 MFMA peak, the
        # published peak of the arithmetic type the path computes; the kernel issues six bf16 MFMA flops for each of them,
        # and `bf16_pipe` prices those against the bf16 peak
        "roofline": {"bound": "mfma", "kernel": "attnBackwardDkvPipedKernel<64,..,store dS> (dK, dV and the dS hand-over; key-tile owner)",
                     "achieved": round(achieved, 3), "peak": PEAK_FP32_MFMA_TFLOPS, "unit": "TFLOP/s",
                     "frac": round(achieved / PEAK_FP32_MFMA_TFLOPS, 4),
                     # what the kernel executes: six bf16 MFMA flops per algorithmic fp32 flop, on the bf16 matrix pipe;
                     # mfma_busy is the share of cycles the matrix pipe is busy by counter (SQ_VALU_MFMA_BUSY_CYCLES over
                     # GRBM_GUI_ACTIVE / 8 x 1024 SIMDs for this kernel on this workload, profiles/attention_c3_kernel_trace.md)
                     "executed": {"pipe": "bf16", "instruction": "v_mfma_f32_32x32x16_bf16", "flops_per_launch": 6 * fl["dkv"],
                                  "achieved": round(6 * achieved, 2), "peak": PEAK_BF16_MFMA_TFLOPS, "unit": "TFLOP/s",
                                  "frac_of_pipe": round(6 * achieved / PEAK_BF16_MFMA_TFLOPS, 4), "mfma_busy": MEASURED_MFMA_BUSY["attnBackwardDkvPipedKernel"]},
                     "traffic": MEASURED_TRAFFIC_BYTES["attnBackwardDkvPipedKernel"],
                     "traffic_source": "rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE runs of this kernel on this workload, recorded in "
                                       "profiles/attention_c3_kernel_trace.md (counters cannot be read from inside this run)",
                     "flops_per_launch": fl["dkv"], "launch_ms": round(dkv_ms, 4)},
        "frac_of_fp32_mfma_peak": round(value / PEAK_FP32_MFMA_TFLOPS, 4),
        "kernel_ms": {k: round(v, 4) for k, v in res["kernel_ms"].items()},
        "kernel_tflops": {"forward": round(fl["fwd"] / res["kernel_ms"]["forward"] / 1e9, 2),
                          "dkv": round(fl["dkv"] / res["kernel_ms"]["dkv"] / 1e9, 2),
                          "dq": round(fl["dq"] / res["kernel_ms"]["dq"] / 1e9, 2),
                          "dkv_recompute": round(fl["dkv"] / res["kernel_ms"]["dkv_recompute"] / 1e9, 2),
                          "dq_recompute": round(fl["dq_recompute"] / res["kernel_ms"]["dq_recompute"] / 1e9, 2)},
        "wall_ms_per_step": round(res["wall_ms_per_step"], 4),
        # bf_hip_attention_set_route(0), NOT what `value` measures: every product on v_mfma_f32_32x32x2_f32
        "fp32_mfma_route": {
            "forward_ms": round(res["fp32_mfma_route"]["forward_ms"], 4),
            "forward_tflops": round(fl["fwd"] / res["fp32_mfma_route"]["forward_ms"] / 1e9, 2),
            "dkv_ms": round(res["fp32_mfma_route"]["dkv_ms"], 4),
            "dkv_tflops": round(fl["dkv"] / res["fp32_mfma_route"]["dkv_ms"] / 1e9, 2),
            "dkv_frac_of_fp32_mfma_peak": round(fl["dkv"] / res["fp32_mfma_route"]["dkv_ms"] / 1e9 / PEAK_FP32_MFMA_TFLOPS, 4),
            "step_ms": round(res["fp32_mfma_route"]["step_ms"], 4),
            "step_tflops": round(total_flops / res["fp32_mfma_route"]["step_ms"] / 1e9, 2)},
        "device": {"name": props.name.decode(), "arch": props.arch.decode(), "compute_units": props.compute_units},
    }
    if args.train != "none":
        line["train_step"] = {name: (bench_mlp if name == "mlp" else lambda b, s_, w_: bench_train_step(b, name, s_, w_, not args.no_graph))(
                                  bf, max(3, args.steps // 2), max(1, args.warmup // 2))
                              for name in args.train.split(",")}
    if args.decode or not (args.no_decode or args.no_extras):
        line["decode"] = bench_decode(bf)
    if not args.no_extras:
        line["extras"] = bench_extras(bf, min(10, max(5, args.steps // 2)))   # ten launches a kernel: what profiles/hbm_kernels_and_gemm.md describes
        line["extras_summary"] = extras_summary(line["extras"])
    if not args.no_cpu_baseline:
        line["cpu_baseline"] = cpu_baseline_attention()
        line["cpu_baseline"]["host_cores"] = os.cpu_count()
        if "decode" in line:
            line["decode"]["cpu_baseline"] = cpu_baseline_decode()
        for name in line.get("train_step", {}):
            line["train_step"][name]["cpu_baseline"] = cpu_baseline_mlp() if name == "mlp" else cpu_baseline_train_step(name)
    print(json.dumps(line))


if __name__ == "__main__":
    main()
