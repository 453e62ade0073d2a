#!/usr/bin/env python3
"""Decode benchmark of the MI355X HipBackend path.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

Workload (the configuration the headline metric is quoted on):
Llama decode, dModel 2048, 16 layers, 32 heads (head dim 64), SwiGLU hidden 5632, vocab
32000, maxSeq 2048; weights = new LlamaModel(cfg, 42) (java.util.Random Gaussians x 0.1),
all matmul weights Q8; prompt = 512 ids from Random(3).nextInt(32000); batch-1 greedy decode
with a device-resident fp32 KV cache.  A step = one decoded token (one replay of the
per-token HIP graph).  Prints ONE JSON line.

Besides tok/s the line carries
  roofline     - the Q8 matvec kernel (the dominant kernel): algorithmic bytes per launch /
                 mean kernel duration, measured live with a start and a stop HIP event on every
                 dispatch of the per-token stream run in order on the model's own weights (1 GB of
                 distinct weights per token, so nothing is served from the 256 MB Infinity Cache) -
                 the quantity rocprofv3 --kernel-trace reports; `per_kernel` holds the same for
                 every kernel of the token, `floor` an empty kernel and a pure streaming read of the
                 very same weight buffers by the same method; the back-to-back launch period
                 (no events, launch cost hidden behind the previous kernel) is reported beside it
  cpu_baseline - the CPU oracle (a C restatement of the reference's CpuBackend + layers,
                 not the JVM) on this box's host cores, on a bounded sample of the workload
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0          # MI355X HBM3E, published
# HBM bytes read + written per matvec launch (mean over the 65 launches of one token).  rocprofv3 cannot collect
# counters over the decode stream on this build (profiles/README.md), so the figure is the algorithmic 15.40 MB times
# the fetched / algorithmic ratios its FETCH_SIZE counter gives for the same kernel on buffers of the same sizes in the
# isolated sweep (profiles/q8_matvec_c2_sweep_hbm_traffic.txt: 1.032 at 4.7 MB, 1.014-1.024 at 13 MB, 1.010 at 51 MB).
MATVEC_TRAFFIC_BYTES_PER_LAUNCH = 15_700_000


def q8_linear_bytes(k: int, n_rows: int) -> int:
    """Algorithmic bytes of one M = 1 Q8 matvec: int8 weights + one fp32 scale per 32 + x + y."""
    return k * n_rows + 4 * k * n_rows // 32 + 4 * k + 4 * n_rows


VARIANTS = {  # (K, Q8 rows) of the workload's five matvec shapes
    (2048, 6144): "qkv", (2048, 2048): "wo", (2048, 11264): "gate_up", (5632, 2048): "down", (2048, 32000): "lm_head"}


def decode_ops(stream):
    """(opcode, words) of every op of a fused command stream."""
    from deepj_amd import opcodes as op
    pos, ops = 0, []
    while pos < len(stream):
        code = int(stream[pos])
        n = op.FUSED_STRIDES[code]
        ops.append((code, [int(x) for x in stream[pos:pos + n]]))
        pos += n
    return ops


def matvec_roofline(model, position: int, iters: int = 12):
    """Per-kernel durations of one decoded token, measured live: the per-token stream runs in order (1 GB of distinct
    weights per pass, so nothing is served from the 256 MB Infinity Cache) with a start and a stop event on every
    dispatch; a kernel's duration is the time between the two on the device - what a kernel trace reports for it.
    `achieved` = algorithmic bytes of the 65 Q8 matvec launches / the sum of their durations."""
    from deepj_amd import HipNative, opcodes as op
    from deepj_amd.fused import DeviceBuffers, Stream
    cfg = model.cfg
    stream = model.decodeStream()
    ops = decode_ops(stream)
    HipNative.profileOps(stream, 2)                               # warm-up
    us = HipNative.profileOps(stream, iters)
    table, lin, lin_bytes, lin_us, weights, kv_cache_id = {}, [], 0, 0.0, [], None

    def add(name, nbytes, t):
        e = table.setdefault(name, {"launches_per_token": 0, "bytes": int(nbytes), "us": 0.0})
        e["launches_per_token"] += 1
        e["us"] += float(t)

    for (code, w), t in zip(ops, us):
        if code == op.OP_Q8_LINEAR and w[4] == 1:
            k, nn, flags = w[5], w[6], w[7]
            rows = 2 * nn if flags & op.LIN_SWIGLU else nn
            nbytes = q8_linear_bytes(k, rows)
            add(VARIANTS.get((k, rows), f"{k}x{rows}"), nbytes, t)
            lin_bytes += nbytes
            lin_us += float(t)
            lin.extend(w)
            weights.append((w[2], HipNative.q8Floats(k, rows), VARIANTS.get((k, rows), f"{k}x{rows}")))
        elif code == op.OP_ATTN_DECODE_RECORDS:
            add("attention", 2 * position * cfg.dModel * 4, t)    # K and V rows of the live context, fp32
            kv_cache_id = w[2]
        elif code == op.OP_DECODE_NEXT:
            add("decode_next", 4 * cfg.vocabSize, t)
    for e in table.values():
        e["us"] = round(e["us"] / e["launches_per_token"], 3)
        e["GBs"] = round(e["bytes"] / e["us"] / 1e3, 1)
        e["frac"] = round(e["bytes"] / e["us"] / 1e3 / HBM_PEAK_GBS, 4)
    launches = len(weights)
    achieved = lin_bytes / lin_us / 1e3

    # the same 65 launches back to back without events (launch cost hidden behind the previous kernel, gaps included)
    lin = np.asarray(lin, dtype=np.int32)
    HipNative.timeOps(lin, 2)
    b2b_us = HipNative.timeOps(lin, iters) * 1e3 / (iters * launches)
    words = len(lin) // launches
    warm_n = min(16, launches)                                    # first four layers: 232 MB, Infinity-Cache resident
    warm = lin[:warm_n * words]
    HipNative.timeOps(warm, 4)
    warm_us = HipNative.timeOps(warm, 4 * iters) * 1e3 / (4 * iters * warm_n)

    # floors, by the same method: an empty kernel of the matvec's grid size (what a dependent launch costs with no
    # work in it), and a pure streaming read of the very same weight buffers in the same order
    dev = DeviceBuffers()
    sink = dev.alloc(4)
    nops = Stream()
    for _ in range(64):
        nops.nop(768)
    nops.profile(2)
    empty_us = float(np.mean(nops.profile(iters)))
    empty_period_us = nops.time(iters) * 1e3 / (iters * 64)
    reads = Stream()
    for wid, floats, _ in weights:
        reads.stream_read(wid, sink, floats)
    reads.profile(2)
    rus = reads.profile(iters)
    read_tab = {}
    for (wid, floats, name), t in zip(weights, rus):
        e = read_tab.setdefault(name, {"bytes": floats * 4, "us": 0.0, "n": 0})
        e["us"] += float(t)
        e["n"] += 1
    for e in read_tab.values():
        e["us"] = round(e["us"] / e.pop("n"), 3)
        e["GBs"] = round(e["bytes"] / e["us"] / 1e3, 1)
    read_avg_us = float(np.sum(rus)) / launches
    read_b2b_us = reads.time(iters) * 1e3 / (iters * launches)
    # the decode attention's floor: as many bytes of the K cache as one layer's K and V rows of the live context
    kv = Stream()
    for _ in range(cfg.nLayers):
        kv.stream_read(kv_cache_id, sink, 2 * position * cfg.dModel)
    kv.profile(2)
    kv_us = float(np.mean(kv.profile(iters)))
    read_tab["attention_kv"] = {"bytes": 2 * position * cfg.dModel * 4, "us": round(kv_us, 3),
                                "GBs": round(2 * position * cfg.dModel * 4 / kv_us / 1e3, 1)}
    dev.release_all()
    return {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
            "frac": round(achieved / HBM_PEAK_GBS, 4), "traffic": MATVEC_TRAFFIC_BYTES_PER_LAUNCH,
            "traffic_source": "not measured in this run: algorithmic bytes x the fetched / algorithmic ratio of the same kernel "
                              "in profiles/q8_matvec_c2_sweep_hbm_traffic.txt (rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE over "
                              "bench.py --sweep, scaled by k_copy)",
            "kernel": "k_q8_matvec", "launches_per_token": launches, "bytes_per_launch": lin_bytes // launches,
            "avg_launch_us": round(lin_us / launches, 3),
            "timing": "mean kernel duration (start/stop events on each dispatch, whole token in order, HBM-cold); "
                      "rocprofv3 --kernel-trace reports the same quantity",
            "back_to_back_avg_launch_us": round(b2b_us, 3), "cache_warm_avg_launch_us": round(warm_us, 3),
            "per_kernel": table,
            "floor": {"empty_kernel_us": round(empty_us, 3), "empty_launch_period_us": round(empty_period_us, 3),
                      "stream_read": read_tab, "stream_read_avg_us": round(read_avg_us, 3),
                      "stream_read_back_to_back_avg_us": round(read_b2b_us, 3),
                      # what a kernel that only READS the same weight buffers reaches by the same measure
                      "stream_read_frac_of_peak": round(lin_bytes / launches / read_avg_us / 1e3 / HBM_PEAK_GBS, 4),
                      "matvec_time_over_stream_read_time": round(lin_us / launches / read_avg_us, 3)}}


MFMA_PEAK_TFLOPS = 2500.0       # MI355X dense fp16 / bf16 matrix-core peak


def prefill_roofline(model, n: int, iters: int = 6):
    """Per-op durations of the n-token prompt's command stream, measured live like the decode table: a start and a stop
    event on EVERY dispatch of every op, summed per op - so a projection's figure holds its GEMM and the helpers the
    op cannot do without (the split of the activations into fp16 planes, with the norm; the sum of partial products
    when workgroups share K; the per-call conversion of the weights when the runner holds no fp16 copy).  `gemm_us` is
    the op's longest dispatch alone.  A projection's algorithmic work is one multiply-add per weight per row,
    2 M K N flops; the fp16 kernels issue two matrix-core products for it (hi and lo halves of the activation), the
    bf16 kernels three - `issued` counts those against the same peak."""
    from deepj_amd import HipNative, opcodes as op
    stream = model.prefillStream(n)
    ops = decode_ops(stream)
    HipNative.profileOps(stream, 2)
    us, top, count = HipNative.profileOps(stream, iters, detail=True)
    names = {(2048, 6144): "qkv", (2048, 2048): "wo", (2048, 11264): "gate_up", (5632, 2048): "down"}
    other_names = {op.OP_ROPE_KV_STORE: "rope_kv_store", op.OP_EMBED_GATHER: "embed_gather", op.OP_DECODE_NEXT: "decode_next",
                   op.OP_COPY: "copy_last_row"}
    table, flops, gemm_us, issued, all_us = {}, 0.0, 0.0, 0.0, 0.0
    for (code, w), t, t_top, c in zip(ops, us, top, count):
        if t <= 0:
            continue
        all_us += float(t)
        if (code == op.OP_Q8_LINEAR and w[4] > 1) or code == op.OP_Q8_LINEAR_ROPE:
            fused_rope = code == op.OP_Q8_LINEAR_ROPE
            m, k, nn, flags = w[4], w[5], (3 * w[6] if fused_rope else w[6]), w[7]
            rows = 2 * nn if flags & op.LIN_SWIGLU else nn
            tile, tile_cols, shares = HipNative.q8GemmTile(m, k, rows)
            f = 2.0 * m * k * rows
            e = table.setdefault(names.get((k, rows), f"{k}x{rows}") + ("_rope_kv_store" if fused_rope else ""), {
                "launches": 0, "us": 0.0, "gemm_us": 0.0, "dispatches_per_op": int(c), "flops": f,
                "kernel": (f"k_gemm_q8_f16 ({tile} x {tile_cols} tiles" + (f", K shared by {shares}" if shares > 1 else "") +
                           ", fp16 x 2" + (", RoPE + cache append as the epilogue)" if fused_rope else ")")) if tile else "k_gemm_q8 (bf16 x 3)"})
            e["launches"] += 1
            e["us"] += float(t)
            e["gemm_us"] += float(t_top)
            flops += f
            gemm_us += float(t)
            issued += f * (2 if tile else 3)
        elif code == op.OP_ATTENTION:
            e = table.setdefault("attention", {"launches": 0, "us": 0.0, "kernel": "k_attention_tiled (scores: bf16 x 6 on split planes; values: fp32 matrix instructions at this shape)"})
            e["launches"] += 1
            e["us"] += float(t)
        elif code in other_names or (code == op.OP_Q8_LINEAR and w[4] == 1):
            e = table.setdefault(other_names.get(code, "lm_head_last_row"), {"launches": 0, "us": 0.0})
            e["launches"] += 1
            e["us"] += float(t)
    for e in table.values():
        e["us"] = round(e["us"] / e["launches"], 2)
        if "gemm_us" in e:
            e["gemm_us"] = round(e["gemm_us"] / e["launches"], 2)
        if "flops" in e:
            e["TFLOPs"] = round(e.pop("flops") / e["us"] / 1e6, 1)
            e["frac"] = round(e["TFLOPs"] / MFMA_PEAK_TFLOPS, 4)
    # HBM-bound helpers of the prompt against the HBM peak: RoPE + cache append moves 24 bytes per element of [n x d]
    d = model.cfg.dModel
    if "rope_kv_store" in table:
        e = table["rope_kv_store"]
        e["bytes"] = 24 * n * d
        e["frac_of_hbm_peak"] = round(e["bytes"] / e["us"] / 1e3 / HBM_PEAK_GBS, 4)
    achieved = flops / gemm_us / 1e6
    return {"bound": "mfma", "achieved": round(achieved, 1), "peak": MFMA_PEAK_TFLOPS, "unit": "TFLOP/s",
            "frac": round(achieved / MFMA_PEAK_TFLOPS, 4), "issued_frac": round(issued / gemm_us / 1e6 / MFMA_PEAK_TFLOPS, 4),
            "kernel": "Q8_LINEAR ops of the prompt's projections (GEMM + their helper kernels)", "rows": n,
            "kernel_time_us_all_ops": round(all_us, 1), "per_kernel": table,
            "timing": "per op: sum of the begin-to-end times of all its dispatches (start/stop events on each, whole prompt in order)"}


C2_SHAPES = [(2048, 2048), (2048, 5632), (5632, 2048), (4096, 11008)]     # K x N of the isolated linear-op sweep
C2_ROTATION_BYTES = 512 << 20      # distinct Q8 copies a cache-cold row rotates over: twice the 256 MB Infinity Cache


def _best_of(fn, reps: int) -> float:
    best = float("inf")
    for _ in range(reps):
        t0 = time.perf_counter()
        fn()
        best = min(best, time.perf_counter() - t0)
    return best


def c2_sweep(iters: int = 10, cpu: bool = True):
    """The isolated linear-op sweep as a measurement: the four weight shapes at M = 1 (decode matvec; cache-cold
    over a rotation of distinct Q8 copies and cache-warm on one copy), M = 64 and M = 512 (prompt GEMM), and the
    fused RMSNorm / SiLU-times-up / RoPE-and-cache-append ops on [M x 2048] and [M x 5632] rows; next to each row
    the CPU oracle's matmul, RMSNorm or SiLU-times-up on the same shape (best of a few runs after a warm-up, like the
    reference's own harness: MetalBackendAllOpsPerformanceTest.java:85-107).  Weight VALUES come from numpy here
    (a timing does not depend on them; the parity of this sweep, on the java.util.Random streams the baseline
    states, is tests/test_gpu_c2_sweep.py).  GPU times are launch periods of back-to-back launches (HIP events
    around the whole run, every helper kernel of an op included)."""
    from deepj_amd import HipNative
    from deepj_amd.fused import DeviceBuffers, Stream
    rng = np.random.default_rng(1)
    dev = DeviceBuffers()
    ref = None
    threads = 1
    if cpu:
        from oracle import cpu_ref as ref
        threads = ref.default_threads()
        ref.set_threads(threads)
        ref.set_column_parallel(False)
    linear, fused = [], []

    def period_us(stream, launches, n_iters=iters):
        stream.time(2)
        return stream.time(n_iters) * 1e3 / (n_iters * launches)

    for k, n in C2_SHAPES:
        w = (rng.standard_normal((k, n)) * 0.02).astype(np.float32)
        q_floats = HipNative.q8Floats(k, n)
        nbytes = q8_linear_bytes(k, n)
        copies = max(2, -(-C2_ROTATION_BYTES // (4 * q_floats)))
        src = dev.upload(w)
        qs = [dev.alloc(q_floats) for _ in range(copies)]
        Stream().q8_quantize(src, qs[0], k, n).run()
        dev.release(src)
        dup = Stream()
        for q in qs[1:]:
            dup.copy(qs[0], q, q_floats)
        dup.run()
        for m in (1, 64, 512):
            x_host = rng.standard_normal((m, k)).astype(np.float32)
            x, out = dev.upload(x_host), dev.alloc(m * n)
            row = {"K": k, "N": n, "M": m}
            if m == 1:
                cold, warm = Stream(), Stream()
                for q in qs:
                    cold.q8_linear(x, q, out, 1, k, n)
                    warm.q8_linear(x, qs[0], out, 1, k, n)
                cold.profile(2)
                ev = float(np.mean(cold.profile(iters)))
                cold_us, warm_us = period_us(cold, copies), period_us(warm, copies)
                row.update({"kernel": "k_q8_matvec", "bytes": nbytes, "rotation_copies": copies,
                            "cold_us": round(cold_us, 3), "cold_GBs": round(nbytes / cold_us / 1e3, 1),
                            "cold_frac_of_hbm_peak": round(nbytes / cold_us / 1e3 / HBM_PEAK_GBS, 4),
                            "cold_kernel_us": round(ev, 3),
                            "cold_kernel_frac_of_hbm_peak": round(nbytes / ev / 1e3 / HBM_PEAK_GBS, 4),
                            "warm_us": round(warm_us, 3), "warm_GBs": round(nbytes / warm_us / 1e3, 1)})
            else:
                tile, tile_cols, shares = HipNative.q8GemmTile(m, k, n)
                flops = 2.0 * m * k * n
                use = qs[:min(copies, 4)]
                plain = Stream()
                for q in use:
                    plain.q8_linear(x, q, out, m, k, n)
                us = period_us(plain, len(use))
                row.update({"kernel": (f"k_gemm_q8_f16 ({tile} x {tile_cols} tiles" + (f", K shared by {shares}" if shares > 1 else "") +
                                       ", fp16 x 2) + k_split_f16 + k_q8_to_f16") if tile else "k_gemm_q8 (bf16 x 3)",
                            "flops": flops, "us": round(us, 2), "TFLOPs": round(flops / us / 1e6, 1),
                            "frac_of_mfma_peak": round(flops / us / 1e6 / MFMA_PEAK_TFLOPS, 4)})
                ptile, ptile_cols, pshares = HipNative.q8GemmTilePrepared(m, k, n)
                if ptile:
                    # with the weight kept in the GEMM's own layout (OP_Q8_PREPARE), as the decode driver keeps them
                    # (fewer than 256 rows reach the fp16 GEMM only this way)
                    prep = [dev.alloc(HipNative.q8PreparedFloats(k, n)) for _ in use[:2]]
                    ps = Stream()
                    for q, pb in zip(use, prep):
                        ps.q8_prepare(q, pb, k, n)
                    ps.run()
                    prepared = Stream()
                    for q in use[:2]:
                        prepared.q8_linear(x, q, out, m, k, n)
                    pus = period_us(prepared, len(use[:2]))
                    row.update({"prepared_us": round(pus, 2), "prepared_TFLOPs": round(flops / pus / 1e6, 1),
                                "prepared_frac_of_mfma_peak": round(flops / pus / 1e6 / MFMA_PEAK_TFLOPS, 4),
                                "prepared_kernel": f"k_gemm_q8_f16 ({ptile} x {ptile_cols} tiles" + (f", K shared by {pshares}" if pshares > 1 else "") + ", fp16 x 2) + k_split_f16"})
                    dev.release(*prep)       # releasing a prepared copy ends its association with the weight
            if ref is not None:
                reps = 1 if m * k * n > 2e9 else 3      # (the oracle multiplies the fp32 weights, as CpuBackend.matmul does)
                if reps > 1:
                    ref.matmul(x_host, w)
                t = _best_of(lambda: ref.matmul(x_host, w), reps)
                row["cpu_us"] = round(t * 1e6, 1)
                row["cpu_threads"] = 1 if m == 1 else min(threads, m)
            dev.release(x, out)
            linear.append(row)
        dev.release(*qs)

    # fused element-wise and norm ops: rows rotate over enough buffers that the larger ones come from HBM
    H, hd = 32, 64
    for d in (2048, 5632):
        for m in (1, 64, 512):
            n_el = m * d
            x_host = rng.standard_normal((m, d)).astype(np.float32)
            g_host = (1.0 + 0.02 * rng.standard_normal((1, d))).astype(np.float32)
            rot = int(max(2, min(48, -(-C2_ROTATION_BYTES // (12 * n_el)))))
            xs = [dev.upload(x_host) for _ in range(rot)]
            ys = [dev.upload(x_host) for _ in range(rot)]
            outs = [dev.alloc(n_el) for _ in range(rot)]
            gam = dev.upload(g_host)
            s1, s2 = Stream(), Stream()
            for a, b, o in zip(xs, ys, outs):
                s1.rmsnorm(a, gam, o, m, d)
                s2.silu_mul(a, b, o, n_el)
            for name, st, nbytes in (("rmsnorm", s1, 4 * (2 * n_el + d)), ("silu_mul", s2, 12 * n_el)):
                us = period_us(st, rot)
                st.profile(2)
                ev = float(np.mean(st.profile(iters)))
                row = {"op": name, "M": m, "cols": d, "bytes": nbytes, "rotation_buffers": rot, "us": round(us, 3),
                       "GBs": round(nbytes / us / 1e3, 1), "frac_of_hbm_peak": round(nbytes / us / 1e3 / HBM_PEAK_GBS, 4),
                       "kernel_us": round(ev, 3), "kernel_frac_of_hbm_peak": round(nbytes / ev / 1e3 / HBM_PEAK_GBS, 4)}
                if ref is not None:
                    fn = (lambda: ref.rmsnorm(x_host, g_host)) if name == "rmsnorm" else (lambda: ref.multiply(ref.silu(x_host), x_host))
                    fn()
                    row["cpu_us"] = round(_best_of(fn, 3) * 1e6, 1)
                    row["cpu_threads"] = min(threads, m)
                fused.append(row)
            dev.release(*xs, *ys, *outs, gam)
    # RoPE on Q and K with the append of K and V to the cache (ROPE_KV_STORE), d = 2048 as 32 heads of 64
    d = H * hd
    theta = np.arange(2048, dtype=np.float64)[:, None] / np.power(10000.0, 2.0 * np.arange(hd // 2) / hd)[None, :]
    cos, sin = np.cos(theta).astype(np.float32), np.sin(theta).astype(np.float32)
    cos_b, sin_b = dev.upload(cos), dev.upload(sin)
    state = dev.upload(np.zeros(4, np.int32))
    for m in (1, 64, 512):
        rot = int(max(2, min(32, -(-C2_ROTATION_BYTES // (40 * m * d)))))
        qkvs = [dev.upload(rng.standard_normal((m, 3 * d)).astype(np.float32)) for _ in range(rot)]
        qo = [dev.alloc(m * d) for _ in range(rot)]
        kc, vc = dev.alloc(2048 * d), dev.alloc(2048 * d)
        st = Stream()
        for a, o in zip(qkvs, qo):
            st.rope_kv_store(a, o, kc, vc, state, cos_b, sin_b, m, H, hd, 2048, 0)
        us = period_us(st, rot)
        st.profile(2)
        ev = float(np.mean(st.profile(iters)))
        nbytes = 16 * m * d                      # Q and K read and written; the V rows' move to the cache is extra
        moved = 24 * m * d + 2 * 4 * m * (hd // 2)
        fused.append({"op": "rope_kv_store", "M": m, "cols": d, "bytes": nbytes, "bytes_moved": moved,
                      "rotation_buffers": rot, "us": round(us, 3), "GBs": round(nbytes / us / 1e3, 1),
                      "frac_of_hbm_peak": round(nbytes / us / 1e3 / HBM_PEAK_GBS, 4), "kernel_us": round(ev, 3),
                      "kernel_frac_of_hbm_peak": round(nbytes / ev / 1e3 / HBM_PEAK_GBS, 4),
                      "moved_frac_of_hbm_peak": round(moved / ev / 1e3 / HBM_PEAK_GBS, 4)})
        dev.release(*qkvs, *qo, kc, vc)
    dev.release_all()
    if ref is not None:
        ref.set_threads(1)
    return {"workload": "isolated Q8 linear-op sweep: 2048x2048, 2048x5632, 5632x2048, 4096x11008 at M = 1 / 64 / 512; "
                        "fused RMSNorm, SiLU x up and RoPE + cache append on [M x 2048] and [M x 5632]",
            "timing": "launch period of back-to-back launches (HIP events around the run; an op's helper kernels "
                      "included); *kernel_us: mean begin-to-end time of the dispatch alone; cold = rotation over "
                      f"{C2_ROTATION_BYTES >> 20} MiB of distinct buffers, warm = one buffer",
            "hbm_peak_GBs": HBM_PEAK_GBS, "mfma_peak_TFLOPs": MFMA_PEAK_TFLOPS,
            "cpu": "C restatement of CpuBackend (not the JVM): matmul parallel over rows of A like DeepJExecutor.forRange, "
                   f"{threads} threads available" if ref is not None else None,
            "linear": linear, "fused": fused}


def calibration_copy(mib: int = 256, repeats: int = 3) -> None:
    """A plain device copy of known size (reads `mib` MiB, writes `mib` MiB per launch), so that a
    hardware-counter run of this script has a kernel (k_copy) whose FETCH_SIZE / WRITE_SIZE readings
    can be compared with its known traffic."""
    from deepj_amd.fused import DeviceBuffers, Stream
    dev = DeviceBuffers()
    n = mib * (1 << 20) // 4
    src, dst = dev.alloc(n), dev.alloc(n)
    Stream().fill(src, 0x3F800000, n).run()
    for _ in range(repeats):
        Stream().copy(src, dst, n).run()
    dev.release_all()


def clock_probe():
    """The shader clock under the library's own kernels: a one-wavefront sampler on a second stream reads the shader
    clock counter against the 100 MHz wall clock every few microseconds while a stream runs (deepj_hip_clock_probe).
    Workloads: nothing (idle), a pure read of 1 GiB (STREAM_READ), the prompt's gate/up GEMM at 512 rows, a
    2048 x 12288 x 4096 GEMM (prepared weights), and the empty kernel.  Reported: median / 10th / 90th percentile of the clock
    over the sampling intervals that lie inside the stream's runs, and how long the runs took."""
    from deepj_amd import HipNative
    from deepj_amd.fused import DeviceBuffers, Stream
    rng = np.random.default_rng(5)
    dev = DeviceBuffers()
    rows = []

    def measure(name, stream, iters, samples):
        if iters:
            stream.run()
            HipNative.synchronize()
        mhz, t, win = HipNative.clockProbe(stream.array(), iters, samples, 1)
        inside = mhz[(t > win[0] + 20.0) & (t < win[1] - 5.0)] if iters else mhz
        if inside.size == 0:
            inside = mhz
        rows.append({"workload": name, "run_us": round(win[1] - win[0], 1) if iters else 0.0, "intervals": int(inside.size),
                     "interval_us": round(float(np.median(np.diff(t))), 2),
                     "clock_MHz_median": round(float(np.median(inside)), 0), "clock_MHz_p10": round(float(np.percentile(inside, 10)), 0),
                     "clock_MHz_p90": round(float(np.percentile(inside, 90)), 0)})

    smi = []

    def smi_during(name, stream, iters):
        """The driver's own view beside the sampler's: rocm-smi's sclk, read a few times while the stream loops for a
        second or two (None where the tool is not there or prints no clock)."""
        import re, subprocess, threading
        reads = []

        def poll():
            for _ in range(6):
                try:
                    r = subprocess.run(["rocm-smi", "--showclocks"], capture_output=True, text=True, timeout=20)
                except (OSError, subprocess.SubprocessError):
                    return
                found = re.search(r"sclk clock level: *\d+: *\((\d+)Mhz\)", r.stdout)
                if found:
                    reads.append((time.perf_counter(), int(found.group(1))))
                time.sleep(0.2)

        stream.run()
        HipNative.synchronize()
        th = threading.Thread(target=poll)
        t0 = time.perf_counter()
        th.start()
        ms = stream.time(iters)
        t1 = time.perf_counter()
        th.join()
        inside = [mhz for t, mhz in reads if t0 + 0.3 < t < t1]
        return {"workload": name, "loop_s": round(t1 - t0, 2), "us_per_launch": round(ms * 1e3 / iters, 1),
                "rocm_smi_sclk_MHz": inside or None}

    measure("idle (sampler alone)", Stream().nop(1), 0, 400)
    measure("empty kernels back to back", Stream().nop(768), 4000, 1500)
    n = 1 << 28
    big, sink = dev.alloc(n), dev.alloc(64)
    Stream().fill(big, 0x3F800000, n).run()
    measure("pure read of 1 GiB (STREAM_READ)", Stream().stream_read(big, sink, n), 24, 1500)
    smi.append(smi_during("pure read of 1 GiB (STREAM_READ)", Stream().stream_read(big, sink, n), 10000))
    dev.release(big, sink)
    k, nn = 2048, 5632                       # the decode matvec over a rotation of distinct weight copies (HBM-cold)
    wf = dev.upload((rng.standard_normal((k, nn)) * 0.02).astype(np.float32))
    q_floats = HipNative.q8Floats(k, nn)
    qs = [dev.alloc(q_floats) for _ in range(40)]
    Stream().q8_quantize(wf, qs[0], k, nn).run()
    dup = Stream()
    for q in qs[1:]:
        dup.copy(qs[0], q, q_floats)
    dup.run()
    x, out = dev.upload(rng.standard_normal((1, k)).astype(np.float32)), dev.alloc(nn)
    mv = Stream()
    for q in qs:
        mv.q8_linear(x, q, out, 1, k, nn)
    measure("Q8 matvec 2048 x 5632, 40 distinct copies in turn", mv, 40, 1500)
    dev.release(wf, x, out, *qs)
    for m, k, nn, iters in ((512, 2048, 11264, 96), (2048, 4096, 12288, 14)):
        x = dev.upload(rng.standard_normal((m, k)).astype(np.float32))
        wf = dev.upload((rng.standard_normal((k, nn)) * 0.02).astype(np.float32))
        wq = dev.alloc(HipNative.q8Floats(k, nn))
        Stream().q8_quantize(wf, wq, k, nn).run()
        dev.release(wf)
        prep = dev.alloc(HipNative.q8PreparedFloats(k, nn))
        Stream().q8_prepare(wq, prep, k, nn).run()
        out = dev.alloc(m * nn)
        tile = HipNative.q8GemmTile(m, k, nn)
        gemm = Stream().q8_linear(x, wq, out, m, k, nn)
        measure(f"Q8 GEMM {m} x {nn} x {k} (fp16 x 2, {tile[0]} x {tile[1]} tiles)", gemm, iters, 2000)
        if m == 2048:
            smi.append(smi_during(f"Q8 GEMM {m} x {nn} x {k}", gemm, 4000))
        dev.release(x, wq, prep, out)
    return {"method": "one wavefront on a second stream samples s_memtime (shader clock counter) against s_memrealtime (100 MHz) "
                      "while the workload runs on the library's stream; clock = counter difference / wall difference x 100 MHz "
                      "per sampling interval; intervals inside the workload's runs only", "rows": rows,
            "rocm_smi": smi}


def cpu_baseline(cfg, ctx: int, tokens: int = 12):
    """Oracle timing, like for like: the whole 16-layer model, S = 1 with a KV cache at context `ctx`.

    The model has the workload's dimensions and fp32 weights (4.3 GB, every layer its own, so a
    token streams them from DRAM as the reference would); they are filled by a cheap hash rather
    than the seeded Gaussian stream, which alone would take minutes - values do not affect speed.
    CpuBackend.matmul parallelises over the rows of A only (CpuBackend.java:175), so an M = 1
    product runs on one thread by construction."""
    from oracle import cpu_ref as ref
    threads = ref.default_threads()
    ref.set_threads(threads)
    ref.set_column_parallel(False)
    m = ref.Model(vocab=cfg.vocabSize, max_seq=cfg.maxSeqLen, d=cfg.dModel, heads=cfg.nHeads, layers=cfg.nLayers,
                  dff=cfg.dFF, seed=42, timing_only_fill=True)
    ids = ref.JavaRandom(3).ints(ctx + tokens, cfg.vocabSize)
    m.reset_cache()
    t0 = time.perf_counter()
    m.forward_cached(ids[:ctx], last_only=True)                  # fills the cache (rows run in parallel)
    t_prefill = time.perf_counter() - t0
    m.forward_cached(ids[ctx:ctx + 1], last_only=True)           # one untimed token
    t0 = time.perf_counter()
    for i in range(1, tokens):
        m.forward_cached(ids[ctx + i:ctx + i + 1], last_only=True)
    per_token = (time.perf_counter() - t0) / (tokens - 1)
    # the reference itself has no KV cache: every new token is a forward of the whole context, logits for every row
    # (TextGenerator.java:91-100, DecoderOnlyModel.java:58-64) - one such forward, timed
    t0 = time.perf_counter()
    m.forward(ids[:ctx + 1])
    t_full = time.perf_counter() - t0
    m.close()
    ref.set_threads(1)
    return {"value": round(1.0 / per_token, 4), "unit": "tok/s", "cores": 1, "kind": "port",
            "sample": f"C restatement of CpuBackend + layers (not the JVM), full {cfg.nLayers}-layer model with fp32 "
                      f"weights, KV cache at context {ctx}, {tokens - 1} timed tokens; S=1 matmul is single-threaded "
                      f"by construction (CpuBackend.java:175)",
            "prefill_tok_s": round(ctx / t_prefill, 2), "prefill_threads": threads,
            "no_kv_cache_s_per_token": round(t_full, 2), "no_kv_cache_threads": threads}


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=256)
    ap.add_argument("--warmup", type=int, default=16)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--prompt", type=int, default=512)
    ap.add_argument("--eager", action="store_true",
                    help="decode without the HIP graph (same kernels, launched one by one): for runs under a tracer")
    ap.add_argument("--prefill-only", action="store_true",
                    help="stop after the prompt: prints the prefill object alone (short runs under a counter-collecting profiler)")
    ap.add_argument("--sweep", action="store_true",
                    help="only the isolated linear-op sweep (four weight shapes x M = 1 / 64 / 512, fused norm and element-wise ops)")
    ap.add_argument("--no-sweep", action="store_true", help="leave the sweep out of the default line")
    ap.add_argument("--clock-probe", action="store_true",
                    help="only sample the shader clock under a pure read and under the prompt GEMMs (one JSON line)")
    ap.add_argument("--table-iters", type=int, default=12,
                    help="passes behind the per-kernel tables; counter-collecting profilers serialise every dispatch, 1 keeps such runs short")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs on ONE GPU (one MI355X per box); --gpus > 1 is not supported", file=sys.stderr)
        return 2

    from deepj_amd import HipNative, JavaRandom, LlamaConfig, LlamaModel

    if args.clock_probe:
        HipNative.init(0)
        print(json.dumps({"metric": "shader clock under load, MHz", "n_gpus": 1, "clock_probe": clock_probe()}))
        return 0
    if args.sweep:
        HipNative.init(0)
        sw = c2_sweep(max(2, args.table_iters), cpu=not args.no_cpu_baseline)
        calibration_copy()
        print(json.dumps({"metric": "Q8 matvec HBM GB/s vs peak; Q8 GEMM TFLOP/s vs peak (isolated linear-op sweep)",
                          "n_gpus": 1, "sweep": sw}))
        return 0
    cfg = LlamaConfig(vocabSize=32000, maxSeqLen=2048, dModel=2048, nHeads=32, nLayers=16, dFF=5632)
    if args.prompt + args.warmup + args.steps > cfg.maxSeqLen:
        print("bench.py: prompt + warmup + steps exceeds maxSeq 2048", file=sys.stderr)
        return 2
    t0 = time.perf_counter()
    model = LlamaModel(cfg, 42)
    t_build = time.perf_counter() - t0
    prompt = JavaRandom(3).ints(args.prompt, cfg.vocabSize)

    model.reset()
    t0 = time.perf_counter()
    model.prefill(prompt)
    HipNative.synchronize()
    t_first_prefill = time.perf_counter() - t0      # the first request after the model was built
    times = []                                      # then the median of five more (each from an empty cache, host clock, synchronised)
    for _ in range(5):
        model.reset()
        t0 = time.perf_counter()
        model.prefill(prompt)
        HipNative.synchronize()
        times.append(time.perf_counter() - t0)
    t_prefill = sorted(times)[len(times) // 2]
    if args.prefill_only:
        model.reset()
        prefill_roof = prefill_roofline(model, args.prompt, max(1, args.table_iters // 2))
        print(json.dumps({"metric": "prefill tok/s, Q8 Llama d=2048 L=16, 1 GPU", "value": round(args.prompt / t_prefill, 1),
                          "unit": "tok/s", "n_gpus": 1, "prompt_tokens": args.prompt, "prefill": prefill_roof}))
        model.close()
        return 0

    graph = False if args.eager else None
    model.decode(args.warmup, use_graph=graph)      # captures the graph on first use
    HipNative.synchronize()
    t0 = time.perf_counter()
    model.decode(args.steps, use_graph=graph)
    HipNative.synchronize()
    elapsed = time.perf_counter() - t0
    toks = model.tokens()
    assert len(toks) == 1 + args.warmup + args.steps

    roof = matvec_roofline(model, args.prompt + args.warmup + args.steps, args.table_iters)
    model.reset()
    # the same decode at three times the context (the cache read grows with the position, the weights do not)
    long_prompt = JavaRandom(3).ints(1536, cfg.vocabSize)
    model.prefill(long_prompt)
    model.decode(8, use_graph=graph)
    HipNative.synchronize()
    t0 = time.perf_counter()
    model.decode(128, use_graph=graph)
    HipNative.synchronize()
    t_long = (time.perf_counter() - t0) / 128
    model.reset()
    model.prefill(prompt)
    model.reset()
    prefill_roof = prefill_roofline(model, args.prompt, max(1, args.table_iters // 2))
    model.reset()
    calibration_copy()
    cpu = None if args.no_cpu_baseline else cpu_baseline(cfg, args.prompt)
    sweep = None if args.no_sweep else c2_sweep(max(2, args.table_iters), cpu=not args.no_cpu_baseline)

    # per-token algorithmic bytes at the mean decoded position (weights + fp32 KV read)
    weights = sum(q8_linear_bytes(k, n) for k, n in
                  [(2048, 6144), (2048, 2048), (2048, 11264), (5632, 2048)]) * cfg.nLayers + q8_linear_bytes(2048, 32000)
    mean_pos = args.prompt + args.warmup + args.steps / 2
    kv = cfg.nLayers * 2 * mean_pos * cfg.dModel * 4
    tok_s = args.steps / elapsed
    mem, prepared_bytes = HipNative.poolStats(), model.preparedBytes()
    line = {
        "metric": "decode tok/s, Q8 Llama d=2048 L=16, 1 GPU; Q8 matvec HBM GB/s vs peak",
        "value": round(tok_s, 2), "unit": "tok/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(elapsed * 1e3 / args.steps, 4), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "q8 weights (int8 + fp32 scale per 32), fp32 activations/accumulate",
        "data": "synthetic: seeded random-init weights (java.util.Random seed 42), random prompt ids (seed 3)",
        "config": {"workload": "llama-decode d2048 L16 H32 dFF5632 V32000, prompt 512, batch 1, greedy, fp32 KV cache",
                   "prompt_tokens": args.prompt, "decode_tokens": args.steps},
        "roofline": roof,
        "cpu_baseline": cpu,
        "end_to_end": {"bytes_per_token": int(weights + kv), "achieved_GBs": round((weights + kv) * tok_s / 1e9, 1),
                       "frac_of_hbm_peak": round((weights + kv) * tok_s / 1e9 / HBM_PEAK_GBS, 4),
                       "prefill_tok_s": round(args.prompt / t_prefill, 1),
                       "first_prefill_ms": round(t_first_prefill * 1e3, 2), "model_build_s": round(t_build, 1),
                       # device memory: everything the library holds for this model, the Q8 weights (1.125 B/weight), and
                       # the fp16 copies of the projections the prompt GEMM reads (2 B/weight; LlamaModel.setPreparedBudget
                       # bounds them, 0 = none at about 40 us per layer and prompt)
                       "device_bytes_live": int(mem["live_bytes"]), "q8_weight_bytes": int(weights),
                       "prepared_weight_bytes": prepared_bytes,
                       "decode_tok_s_at_context_1536": round(1.0 / t_long, 1)},
        "prefill": prefill_roof,
        "sweep": sweep,
    }
    print(json.dumps(line))
    model.close()
    return 0


if __name__ == "__main__":
    sys.exit(main())
