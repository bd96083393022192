#!/usr/bin/env python3
"""Benchmark of the block-quantized matmul hot path on one MI355X.

A "step" is one pass of the decode hot path over the LFM2-350M-shaped weight set
(hidden 1024, 10 short-conv + 6 attention layers, FFN 4608, tied LM head
65536 x 1024) at n = 1: 93 weight matrices in 65 GEMV launches ({Q,K,V} and
{gate,up} share one activation and one launch, like the reference's call sites; the
Q8_0 quantization of the activation runs inside the GEMV kernel), submitted as ONE
HIP graph per token.  Two distinct device copies of the weight set are alternated
so every step streams its weights from HBM, not from the 256 MB Infinity Cache.

Prints one JSON line: `value` = algorithmic GEMV bytes per step / step time, plus
  roofline        the GEMV kernel over the timed steps: algorithmic bytes / summed kernel
                  execution time (per-dispatch timestamps, the quantity a kernel trace reports)
  gemm            prefill GEMM leg (Q4_0, m=6912, n=2002, k=2048) with its own roofline
  gemv_6912x2048  the single-GEMV shape the HBM target is quoted on, HBM-cold
  decode_step_q8_0, prefill_sites, lm_head_sweep   the other configurations
  cpu_baseline    the reference's x86 CPU path (f32 per-token GEMV, serial for Q4_0)
                  timed on this host on a bounded sample of the same step

`--leg NAME` runs one leg only (used for profiling): decode, decode_q8, gemv, gemm,
prefill_sites, lm_head, copy, cpu.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time
from concurrent.futures import ThreadPoolExecutor

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0      # MI355X HBM3E
INT8_PEAK_TOPS = 5000.0    # MI355X dense int8 MFMA (5.0 POP/s)

HS, IS, KV, VOCAB = 1024, 4608, 512, 65536
N_CONV, N_ATTN = 10, 6
BW = {2: 18, 8: 34}


def gemv_bytes(dtype: int, m: int, k: int, n: int = 1) -> int:
    """Algorithmic bytes of one GEMV: weights once + Q8_0 activations (34 B / block) + f32 output."""
    nb = k // 32
    wbytes = m * (k // 256) * 210 if dtype == 14 else m * nb * BW[dtype]  # 14 = Q6_K
    return wbytes + nb * 34 * n + 4 * m * n


def quant_bytes(n: int, k: int) -> int:
    return 4 * n * k + n * k + 2 * n * k // 32


def decode_call_sites():
    """(name, [m...], k) per launch of one decode step, in call order."""
    sites = []
    for layer in range(N_CONV + N_ATTN):
        if layer < N_CONV:
            sites.append((f"L{layer}.conv_in", [3 * HS], HS))
            sites.append((f"L{layer}.conv_out", [HS], HS))
        else:
            sites.append((f"L{layer}.attn_qkv", [HS, KV, KV], HS))
            sites.append((f"L{layer}.attn_o", [HS], HS))
        sites.append((f"L{layer}.ffn_gate_up", [IS, IS], HS))
        sites.append((f"L{layer}.ffn_down", [HS], IS))
    sites.append(("lm_head", [VOCAB], HS))
    return sites


def synth_many(O, jobs):
    """jobs: [(dtype, m, k, seed)] -> block bytes, generated on a thread pool (N(0, 0.02^2))."""
    with ThreadPoolExecutor(max_workers=min(16, os.cpu_count() or 4)) as pool:
        return list(pool.map(lambda j: O.synth_weight(j[0], j[1], j[2], seed=j[3]), jobs))


def synth_decode_weights(O, dtype: int):
    """Host block bytes for every weight of the step: {site: [bytes per matrix]}."""
    jobs, keys = [], []
    for si, (name, ms, k) in enumerate(decode_call_sites()):
        for wi, m in enumerate(ms):
            jobs.append((dtype, m, k, 1000 * dtype + 17 * si + wi))
            keys.append(name)
    out = {}
    for name, b in zip(keys, synth_many(O, jobs)):
        out.setdefault(name, []).append(b)
    return out


class DecodeStep:
    """Device state of one copy of the weight set + the enqueue order of a step."""

    def __init__(self, ctx, dtype, host_weights, d_x_hs, d_x_is):
        self.ctx, self.dtype = ctx, dtype
        self.sites = []
        for name, ms, k in decode_call_sites():
            ws = [ctx.upload_weight(b, dtype, m, k) for b, m in zip(host_weights[name], ms)]
            ys = [ctx.alloc(m * 4) for m in ms]
            self.sites.append((ws, ys, k))
        self.d_x = {HS: d_x_hs, IS: d_x_is}
        self.d_q = ctx.alloc(IS)
        self.d_s = ctx.alloc(IS // 32 * 4)

    def enqueue(self, fused=True):
        """fused: one launch per call site, the Q8_0 quantization of the activation is done
        inside the GEMV kernel.  Otherwise quantize and GEMV are separate launches."""
        ctx = self.ctx
        for ws, ys, k in self.sites:
            if fused:
                ctx.encode_gemv_fused(ws, self.d_x[k], 0, ys)
            else:
                ctx.quantize_q8_0(self.d_x[k], 1, k, k, self.d_q, self.d_s)
                ctx.gemv_with_preq_multi(ws, self.d_s, self.d_q, ys)

    def free(self):
        for ws, ys, _ in self.sites:
            for w in ws:
                w.free()
            for y in ys:
                y.free()
        self.d_q.free(), self.d_s.free()


def time_graphs(ctx, graphs, steps, warmup):
    """Events around `steps` graph launches (round-robin over `graphs`); returns ms per step."""
    for i in range(warmup):
        ctx.graph_launch(graphs[i % len(graphs)])
    ctx.sync()
    e0, e1 = ctx.event(), ctx.event()
    ctx.record(e0)
    for i in range(steps):
        ctx.graph_launch(graphs[i % len(graphs)])
    ctx.record(e1)
    ms = ctx.elapsed_ms(e0, e1)
    ctx.sync()
    ctx.event_destroy(e0), ctx.event_destroy(e1)
    return ms / steps


def bench_decode(ctx, W, O, dtype, steps, warmup, host_weights, with_unfused=True):
    x_hs = ctx.to_device(O.fill_normal(1, 1.0, HS))
    x_is = ctx.to_device(O.fill_normal(2, 1.0, IS))
    copies = [DecodeStep(ctx, dtype, host_weights, x_hs, x_is) for _ in range(2)]
    graphs = []
    for c in copies:
        ctx.graph_begin()
        c.enqueue()
        graphs.append(ctx.graph_end())
    ms_step = time_graphs(ctx, graphs, steps, warmup)
    # kernel-only durations: the same launches, eager, with per-dispatch timestamps
    ctx.kernel_timing_begin()
    for i in range(steps):
        copies[i % 2].enqueue()
    kt = ctx.kernel_timing_end()
    sites = decode_call_sites()
    gbytes = sum(gemv_bytes(dtype, m, k) for _, ms, k in sites for m in ms)
    wbytes = sum(m * (k // 32) * BW[dtype] for _, ms, k in sites for m in ms)
    res = {
        "dtype": dtype,
        "ms_per_step": ms_step,
        "gemv_bytes_per_step": gbytes,
        "weight_bytes_per_step": wbytes,
        "quantize_bytes_per_step": sum(quant_bytes(1, k) for _, _, k in sites),
        "gemv_launches_per_step": len(sites),
        "gemvs_per_step": sum(len(ms) for _, ms, _ in sites),
        "step_GBps": gbytes / ms_step / 1e6,
        "us_per_launch_in_graph": ms_step * 1e3 / len(sites),
        "gemv_kernel_ms_per_step": kt["gemv"][0] / steps,
        "gemv_kernel_GBps": gbytes / (kt["gemv"][0] / steps) / 1e6,
        "gemv_kernel_avg_us": kt["gemv"][0] / kt["gemv"][1] * 1e3,
    }
    if with_unfused:  # the same step with the quantizer as its own launch (two launches per call site)
        graphs2 = []
        for c in copies:
            ctx.graph_begin()
            c.enqueue(fused=False)
            graphs2.append(ctx.graph_end())
        res["ms_per_step_unfused_quantizer"] = time_graphs(ctx, graphs2, steps, warmup)
        for g in graphs2:
            ctx.graph_destroy(g)
    for g in graphs:
        ctx.graph_destroy(g)
    for c in copies:
        c.free()
    x_hs.free(), x_is.free()
    return res


def bench_single_gemv(ctx, W, O, dtype, m, k, launches=200, wb=None):
    """One GEMV shape, HBM-cold: rotate over enough weight copies to exceed the Infinity Cache."""
    wb = O.synth_weight(dtype, m, k, seed=4242) if wb is None else wb
    copies = max(3, int(300e6 // wb.nbytes) + 1)
    ws = [ctx.upload_weight(wb, dtype, m, k) for _ in range(copies)]
    s, q = O.quantize_q8_0(O.fill_normal(3, 1.0, k))
    d_q, d_s, d_y = ctx.to_device(q), ctx.to_device(s), ctx.alloc(m * 4)
    ctx.graph_begin()
    for w in ws:
        ctx.gemv_with_preq(w, d_s, d_q, d_y)
    g = ctx.graph_end()
    reps = max(1, launches // copies)
    ms = time_graphs(ctx, [g], reps, 2) / copies
    ctx.kernel_timing_begin()
    for _ in range(reps):
        for w in ws:
            ctx.gemv_with_preq(w, d_s, d_q, d_y)
    kt = ctx.kernel_timing_end()
    ctx.graph_destroy(g)
    kus = kt["gemv"][0] / kt["gemv"][1] * 1e3
    b = gemv_bytes(dtype, m, k)
    for w in ws:
        w.free()
    d_q.free(), d_s.free(), d_y.free()
    return {"m": m, "k": k, "dtype": dtype, "bytes": b, "weight_copies": copies, "us_per_launch_in_graph": ms * 1e3,
            "GBps_in_graph": b / ms / 1e6, "frac_of_hbm_peak_in_graph": b / ms / 1e6 / HBM_PEAK_GBS,
            "kernel_us": kus, "kernel_GBps": b / kus / 1e3, "kernel_frac_of_hbm_peak": b / kus / 1e3 / HBM_PEAK_GBS}


def lfm2_350m_image(O, body=2, embd=14, HS=HS, IS=IS, KV=KV):
    """A randomly initialised LFM2-350M-shaped model as a GGUF image: 16 layers (gated conv except attention at
    2, 5, 8, 10, 12, 14), hidden 1024, FFN 4608, 16 heads / 8 KV heads, vocabulary 65536, Q4_0 body with the tied
    embedding in Q6_K like the shipped Q4_0 files (tensor names of wick/src/model/lfm2.rs:97-300).  Other hidden / FFN /
    KV widths give the other sizes of the family (head_dim stays 64)."""
    from wick_amd import gguf as G

    attn = {2, 5, 8, 10, 12, 14}
    n_layers, hd = N_CONV + N_ATTN, 64
    names, jobs = ["token_embd.weight"], [(embd, VOCAB, HS, 9000)]
    for i in range(n_layers):
        p = f"blk.{i}."
        mats = ([("attn_q", HS, HS), ("attn_k", KV, HS), ("attn_v", KV, HS), ("attn_output", HS, HS)] if i in attn else
                [("shortconv.in_proj", 3 * HS, HS), ("shortconv.out_proj", HS, HS)])
        for j, (n, m, k) in enumerate(mats + [("ffn_gate", IS, HS), ("ffn_up", IS, HS), ("ffn_down", HS, IS)]):
            names.append(p + n + ".weight")
            jobs.append((body, m, k, 9100 + 16 * i + j))
    tensors = [(n, [j[2], j[1]], j[0], b) for n, j, b in zip(names, jobs, synth_many(O, jobs))]
    rng = np.random.default_rng(5)
    norm = lambda n: (1.0 + 0.1 * rng.standard_normal(n)).astype(np.float32)
    tensors.append(("token_embd_norm.weight", [HS], 0, norm(HS)))
    for i in range(n_layers):
        p = f"blk.{i}."
        tensors += [(p + "attn_norm.weight", [HS], 0, norm(HS)), (p + "ffn_norm.weight", [HS], 0, norm(HS))]
        if i in attn:
            tensors += [(p + "attn_q_norm.weight", [hd], 0, norm(hd)), (p + "attn_k_norm.weight", [hd], 0, norm(hd))]
        else:
            tensors.append((p + "shortconv.conv.weight", [3, HS], 0, (0.3 * rng.standard_normal(3 * HS)).astype(np.float32)))
    meta = [("general.architecture", G.T_STRING, "lfm2"), ("lfm2.block_count", G.T_U32, n_layers), ("lfm2.embedding_length", G.T_U32, HS),
            ("lfm2.feed_forward_length", G.T_U32, IS), ("lfm2.attention.head_count", G.T_U32, HS // hd), ("lfm2.vocab_size", G.T_U32, VOCAB),
            ("lfm2.rope.freq_base", G.T_F32, 1000000.0), ("lfm2.attention.layer_norm_rms_epsilon", G.T_F32, 1e-5),
            ("lfm2.shortconv.l_cache", G.T_U32, 3),
            ("lfm2.attention.head_count_kv", G.T_ARRAY, (G.T_I32, [KV // hd if i in attn else 0 for i in range(n_layers)]))]
    return G.build_image(meta, tensors)


def trace_lfm2_step(ctx, W, O, tokens=32, context=4096):
    """The same decode steps enqueued one by one (no graph replay), for a kernel tracer: 32 tokens from position 1024."""
    from wick_amd import gguf as G
    from wick_amd.lfm2 import RocmLfm2Model

    with G.GgufFile.from_bytes(lfm2_350m_image(O)) as g:
        model = RocmLfm2Model(ctx, g, context)
    model.set_graph_replay(False)
    picks = model.generate_greedy(1, 1024, tokens)
    model.free()
    return {"tokens": tokens, "start_pos": 1024, "last_pick": int(picks[-1])}


def bench_lfm2_step(ctx, W, O, tokens=64, context=4096, body=2, embd=14, dims=None, label="LFM2-350M-shaped"):
    """Whole decode steps of the model handle (embedding, 16 layers with their norms / conv / attention / gates, tied
    LM head, greedy pick), replayed as one graph per token with token and position resident on the device."""
    from wick_amd import gguf as G
    from wick_amd.lfm2 import RocmLfm2Model

    with G.GgufFile.from_bytes(lfm2_350m_image(O, body=body, embd=embd, **(dims or {}))) as g:
        model = RocmLfm2Model(ctx, g, context)
    model.generate_greedy(1, 0, 8)  # captures the graph, warms up
    names = {2: "Q4_0", 8: "Q8_0", 14: "Q6_K"}
    out = {"model": f"{label}, {names[body]} body + {names[embd]} tied embedding, random init", "context": context,
           "gpu_memory_MB": model.gpu_memory_bytes() / 1e6, "runs": []}
    for start in (0, 1024, context - tokens):  # attention cost grows with the position
        model.reset()
        t0 = time.perf_counter()
        model.generate_greedy(1, start, tokens)
        dt = time.perf_counter() - t0
        out["runs"].append({"start_pos": start, "tokens": tokens, "ms_per_token": dt / tokens * 1e3, "tokens_per_s": tokens / dt})
    # prompts: the batched pass (projections on the int8-MFMA GEMM)
    out["prefill"] = []
    for n in (512, 2002):
        toks = np.random.default_rng(n).integers(0, VOCAB, n)
        model.reset()
        model.forward_prefill(toks[:64], 0)  # buffers allocated, kernels warm
        model.reset()
        t0 = time.perf_counter()
        model.forward_prefill(toks, 0)
        dt = time.perf_counter() - t0
        out["prefill"].append({"prompt_tokens": n, "ms": dt * 1e3, "tokens_per_s": n / dt})
    # where the time goes: the same steps enqueued one by one with per-dispatch timestamps
    model.set_graph_replay(False)
    model.reset()
    model.generate_greedy(1, 1024, 4)
    ctx.kernel_timing_begin()
    model.generate_greedy(1, 1028, 16)
    kt = ctx.kernel_timing_end()
    out["kernel_time_per_token_at_pos_1024"] = {fam: {"us": ms / 16 * 1e3, "launches": n // 16} for fam, (ms, n) in kt.items() if n}
    model.free()
    return out


def bench_gemm(ctx, W, O, dtype, m, n, k, reps=20, wb=None, with_quantize=True):
    wb = O.synth_weight(dtype, m, k, seed=777) if wb is None else wb
    w = ctx.upload_weight(wb, dtype, m, k)
    d_x = ctx.to_device(O.fill_normal(9, 1.0, n * k))
    d_q, d_s, d_y = ctx.alloc(n * k), ctx.alloc(n * (k // 32) * 4), ctx.alloc(m * n * 4)

    def run():
        ctx.quantize_q8_0(d_x, n, k, k, d_q, d_s)
        ctx.gemm_preq(w, d_s, d_q, n, d_y, layout=W.LAYOUT_TOKEN_MAJOR)

    for _ in range(3):
        run()
    ctx.sync()
    e0, e1 = ctx.event(), ctx.event()
    ctx.record(e0)
    for _ in range(reps):
        run()
    ctx.record(e1)
    ms_both = ctx.elapsed_ms(e0, e1) / reps
    ctx.kernel_timing_begin()
    for _ in range(reps):
        run()
    kt = ctx.kernel_timing_end()
    ops = 2.0 * m * n * k
    fam = "gemm" if kt["gemm"][1] else "gemv"  # small n is served by the multi-token GEMV
    gemm_ms = kt[fam][0] / kt[fam][1]
    quant_ms = kt["quantize"][0] / kt["quantize"][1]
    w.free()
    for b in (d_x, d_q, d_s, d_y):
        b.free()
    return {"m": m, "n": n, "k": k, "dtype": dtype, "ops": ops, "kernel_family": fam, "quantize_plus_gemm_ms": ms_both,
            "quantize_plus_gemm_TOPS": ops / ms_both / 1e9, "gemm_kernel_ms": gemm_ms, "gemm_kernel_TOPS": ops / gemm_ms / 1e9,
            "frac_of_int8_peak": ops / gemm_ms / 1e9 / INT8_PEAK_TOPS,
            "quantize_kernel_ms": quant_ms, "quantize_kernel_GBps": quant_bytes(n, k) / quant_ms / 1e6}


def bench_prefill_sites(ctx, W, O, n=4096, dtype=8):
    """The nine per-layer prefill GEMMs of an LFM2-1.2B-shaped layer at n tokens (Q8_0)."""
    hs, is_, kv = 2048, 6912, 512
    sites = [("conv_in", 3 * hs, hs), ("conv_out", hs, hs), ("attn_q", hs, hs), ("attn_k", kv, hs), ("attn_v", kv, hs),
             ("attn_o", hs, hs), ("ffn_gate", is_, hs), ("ffn_up", is_, hs), ("ffn_down", hs, is_)]
    blobs = synth_many(O, [(dtype, m, k, 300 + i) for i, (_, m, k) in enumerate(sites)])
    out, tot_ops, tot_ms = [], 0.0, 0.0
    for (name, m, k), wb in zip(sites, blobs):
        r = bench_gemm(ctx, W, O, dtype, m, n, k, reps=5, wb=wb)
        out.append({"site": name, "m": m, "k": k, "gemm_kernel_ms": r["gemm_kernel_ms"], "TOPS": r["gemm_kernel_TOPS"],
                    "frac_of_int8_peak": r["frac_of_int8_peak"]})
        tot_ops += r["ops"]
        tot_ms += r["gemm_kernel_ms"]
    return {"n": n, "dtype": dtype, "sites": out, "total_ops": tot_ops, "total_gemm_ms": tot_ms, "TOPS": tot_ops / tot_ms / 1e9}


def bench_lm_head_sweep(ctx, W, O, dtype=8, m=65536, k=2048, ns=(1, 4, 16, 64)):
    """Tied LM head: where the bandwidth-bound multi-token GEMV hands off to the MFMA GEMM.
    Each n is timed through both kernels (hand-off forced), HBM-cold over three weight copies."""
    wb = O.synth_weight(dtype, m, k, seed=999)
    ws = [ctx.upload_weight(wb, dtype, m, k) for _ in range(3)]
    nmax = max(ns)
    x = O.fill_normal(5, 1.0, nmax * k)
    s, q = O.quantize_q8_0_batch(x, nmax, k)
    d_q, d_s, d_y = ctx.to_device(q), ctx.to_device(s), ctx.alloc(m * nmax * 4)
    rows = []
    for n in ns:
        row = {"n": n, "bytes": gemv_bytes(dtype, m, k, n), "ops": 2.0 * m * n * k}
        for label, min_n in (("gemv", 1 << 30), ("mfma", 1)):
            if label == "mfma" and n == 1:
                continue
            ctx.set_gemm_min_n(min_n)
            ctx.graph_begin()
            for w in ws:
                ctx.gemm_preq(w, d_s, d_q, n, d_y, y_stride=m, layout=W.LAYOUT_TOKEN_MAJOR)
            g = ctx.graph_end()
            ms = time_graphs(ctx, [g], 4, 1) / len(ws)
            ctx.graph_destroy(g)
            row[label] = {"us": ms * 1e3, "GBps": row["bytes"] / ms / 1e6, "TOPS": row["ops"] / ms / 1e9}
        ctx.set_gemm_min_n(0)
        rows.append(row)
    for w in ws:
        w.free()
    d_q.free(), d_s.free(), d_y.free()
    crossover = next((r["n"] for r in rows if "mfma" in r and r["mfma"]["us"] < r["gemv"]["us"]), None)
    return {"dtype": dtype, "m": m, "k": k, "rows": rows, "first_n_where_mfma_wins": crossover, "library_hand_off_n": W.GEMM_MIN_N}


def bench_probe(ctx, iters=20000):
    """Register-only ceilings of this GPU for the GEMM's two bounds (no memory traffic)."""
    out = {}
    for shape, name, unit in [(0, "mfma_i32_32x32x32_i8", "TOP/s"), (1, "mfma_i32_16x16x32_i8", "TOP/s"), (2, "v_fma_f32", "TFLOP/s"),
                              (3, "block_loop_8xmfma16_plus_64_scaling_fma", "TOP/s"), (4, "block_loop_2xmfma32_plus_64_scaling_fma", "TOP/s")]:
        ctx.probe_rate(shape, iters)
        ctx.sync()
        e0, e1 = ctx.event(), ctx.event()
        ctx.record(e0)
        ops = ctx.probe_rate(shape, iters)
        ctx.record(e1)
        ms = ctx.elapsed_ms(e0, e1)
        ctx.event_destroy(e0), ctx.event_destroy(e1)
        out[name] = {"value": ops / ms / 1e9, "unit": unit, "ms": ms}
    return out


def bench_copy(ctx, nbytes=256 << 20, reps=10):
    """Device-to-device copy of a known size: calibration of the FETCH_SIZE / WRITE_SIZE counters."""
    a, b = ctx.alloc(nbytes), ctx.alloc(nbytes)
    ctx.copy(b, a, nbytes)
    ctx.sync()
    e0, e1 = ctx.event(), ctx.event()
    ctx.record(e0)
    for _ in range(reps):
        ctx.copy(b, a, nbytes)
    ctx.record(e1)
    ms = ctx.elapsed_ms(e0, e1) / reps
    a.free(), b.free()
    return {"bytes": nbytes, "ms": ms, "GBps_read_plus_write": 2 * nbytes / ms / 1e6}


def bench_upload(ctx, nbytes=256 << 20, reps=3):
    """Host -> device rate of wick_rocm_upload from ordinary (pageable) host memory: what loading a model's weights costs
    once; no step of the path crosses PCIe afterwards."""
    host = np.ones(nbytes, np.uint8)
    d = ctx.alloc(nbytes)
    d.upload(host)
    ctx.sync()
    t0 = time.perf_counter()
    for _ in range(reps):
        d.upload(host)
    ctx.sync()
    dt = (time.perf_counter() - t0) / reps
    d.free()
    return {"bytes": nbytes, "ms": dt * 1e3, "GBps": nbytes / dt / 1e9}


def cpu_baseline(O, dtype, host_weights, budget_s=12.0):
    """The reference's x86 path for the same step: per call site a serial f32 GEMV
    (wick/src/backend/cpu.rs:293-306; Q8_0 rows would be chunked over threads).  Runs
    whole steps until ~budget_s of CPU time, at least one."""
    sites = decode_call_sites()
    xs = {HS: O.fill_normal(1, 1.0, HS), IS: O.fill_normal(2, 1.0, IS)}
    threads = os.cpu_count() or 1
    gbytes = sum(gemv_bytes(dtype, m, k) for _, ms, k in sites for m in ms)
    used = 1
    t0 = time.perf_counter()
    steps = 0
    while True:
        for name, ms, k in sites:
            for b, m in zip(host_weights[name], ms):
                _, u = O.x86_gemv_f32(dtype, b, xs[k], m, k, threads=threads)
                used = max(used, u)
        steps += 1
        if time.perf_counter() - t0 >= budget_s:
            break
    dt = time.perf_counter() - t0
    return {"value": gbytes * steps / dt / 1e9, "unit": "GB/s", "cores": used, "kind": "port",
            "sample": f"{steps} full decode steps ({gbytes * steps / 1e6:.0f} MB of GEMV work) in {dt:.1f} s; x86 f32 per-block AVX2 path "
                      "restated in C (the reference's integer kernels are aarch64-only)",
            "ms_per_step": dt / steps * 1e3}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--skip-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--skip-extra", action="store_true", help="only the headline decode step (+ CPU baseline)")
    ap.add_argument("--leg", default="all", help="all | decode | decode_q8 | gemv | gemm | prefill_sites | lm_head | lm_head_q6k | upload | lfm2_step | lfm2_step_q8 | lfm2_step_1p2b | lfm2_step_trace | copy | probe | cpu")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs on ONE GPU only (no collectives, no sharding); use --gpus 1", file=sys.stderr)
        sys.exit(2)

    import wick_amd as W
    from oracle import oracle as O  # cpu_baseline leg + synthetic inputs only; never in the timed GPU path

    leg = args.leg
    if leg == "cpu":
        print(json.dumps({"cpu_baseline": cpu_baseline(O, W.Q4_0, synth_decode_weights(O, W.Q4_0))}))
        return
    ctx = W.RocmContext(0)
    if leg != "all":
        one = {
            "decode": lambda: bench_decode(ctx, W, O, W.Q4_0, args.steps, args.warmup, synth_decode_weights(O, W.Q4_0), with_unfused=False),
            "decode_q8": lambda: bench_decode(ctx, W, O, W.Q8_0, args.steps, args.warmup, synth_decode_weights(O, W.Q8_0), with_unfused=False),
            "gemv": lambda: bench_single_gemv(ctx, W, O, W.Q4_0, 6912, 2048),
            "gemm": lambda: bench_gemm(ctx, W, O, W.Q4_0, 6912, 2002, 2048),
            "prefill_sites": lambda: bench_prefill_sites(ctx, W, O),
            "lm_head": lambda: bench_lm_head_sweep(ctx, W, O),
            "lm_head_q6k": lambda: bench_single_gemv(ctx, W, O, W.Q6_K, 65536, 1024),
            "lfm2_step": lambda: bench_lfm2_step(ctx, W, O),
            "lfm2_step_q8": lambda: bench_lfm2_step(ctx, W, O, body=8, embd=8),
            # the per-layer shapes of BASELINE's LFM2-1.2B call sites: hidden 2048, FFN 6912, 32 heads / 8 KV heads
            "lfm2_step_1p2b": lambda: bench_lfm2_step(ctx, W, O, dims=dict(HS=2048, IS=6912, KV=512), label="LFM2-1.2B-shaped"),
            "lfm2_step_trace": lambda: trace_lfm2_step(ctx, W, O),
            "copy": lambda: bench_copy(ctx),
            "upload": lambda: bench_upload(ctx),
            "probe": lambda: bench_probe(ctx),
        }
        if leg not in one:
            print(f"bench.py: unknown leg {leg}", file=sys.stderr)
            sys.exit(2)
        print(json.dumps({leg: one[leg]()}))
        ctx.close()
        return

    dtype = W.Q4_0
    host_weights = synth_decode_weights(O, dtype)
    dec = bench_decode(ctx, W, O, dtype, args.steps, args.warmup, host_weights)

    out = {
        "metric": "Q4_0 GEMV GB/s (% HBM peak) + prefill int8 GEMM TOPS (% MFMA peak)",
        "value": dec["step_GBps"],
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": dec["ms_per_step"],
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "i8",
        "data": "synthetic",
        "config": {
            "workload": "LFM2-350M-shaped decode-step weight set, Q4_0 weights x Q8_0 activations, n=1: 93 GEMVs in 65 launches, "
                        "each quantizing its f32 activation in-kernel; one HIP graph per step, two weight copies alternated (HBM-cold)",
            "device": ctx.device_name,
            "value_definition": "algorithmic GEMV bytes per step (weights + Q8_0 activations + f32 outputs) / step time, activation quantization included in the time",
        },
        "roofline": {
            "bound": "hbm",
            "kernel": "gemv_pairs_kernel (all instantiations of the step, fused quantizer)",
            "achieved": dec["gemv_kernel_GBps"],
            "peak": HBM_PEAK_GBS,
            "unit": "GB/s",
            "frac": dec["gemv_kernel_GBps"] / HBM_PEAK_GBS,
            # HBM bytes per launch (average over the 65 launches of a step) from the calibrated FETCH_SIZE / WRITE_SIZE passes
            # recorded in profiles/decode_step_lfm2_350m_q4_0.txt: mean over all GEMV dispatches of the step, 3.21 MB read + 0.02 MB written
            "traffic": 3.23e6,
            "traffic_source": "profiles/decode_step_lfm2_350m_q4_0.txt (rocprofv3 --pmc FETCH_SIZE x2.0, WRITE_SIZE x1.0; copy-calibrated)",
            "bytes_per_launch_avg": dec["gemv_bytes_per_step"] / dec["gemv_launches_per_step"],
            "avg_launch_us": dec["gemv_kernel_avg_us"],
            "note": "per-dispatch timestamps include a fixed dispatch cost per launch; in the graph the same launches average "
                    f"{dec['us_per_launch_in_graph']:.2f} us each",
        },
        "decode_step": dec,
    }

    if not args.skip_extra:
        out["gemv_6912x2048"] = bench_single_gemv(ctx, W, O, W.Q4_0, 6912, 2048)
        g = bench_gemm(ctx, W, O, W.Q4_0, 6912, 2002, 2048)
        g["roofline"] = {"bound": "mfma", "kernel": "gemm_mfma_kernel<Q4_0>", "achieved": g["gemm_kernel_TOPS"], "peak": INT8_PEAK_TOPS,
                         "unit": "TOP/s", "frac": g["gemm_kernel_TOPS"] / INT8_PEAK_TOPS,
                         # 88.97 MB read + 55.39 MB written per launch (algorithmic 12.57 + 55.35 MB), profiles/gemm_q4_0_6912x2002x2048.txt
                         "traffic": 144.4e6, "traffic_source": "profiles/gemm_q4_0_6912x2002x2048.txt"}
        out["gemm"] = g
        out["measured_ceilings"] = bench_probe(ctx)
        g["roofline"]["frac_of_measured_mfma_ceiling"] = g["gemm_kernel_TOPS"] / out["measured_ceilings"]["mfma_i32_32x32x32_i8"]["value"]
        del host_weights  # the CPU leg regenerates what it needs; keep host memory low
        dq = bench_decode(ctx, W, O, W.Q8_0, max(10, args.steps // 2), args.warmup, synth_decode_weights(O, W.Q8_0), with_unfused=False)
        out["decode_step_q8_0"] = dq
        out["prefill_sites"] = bench_prefill_sites(ctx, W, O)
        out["lm_head_sweep"] = bench_lm_head_sweep(ctx, W, O)
        # shipped LFM2 Q4_0 files keep the tied embedding / LM head in Q6_K (wick/src/model/metal_lfm2.rs:175-180)
        out["lm_head_q6_k_65536x1024"] = bench_single_gemv(ctx, W, O, W.Q6_K, 65536, 1024)
        out["lfm2_decode_step"] = bench_lfm2_step(ctx, W, O)
        host_weights = None
    ctx.close()
    if not args.skip_cpu:
        out["cpu_baseline"] = cpu_baseline(O, dtype, host_weights or synth_decode_weights(O, dtype))
    print(json.dumps(out))


if __name__ == "__main__":
    main()
