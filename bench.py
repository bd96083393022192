#!/usr/bin/env python3
"""Benchmark of the block-quantized matmul hot path on one MI355X.

Headline (what `value`, `ms_per_step`, `config` and `roofline` describe): the single decode GEMV the HBM target is
quoted on, Q4_0 6912 x 2048 (LFM2-1.2B ffn_up) against one Q8_0-quantized token.  A "step" is one replay of a HIP graph
that runs this GEMV once on each of 38 distinct device copies of the weight (303 MB, more than the 256 MB Infinity Cache),
so every launch streams its 8 MB of weights from HBM.  The launches of a graph are chained on one stream, like the
GEMVs of a decode step are.  Each replay is bracketed by its own pair of events: mean (= ms_per_step), median, min,
p10 / p90 over the timed steps are reported.

Beside it, in the same JSON line:
  roofline         the GEMV kernel: algorithmic bytes per launch / average launch duration of the timed region
                   (step time / 38; the kernel runs nowhere else in that region), against 8 TB/s.  Inside it:
                   kernel_span_* = the launch clocked by the kernel itself inside the same graph (first wave's first
                   instruction -> last wave's last store acknowledged) and gap_between_dependent_launches_us, both from the
                   timing-hook instantiation in libwick_rocm_bench.so; independent_streams_* = gemv_concurrent's figure;
                   gemm = the prefill GEMM's roofline object (bound "mfma"), so that both halves of the metric sit in one
                   place; lm_head_* = where the hand-off sweep says the MFMA kernel starts to win and where the library
                   hands off
  gemv_concurrent  the same launches as INDEPENDENT work on four streams: what the kernel sustains when the gap between
                   dependent launches is taken out of the picture
  gemm             the prefill GEMM the matrix-core target is quoted on (Q4_0, m=6912, n=2002, k=2048) with its own
                   roofline object (per-launch kernel timestamps, median / min over 100 launches)
  decode_step, decode_step_q8_0, prefill_sites, lm_head_sweep, lm_head_q6_k_65536x1024, lfm2_decode_step
                   the other configurations (LFM2-350M-shaped decode weight set, the nine LFM2-1.2B prefill call sites at
                   n = 4096, the 65536 x 2048 head at n = 1 / 4 / 5 / 6 / 8 / 12 / 16 / 64, a whole model step;
                   `--leg lfm2_step_kv16` times the same model with f16 KV caches)
  cpu_baseline     the reference's x86 CPU path (f32 per-token GEMV; Q4_0 rows serial, Q8_0 rows over T threads) timed on
                   this host on bounded samples of the same workloads

`--leg NAME` runs one leg only (used for profiling; `c1` replays graphs and launches nothing else).
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


def stats(samples_ms, per=1):
    """mean / median / min / p10 / p90 of per-step samples, in microseconds per `per` launches."""
    a = np.asarray(samples_ms, np.float64) * 1e3 / per
    return {"mean_us": float(a.mean()), "median_us": float(np.median(a)), "min_us": float(a.min()), "p10_us": float(np.percentile(a, 10)),
            "p90_us": float(np.percentile(a, 90)), "samples": int(a.size)}


def time_graph_steps(ctx, graphs, steps, warmup):
    """Like time_graphs, with an event between consecutive replays: returns (ms per step over the whole timed region,
    [ms of each step])."""
    for i in range(warmup):
        ctx.graph_launch(graphs[i % len(graphs)])
    ctx.sync()
    ev = [ctx.event() for _ in range(steps + 1)]
    ctx.record(ev[0])
    for i in range(steps):
        ctx.graph_launch(graphs[i % len(graphs)])
        ctx.record(ev[i + 1])
    total = ctx.elapsed_ms(ev[0], ev[steps])
    each = [ctx.elapsed_ms(ev[i], ev[i + 1]) for i in range(steps)]
    ctx.sync()
    for e in ev:
        ctx.event_destroy(e)
    return total / steps, each


C1 = (6912, 2048)  # LFM2-1.2B ffn_up: the shape the HBM target is quoted on


def bench_c1(ctx, W, O, steps, warmup, with_concurrent=True):
    """Q4_0 6912 x 2048 decode GEMV, HBM-cold: one step = one graph replay = one launch on each of `copies` weight copies."""
    m, k = C1
    dtype = W.Q4_0
    wb = O.synth_weight(dtype, m, k, seed=4242)
    copies = int(300e6 // wb.nbytes) + 1  # 38: beyond the 256 MB Infinity Cache
    ws = [ctx.upload_weight(wb, dtype, m, k) for _ in range(copies)]
    s, q = O.quantize_q8_0(O.fill_normal(3, 1.0, k))
    d_q, d_s, d_y = ctx.to_device(q), ctx.to_device(s), ctx.alloc(m * 4)
    ctx.graph_begin()
    for w in ws:
        ctx.gemv_with_preq(w, d_s, d_q, d_y)
    g = ctx.graph_end()
    ms_step, each = time_graph_steps(ctx, [g], steps, warmup)
    ctx.graph_destroy(g)
    b = gemv_bytes(dtype, m, k)
    res = {"m": m, "k": k, "dtype": dtype, "bytes_per_launch": b, "weight_copies": copies, "launches_per_step": copies, "ms_per_step": ms_step,
           "per_launch_in_graph": stats(each, copies), "GBps": b * copies / ms_step / 1e6}
    res["kernel_span"] = bench_c1_span(ctx, W, ws, d_q, d_s, d_y, m, steps=min(steps, 20), warmup=warmup)
    if with_concurrent:
        res["concurrent"] = bench_c1_concurrent(ctx, W, ws, d_q, d_s, b, m)
    for w in ws:
        w.free()
    d_q.free(), d_s.free(), d_y.free()
    return res


def bench_c1_span(ctx, W, ws, d_q, d_s, d_y, m, steps, warmup):
    """Execution span of the GEMV launches INSIDE a graph replay: the same chain of launches through the product kernel with its
    timing hook (two reads of the 100 MHz wall clock per wave, libwick_rocm_bench.so); span of a launch = first wave's first
    instruction -> last wave's last store acknowledged.  A kernel tracer cannot give this figure (it splits a replay into single
    dispatches and inflates each); per-dispatch events cannot either (graph nodes carry none)."""
    from wick_amd import benchlib as B

    spans = [ctx.alloc(m * 16) for _ in ws]
    ctx.graph_begin()
    waves = [B.gemv_q8_span(ctx, w, d_s, d_q, d_y, sp, m) for w, sp in zip(ws, spans)]
    g = ctx.graph_end()
    ms_step, _ = time_graph_steps(ctx, [g], steps, warmup)
    per_launch, gaps, start_off, wave_dur = [], [], [], []
    for _ in range(3):  # three more replays, each read back
        ctx.graph_launch(g)
        ctx.sync()
        rec = [sp.download(np.uint64, 2 * nw).reshape(nw, 2) for sp, nw in zip(spans, waves)]
        per_launch += [B.span_us(r) for r in rec]
        start_off += [(r[:, 0] - r[:, 0].min()).astype(np.float64) / 100.0 for r in rec]
        wave_dur += [(r[:, 1] - r[:, 0]).astype(np.float64) / 100.0 for r in rec]
        starts, ends = [int(r[:, 0].min()) for r in rec], [int(r[:, 1].max()) for r in rec]
        gaps += [(starts[i + 1] - ends[i]) / 100.0 for i in range(len(rec) - 1)]
    ctx.graph_destroy(g)
    for sp in spans:
        sp.free()
    a, gp = np.asarray(per_launch), np.asarray(gaps)
    so, wd = np.concatenate(start_off), np.concatenate(wave_dur)
    inside = {"wave_start_after_first_wave_us": {f"p{q}": float(np.percentile(so, q)) for q in (50, 90, 99, 100)},
              "wave_duration_us": {f"p{q}": float(np.percentile(wd, q)) for q in (1, 50, 90, 100)}}
    return {"launches_per_step": len(ws), "waves_per_launch": waves[0], **inside, "span_us_mean": float(a.mean()), "span_us_median": float(np.median(a)),
            "span_us_min": float(a.min()), "span_us_p90": float(np.percentile(a, 90)), "samples": int(a.size),
            "gap_to_next_launch_us_mean": float(gp.mean()), "gap_to_next_launch_us_median": float(np.median(gp)),
            "step_ms_with_hook": ms_step, "sum_of_spans_ms": float(a.mean()) * len(ws) / 1e3, "clock": "100 MHz wall clock (s_memrealtime), 10 ns steps"}


def bench_c1_concurrent(ctx, W, ws, d_q, d_s, b, m, streams=4, passes=8, reps=12):
    """The same GEMVs as independent work: `streams` contexts (one stream each, default priority, within the four hardware
    queues of a process), each replaying a graph over its own share of the weight copies with its own output.  Nothing
    orders a launch after a launch of another stream, so the time per launch is what the kernel sustains, not the gap
    between dependent dispatches.  Timed on the host around launch ... sync of all streams (>= 10 ms of GPU work)."""
    ctxs = [ctx] + [W.RocmContext(0) for _ in range(streams - 1)]
    graphs, outs, count = [], [], 0
    for i, c in enumerate(ctxs):
        mine = ws[i::streams]
        d_y = c.alloc(m * 4)
        outs.append(d_y)
        c.graph_begin()
        for _ in range(passes):
            for w in mine:
                c.gemv_with_preq(w, d_s, d_q, d_y)
        graphs.append(c.graph_end())
        count += passes * len(mine)

    def round_trip():
        for c, g in zip(ctxs, graphs):
            c.graph_launch(g)

    for _ in range(2):
        round_trip()
    for c in ctxs:
        c.sync()
    samples = []
    for _ in range(reps):
        t0 = time.perf_counter()
        for _ in range(4):
            round_trip()
        for c in ctxs:
            c.sync()
        samples.append((time.perf_counter() - t0) * 1e3 / 4)
    for c, g, y in zip(ctxs, graphs, outs):
        c.graph_destroy(g)
        y.free()
    for c in ctxs[1:]:
        c.close()
    st = stats(samples, count)
    return {"streams": streams, "launches_per_round": count, "per_launch": st, "GBps_median": b / st["median_us"] / 1e3,
            "GBps_best": b / st["min_us"] / 1e3, "frac_of_hbm_peak_median": b / st["median_us"] / 1e3 / HBM_PEAK_GBS,
            "timing": "host clock around 4 rounds of graph launches on every stream + sync of all streams"}


def bench_decode(ctx, W, O, dtype, steps, warmup, host_weights, with_unfused=True, graph_only=False):
    x_hs = ctx.to_device(O.fill_normal(1, 1.0, HS))
    x_is = ctx.to_device(O.fill_normal(2, 1.0, IS))
    copies = [DecodeStep(ctx, dtype, host_weights, x_hs, x_is) for _ in range(2)]
    graphs = []
    for c in copies:
        ctx.graph_begin()
        c.enqueue()
        graphs.append(ctx.graph_end())
    ms_step, each = time_graph_steps(ctx, graphs, steps, warmup)
    # kernel-only durations: the same launches, eager, with per-dispatch timestamps (not under a kernel tracer: graph_only)
    kt = {"gemv": (float("nan"), 1)}
    if not graph_only:
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
        "per_step": stats(each),
        "gemv_bytes_per_step": gbytes,
        "weight_bytes_per_step": wbytes,
        "quantize_bytes_per_step": sum(quant_bytes(1, k) for _, _, k in sites),
        "gemv_launches_per_step": len(sites),
        "gemvs_per_step": sum(len(ms) for _, ms, _ in sites),
        "step_GBps": gbytes / ms_step / 1e6,
        "us_per_launch_in_graph": ms_step * 1e3 / len(sites),
        "eager_gemv_kernel_ms_per_step": kt["gemv"][0] / steps,
        "eager_gemv_kernel_avg_us": kt["gemv"][0] / kt["gemv"][1] * 1e3,
        "eager_note": "per-dispatch timestamps of the same launches issued one by one, outside a graph: each carries dispatch cost that a graph "
                      "replay does not pay, so their sum exceeds the replayed step",
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


def trace_lfm2_prefill(ctx, W, O, n=2002, context=4096):
    """One warm prompt pass of n tokens, for a kernel tracer (eager launches only)."""
    from wick_amd import gguf as G
    from wick_amd.lfm2 import RocmLfm2Model

    with G.GgufFile.from_bytes(lfm2_350m_image(O)) as g:
        model = RocmLfm2Model(ctx, g, context)
    toks = np.random.default_rng(n).integers(0, VOCAB, n)
    for _ in range(2):
        model.reset()
        logits = model.forward_prefill(toks, 0)
    model.free()
    return {"prompt_tokens": n, "passes": 2, "argmax": int(np.argmax(logits))}


def bench_lfm2_step(ctx, W, O, tokens=64, context=4096, body=2, embd=14, dims=None, label="LFM2-350M-shaped", kernel_times=True, kv_f16=False):
    """Whole decode steps of the model handle (embedding, 16 layers with their norms / conv / attention / gates, tied
    LM head, greedy pick), replayed as one graph per token with token and position resident on the device."""
    from wick_amd import gguf as G
    from wick_amd.lfm2 import RocmLfm2Model

    with G.GgufFile.from_bytes(lfm2_350m_image(O, body=body, embd=embd, **(dims or {}))) as g:
        model = RocmLfm2Model(ctx, g, context, kv_f16=kv_f16)
    model.generate_greedy(1, 0, 8)  # captures the graph, warms up
    names = {2: "Q4_0", 8: "Q8_0", 14: "Q6_K"}
    out = {"model": f"{label}, {names[body]} body + {names[embd]} tied embedding, random init", "context": context, "kv_cache": "f16" if kv_f16 else "f32",
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
        model.forward_prefill(toks, 0)  # buffers sized for this prompt, kernels warm
        ts = []
        for _ in range(7):
            model.reset()
            t0 = time.perf_counter()
            model.forward_prefill(toks, 0)  # tokens up, the batched pass, the last token's logits down
            ts.append(time.perf_counter() - t0)
        dt = float(np.median(ts))
        out["prefill"].append({"prompt_tokens": n, "ms": dt * 1e3, "ms_min": min(ts) * 1e3, "samples": len(ts), "tokens_per_s": n / dt})
    if kernel_times:
        ctx.kernel_timing_begin()
        model.reset()
        model.forward_prefill(toks, 0)
        kt = ctx.kernel_timing_end()
        out["prefill_kernel_time_2002"] = {fam: {"us": ms * 1e3, "launches": n} for fam, (ms, n) in kt.items() if n}
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


def bench_gemm(ctx, W, O, dtype, m, n, k, reps=20, wb=None, samples=20):
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
    gemm_samples, quant_samples, fam = [], [], "gemm"
    for _ in range(samples):  # one launch per timing window: a sample per launch (per-dispatch timestamps, the quantity a kernel trace reports)
        ctx.kernel_timing_begin()
        run()
        kt = ctx.kernel_timing_end()
        fam = "gemm" if kt["gemm"][1] else "gemv"  # small n is served by the multi-token GEMV
        gemm_samples.append(kt[fam][0])
        quant_samples.append(kt["quantize"][0])
    ops = 2.0 * m * n * k
    gemm_ms = float(np.mean(gemm_samples))
    quant_ms = float(np.mean(quant_samples))
    w.free()
    for b in (d_x, d_q, d_s, d_y):
        b.free()
    return {"m": m, "n": n, "k": k, "dtype": dtype, "ops": ops, "kernel_family": fam, "quantize_plus_gemm_ms": ms_both,
            "quantize_plus_gemm_TOPS": ops / ms_both / 1e9, "gemm_kernel_ms": gemm_ms, "gemm_kernel_TOPS": ops / gemm_ms / 1e9,
            "frac_of_int8_peak": ops / gemm_ms / 1e9 / INT8_PEAK_TOPS, "gemm_kernel_per_launch": stats(gemm_samples),
            "gemm_kernel_TOPS_median": ops / float(np.median(gemm_samples)) / 1e9, "gemm_kernel_TOPS_best": ops / float(np.min(gemm_samples)) / 1e9,
            "quantize_kernel_ms": quant_ms, "quantize_kernel_GBps": quant_bytes(n, k) / quant_ms / 1e6}


def bench_gemm_multi(ctx, W, O, dtype, ms, n, k, blobs, samples=5):
    """1..3 weights over the same quantized activations in ONE launch (Q | K | V, gate | up of a prompt pass)."""
    ws = [ctx.upload_weight(b, dtype, m, k) for b, m in zip(blobs, ms)]
    d_x = ctx.to_device(O.fill_normal(9, 1.0, n * k))
    stride = sum(ms)
    d_q, d_s, d_y = ctx.alloc(n * k), ctx.alloc(n * (k // 32) * 4), ctx.alloc(stride * n * 4)
    ctx.quantize_q8_0(d_x, n, k, k, d_q, d_s)
    ys = [d_y.ptr + 4 * int(o) for o in np.concatenate([[0], np.cumsum(ms)[:-1]])]
    run = lambda: ctx.gemm_preq_multi(ws, d_s, d_q, n, ys, stride, layout=W.LAYOUT_TOKEN_MAJOR)
    for _ in range(2):
        run()
    ctx.sync()
    ts = []
    for _ in range(samples):
        ctx.kernel_timing_begin()
        run()
        ts.append(ctx.kernel_timing_end()["gemm"][0])
    for w in ws:
        w.free()
    for b in (d_x, d_q, d_s, d_y):
        b.free()
    ops = 2.0 * sum(ms) * n * k
    return {"ops": ops, "gemm_kernel_ms": float(np.mean(ts)), "gemm_kernel_TOPS": ops / float(np.mean(ts)) / 1e9, "per_launch": stats(ts)}


def bench_prefill_sites(ctx, W, O, n=4096, dtype=8):
    """The nine per-layer prefill GEMMs of an LFM2-1.2B-shaped layer at n tokens (Q8_0), launched the way the prompt pass
    launches them (wick_rocm_lfm2_forward_prefill): projections that share their input -- Q | K | V and gate | up -- as one
    launch over their weights, the others on their own.  K and V alone (512 rows each: half the chip has no tile) are
    listed too, for reference."""
    hs, is_, kv = 2048, 6912, 512
    sites = [("conv_in", 3 * hs, hs), ("conv_out", hs, hs), ("attn_q", hs, hs), ("attn_k", kv, hs), ("attn_v", kv, hs),
             ("attn_o", hs, hs), ("ffn_gate", is_, hs), ("ffn_up", is_, hs), ("ffn_down", hs, is_)]
    blobs = dict(zip([s_[0] for s_ in sites], synth_many(O, [(dtype, m, k, 300 + i) for i, (_, m, k) in enumerate(sites)])))
    dims = {name: (m, k) for name, m, k in sites}
    launches = [("conv_in",), ("conv_out",), ("attn_q", "attn_k", "attn_v"), ("attn_o",), ("ffn_gate", "ffn_up"), ("ffn_down",)]
    out, tot_ops, tot_ms = [], 0.0, 0.0
    for group in launches:
        ms, k = [dims[g][0] for g in group], dims[group[0]][1]
        if len(group) == 1:
            r = bench_gemm(ctx, W, O, dtype, ms[0], n, k, reps=3, wb=blobs[group[0]], samples=5)
        else:
            r = bench_gemm_multi(ctx, W, O, dtype, ms, n, k, [blobs[g] for g in group])
        out.append({"launch": "+".join(group), "m": ms, "k": k, "gemm_kernel_ms": r["gemm_kernel_ms"], "TOPS": r["gemm_kernel_TOPS"],
                    "frac_of_int8_peak": r["gemm_kernel_TOPS"] / INT8_PEAK_TOPS})
        tot_ops += r["ops"]
        tot_ms += r["gemm_kernel_ms"]
    alone = []
    for name in ("attn_k", "attn_v"):
        r = bench_gemm(ctx, W, O, dtype, dims[name][0], n, dims[name][1], reps=3, wb=blobs[name], samples=5)
        alone.append({"site": name, "m": dims[name][0], "gemm_kernel_ms": r["gemm_kernel_ms"], "TOPS": r["gemm_kernel_TOPS"]})
    res = {"n": n, "dtype": dtype, "launches": out, "k_v_on_their_own": alone, "total_ops": tot_ops, "total_gemm_ms": tot_ms,
           "TOPS": tot_ops / tot_ms / 1e9}
    res["ffn_gate_up_to_q8"] = [bench_gate_up_fused(ctx, W, O, dtype, is_, hs, n, blobs["ffn_gate"], blobs["ffn_up"]),
                                bench_gate_up_fused(ctx, W, O, W.Q4_0, 4608, 1024, 2002), bench_gate_up_fused(ctx, W, O, W.Q8_0, 4608, 1024, 2002),
                                bench_gate_up_fused(ctx, W, O, W.Q4_0, 6912, 2048, 2002), bench_gate_up_fused(ctx, W, O, W.Q4_0, 6912, 1024, 2002),
                                bench_gate_up_fused(ctx, W, O, W.Q4_0, 4608, 2048, 2002), bench_gate_up_fused(ctx, W, O, W.Q4_0, 4608, 2048, 1024)]
    return res


def bench_gate_up_fused(ctx, W, O, dtype, m, k, n, wg=None, wu=None, reps=5):
    """gate | up of a prompt pass up to the down projection's Q8_0 input: one GEMM launch over both weights + the SiLU gate /
    quantizer kernel, against the GEMM whose epilogue gates and quantizes (same bits).  Per-dispatch timestamps, median."""
    from wick_amd.lfm2 import Lfm2Ops
    ops = Lfm2Ops(ctx)
    wg = O.synth_weight(dtype, m, k, seed=41) if wg is None else wg
    wu = O.synth_weight(dtype, m, k, seed=42) if wu is None else wu
    d_wg, d_wu = ctx.upload_weight(wg, dtype, m, k), ctx.upload_weight(wu, dtype, m, k)
    s, q = O.quantize_q8_0_batch(O.fill_normal(9, 1.0, n * k), n, k)
    d_q, d_s = ctx.to_device(q), ctx.to_device(s)
    d_g, d_u, d_oq, d_os = ctx.alloc(n * m * 4), ctx.alloc(n * m * 4), ctx.alloc(n * m), ctx.alloc(n * (m // 32) * 4)

    def separate():
        ctx.gemm_preq_multi([d_wg, d_wu], d_s, d_q, n, [d_g, d_u], m)
        ops.silu_mul_quantize(d_g, d_u, n, m, d_oq, d_os)

    def fused():
        ops.encode_ffn_gate_up_silu_quantize(d_wg, d_wu, d_s, d_q, n, d_oq, d_os)

    out = {"dtype": dtype, "m": m, "k": k, "n": n}
    for name, fn in (("separate_us", separate), ("fused_us", fused)):
        fn()
        ts = []
        for _ in range(reps):
            ctx.kernel_timing_begin()
            fn()
            kt = ctx.kernel_timing_end()
            ts.append(sum(ms for ms, cnt in kt.values()) * 1e3)
            out[name.replace("_us", "_gemm_us")] = kt["gemm"][0] * 1e3
        out[name] = float(np.median(ts))
    for b in (d_q, d_s, d_g, d_u, d_oq, d_os):
        b.free()
    d_wg.free(), d_wu.free()
    return out


def bench_lm_head_sweep(ctx, W, O, dtype=8, m=65536, k=2048, ns=(1, 4, 5, 6, 8, 12, 16, 64)):
    """Tied LM head: where the bandwidth-bound multi-token GEMV hands off to the MFMA GEMM.
    Each n is timed through both kernels (hand-off forced), HBM-cold over three weight copies: the configuration's n = 1, 4, 16, 64
    and the n between 4 and 16 where the routes cross, so that the crossing and the library's own hand-off come from the same data."""
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
    return {"dtype": dtype, "m": m, "k": k, "rows": rows, "first_n_where_mfma_wins": crossover, "library_hand_off_n": W.GEMM_MIN_N_LARGE if m * (k // 32) * 34 >= (16 << 20) else W.GEMM_MIN_N}


def bench_probe(ctx, iters=20000):
    """Register-only ceilings of this GPU for the GEMM's two bounds (no memory traffic)."""
    from wick_amd import benchlib as B

    out = {}
    for shape, name, unit in [(0, "mfma_i32_32x32x32_i8", "TOP/s"), (1, "mfma_i32_16x16x32_i8", "TOP/s"), (2, "v_fma_f32", "TFLOP/s"),
                              (3, "block_loop_8xmfma16_plus_64_scaling_fma", "TOP/s"), (4, "block_loop_2xmfma32_plus_64_scaling_fma", "TOP/s")]:
        B.probe_rate(ctx, shape, iters)
        ctx.sync()
        e0, e1 = ctx.event(), ctx.event()
        ctx.record(e0)
        ops = B.probe_rate(ctx, shape, iters)
        ctx.record(e1)
        ms = ctx.elapsed_ms(e0, e1)
        ctx.event_destroy(e0), ctx.event_destroy(e1)
        out[name] = {"value": ops / ms / 1e9, "unit": unit, "ms": ms}
    return out


def bench_copy(ctx, nbytes=256 << 20, reps=10):
    """Device-to-device copy of a known size: calibration of the FETCH_SIZE / WRITE_SIZE counters."""
    from wick_amd import benchlib as B

    a, b = ctx.alloc(nbytes), ctx.alloc(nbytes)
    B.copy(ctx, b, a, nbytes)
    ctx.sync()
    e0, e1 = ctx.event(), ctx.event()
    ctx.record(e0)
    for _ in range(reps):
        B.copy(ctx, b, a, nbytes)
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


def cpu_model_name():
    try:
        for line in open("/proc/cpuinfo"):
            if line.startswith("model name"):
                return line.split(":", 1)[1].strip()
    except OSError:
        pass
    return "unknown"


def cpu_baseline(O, W):
    """The reference's x86 path (what it executes on this host: f32 per-block AVX2 dots restated in C, the integer kernels
    being aarch64-only), timed on bounded samples of the benchmark's workloads:
      headline   the single Q4_0 6912 x 2048 GEMV: rows serial on ONE core (wick/src/backend/cpu.rs:293-306)
      legs       the Q4_0 decode step (serial), the Q8_0 decode step with rows split over T threads
                 (wick/src/backend/cpu.rs:222-234, 401-420), the prefill GEMM as a loop of per-token GEMVs
                 (wick/src/model/lfm2.rs:2111-2169) on a 64-token subset, scaled to 2002 tokens."""
    threads = os.cpu_count() or 1
    m, k = C1
    wb = O.synth_weight(W.Q4_0, m, k, seed=4242)
    x = O.fill_normal(3, 1.0, k)
    b = gemv_bytes(W.Q4_0, m, k)
    O.x86_gemv_f32(W.Q4_0, wb, x, m, k)
    t0, reps = time.perf_counter(), 0
    while time.perf_counter() - t0 < 4.0:
        O.x86_gemv_f32(W.Q4_0, wb, x, m, k)
        reps += 1
    dt = time.perf_counter() - t0
    out = {"value": b * reps / dt / 1e9, "unit": "GB/s", "cores": 1, "kind": "port", "cpu": cpu_model_name(), "host_threads": threads,
           "sample": f"{reps} GEMVs of the headline shape (Q4_0 {m} x {k}, {b * reps / 1e6:.0f} MB) in {dt:.1f} s on one core: the reference runs "
                     "Q4_0 rows serially on x86; f32 per-block AVX2 path restated in C (its integer kernels are aarch64-only)",
           "us_per_gemv": dt / reps * 1e6, "legs": {}}
    sites = decode_call_sites()
    xs = {HS: O.fill_normal(1, 1.0, HS), IS: O.fill_normal(2, 1.0, IS)}
    for dtype, name, budget in ((W.Q4_0, "decode_step_q4_0_serial", 6.0), (W.Q8_0, "decode_step_q8_0_threaded", 4.0)):
        host_weights = synth_decode_weights(O, dtype)
        gbytes = sum(gemv_bytes(dtype, mm, kk) for _, ms, kk in sites for mm in ms)
        used, steps, t0 = 1, 0, time.perf_counter()
        while True:
            for sname, ms, kk in sites:
                for blob, mm in zip(host_weights[sname], ms):
                    _, u = O.x86_gemv_f32(dtype, blob, xs[kk], mm, kk, threads=threads)
                    used = max(used, u)
            steps += 1
            if time.perf_counter() - t0 >= budget:
                break
        dt = time.perf_counter() - t0
        out["legs"][name] = {"value": gbytes * steps / dt / 1e9, "unit": "GB/s", "cores": used, "ms_per_step": dt / steps * 1e3,
                             "sample": f"{steps} full LFM2-350M-shaped decode steps ({gbytes * steps / 1e6:.0f} MB of GEMV work) in {dt:.1f} s"}
        del host_weights
    mm, n, kk, sub = 6912, 2002, 2048, 64
    wb = O.synth_weight(W.Q4_0, mm, kk, seed=777)
    xsub = O.fill_normal(9, 1.0, sub * kk)
    t0 = time.perf_counter()
    _, used = O.x86_prefill_f32(W.Q4_0, wb, xsub, mm, sub, kk, threads=threads)
    dt = time.perf_counter() - t0
    out["legs"]["prefill_gemm_q4_0_6912x2002x2048"] = {
        "value": 2.0 * mm * sub * kk / dt / 1e12, "unit": "TOP/s", "cores": used, "ms_scaled_to_2002_tokens": dt * 1e3 * n / sub,
        "sample": f"{sub} of the 2002 tokens as a loop of per-token f32 GEMVs ({dt:.2f} s), scaled linearly to the whole prompt"}
    return out


def profile_figure(name, key):
    """A `key: number` line of a committed profile summary (profiles/<name>), or None: the counter-derived figures of the
    JSON line are read from the file they were measured into instead of being repeated here."""
    try:
        for line in open(os.path.join(ROOT, "profiles", name)):
            if line.strip().startswith(key + ":"):
                return float(line.split(":", 1)[1].split()[0])
    except (OSError, ValueError):
        pass
    return None


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=100, help="timed graph replays of the headline GEMV (38 launches each)")
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--skip-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--skip-extra", action="store_true", help="only the headline GEMV, the GEMM (+ CPU baseline)")
    ap.add_argument("--prompt-tokens", type=int, default=2002, help="lfm2_prefill_trace: tokens of the traced prompt pass")
    ap.add_argument("--graph-only", action="store_true", help="decode legs: graph replays only, no eager launches (for kernel tracers)")
    ap.add_argument("--mfma-shape", type=int, default=0, help="block loop of the wide GEMM tile: 0 / 32 (default) or 16 (A/B runs)")
    ap.add_argument("--leg", default="all", help="all | c1 | gemm | decode | decode_q8 | gemv | prefill_sites | lm_head | lm_head_q6k | upload | lfm2_step | lfm2_step_q8 | lfm2_step_kv16 | lfm2_step_1p2b | lfm2_step_trace | lfm2_prefill_trace | copy | probe | cpu")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs on ONE GPU only (no collectives, no sharding); use --gpus 1", file=sys.stderr)
        sys.exit(2)

    import wick_amd as W
    from oracle import oracle as O  # cpu_baseline leg + synthetic inputs only; never in the timed GPU path

    leg = args.leg
    if leg == "cpu":
        print(json.dumps({"cpu_baseline": cpu_baseline(O, W)}))
        return
    ctx = W.RocmContext(0)
    ctx.set_gemm_mfma_shape(args.mfma_shape)
    if leg != "all":
        one = {
            # graph replays only (warm-up included): every gemv_pairs_kernel dispatch a kernel tracer sees belongs to the timed workload
            "c1": lambda: bench_c1(ctx, W, O, args.steps, args.warmup, with_concurrent=False),
            "c1_concurrent": lambda: bench_c1(ctx, W, O, args.steps, args.warmup),
            "decode": lambda: bench_decode(ctx, W, O, W.Q4_0, args.steps, args.warmup, synth_decode_weights(O, W.Q4_0), with_unfused=False, graph_only=args.graph_only),
            "decode_q8": lambda: bench_decode(ctx, W, O, W.Q8_0, args.steps, args.warmup, synth_decode_weights(O, W.Q8_0), with_unfused=False, graph_only=args.graph_only),
            "gemv": lambda: bench_single_gemv(ctx, W, O, W.Q4_0, 6912, 2048),
            "gemm": lambda: bench_gemm(ctx, W, O, W.Q4_0, 6912, 2002, 2048, samples=100),
            "prefill_sites": lambda: bench_prefill_sites(ctx, W, O),
            "lm_head": lambda: bench_lm_head_sweep(ctx, W, O),
            "lm_head_q6k": lambda: bench_single_gemv(ctx, W, O, W.Q6_K, 65536, 1024),
            "lfm2_step": lambda: bench_lfm2_step(ctx, W, O),
            "lfm2_step_q8": lambda: bench_lfm2_step(ctx, W, O, body=8, embd=8),
            "lfm2_step_kv16": lambda: bench_lfm2_step(ctx, W, O, kv_f16=True),  # KV caches of f16 rows
            # the per-layer shapes of an LFM2-1.2B: hidden 2048, FFN 6912, 32 heads / 8 KV heads
            "lfm2_step_1p2b": lambda: bench_lfm2_step(ctx, W, O, dims=dict(HS=2048, IS=6912, KV=512), label="LFM2-1.2B-shaped"),
            "lfm2_step_trace": lambda: trace_lfm2_step(ctx, W, O),
            "lfm2_prefill_trace": lambda: trace_lfm2_prefill(ctx, W, O, n=args.prompt_tokens),
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

    c1 = bench_c1(ctx, W, O, args.steps, args.warmup)
    avg_launch_us = c1["ms_per_step"] * 1e3 / c1["launches_per_step"]
    achieved = c1["bytes_per_launch"] / avg_launch_us / 1e3  # GB/s
    c1_profile = "gemv_q4_0_6912x2048_hbm_cold.txt"
    span = c1["kernel_span"]
    conc = c1.pop("concurrent", None)
    roofline = {
        "bound": "hbm",
        "kernel": "gemv_pairs_kernel<Q4_0> (pre-quantized activation, span loads)",
        "achieved": achieved,
        "peak": HBM_PEAK_GBS,
        "unit": "GB/s",
        "frac": achieved / HBM_PEAK_GBS,
        "bytes_per_launch": c1["bytes_per_launch"],
        "avg_launch_us": avg_launch_us,
        "avg_launch_definition": "timed region / launches in it: kernel execution + the gap to the next dependent launch, an upper bound of the "
                                 "kernel's own duration",
        "per_launch": c1["per_launch_in_graph"],
        "frac_best_step": c1["bytes_per_launch"] / c1["per_launch_in_graph"]["min_us"] / 1e3 / HBM_PEAK_GBS,
        # the kernel's own execution inside the same chain (first wave's first instruction -> last wave's last store), from the
        # timing hook: kernel_span_us x launches <= ms_per_step, the rest is the gap between dependent launches
        "kernel_span_us": span["span_us_mean"],
        "kernel_span_GBps": c1["bytes_per_launch"] / span["span_us_mean"] / 1e3,
        "kernel_span_frac": c1["bytes_per_launch"] / span["span_us_mean"] / 1e3 / HBM_PEAK_GBS,
        "gap_between_dependent_launches_us": span["gap_to_next_launch_us_mean"],
        # HBM bytes per launch from the copy-calibrated FETCH_SIZE / WRITE_SIZE passes recorded in the profile summary
        "traffic": profile_figure(c1_profile, "traffic_bytes_per_launch"),
        "traffic_source": "profiles/" + c1_profile,
    }
    if conc:  # the same launches as independent work on four streams
        roofline["independent_streams_us_per_launch"] = conc["per_launch"]["median_us"]
        roofline["independent_streams_frac"] = conc["frac_of_hbm_peak_median"]
    out = {
        "metric": "Q4_0 GEMV GB/s (% HBM peak) + prefill int8 GEMM TOPS (% MFMA peak)",
        "value": c1["GBps"],
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": c1["ms_per_step"],
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "i8",
        "data": "synthetic",
        "config": {
            "workload": "single decode GEMV, LFM2-1.2B ffn_up shape: Q4_0 weight 6912 x 2048 x one Q8_0-quantized token (n = 1), HBM-cold; "
                        f"one step = one HIP-graph replay = {c1['launches_per_step']} chained launches, one per distinct device copy of the weight "
                        "(303 MB, beyond the 256 MB Infinity Cache)",
            "device": ctx.device_name,
            "value_definition": "algorithmic GEMV bytes per step (38 x (weights + Q8_0 activation + f32 output) = 38 x 7 992 448 B) / step time",
        },
        "gemv_6912x2048": c1,
    }
    if conc:
        out["gemv_concurrent"] = conc

    gemm_profile = "gemm_q4_0_6912x2002x2048.txt"
    g = bench_gemm(ctx, W, O, W.Q4_0, 6912, 2002, 2048, samples=100)
    g["roofline"] = {"bound": "mfma", "kernel": "gemm_mfma32_kernel<Q4_0>", "workload": "prefill GEMM Q4_0 m=6912, n=2002, k=2048 (2 m n k int8 ops per launch)",
                     "achieved": g["gemm_kernel_TOPS"], "peak": INT8_PEAK_TOPS,
                     "unit": "TOP/s", "frac": g["gemm_kernel_TOPS"] / INT8_PEAK_TOPS, "frac_median": g["gemm_kernel_TOPS_median"] / INT8_PEAK_TOPS,
                     "frac_best": g["gemm_kernel_TOPS_best"] / INT8_PEAK_TOPS, "avg_launch_us": g["gemm_kernel_ms"] * 1e3,
                     "traffic": profile_figure(gemm_profile, "traffic_bytes_per_launch"), "traffic_source": "profiles/" + gemm_profile}
    out["gemm"] = g
    roofline["gemm"] = g["roofline"]  # the matrix-core half of the metric, inside the object the record keeps

    if not args.skip_extra:
        out["measured_ceilings"] = bench_probe(ctx)
        g["roofline"]["frac_of_measured_block_loop_ceiling"] = g["gemm_kernel_TOPS"] / out["measured_ceilings"]["block_loop_2xmfma32_plus_64_scaling_fma"]["value"]
        roofline["lm_head_first_n_where_mfma_wins"] = None  # filled below from the sweep
        dec = bench_decode(ctx, W, O, W.Q4_0, 50, args.warmup, synth_decode_weights(O, W.Q4_0))
        out["decode_step"] = dec
        dq = bench_decode(ctx, W, O, W.Q8_0, 25, args.warmup, synth_decode_weights(O, W.Q8_0), with_unfused=False)
        out["decode_step_q8_0"] = dq
        out["prefill_sites"] = bench_prefill_sites(ctx, W, O)
        out["lm_head_sweep"] = bench_lm_head_sweep(ctx, W, O)
        roofline["lm_head_first_n_where_mfma_wins"] = out["lm_head_sweep"]["first_n_where_mfma_wins"]
        roofline["lm_head_library_hand_off_n"] = out["lm_head_sweep"]["library_hand_off_n"]
        # shipped LFM2 Q4_0 files keep the tied embedding / LM head in Q6_K (wick/src/model/metal_lfm2.rs:175-180)
        out["lm_head_q6_k_65536x1024"] = bench_single_gemv(ctx, W, O, W.Q6_K, 65536, 1024)
        out["lfm2_decode_step"] = bench_lfm2_step(ctx, W, O)
        out["lfm2_decode_step_kv_f16"] = bench_lfm2_step(ctx, W, O, kernel_times=False, kv_f16=True)  # the same model on f16 K / V rows
    ctx.close()
    out["roofline"] = roofline  # (last, with cpu_baseline: the end of the line is what a truncated log still shows)
    if not args.skip_cpu:
        out["cpu_baseline"] = cpu_baseline(O, W)
    print(json.dumps(out))


if __name__ == "__main__":
    main()
