"""The benchmark's own decode-step launch list (bench.py DecodeStep: the 93 GEMVs of an LFM2-350M-shaped step in 65 fused
launches, incl. the tied 65536 x 1024 head at its exact shape) replayed once as a graph and compared, output by output,
with the oracle's GEMV (the decode call sites of wick/src/model/lfm2.rs:1020-1124: which projections share one
quantization)."""
import numpy as np
import pytest

import wick_amd as W
from conftest import assert_f32_parity

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("dtype", [W.Q4_0, W.Q8_0])
def test_bench_decode_step_launch_list_against_the_oracle(ctx, oracle, dtype):
    import bench

    host = bench.synth_decode_weights(oracle, dtype)
    x = {bench.HS: oracle.fill_normal(1, 1.0, bench.HS), bench.IS: oracle.fill_normal(2, 1.0, bench.IS)}
    d_x = {k: ctx.to_device(v) for k, v in x.items()}
    step = bench.DecodeStep(ctx, dtype, host, d_x[bench.HS], d_x[bench.IS])
    ctx.graph_begin()
    step.enqueue()
    g = ctx.graph_end()
    ctx.graph_launch(g)
    ctx.sync()
    quant = {k: oracle.quantize_q8_0(v) for k, v in x.items()}
    sites = bench.decode_call_sites()
    assert len(sites) == 65 and sum(len(ms) for _, ms, _ in sites) == 93
    for (name, ms, k), (ws, ys, _) in zip(sites, step.sites):
        s, q = quant[k]
        for i, (m, d_y) in enumerate(zip(ms, ys)):
            ref = oracle.gemv_q8(dtype, host[name][i], s, q, m, k)
            assert_f32_parity(d_y.download(np.float32, m), ref, f"{name}[{i}] {m}x{k}")
    ctx.graph_destroy(g)
    step.free()
    for b in d_x.values():
        b.free()
