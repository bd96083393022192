"""Batched prefill GEMM on the GPU against the oracle, both output layouts, both
kernel paths (multi-token GEMV below the hand-off n or when k % 128 != 0; int8 MFMA
otherwise).  Block dots BIT-EXACT, f32 within rel-L2 1e-5 / max-abs 1e-4 x RMS."""
import numpy as np
import pytest

import wick_amd as W
from conftest import assert_f32_parity, rel_l2
from gpu_util import Problem, fetch_gemm
from test_oracle_matmul import ref_inputs, ref_weights

pytestmark = pytest.mark.gpu

# (m, n, k)
SHAPES = [
    (8, 1, 64), (8, 5, 64), (8, 7, 64), (8, 8, 64), (8, 11, 64), (8, 16, 64),  # the reference's own test shapes
    (4, 1, 32), (64, 4, 32), (64, 20, 96), (33, 3, 2080),                        # generic path
    (64, 2, 256), (100, 15, 512),                                                # multi-token GEMV
    (128, 16, 256), (128, 128, 256), (1, 16, 256), (130, 129, 512), (200, 50, 512), (256, 300, 1024),
    (512, 100, 2048), (1000, 257, 4608), (300, 64, 6912),                        # MFMA, ragged tiles
    (129, 17, 128), (16, 33, 256), (250, 63, 384), (131, 64, 1024), (257, 65, 512),  # narrow kernel (n <= 64) and its hand-off
]


@pytest.mark.parametrize("dtype", [W.Q4_0, W.Q8_0])
@pytest.mark.parametrize("m,n,k", SHAPES)
def test_gemm_parity(ctx, oracle, dtype, m, n, k):
    with Problem(ctx, oracle, dtype, m, k, n, seed=m + 5 * n + 11 * k + dtype) as p:
        ref = oracle.gemm_q8(dtype, p.wb, p.s, p.q, m, n, k)
        for layout, stride in ((W.LAYOUT_ROW_MAJOR, n), (W.LAYOUT_TOKEN_MAJOR, m), (W.LAYOUT_ROW_MAJOR, n + 3), (W.LAYOUT_TOKEN_MAJOR, m + 5)):
            rows = m if layout == W.LAYOUT_ROW_MAJOR else n
            d_y = p.to_device(np.full(rows * stride, -7.0, np.float32))
            ctx.gemm_preq(p.w, p.d_s, p.d_q, n, d_y, y_stride=stride, layout=layout)
            assert_f32_parity(fetch_gemm(d_y, m, n, stride, layout), ref, f"gemm {dtype} {m}x{n}x{k} layout {layout}")
            # padding between rows is left untouched
            full = d_y.download(np.float32, rows * stride).reshape(rows, stride)
            used = n if layout == W.LAYOUT_ROW_MAJOR else m
            assert np.all(full[:, used:] == -7.0)
        d_d = p.alloc(n * m * (k // 32) * 4)
        ctx.block_dots_i32(p.w, p.d_q, n, d_d)
        dots = d_d.download(np.int32, n * m * (k // 32)).reshape(n, m, k // 32)
        assert np.array_equal(dots, oracle.block_dots_i32(dtype, p.wb, p.q, m, n, k))


# more than 256 wide tiles (fewer run on the narrow tile), ragged in rows and tokens; the fourth is cut over K on the wide tile;
# the last two take the narrow tile (n > 48: both of its block loops exist), the very last one cut over K
WIDE_SHAPES = [(2100, 2010, 128, True), (2100, 1990, 256, False), (4700, 1100, 384, False), (1024, 2002, 4608, False),
               (300, 64, 512, True), (1000, 700, 1024, False)]


@pytest.mark.parametrize("dtype", [W.Q4_0, W.Q8_0])
@pytest.mark.parametrize("m,n,k,with_dots", WIDE_SHAPES)
def test_wide_tile_on_either_mfma_shape(ctx, oracle, dtype, m, n, k, with_dots):
    """The two block loops of the wide tile and of the full narrow tile (32x32x32, the default, and 16x16x32): each against the oracle (two row bands over all
    tokens) in both layouts with ragged strides and with the accumulate flag, block dots bit-exact through either, and the
    two within 1e-6 of each other everywhere."""
    rb = (k // 32) * (18 if dtype == W.Q4_0 else 34)
    bands = [(0, 96), (m - 70, m)]
    with Problem(ctx, oracle, dtype, m, k, n, seed=3 * m + 7 * n + k + dtype) as p:
        refs = [oracle.gemm_q8(dtype, p.wb[r0 * rb:r1 * rb], p.s, p.q, r1 - r0, n, k) for r0, r1 in bands]
        outs = {}
        try:
            for shape in (32, 16):
                ctx.set_gemm_mfma_shape(shape)
                for layout, stride in ((W.LAYOUT_TOKEN_MAJOR, m), (W.LAYOUT_ROW_MAJOR, n + 3), (W.LAYOUT_TOKEN_MAJOR, m + 5)):
                    rows = m if layout == W.LAYOUT_ROW_MAJOR else n
                    d_y = ctx.to_device(np.full(rows * stride, -7.0, np.float32))
                    ctx.gemm_preq(p.w, p.d_s, p.d_q, n, d_y, y_stride=stride, layout=layout)
                    got = fetch_gemm(d_y, m, n, stride, layout)
                    for (r0, r1), ref in zip(bands, refs):
                        assert_f32_parity(got[r0:r1], ref, f"gemm {dtype} {m}x{n}x{k} layout {layout} mfma {shape} rows {r0}..{r1}")
                    full = d_y.download(np.float32, rows * stride).reshape(rows, stride)
                    assert np.all(full[:, (n if layout == W.LAYOUT_ROW_MAJOR else m):] == -7.0)
                    if layout == W.LAYOUT_TOKEN_MAJOR and stride == m:
                        outs[shape] = got
                        ctx.gemm_preq(p.w, p.d_s, p.d_q, n, d_y, y_stride=stride, layout=layout, accumulate=True)  # y += W x
                        twice = fetch_gemm(d_y, m, n, stride, layout)
                        for (r0, r1), ref in zip(bands, refs):
                            assert_f32_parity(twice[r0:r1], 2.0 * ref, f"accumulate, mfma {shape}")
                    d_y.free()
                if with_dots:
                    d_d = p.alloc(n * m * (k // 32) * 4)
                    ctx.block_dots_i32(p.w, p.d_q, n, d_d)
                    dots = d_d.download(np.int32, n * m * (k // 32)).reshape(n, m, k // 32)
                    assert np.array_equal(dots, oracle.block_dots_i32(dtype, p.wb, p.q, m, n, k))
        finally:
            ctx.set_gemm_mfma_shape(0)
        assert rel_l2(outs[16], outs[32]) < 1e-6


def test_mfma_shape_knob_rejects_other_values(ctx):
    with pytest.raises(W.RocmError):
        ctx.set_gemm_mfma_shape(8)
    ctx.set_gemm_mfma_shape(0)


@pytest.mark.parametrize("dtype,n", [(W.Q4_0, 7), (W.Q8_0, 5), (W.Q4_0, 8), (W.Q4_0, 11), (W.Q4_0, 16)])
def test_reference_gemm_vs_gemv_inputs(ctx, oracle, dtype, n):
    """The reference's GEMM == sequential GEMV tests (simd.rs:1440-1623) on their own
    weights/inputs: GPU GEMM column j vs GPU GEMV of column j within the reference's 1e-4."""
    m, k = 8, 64
    wb = oracle.build_matrix(dtype, ref_weights(m, k), m, k)
    s, q = oracle.quantize_q8_0_batch(ref_inputs(n, k), n, k)
    w = ctx.upload_weight(wb, dtype, m, k)
    d_q, d_s = ctx.to_device(q), ctx.to_device(s)
    d_c, d_y = ctx.alloc(m * n * 4), ctx.alloc(m * 4)
    ctx.gemm_preq(w, d_s, d_q, n, d_c, layout=W.LAYOUT_ROW_MAJOR)
    c = d_c.download(np.float32, m * n).reshape(m, n)
    assert_f32_parity(c, oracle.gemm_q8(dtype, wb, s, q, m, n, k), "reference inputs")
    for j in range(n):
        ctx.gemv_with_preq(w, d_s.ptr + j * (k // 32) * 4, d_q.ptr + j * k, d_y)
        assert np.abs(c[:, j] - d_y.download(np.float32, m)).max() < 1e-4
    w.free()
    for b in (d_q, d_s, d_c, d_y):
        b.free()


def test_q8_0_closed_form(ctx, oracle):
    """test_q8_0_gemm_standalone (wick/tests/bench_perf.rs:852-971): m=64, k=32, n=4,
    scale 1/(row+1), quants -16..15, x == 1, x_stride = k, y_stride = m, through the
    f32 call-site entry point."""
    m, k, n = 64, 32, 4
    rows = []
    for r in range(m):
        h = int(np.float16(1.0 / (r + 1.0)).view(np.uint16))
        rows.append(np.concatenate([np.array([h & 0xFF, h >> 8], np.uint8), (np.arange(32) - 16).astype(np.int8).view(np.uint8)]))
    w = ctx.upload_weight(np.concatenate(rows), W.Q8_0, m, k)
    d_x = ctx.to_device(np.ones(n * k, np.float32))
    d_y = ctx.alloc(m * n * 4)
    ctx.encode_gemm(w, d_x, 0, d_y, 0, n, k, m)
    y = d_y.download(np.float32, m * n).reshape(n, m)
    expect = np.array([-16.0 * float(np.float16(1.0 / (r + 1.0))) for r in range(m)]) * 127.0 * float(np.float16(1.0 / 127.0))
    for col in range(n):
        assert np.abs(y[col] - (-16.0 / (np.arange(m) + 1.0))).max() < 1.0  # the reference's bound
        assert np.allclose(y[col], expect, rtol=1e-6)
    w.free(), d_x.free(), d_y.free()


@pytest.mark.parametrize("dtype", [W.Q4_0, W.Q8_0])
@pytest.mark.parametrize("n", [3, 40])
def test_accumulate(ctx, oracle, dtype, n):
    m, k = 256, 512
    with Problem(ctx, oracle, dtype, m, k, n, seed=8) as p:
        y0 = oracle.fill_normal(4, 1.0, n * m)
        d_y = p.to_device(y0)
        ctx.gemm_preq(p.w, p.d_s, p.d_q, n, d_y, layout=W.LAYOUT_TOKEN_MAJOR, accumulate=True)
        ref = y0.reshape(n, m).T.astype(np.float64) + oracle.gemm_q8(dtype, p.wb, p.s, p.q, m, n, k, f64=True)
        assert_f32_parity(fetch_gemm(d_y, m, n, m, W.LAYOUT_TOKEN_MAJOR), ref, "gemm accumulate")


def test_weight_free_releases_both_copies(ctx, oracle):
    """Uploading and freeing a weight over and over leaves the device's free memory where it was: the raw blocks and the
    GEMM's copy both go (read through hipMemGetInfo of the HIP runtime the library itself is linked against)."""
    import ctypes

    hip = ctypes.CDLL("libamdhip64.so")
    free, total = ctypes.c_size_t(), ctypes.c_size_t()

    def free_bytes():
        ctx.sync()
        assert hip.hipMemGetInfo(ctypes.byref(free), ctypes.byref(total)) == 0
        return free.value

    m, k = 16384, 2048  # 36 MB of Q8_0 blocks + 42 MB of slabs
    wb = np.tile(oracle.synth_weight(W.Q8_0, 256, k, 9, 0.02), m // 256)
    ctx.upload_weight(wb, W.Q8_0, m, k).free()  # the runtime's own pools settle on the first round
    before = free_bytes()
    for _ in range(12):
        w = ctx.upload_weight(wb, W.Q8_0, m, k)
        assert w.device_bytes > 2 * 36_000_000
        w.free()
    assert abs(before - free_bytes()) <= 8 << 20


def test_weights_without_the_gemm_copy_take_the_gemv_route(ctx, oracle):
    """wick_rocm_set_gemm_packing(0): weights uploaded from then on hold the raw blocks only (no second layout for the
    matrix-core kernel) and run as multi-token GEMVs for any n -- same block dots bit for bit, f32 results to the bar."""
    m, n, k = 200, 70, 512
    for dtype, raw_per_block in ((W.Q4_0, 18), (W.Q8_0, 34)):
        wb = oracle.synth_weight(dtype, m, k, 5, 0.02)
        s, q = oracle.quantize_q8_0_batch(oracle.fill_normal(6, 1.0, n * k), n, k)
        packed = ctx.upload_weight(wb, dtype, m, k)
        ctx.set_gemm_packing(False)
        try:
            plain = ctx.upload_weight(wb, dtype, m, k)
        finally:
            ctx.set_gemm_packing(True)
        raw = m * (k // 32) * raw_per_block
        assert plain.device_bytes == raw
        # whole pairs of 32-row granules, 5 KB per granule and 128 K-elements
        assert packed.device_bytes == raw + 2 * ((m + 63) // 64) * (k // 128) * 5120
        d_q, d_s = ctx.to_device(q), ctx.to_device(s)
        ref = oracle.gemm_q8(dtype, wb, s, q, m, n, k)
        outs, dots = [], []
        for w in (packed, plain):
            d_y, d_d = ctx.alloc(n * m * 4), ctx.alloc(n * m * (k // 32) * 4)
            ctx.gemm_preq(w, d_s, d_q, n, d_y, y_stride=m, layout=W.LAYOUT_TOKEN_MAJOR)
            ctx.block_dots_i32(w, d_q, n, d_d)
            outs.append(fetch_gemm(d_y, m, n, m, W.LAYOUT_TOKEN_MAJOR))
            dots.append(d_d.download(np.int32, n * m * (k // 32)))
            d_y.free(), d_d.free()
        assert_f32_parity(outs[0], ref, "packed weight")
        assert_f32_parity(outs[1], ref, "raw-only weight")
        assert np.array_equal(dots[0], dots[1])
        assert np.array_equal(dots[0].reshape(n, m, k // 32), oracle.block_dots_i32(dtype, wb, q, m, n, k))
        # a launch over several weights falls back to one call per weight when one of them has no copy
        d_a, d_b = ctx.alloc(n * 2 * m * 4), ctx.alloc(n * 2 * m * 4)
        ctx.gemm_preq_multi([packed, plain], d_s, d_q, n, [d_a.ptr, d_a.ptr + m * 4], 2 * m)
        ctx.gemm_preq(packed, d_s, d_q, n, d_b.ptr, y_stride=2 * m, layout=W.LAYOUT_TOKEN_MAJOR)
        ctx.gemm_preq(plain, d_s, d_q, n, d_b.ptr + m * 4, y_stride=2 * m, layout=W.LAYOUT_TOKEN_MAJOR)
        assert np.array_equal(d_a.download(np.uint32, n * 2 * m), d_b.download(np.uint32, n * 2 * m))
        for b in (d_q, d_s, d_a, d_b):
            b.free()
        packed.free(), plain.free()


@pytest.mark.parametrize("dtype", [W.Q4_0, W.Q8_0])
@pytest.mark.parametrize("ms,n,k,layout,acc", [
    ((256, 128, 128), 200, 512, W.LAYOUT_TOKEN_MAJOR, False),   # Q / K / V into one [n][q|k|v] row
    ((300, 300), 130, 1024, W.LAYOUT_TOKEN_MAJOR, True),         # gate / up, ragged row tiles, accumulate
    ((129, 1, 257), 40, 256, W.LAYOUT_TOKEN_MAJOR, False),       # narrow tile
    ((128, 64), 17, 128, W.LAYOUT_ROW_MAJOR, False),
    ((64, 96), 5, 256, W.LAYOUT_TOKEN_MAJOR, False),             # below the MFMA hand-off: one call per weight
])
def test_gemm_multi_equals_one_launch_per_weight(ctx, oracle, dtype, ms, n, k, layout, acc):
    """Up to three weights over the same activations in one launch: bit-identical to one launch per weight (each taken unsplit:
    a single weight's launch with few tiles may otherwise walk K in shares, which moves its sums by a few 1e-7)."""
    with Problem(ctx, oracle, dtype, ms[0], k, n, seed=sum(ms) + n) as p:
        ws = [p.w] + [ctx.upload_weight(oracle.synth_weight(dtype, m, k, 50 + i, 0.02), dtype, m, k) for i, m in enumerate(ms[1:])]
        tm = layout == W.LAYOUT_TOKEN_MAJOR
        stride = sum(ms) + 3 if tm else n + 1
        y0 = oracle.fill_normal(9, 1.0, (n if tm else sum(ms)) * stride)
        d_a, d_b = p.to_device(y0), p.to_device(y0)
        offs = np.concatenate([[0], np.cumsum(ms)[:-1]])
        elem = lambda o: int(o) * 4 if tm else int(o) * stride * 4  # byte offset of a weight's first output
        ya = [d_a.ptr + elem(o) for o in offs]
        yb = [d_b.ptr + elem(o) for o in offs]
        ctx.gemm_preq_multi(ws, p.d_s, p.d_q, n, ya, stride, layout=layout, accumulate=acc)
        ctx.set_gemm_max_k_splits(1)
        try:
            for w, y in zip(ws, yb):
                ctx.gemm_preq(w, p.d_s, p.d_q, n, y, y_stride=stride, layout=layout, accumulate=acc)
        finally:
            ctx.set_gemm_max_k_splits(0)
        a, b = d_a.download(np.float32, y0.size), d_b.download(np.float32, y0.size)
        assert np.array_equal(a.view(np.uint32), b.view(np.uint32))
        assert not np.array_equal(a, y0)
        d_c = p.to_device(y0)  # the same launches as the library routes them by default: equal to the f32 bar
        for w, o in zip(ws, offs):
            ctx.gemm_preq(w, p.d_s, p.d_q, n, d_c.ptr + elem(o), y_stride=stride, layout=layout, accumulate=acc)
        c = d_c.download(np.float32, y0.size)
        assert np.linalg.norm(c.astype(np.float64) - a) <= 1e-6 * np.linalg.norm(a)
        with pytest.raises(W.RocmError, match="share k and dtype"):
            other = ctx.upload_weight(oracle.synth_weight(dtype, 32, k + 128, 3, 0.02), dtype, 32, k + 128)
            ws.append(other)
            ctx.gemm_preq_multi([ws[0], other], p.d_s, p.d_q, n, ya[:2], stride, layout=layout)
        for w in ws[1:]:
            w.free()


@pytest.mark.parametrize("dtype", [W.Q4_0, W.Q8_0])
def test_full_size_prefill_shape(ctx, oracle, dtype):
    """m=6912, n=2002, k=2048 (the LFM2-1.2B ffn_up prefill shape).  The oracle checks a
    band of rows across ALL tokens plus scattered rows; size-independent properties cover
    the rest: column j of the GEMM equals the GEMV of column j, and both layouts agree."""
    m, n, k = 6912, 2002, 2048
    with Problem(ctx, oracle, dtype, m, k, n, seed=2026) as p:
        d_y = p.alloc(m * n * 4)
        ctx.gemm_preq(p.w, p.d_s, p.d_q, n, d_y, layout=W.LAYOUT_TOKEN_MAJOR)
        y = fetch_gemm(d_y, m, n, m, W.LAYOUT_TOKEN_MAJOR)
        assert np.isfinite(y).all()
        bb = 18 if dtype == W.Q4_0 else 34
        rows = np.concatenate([np.arange(0, 40), np.arange(6890, 6912), np.arange(100, 6800, 397)])
        sub = np.concatenate([p.wb.reshape(m, -1)[r] for r in rows])
        assert sub.size == len(rows) * (k // 32) * bb
        assert_f32_parity(y[rows], oracle.gemm_q8(dtype, sub, p.s, p.q, len(rows), n, k), "C3 row band")
        d_v = p.alloc(m * 4)
        for j in (0, 1, 127, 128, 1000, 1983, 1984, 2001):
            ctx.gemv_with_preq(p.w, p.d_s.ptr + j * (k // 32) * 4, p.d_q.ptr + j * k, d_v)
            assert rel_l2(y[:, j], d_v.download(np.float32, m)) < 1e-6
        ctx.gemm_preq(p.w, p.d_s, p.d_q, n, d_y, layout=W.LAYOUT_ROW_MAJOR)
        y2 = fetch_gemm(d_y, m, n, n, W.LAYOUT_ROW_MAJOR)
        assert np.array_equal(y, y2)


def test_argument_errors(ctx, oracle):
    with Problem(ctx, oracle, W.Q4_0, 64, 256, 20) as p:
        d_y = p.alloc(64 * 20 * 4)
        with pytest.raises(W.RocmError) as e:
            ctx.gemm_preq(p.w, p.d_s, p.d_q, 20, d_y, y_stride=10, layout=W.LAYOUT_ROW_MAJOR)
        assert e.value.status == -1
        with pytest.raises(W.RocmError) as e:
            ctx.gemm_preq(p.w, p.d_s, p.d_q, 20, d_y, y_stride=63, layout=W.LAYOUT_TOKEN_MAJOR)
        assert e.value.status == -1
        with pytest.raises(W.RocmError) as e:
            ctx.gemm_preq(p.w, p.d_s, p.d_q, 20, d_y, y_stride=64, layout=5)
        assert e.value.status == -1
        ctx.gemm_preq(p.w, p.d_s, p.d_q, 0, d_y, y_stride=64, layout=W.LAYOUT_TOKEN_MAJOR)  # n = 0: no-op


@pytest.mark.parametrize("dtype,m,n,k,layout,accumulate", [
    (W.Q4_0, 1024, 512, 4608, "token", True),    # the down projection of a 512-token prompt: 64 tiles, 4 shares
    (W.Q8_0, 1024, 100, 2048, "token", False),   # 16 tiles, 4 shares of 4 stages
    (W.Q4_0, 300, 70, 4608, "row", True),        # ragged rows and tokens, 8 shares, row-major output
    (W.Q8_0, 2048, 640, 6912, "token", False),   # 160 narrow tiles (80 wide): 4 shares on the wide tile
    (W.Q4_0, 1024, 2002, 4608, "token", False),  # 256 narrow tiles = 128 wide ones with a long K: 4 shares on the wide tile
    (W.Q8_0, 2048, 700, 4224, "row", True),      # 96 wide tiles, 33 stages: 4 shares of 8 or 9 on the wide tile, ragged tokens
    (W.Q8_0, 1024, 2002, 2048, "token", False),  # 16 stages: too short for the wide split, too many tiles for the narrow one
    (W.Q4_0, 256, 300, 1024, "row", False),      # 10 tiles (not a multiple of the 8 slots the tile map deals out), 4 shares of 2 stages
    (W.Q8_0, 640, 200, 2048, "token", True),     # 20 tiles, 4 shares
    (W.Q4_0, 384, 130, 1152, "token", False),    # 9 stages in 4 shares: 2, 2, 2, 3
    (W.Q8_0, 200, 40, 4224, "row", True),        # 33 stages in 8 shares: 4 or 5 each
    (W.Q4_0, 3072, 128, 1024, "token", False),   # the in projection of a short prompt: 48 tiles, 4 shares
])
def test_gemm_split_over_k(ctx, oracle, dtype, m, n, k, layout, accumulate):
    """GEMM launches with few tiles and a long K walk K in shares (one workgroup per tile and share, a second launch adds the
    shares in a fixed order): held against the oracle like every other launch, equal to the unsplit launch to a few 1e-7,
    and the same bits on every run."""
    wb = oracle.synth_weight(dtype, m, k, seed=77)
    w = ctx.upload_weight(wb, dtype, m, k)
    s, q = oracle.quantize_q8_0_batch(oracle.fill_normal(5, 1.0, n * k), n, k)
    d_q, d_s = ctx.to_device(q), ctx.to_device(s)
    lay = W.LAYOUT_TOKEN_MAJOR if layout == "token" else W.LAYOUT_ROW_MAJOR
    stride = (m + 8) if layout == "token" else (n + 4)
    size = n * stride if layout == "token" else m * stride
    y0 = oracle.fill_normal(6, 1.0, size)
    outs = []
    for splits in (0, 0, 1):  # default twice, then switched off
        ctx.set_gemm_max_k_splits(splits)
        d_y = ctx.to_device(y0)
        ctx.gemm_preq(w, d_s, d_q, n, d_y, y_stride=stride, layout=lay, accumulate=accumulate)
        y = d_y.download(np.float32, size)
        outs.append((y.reshape(n, stride)[:, :m].T if layout == "token" else y.reshape(m, stride)[:, :n]).copy())
        pad = y.reshape(n, stride)[:, m:] if layout == "token" else y.reshape(m, stride)[:, n:]
        assert np.array_equal(pad, (y0.reshape(n, stride)[:, m:] if layout == "token" else y0.reshape(m, stride)[:, n:]))
        d_y.free()
    ctx.set_gemm_max_k_splits(0)
    assert np.array_equal(outs[0].view(np.uint32), outs[1].view(np.uint32))
    ref = oracle.gemm_q8(dtype, wb, s, q, m, n, k, f64=True)
    if accumulate:
        ref = ref + (y0.reshape(n, stride)[:, :m].T if layout == "token" else y0.reshape(m, stride)[:, :n])
    assert_f32_parity(outs[0], ref, "split GEMM")
    assert_f32_parity(outs[2], ref, "unsplit GEMM")
    assert np.linalg.norm(outs[0].astype(np.float64) - outs[2]) <= 1e-6 * np.linalg.norm(outs[2])
    w.free(), d_q.free(), d_s.free()


@pytest.mark.parametrize("dtype,m,n,k,pad", [
    (W.Q4_0, 1024, 512, 4608, 0),   # the down projection of a 512-token prompt: split, the norm's kernel adds the shares up
    (W.Q8_0, 1024, 100, 1024, 8),   # an out projection of a short prompt: split in 4, padded rows
    (W.Q4_0, 256, 300, 1024, 0),    # 10 tiles
    (W.Q4_0, 1024, 2002, 4608, 0),  # 256 tiles: unsplit, the plain norm kernel
    (W.Q8_0, 512, 7, 256, 4),       # below the MFMA hand-off: multi-token GEMV, then the norm
])
def test_residual_projection_with_norm_and_quantizer(ctx, oracle, dtype, m, n, k, pad):
    """x += W a, then Q8_0(rmsnorm(x)): one call == wick_rocm_gemm_q8 (accumulate) + wick_rocm_rmsnorm_quantize_q8_0, bit for bit -- the
    residual rows, the quants and the scales -- whether or not the projection is split over K; and x against the oracle."""
    from wick_amd.lfm2 import Lfm2Ops
    ops, eps, stride = Lfm2Ops(ctx), 1e-5, m + pad
    wb = oracle.synth_weight(dtype, m, k, seed=31)
    w = ctx.upload_weight(wb, dtype, m, k)
    s, q = oracle.quantize_q8_0_batch(oracle.fill_normal(5, 1.0, n * k), n, k)
    d_q, d_s = ctx.to_device(q), ctx.to_device(s)
    x0 = oracle.fill_normal(6, 1.0, n * stride)
    nw = (1 + 0.3 * oracle.fill_normal(7, 1.0, m)).astype(np.float32)
    d_nw = ctx.to_device(nw)
    res = []
    for fused in (True, False):
        d_x, d_oq, d_os = ctx.to_device(x0), ctx.alloc(n * m), ctx.alloc(n * (m // 32) * 4)
        if fused:
            ctx.gemm_preq_residual_rmsnorm_quantize(w, d_s, d_q, n, d_x, stride, d_nw, eps, d_oq, d_os)
        else:
            ctx.gemm_preq(w, d_s, d_q, n, d_x, y_stride=stride, layout=W.LAYOUT_TOKEN_MAJOR, accumulate=True)
            ops.rmsnorm_quantize(d_x, d_nw, n, m, eps, d_oq, d_os, x_stride=stride)
        res.append((d_x.download(np.float32, n * stride), d_oq.download(np.int8, n * m), d_os.download(np.float32, n * (m // 32))))
        for b in (d_x, d_oq, d_os):
            b.free()
    for a, b in zip(*res):
        assert np.array_equal(a.view(np.uint8), b.view(np.uint8))
    x = res[0][0].reshape(n, stride)
    assert np.array_equal(x[:, m:], x0.reshape(n, stride)[:, m:])  # padding untouched
    ref = oracle.gemm_q8(dtype, wb, s, q, m, n, k, f64=True).T + x0.reshape(n, stride)[:, :m]
    assert_f32_parity(x[:, :m], ref, "residual projection")
    # quantizing the input in place of the projection's own input buffers is what the prompt pass does
    if m == k:
        d_x, d_q2, d_s2 = ctx.to_device(x0), ctx.to_device(q), ctx.to_device(s)
        ctx.gemm_preq_residual_rmsnorm_quantize(w, d_s2, d_q2, n, d_x, stride, d_nw, eps, d_q2, d_s2)
        assert np.array_equal(d_q2.download(np.int8, n * m), res[0][1]) and np.array_equal(d_s2.download(np.float32, n * (m // 32)).view(np.uint32), res[0][2].view(np.uint32))
        for b in (d_x, d_q2, d_s2):
            b.free()
    with pytest.raises(W.RocmError, match="multiple of 32"):
        w2 = ctx.upload_weight(oracle.synth_weight(dtype, 48, 256, seed=1), dtype, 48, 256)
        ctx.gemm_preq_residual_rmsnorm_quantize(w2, d_s, d_q, 1, d_nw, 48, d_nw, eps, d_q, d_s)
    w.free(), w2.free(), d_q.free(), d_s.free(), d_nw.free()
