"""Helpers shared by the GPU parity tests (not collected by pytest)."""
import numpy as np

import wick_amd as W


class Problem:
    """Seeded weight + activations on host and device, quantized by the ORACLE so
    the GEMV/GEMM tests do not depend on the device quantizer."""

    def __init__(self, ctx, oracle, dtype, m, k, n=1, seed=1, w_sigma=0.02, weight_bytes=None):
        self.ctx, self.dtype, self.m, self.k, self.n = ctx, dtype, m, k, n
        self.wb = weight_bytes if weight_bytes is not None else oracle.synth_weight(dtype, m, k, seed, w_sigma)
        self.x = oracle.fill_normal(seed * 7919 + 13, 1.0, n * k)
        self.s, self.q = oracle.quantize_q8_0_batch(self.x, n, k)
        self.w = ctx.upload_weight(self.wb, dtype, m, k)
        self.d_q = ctx.to_device(self.q)
        self.d_s = ctx.to_device(self.s)
        self._bufs = [self.d_q, self.d_s]

    def alloc(self, nbytes):
        b = self.ctx.alloc(nbytes)
        self._bufs.append(b)
        return b

    def to_device(self, arr):
        b = self.ctx.to_device(arr)
        self._bufs.append(b)
        return b

    def free(self):
        self.w.free()
        for b in self._bufs:
            b.free()

    def __enter__(self):
        return self

    def __exit__(self, *exc):
        self.free()


def fetch_gemm(buf, m, n, stride, layout):
    """Device GEMM output -> [m, n] regardless of layout."""
    if layout == W.LAYOUT_ROW_MAJOR:
        return buf.download(np.float32, m * stride).reshape(m, stride)[:, :n]
    return buf.download(np.float32, n * stride).reshape(n, stride)[:, :m].T
