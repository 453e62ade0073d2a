"""deepj_hip_flush_ops_noalloc against deepj_hip_flush_ops through the C ABI: the same stream gives bit-identical
results over the library's static scratch array as over the runtime's own workspace and counters, on two calls in a
row (the second with a smaller input, so that it meets the first call's leftovers in the array), no driver
allocation happens on the way, and a stream whose workspace need exceeds the array is refused before anything
is launched."""
import numpy as np
import pytest

from deepj_amd import HipNative
from deepj_amd.fused import DeviceBuffers, Stream, attn_decode_scratch_floats
from oracle import cpu_ref as ref
from gpu_util import assert_close

pytestmark = pytest.mark.gpu

NOALLOC_WORKSPACE_FLOATS = 2 << 20       # DEEPJ_HIP_NOALLOC_WORKSPACE_FLOATS in include/deepj_hip.h


def gaussian(rows, cols, seed, scale=1.0):
    return (np.random.default_rng(seed).standard_normal((rows, cols)) * scale).astype(np.float32)


class Case:
    """A normalised Q8 GEMM (workspace: M*K floats of normalised rows) followed by one fused decode-attention step
    (scratch: the per-head arrival counters of its key splits)."""

    def __init__(self, dev, m, k, n, H, hd, ctx, seed):
        self.dev, self.m, self.k, self.n, self.H, self.hd = dev, m, k, n, H, hd
        d = H * hd
        self.max_seq = ctx + 8
        w = gaussian(k, n, seed, 0.02)
        self.x = gaussian(m, k, seed + 1)
        self.gamma = 1.0 + gaussian(1, k, seed + 2, 0.02)
        self.wdq = ref.q8_roundtrip(w)
        src = dev.upload(w)
        self.wq = dev.alloc(HipNative.q8Floats(k, n))
        Stream().q8_quantize(src, self.wq, k, n).run()
        dev.release(src)
        self.xb, self.gb = dev.upload(self.x), dev.upload(self.gamma)
        # a cache already holding ctx positions, and the new token's q | k | v row
        self.kcache, self.vcache = gaussian(H * self.max_seq, hd, seed + 3), gaussian(H * self.max_seq, hd, seed + 4)
        self.row = gaussian(1, 3 * d, seed + 5)
        cos, sin = ref.rope_tables(hd, self.max_seq)
        self.cos_b, self.sin_b = dev.upload(cos), dev.upload(sin)
        self.row_b = dev.upload(self.row)
        self.ctx = ctx
        self.att_scratch = dev.alloc(attn_decode_scratch_floats(H, hd))

    def run(self, noalloc):
        dev, d = self.dev, self.H * self.hd
        out, att = dev.alloc(self.m * self.n), dev.alloc(d)
        kc, vc = dev.upload(self.kcache), dev.upload(self.vcache)        # fresh copies: the op appends a row
        state = dev.upload(np.array([self.ctx, 0, 0, 0], np.int32))
        s = (Stream().q8_linear(self.xb, self.wq, out, self.m, self.k, self.n, gamma=self.gb)
             .attn_decode(self.row_b, kc, vc, att, state, self.att_scratch, self.cos_b, self.sin_b, self.H, self.hd,
                          self.max_seq, 0))
        words = s.array()
        if noalloc:
            HipNative.flushOpsNoAlloc(words, words.size)
        else:
            HipNative.nativeFlushOps(words, words.size)
        res = (dev.download(out, (self.m, self.n)), dev.download(att, (1, d)),
               dev.download(kc, (self.H * self.max_seq, self.hd)), dev.download(vc, (self.H * self.max_seq, self.hd)))
        dev.release(out, att, kc, vc, state)
        return res


def test_noalloc_flush_matches_flush_on_two_calls_the_second_smaller():
    HipNative.init(0)
    dev = DeviceBuffers()
    try:
        # the second case is smaller in every dimension: its workspace rows and its counters lie inside what
        # the first call used
        # (GEMM shapes that flush_ops runs as ONE launch of the bf16 kernel, as the allocation-free entry point always
        # does: 288 tiles of 64 x 64, and a K of three steps - too many tiles, too short a K, for workgroups to share it)
        cases = [Case(dev, 192, 2048, 6144, 32, 64, 515, 100), Case(dev, 40, 384, 96, 8, 32, 70, 200)]
        expected = [c.run(noalloc=False) for c in cases]
        # the oracle on the first case's GEMM: the comparison below is between two HIP paths, this pins one of them
        c = cases[0]
        exp = ref.matmul(ref.rmsnorm(c.x, c.gamma), c.wdq)
        scale = float(np.sqrt(np.mean(exp.astype(np.float64) ** 2)))
        assert_close(exp, expected[0][0], atol=1e-4 * scale, rtol=1e-4, what="flush_ops GEMM vs oracle")
        HipNative.synchronize()
        allocs_before = HipNative.poolStats()["driver_allocs"]
        for c, want in zip(cases, expected):
            # inputs, outputs and the cache copies are (re)created by run(); only the flush itself must not allocate,
            # so warm the pool with one throw-away pass of the ordinary entry point first
            c.run(noalloc=False)
            before = HipNative.poolStats()["driver_allocs"]
            got = c.run(noalloc=True)
            assert HipNative.poolStats()["driver_allocs"] == before, "the allocation-free entry point allocated"
            for name, w, g in zip(("gemm", "attention", "k cache", "v cache"), want, got):
                assert np.array_equal(w.view(np.int32), g.view(np.int32)), f"{name} differs between the entry points"
        assert HipNative.poolStats()["driver_allocs"] >= allocs_before
    finally:
        dev.release_all()


def test_noalloc_flush_never_shares_k_among_workgroups():
    """A few-tile, long-K product (64 rows x 2048 x 2048: 32 tiles) runs under flush_ops as eight workgroups per tile
    with their partial products in the workspace; the allocation-free entry point runs it as one launch.  Both are
    held to the oracle at the per-op tolerance."""
    HipNative.init(0)
    dev = DeviceBuffers()
    try:
        m, k, n = 64, 2048, 2048
        w = gaussian(k, n, 41, 0.02)
        x = gaussian(m, k, 42)
        src = dev.upload(w)
        wq = dev.alloc(HipNative.q8Floats(k, n))
        Stream().q8_quantize(src, wq, k, n).run()
        dev.release(src)
        xb, out = dev.upload(x), dev.alloc(m * n)
        exp = ref.matmul(x, ref.q8_roundtrip(w))
        scale = float(np.sqrt(np.mean(exp.astype(np.float64) ** 2)))
        words = Stream().q8_linear(xb, wq, out, m, k, n).array()
        HipNative.nativeFlushOps(words, words.size)
        assert_close(exp, dev.download(out, (m, n)), atol=1e-4 * scale, rtol=1e-4, what="flush_ops (K shared) vs oracle")
        dev.write(out, np.zeros(m * n, np.float32))
        before = HipNative.poolStats()["driver_allocs"]
        HipNative.flushOpsNoAlloc(words, words.size)
        got = dev.download(out, (m, n))
        assert HipNative.poolStats()["driver_allocs"] == before
        assert_close(exp, got, atol=1e-4 * scale, rtol=1e-4, what="noalloc (one launch) vs oracle")
    finally:
        dev.release_all()


def test_noalloc_flush_with_256_rows_and_more_stays_on_the_small_workspace_kernels():
    """From 256 rows on flush_ops may run a Q8_LINEAR on the fp16 GEMM, whose operands live in a workspace sized by the
    shape; the allocation-free entry point never does, whether the fp16 kernel's need would happen to fit the fixed
    array (prepared weights: about 1.1 M floats here) or not (unprepared: about 7.6 M).  Both entry points are
    held to the oracle at the per-op tolerance; the allocation-free result is the same bits with and without a
    prepared copy of the weights (the copy is not used there), which the fp16 kernel's would not be against the
    bf16 kernel's."""
    HipNative.init(0)
    dev = DeviceBuffers()
    try:
        m, k, n = 512, 2048, 6144
        w = gaussian(k, n, 31, 0.02)
        x = gaussian(m, k, 32)
        gamma = 1.0 + gaussian(1, k, 33, 0.02)
        src = dev.upload(w)
        wq = dev.alloc(HipNative.q8Floats(k, n))
        Stream().q8_quantize(src, wq, k, n).run()
        dev.release(src)
        xb, gb, out = dev.upload(x), dev.upload(gamma), dev.alloc(m * n)
        exp = ref.matmul(ref.rmsnorm(x, gamma), ref.q8_roundtrip(w))
        scale = float(np.sqrt(np.mean(exp.astype(np.float64) ** 2)))
        words = Stream().q8_linear(xb, wq, out, m, k, n, gamma=gb).array()

        def noalloc():
            dev.write(out, np.zeros(m * n, np.float32))
            before = HipNative.poolStats()["driver_allocs"]
            HipNative.flushOpsNoAlloc(words, words.size)
            got = dev.download(out, (m, n))
            assert HipNative.poolStats()["driver_allocs"] == before, "the allocation-free entry point allocated"
            assert_close(exp, got, atol=1e-4 * scale, rtol=1e-4, what="noalloc GEMM vs oracle")
            return got

        plain = noalloc()
        HipNative.nativeFlushOps(words, words.size)
        assert_close(exp, dev.download(out, (m, n)), atol=1e-4 * scale, rtol=1e-4, what="flush_ops GEMM vs oracle")
        prepared = dev.alloc(HipNative.q8PreparedFloats(k, n))
        Stream().q8_prepare(wq, prepared, k, n).run()
        assert np.array_equal(noalloc().view(np.int32), plain.view(np.int32)), \
            "a prepared copy of the weights changed the allocation-free result"
        HipNative.nativeFlushOps(words, words.size)
        assert_close(exp, dev.download(out, (m, n)), atol=1e-4 * scale, rtol=1e-4, what="flush_ops GEMM (prepared) vs oracle")
    finally:
        dev.release_all()


def test_noalloc_flush_rejects_what_it_cannot_serve():
    HipNative.init(0)
    dev = DeviceBuffers()
    try:
        m, k, n = 1100, 2048, 64                     # 1100 * 2048 floats of normalised rows: above the static array
        assert m * k > NOALLOC_WORKSPACE_FLOATS
        x, g, out = dev.alloc(m * k), dev.alloc(k), dev.alloc(m * n)
        w = dev.alloc(HipNative.q8Floats(k, n))
        marker = np.full(m * n, 7.0, np.float32)
        dev.write(out, marker)
        words = Stream().q8_linear(x, w, out, m, k, n, gamma=g).array()
        with pytest.raises(RuntimeError, match="static scratch holds"):
            HipNative.flushOpsNoAlloc(words, words.size)
        assert np.array_equal(dev.download(out, (m * n,)), marker), "a refused stream must launch nothing"
        with pytest.raises(RuntimeError, match="Unknown op code in graph: 999"):
            HipNative.flushOpsNoAlloc(np.array([999, 0, 0], np.int32), 3)
        # without a norm prologue the same shape needs no workspace and is served
        words = Stream().fill(x, 0, m * k).q8_linear(x, w, out, m, k, n).array()
        HipNative.flushOpsNoAlloc(words, words.size)
        HipNative.synchronize()
    finally:
        dev.release_all()
