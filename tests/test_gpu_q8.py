"""Q8 weight path through the C ABI: quantiser bit-exact against the host quantiser, decode
matvec and prefill GEMM (with their fused prologue/epilogues) against the CPU oracle run on
the dequantised weights.  Shapes of the isolated linear-op sweep at reduced N
where the oracle would be slow, plus ragged K (688 = 21*32 + 16)."""
import numpy as np
import pytest

from deepj_amd import HipNative
from deepj_amd.fused import DeviceBuffers, Stream
from oracle import cpu_ref as ref
from gpu_util import assert_close

pytestmark = pytest.mark.gpu


def gaussian(rows, cols, seed, scale):
    rng = np.random.default_rng(seed)
    return (rng.standard_normal((rows, cols)) * scale).astype(np.float32)


@pytest.fixture
def dev():
    d = DeviceBuffers()
    yield d
    d.release_all()


def quantize_on_device(dev, w, row_off=0, row_step=1, total_rows=None, dst=None):
    k, n = w.shape
    total = n if total_rows is None else total_rows
    src = dev.upload(w)
    if dst is None:
        dst = dev.alloc(HipNative.q8Floats(k, total))
    Stream().q8_quantize(src, dst, k, n, row_off, row_step, total).run()
    dev.release(src)
    return dst


@pytest.mark.parametrize("k,n", [(64, 3), (688, 70), (2048, 256), (70, 9)])
def test_quantize_and_dequantize_bit_exact_vs_host(dev, k, n):
    w = gaussian(k, n, 1, 0.02)
    w[:, 0] = 0.0                                   # an all-zero column: scale 0, no NaN
    wq = quantize_on_device(dev, w)
    kp = (k + 31) // 32 * 32
    raw = dev.download(wq, (HipNative.q8Floats(k, n),), np.float32).view(np.int8)
    q_dev = raw[: n * kp].reshape(n, kp)
    sc_off = (n * kp + 255) // 256 * 256
    s_dev = raw[sc_off: sc_off + n * (kp // 32) * 4].view(np.float32).reshape(n, kp // 32)
    q_ref, s_ref = ref.q8_quantize(w)
    assert np.array_equal(q_dev, q_ref), "int8 payload differs from the host quantiser"
    assert np.array_equal(s_dev.view(np.int32), s_ref.view(np.int32)), "scales differ bitwise"
    out = dev.alloc(k * n)
    Stream().q8_dequantize(wq, out, k, n).run()
    dq = dev.download(out, (k, n))
    assert np.array_equal(dq.view(np.int32), ref.q8_dequantize(q_ref, s_ref, k).view(np.int32))


def test_quantize_into_interleaved_rows(dev):
    k, n = 96, 10
    wg, wu = gaussian(k, n, 2, 0.02), gaussian(k, n, 3, 0.02)
    dst = dev.alloc(HipNative.q8Floats(k, 2 * n))
    quantize_on_device(dev, wg, 0, 2, 2 * n, dst)
    quantize_on_device(dev, wu, 1, 2, 2 * n, dst)
    og, ou = dev.alloc(k * n), dev.alloc(k * n)
    Stream().q8_dequantize(dst, og, k, n, 0, 2, 2 * n).q8_dequantize(dst, ou, k, n, 1, 2, 2 * n).run()
    assert np.array_equal(dev.download(og, (k, n)), ref.q8_roundtrip(wg))
    assert np.array_equal(dev.download(ou, (k, n)), ref.q8_roundtrip(wu))


def linear_case(dev, m, k, n, *, norm=False, bias=False, residual=False, seed=0):
    w = gaussian(k, n, seed + 1, 0.02)
    x = gaussian(m, k, seed + 2, 1.0)
    wdq = ref.q8_roundtrip(w)
    wq = quantize_on_device(dev, w)
    xb, ob = dev.upload(x), dev.alloc(m * n)
    kw, h = {}, x
    if norm:
        gamma = (1.0 + gaussian(1, k, seed + 3, 0.02))
        kw["gamma"] = dev.upload(gamma)
        h = ref.rmsnorm(x, gamma)
    exp = ref.matmul(h, wdq)
    if bias:
        b = gaussian(1, n, seed + 4, 0.1)
        kw["bias"] = dev.upload(b)
        exp = ref.add_row_vector(exp, b)
    if residual:
        r = gaussian(m, n, seed + 5, 1.0)
        kw["residual"] = dev.upload(r)
        exp = ref.add(r, exp)
    Stream().q8_linear(xb, wq, ob, m, k, n, **kw).run()
    return exp, dev.download(ob, (m, n))


@pytest.mark.parametrize("k,n", [(2048, 2048), (2048, 5632), (5632, 2048), (4096, 1100), (11008, 512), (4096, 11008),
                                 (688, 256), (256, 688), (32, 1), (1024, 5),
                                 # K not a multiple of 4: the scalar staging path, one output per wavefront whatever N
                                 (70, 9), (1023, 300), (2050, 7000)])
def test_q8_matvec_matches_oracle(dev, k, n):
    exp, got = linear_case(dev, 1, k, n)
    # fp32 sums of K terms in a different order: |err| <~ 1e-6 * sqrt(K) * |x||w|; outputs can sit near 0
    scale = float(np.sqrt(np.mean(exp.astype(np.float64) ** 2)))
    assert_close(exp, got, atol=1e-4 * scale, rtol=1e-4, what=f"matvec {k}x{n}")


@pytest.mark.parametrize("flags", [dict(norm=True), dict(bias=True), dict(residual=True),
                                   dict(norm=True, bias=True, residual=True)])
def test_q8_matvec_fused_prologue_epilogue(dev, flags):
    for k, n in [(2048, 768), (688, 256), (1023, 300)]:
        exp, got = linear_case(dev, 1, k, n, seed=10, **flags)
        scale = float(np.sqrt(np.mean(exp.astype(np.float64) ** 2)))
        assert_close(exp, got, atol=1e-4 * scale, rtol=1e-4, what=f"{flags} {k}x{n}")


@pytest.mark.parametrize("m,k,n", [(1, 256, 688), (1, 254, 688), (1, 2050, 6000), (64, 256, 688),
                                   (520, 96, 4500), (1000, 160, 3500), (600, 64, 2000)])   # 64x128, 128x128, many 64x64 tiles
def test_q8_swiglu_gate_up(dev, m, k, n):
    wg, wu = gaussian(k, n, 21, 0.05), gaussian(k, n, 22, 0.05)
    bg, bu = gaussian(1, n, 23, 0.1), gaussian(1, n, 24, 0.1)
    x, gamma = gaussian(m, k, 25, 1.0), 1.0 + gaussian(1, k, 26, 0.02)
    wq = dev.alloc(HipNative.q8Floats(k, 2 * n))
    quantize_on_device(dev, wg, 0, 2, 2 * n, wq)
    quantize_on_device(dev, wu, 1, 2, 2 * n, wq)
    xb, ob = dev.upload(x), dev.alloc(m * n)
    Stream().q8_linear(xb, wq, ob, m, k, n, gamma=dev.upload(gamma), bias=dev.upload(bg), bias2=dev.upload(bu),
                       swiglu=True).run()
    h = ref.rmsnorm(x, gamma)
    gate = ref.linear(h, ref.q8_roundtrip(wg), bg)
    up = ref.linear(h, ref.q8_roundtrip(wu), bu)
    exp = ref.multiply(ref.silu(gate), up)
    assert_close(exp, dev.download(ob, (m, n)), atol=2e-6, rtol=1e-4, what=f"swiglu {m}x{k}x{n}")


@pytest.mark.parametrize("m,k,n", [(64, 2048, 512), (512, 2048, 256), (64, 688, 256), (7, 96, 33), (130, 5632, 128),
                                   (64, 4096, 344), (96, 11008, 128),
                                   (1300, 688, 1400), (1024, 2048, 2100),      # many 64 x 64 tiles, ragged edges
                                   # 440 tiles of 128 x 128 (one well-filled round of 512), ragged in M, N and K; 355 such
                                   # tiles (a mostly empty second round) -> 64 x 128 tiles; exactly 512
                                   (1000, 160, 7000), (520, 96, 9000), (1024, 64, 8192),
                                   # the linear-op sweep's own shapes at M = 512, full width
                                   (512, 2048, 5632), (512, 5632, 2048), (512, 4096, 11008)])
def test_q8_gemm_matches_oracle(dev, m, k, n):
    exp, got = linear_case(dev, m, k, n, norm=True, bias=True, residual=True, seed=30)
    scale = float(np.sqrt(np.mean(exp.astype(np.float64) ** 2)))
    assert_close(exp, got, atol=1e-4 * scale, rtol=1e-4, what=f"gemm {m}x{k}x{n}")


def test_q8_linear_rejects_bad_streams(dev):
    x, w, out = dev.alloc(64), dev.alloc(HipNative.q8Floats(64, 4)), dev.alloc(4)
    with pytest.raises(RuntimeError, match="op needs"):
        Stream().q8_linear(x, w, out, 1, 64, 8).run()                 # weight buffer too small for N=8
    with pytest.raises(RuntimeError, match="SWIGLU cannot be combined"):
        Stream().q8_linear(x, w, out, 1, 64, 2, residual=out, swiglu=True).run()
    with pytest.raises(RuntimeError, match="rows fall outside"):
        Stream().q8_quantize(x, w, 64, 1, 4, 1, 4).run()


def test_fused_rmsnorm_silu_mul_embed_argmax(dev):
    x, gamma = gaussian(9, 2048, 40, 1.0), 1.0 + gaussian(1, 2048, 41, 0.02)
    xb, gb, ob = dev.upload(x), dev.upload(gamma), dev.alloc(x.size)
    Stream().rmsnorm(xb, gb, ob, 9, 2048).run()
    assert_close(ref.rmsnorm(x, gamma), dev.download(ob, x.shape), 1e-6, 1e-5)
    # rows kept in registers (cols a multiple of 4 up to 4096) and the strided fallback (wider or ragged rows)
    for rows, cols in ((3, 36), (600, 4096), (5, 4100), (7, 70), (2, 8192)):
        xr, gr = gaussian(rows, cols, 44, 1.5), 1.0 + gaussian(1, cols, 45, 0.1)
        o = dev.alloc(xr.size)
        Stream().rmsnorm(dev.upload(xr), dev.upload(gr), o, rows, cols).run()
        assert_close(ref.rmsnorm(xr, gr), dev.download(o, xr.shape), 1e-6, 1e-5, what=f"rmsnorm {rows}x{cols}")
    g, u = gaussian(5, 5632, 42, 2.0), gaussian(5, 5632, 43, 1.0)
    o2 = dev.alloc(g.size)
    Stream().silu_mul(dev.upload(g), dev.upload(u), o2, g.size).run()
    assert_close(ref.multiply(ref.silu(g), u), dev.download(o2, g.shape), 1e-7, 1e-6)
    table = gaussian(100, 64, 44, 1.0)
    ids = np.array([5, 99, 0, 5], np.int32)
    o3 = dev.alloc(4 * 64)
    Stream().embed_gather(dev.upload(table), dev.upload(ids), o3, 4, 64, 100).run()
    assert np.array_equal(dev.download(o3, (4, 64)), table[ids])
    logits = gaussian(3, 32000, 45, 4.0)
    logits[1, 777] = logits[1, 31999] = 100.0          # tie -> lowest index
    o4 = dev.alloc(3)
    Stream().argmax_rows(dev.upload(logits), o4, 3, 32000).run()
    got = dev.download(o4, (3,), np.int32)
    assert list(got) == [int(np.argmax(logits[0])), 777, int(np.argmax(logits[2]))]


# ── the two ops the latent KV cache is built from: rows appended at a device-side fill level, and a Q8 product
#    over the rows that exist so far ──────────────────────────────────────────────────────────────────────────

@pytest.mark.parametrize("level,rows", [(0, 3), (5, 1), (9, 4), (12, 2), (-2, 3), (40, 2)])
def test_append_rows_at_the_device_side_fill_level(dev, level, rows):
    """dst[dstOff + (state[0] + i) * rowFloats ...] = src row i; rows that would land outside [0, maxRows) are
    dropped (a fill level that is negative or beyond the cache never makes the kernel write out of bounds)."""
    rf, max_rows, off = 24, 12, 7
    before = gaussian(1, off + max_rows * rf + 5, 61, 1.0).reshape(-1)
    src = gaussian(rows, rf, 62, 1.0)
    dst, sb = dev.upload(before), dev.upload(src)
    state = dev.upload(np.array([level, 0, 0, 0], np.int32))
    Stream().append_rows(sb, dst, state, rows, rf, max_rows, off).run()
    exp = before.copy()
    for i in range(rows):
        r = level + i
        if 0 <= r < max_rows:
            exp[off + r * rf: off + (r + 1) * rf] = src[i]
    assert np.array_equal(dev.download(dst, exp.shape), exp)


@pytest.mark.parametrize("level,extra", [(0, 1), (6, 1), (37, 16), (150, 1), (199, 1), (-3, 1), (500, 4)])
def test_q8_linear_over_the_rows_a_growing_cache_holds(dev, level, extra):
    """Q8_LINEAR_DYN: rows [0, min(Mmax, state[0] + extraRows)) of x + xOff times W; the rows beyond stay untouched."""
    m_max, k, n, x_off = 200, 96, 136, 64
    w = gaussian(k, n, 71, 0.05)
    x = gaussian(m_max, k, 72, 1.0)
    wq = quantize_on_device(dev, w)
    xb = dev.upload(np.concatenate([np.zeros(x_off, np.float32), x.reshape(-1)]))
    marker = np.full((m_max, n), 123.0, np.float32)
    ob = dev.upload(marker)
    state = dev.upload(np.array([level, 0, 0, 0], np.int32))
    Stream().q8_linear_dyn(xb, wq, ob, m_max, k, n, state, extra, x_off).run()
    got = dev.download(ob, (m_max, n))
    live = max(0, min(m_max, level + extra))
    if live:
        exp = ref.matmul(x[:live], ref.q8_roundtrip(w))
        scale = float(np.sqrt(np.mean(exp.astype(np.float64) ** 2)))
        assert_close(exp, got[:live], atol=1e-4 * scale, rtol=1e-4, what=f"live rows at level {level}")
    assert np.array_equal(got[live:], marker[live:]), "rows beyond the fill level were written"


def test_latent_ops_reject_bad_streams(dev):
    a, st = dev.alloc(64), dev.upload(np.zeros(4, np.int32))
    with pytest.raises(RuntimeError, match="op needs"):
        Stream().append_rows(a, a, st, 2, 16, 8, 0).run()                 # dst must hold 8 rows of 16 floats
    with pytest.raises(RuntimeError, match="bad shape"):
        Stream().append_rows(a, a, st, 0, 16, 4, 0).run()
    w = dev.alloc(HipNative.q8Floats(32, 4))
    with pytest.raises(RuntimeError, match="op needs"):
        Stream().q8_linear_dyn(a, w, a, 4, 32, 4, st, 1, 0).run()         # x holds 64 floats, 4 rows of 32 need 128
    with pytest.raises(RuntimeError, match="bad shape"):
        Stream().q8_linear_dyn(a, w, a, 1, 32, 4, st, -1, 0).run()
