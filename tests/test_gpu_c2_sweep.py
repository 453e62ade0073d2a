"""The isolated Q8 linear-op sweep exactly as the baseline states it, through the C ABI against the CPU oracle.

Inputs (java.util.Random streams, like the reference's own GPU test draws its operands,
src/test/java/io/github/kirstenali/deepj/tensor/metal/MetalBackendTest.java:71-78):
  weights      (float)(Random(1).nextGaussian() * 0.02), row-major [K x N], ONE stream that continues across
               2048x2048, 2048x5632, 5632x2048, 4096x11008 in that order (and, for the SwiGLU layer below, on
               into a fifth 2048x5632 matrix, the `up` projection); quantised with the library's Q8 quantiser
  activations  (float)Random(2).nextGaussian(), [M x K], a fresh Random(2) per matrix; M = 1 (decode matvec),
               64 and 512 (prefill GEMM), at FULL width for all four shapes
  RMSNorm      gain 1 + 0.02 g from Random(3); the reference's epsilon 1e-6 (RMSNorm1D.java:30), with the
               baseline's 1e-5 evaluated beside it
Gate: |expected - actual| <= atol + 1e-4 |expected| (MetalBackendTest.java:452-466), atol = 1e-4 of the
output's rms for the contractions.  The expected value is the oracle's fp32 CpuBackend.matmul (ikj order) on the
DEQUANTISED weights; the dequantised weights themselves are checked bit for bit against the host quantiser."""
import numpy as np
import pytest

from deepj_amd import HipNative, JavaRandom
from deepj_amd.fused import DeviceBuffers, Stream
from oracle import cpu_ref as ref
from gpu_util import assert_close

pytestmark = pytest.mark.gpu

SHAPES = [(2048, 2048), (2048, 5632), (5632, 2048), (4096, 11008)]


@pytest.fixture(scope="module")
def sweep():
    ref.set_threads(ref.default_threads())
    rng = JavaRandom(1)
    mats = [rng.tensor(k, n, 0.02) for k, n in SHAPES]
    up = rng.tensor(2048, 5632, 0.02)
    # the stream really is Random(1)'s: its head against the oracle's own java.util.Random
    head = ref.JavaRandom(1).gaussians_f32(1, 64, 0.02)[0]
    assert np.array_equal(mats[0].reshape(-1)[:64].view(np.int32), head.view(np.int32))
    dev = DeviceBuffers()
    bufs, deq = [], []
    for w in mats + [up]:
        k, n = w.shape
        src = dev.upload(w)
        wq = dev.alloc(HipNative.q8Floats(k, n))
        Stream().q8_quantize(src, wq, k, n).run()
        dev.release(src)
        bufs.append(wq)
        deq.append(ref.q8_roundtrip(w))
    yield dev, mats + [up], bufs, deq
    dev.release_all()
    ref.set_threads(1)


def activations(m, k):
    return JavaRandom(2).tensor(m, k, 1.0)


@pytest.mark.parametrize("idx", range(4))
def test_dequantised_weights_bit_exact(sweep, idx):
    dev, mats, bufs, deq = sweep
    k, n = mats[idx].shape
    out = dev.alloc(k * n)
    Stream().q8_dequantize(bufs[idx], out, k, n).run()
    got = dev.download(out, (k, n))
    dev.release(out)
    assert np.array_equal(got.view(np.int32), deq[idx].view(np.int32)), "device dequantisation differs from the host's"
    # and the quantiser's own bound: |w - dequant(quant(w))| <= scale / 2 per element, scale = max|w| of the group / 127
    # (plus the fp32 roundings of w / scale and q * scale: a few 1e-7 of the group's largest weight)
    w = mats[idx].astype(np.float64)
    amax = np.abs(w.reshape(k // 32, 32, n)).max(axis=1, keepdims=True)
    bound = np.broadcast_to(amax / 127.0 * 0.5 + amax * 4e-7, (k // 32, 32, n)).reshape(k, n)
    assert np.all(np.abs(w - deq[idx]) <= bound)


@pytest.mark.parametrize("m", [1, 64, 512])
@pytest.mark.parametrize("idx", range(4))
def test_q8_linear_full_width(sweep, idx, m):
    dev, mats, bufs, deq = sweep
    k, n = mats[idx].shape
    x = activations(m, k)
    exp = ref.matmul(x, deq[idx])
    xb, ob = dev.upload(x), dev.alloc(m * n)
    Stream().q8_linear(xb, bufs[idx], ob, m, k, n).run()
    got = dev.download(ob, (m, n))
    dev.release(xb, ob)
    scale = float(np.sqrt(np.mean(exp.astype(np.float64) ** 2)))
    assert_close(exp, got, atol=1e-4 * scale, rtol=1e-4, what=f"Q8 linear M={m} {k}x{n}")


@pytest.mark.parametrize("idx", range(4))
def test_q8_linear_full_width_on_the_bf16_kernels(sweep, idx):
    """The same 512-row products through the allocation-free entry point, whose fixed workspace keeps them on the bf16
    matrix-core kernels (three-piece activations, 128 x 128 / 64 x 128 / 64 x 64 tiles) that the ordinary entry point
    now leaves to the fp16 GEMM for most of these shapes: both kernels answer to the same oracle and gate."""
    dev, mats, bufs, deq = sweep
    k, n = mats[idx].shape
    m = 512
    x = activations(m, k)
    exp = ref.matmul(x, deq[idx])
    xb, ob = dev.upload(x), dev.alloc(m * n)
    words = Stream().q8_linear(xb, bufs[idx], ob, m, k, n).array()
    HipNative.flushOpsNoAlloc(words, words.size)
    got = dev.download(ob, (m, n))
    dev.release(xb, ob)
    scale = float(np.sqrt(np.mean(exp.astype(np.float64) ** 2)))
    assert_close(exp, got, atol=1e-4 * scale, rtol=1e-4, what=f"Q8 linear (bf16 kernels) M={m} {k}x{n}")


@pytest.mark.parametrize("m", [1, 64, 512])
@pytest.mark.parametrize("cols", [2048, 5632])
def test_fused_rmsnorm_at_both_epsilons(sweep, m, cols):
    """The kernel uses the reference's epsilon (1e-6, RMSNorm1D.java:30).  The baseline's text says 1e-5: on these
    N(0,1) rows mean(x^2) is about 1, so the two differ by 0.5 * 9e-6 relative - twenty times inside the 1e-4 per-op
    gate; the test holds the kernel to the reference's value at 1e-5 relative, shows that it tells the two epsilons
    apart, and that the other one would pass the per-op gate as well."""
    dev = sweep[0]
    x = JavaRandom(2).tensor(m, cols, 1.0)
    gamma = (1.0 + JavaRandom(3).tensor(1, cols, 0.02)).astype(np.float32)
    xb, gb, ob = dev.upload(x), dev.upload(gamma), dev.alloc(m * cols)
    Stream().rmsnorm(xb, gb, ob, m, cols).run()
    got = dev.download(ob, (m, cols)).astype(np.float64)
    dev.release(xb, gb, ob)
    exp6 = ref.rmsnorm(x, gamma)                                   # the oracle: eps 1e-6, six primitive ops
    assert_close(exp6, got, atol=1e-6, rtol=1e-5, what=f"RMSNorm [{m}x{cols}] at the reference's eps 1e-6")
    x64 = x.astype(np.float64)
    ms = (x64 * x64).mean(axis=1, keepdims=True)
    e6, e5 = gamma * x64 / np.sqrt(ms + 1e-6), gamma * x64 / np.sqrt(ms + 1e-5)
    big = np.abs(e6) > 0.5
    d6 = float(np.max(np.abs(got - e6)[big] / np.abs(e6)[big]))
    d5 = float(np.max(np.abs(got - e5)[big] / np.abs(e5)[big]))
    print(f"\n[RMSNorm {m}x{cols}] max relative distance from the exact value at eps 1e-6: {d6:.2e}, at eps 1e-5: {d5:.2e}")
    assert d6 < 1.5e-6 and 3.0e-6 < d5 < 6.0e-6, "the kernel should sit on the eps = 1e-6 value"
    assert_close(e5, got, atol=1e-6, rtol=1e-4, what="the baseline's eps 1e-5 against the per-op gate")


@pytest.mark.parametrize("m", [1, 64, 512])
def test_silu_mul_on_5632_wide_rows(sweep, m):
    dev = sweep[0]
    g, u = JavaRandom(2).tensor(m, 5632, 1.0), JavaRandom(4).tensor(m, 5632, 1.0)
    gb, ub, ob = dev.upload(g), dev.upload(u), dev.alloc(m * 5632)
    Stream().silu_mul(gb, ub, ob, m * 5632).run()
    got = dev.download(ob, (m, 5632))
    dev.release(gb, ub, ob)
    assert_close(ref.multiply(ref.silu(g), u), got, atol=1e-7, rtol=1e-6, what=f"SiLU(gate) * up [{m}x5632]")


@pytest.mark.parametrize("m", [1, 64, 512])
def test_swiglu_layer_on_2048_wide_rows(sweep, m):
    """SwiGLULayer.forward (SwiGLULayer.java:63-70) on [M x 2048]: gate = sweep matrix 2 (2048x5632), up = the
    fifth matrix of the same stream, down = sweep matrix 3 (5632x2048); biases N(0, 0.1) from Random(5)."""
    dev, mats, bufs, deq = sweep
    d, dff = 2048, 5632
    x = activations(m, d)
    br = JavaRandom(5)
    bg, bu, bd = br.tensor(1, dff, 0.1), br.tensor(1, dff, 0.1), br.tensor(1, d, 0.1)
    exp = ref.swiglu(x, deq[1], bg, deq[4], bu, deq[2], bd)
    # the runner's layout: gate and up rows interleaved in one Q8 buffer, SiLU * up in the epilogue
    wgu = dev.alloc(HipNative.q8Floats(d, 2 * dff))
    for w, off in ((mats[1], 0), (mats[4], 1)):
        src = dev.upload(w)
        Stream().q8_quantize(src, wgu, d, dff, off, 2, 2 * dff).run()
        dev.release(src)
    xb, hb, ob = dev.upload(x), dev.alloc(m * dff), dev.alloc(m * d)
    (Stream().q8_linear(xb, wgu, hb, m, d, dff, bias=dev.upload(bg), bias2=dev.upload(bu), swiglu=True)
     .q8_linear(hb, bufs[2], ob, m, dff, d, bias=dev.upload(bd)).run())
    got = dev.download(ob, (m, d))
    dev.release(wgu, xb, hb, ob)
    scale = float(np.sqrt(np.mean(exp.astype(np.float64) ** 2)))
    assert_close(exp, got, atol=1e-4 * scale, rtol=1e-4, what=f"SwiGLU layer [{m}x2048]")
