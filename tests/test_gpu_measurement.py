"""The measurement hooks of the C ABI that bench.py builds its tables on: the floor ops (NOP, STREAM_READ), the launch
period of a stream (time_ops), per-op kernel durations with every dispatch counted (profile_ops) and the shader-clock
sampler (clock_probe).  None has a counterpart in the reference; what is checked is that they measure what they say,
leave results alone and end by themselves."""
import numpy as np
import pytest

from deepj_amd import HipNative
from deepj_amd.fused import DeviceBuffers, Stream

pytestmark = pytest.mark.gpu


@pytest.fixture
def dev():
    d = DeviceBuffers()
    yield d
    d.release_all()


def quantised(dev, k, n, seed):
    w = (np.random.default_rng(seed).standard_normal((k, n)) * 0.05).astype(np.float32)
    src, wq = dev.upload(w), dev.alloc(HipNative.q8Floats(k, n))
    Stream().q8_quantize(src, wq, k, n).run()
    dev.release(src)
    return wq


def test_floor_ops_run_and_touch_nothing(dev):
    data = np.arange(5000, dtype=np.float32)
    src, sink = dev.upload(data), dev.alloc(64)
    Stream().nop(1).nop(768).stream_read(src, sink, data.size).run()
    assert np.array_equal(dev.download(src, (data.size,)), data)
    with pytest.raises(RuntimeError):
        Stream().stream_read(src, sink, data.size + 1).run()          # more floats than the buffer holds
    with pytest.raises(RuntimeError):
        Stream().stream_read(987654, sink, 16).run()                   # unknown buffer


def test_time_ops_is_a_launch_period(dev):
    st = Stream().nop(256)
    one = st.time(200) / 200
    assert 0.0005 < one < 0.05                                          # milliseconds per empty launch: microseconds, not more
    many = Stream()
    for _ in range(8):
        many.nop(256)
    eight = many.time(200) / 200
    assert 4 * one < eight < 16 * one


def test_profile_ops_counts_every_dispatch_of_an_op_and_changes_no_result(dev):
    m, k, n = 512, 2048, 2048
    assert HipNative.q8GemmTile(m, k, n) == (64, 256, 4)                # activation split + GEMM + sum of the K shares
    wq = quantised(dev, k, n, 1)
    x = dev.upload(np.random.default_rng(2).standard_normal((m, k)).astype(np.float32))
    x1 = dev.upload(np.random.default_rng(3).standard_normal((1, k)).astype(np.float32))
    out, out1 = dev.alloc(m * n), dev.alloc(n)
    st = Stream().q8_linear(x, wq, out, m, k, n).q8_linear(x1, wq, out1, 1, k, n).nop(4)
    st.run()
    ref_out, ref_out1 = dev.download(out, (m, n)), dev.download(out1, (1, n))
    total, longest, count = HipNative.profileOps(st.array(), 3, detail=True)
    assert list(count) == [4, 1, 1]                                     # + the per-call weight conversion
    assert all(total > 0) and all(longest > 0)
    assert total[0] > longest[0] > 0.4 * total[0]                       # the GEMM is the bulk of its op, the helpers the rest
    assert abs(total[1] - longest[1]) < 1e-3 and abs(total[2] - longest[2]) < 1e-3
    assert np.array_equal(dev.download(out, (m, n)), ref_out) and np.array_equal(dev.download(out1, (1, n)), ref_out1)
    assert np.allclose(st.profile(2), total, rtol=0.5)


def test_clock_probe_samples_a_plausible_clock_and_ends_by_itself(dev):
    n = 1 << 22
    a, b = dev.alloc(n), dev.alloc(n)
    Stream().fill(a, 0x40000000, n).run()
    st = Stream().copy(a, b, n)
    mhz, t, win = HipNative.clockProbe(st.array(), 50, 300, 1)
    assert mhz.size == 299 and t.size == 299
    assert np.all(np.diff(t) > 0)                                       # the wall clock moves forward
    assert -100.0 < win[0] < win[1] < t[-1] + 1e6                       # the runs begin about when the sampler does, and take time
    assert np.all((mhz > 300.0) & (mhz < 4000.0))                       # a shader clock, whatever the power state
    assert np.all(dev.download(b, (n,)) == 2.0)                         # the stream ran
    idle, _, _ = HipNative.clockProbe(Stream().nop(1).array(), 0, 50, 0)
    assert idle.size == 49
    with pytest.raises(RuntimeError):
        HipNative.clockProbe(st.array(), 1, 0, 1)
    with pytest.raises(RuntimeError):
        HipNative.clockProbe(st.array(), 1, 10, 1 << 20)
