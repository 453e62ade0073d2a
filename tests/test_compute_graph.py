"""The lazy-graph protocol without a GPU: a recording GpuRuntime logs the five calls, as the
reference's own src/test/java/io/github/kirstenali/deepj/tensor/ComputeGraphTest.java:546-591
does.  Each test cites the reference test it mirrors."""
import gc
import struct

import numpy as np
import pytest

from deepj_amd import ComputeGraph, GpuBuffer, HipBackend, Tensor, opcodes as op


class RecordingRuntime:
    def __init__(self):
        self.allocCalls, self.uploads, self.downloads, self.flushCalls, self.releaseCalls = [], [], [], [], []
        self.downloadResult = None

    def allocBuffers(self, ids, sizes, count):
        self.allocCalls.append((np.array(ids).copy(), np.array(sizes).copy(), count))

    def uploadBuffer(self, buf_id, data):
        self.uploads.append((buf_id, np.array(data).copy()))

    def downloadBuffer(self, buf_id, out):
        self.downloads.append(buf_id)
        if self.downloadResult is not None:
            n = min(len(self.downloadResult), out.size)
            out[:n] = self.downloadResult[:n]

    def releaseBuffers(self, ids, count):
        self.releaseCalls.append((np.array(ids).copy(), count))

    def flushOps(self, cmd, length):
        self.flushCalls.append((np.array(cmd[:length]).copy(), length))


@pytest.fixture
def rt():
    return RecordingRuntime()


@pytest.fixture
def graph(rt):
    return ComputeGraph(rt)


def bits(x):
    return struct.unpack("<i", struct.pack("<f", x))[0]


def test_constructor_rejects_null_and_new_graph_is_empty(graph):      # :21-30
    with pytest.raises(TypeError):
        ComputeGraph(None)
    assert graph.isEmpty()


def test_ensure_gpu_buffer_assigns_and_reuses(graph):                 # :34-52
    t = Tensor.from2D([[1, 2], [3, 4]])
    assert t.getGpuTag() is None
    buf = graph.ensureGpuBuffer(t)
    assert buf is t.getGpuTag() and (buf.rows, buf.cols) == (2, 2)
    assert graph.ensureGpuBuffer(t) is buf


def test_reupload_when_needs_upload(graph, rt):                       # :54-74
    t = Tensor.from2D([[1.0]])
    buf = graph.ensureGpuBuffer(t)
    buf.needsUpload = True
    t.data[0, 0] = 99.0
    graph.ensureGpuBuffer(t)
    assert not buf.needsUpload
    graph.flush()
    assert len(rt.uploads) == 2 and rt.uploads[1][1][0] == 99.0


def test_output_buffers(graph):                                       # :78-107
    buf = graph.newOutputBuffer(4, 8)
    assert buf.cpuStale and not buf.allocatedOnGpu and buf.floatCount() == 32
    a, b = graph.newOutputBuffer(1, 1), graph.newOutputBuffer(1, 1)
    assert b.id > a.id
    t = graph.createOutputTensor(graph.newOutputBuffer(3, 5))
    assert (t.rows, t.cols) == (3, 5) and isinstance(t.getGpuTag(), GpuBuffer)


def test_flush_on_empty_graph_is_noop_and_idempotent(graph, rt):      # :176-183,224-231
    for _ in range(3):
        graph.flush()
    assert not rt.allocCalls and not rt.uploads and not rt.flushCalls


def test_flush_allocates_uploads_executes_in_that_order(graph, rt):   # :185-210
    t = Tensor.from2D([[1, 2], [3, 4]])
    inp = graph.ensureGpuBuffer(t)
    out = graph.newOutputBuffer(2, 2)
    graph.recordUnary(op.OP_NEG, inp, out)
    graph.flush()
    assert len(rt.allocCalls) == 1 and list(rt.allocCalls[0][0]) == [inp.id, out.id]
    assert list(rt.allocCalls[0][1]) == [4, 4]
    assert len(rt.uploads) == 1 and rt.uploads[0][0] == inp.id
    assert len(rt.flushCalls) == 1
    assert list(rt.flushCalls[0][0]) == [op.OP_NEG, inp.id, out.id, 4]
    assert graph.isEmpty()                                            # :212-222


def test_second_flush_only_executes_new_ops(graph, rt):               # :233-253
    t = Tensor.from2D([[1]])
    inp = graph.ensureGpuBuffer(t)
    graph.recordUnary(op.OP_SQRT, inp, graph.newOutputBuffer(1, 1))
    graph.flush()
    graph.recordUnary(op.OP_NEG, inp, graph.newOutputBuffer(1, 1))
    graph.flush()
    assert len(rt.allocCalls) == 2 and len(rt.flushCalls) == 2 and len(rt.uploads) == 1


def test_cmd_stream_grows_past_4096_ints(graph, rt):                  # :255-270
    a, b = graph.newOutputBuffer(2, 2), graph.newOutputBuffer(2, 2)
    for _ in range(1000):
        graph.recordBinary(op.OP_ADD, a, b, graph.newOutputBuffer(2, 2))
    graph.flush()
    assert len(rt.flushCalls) == 1 and rt.flushCalls[0][1] == 5000


def test_materialize_flushes_and_downloads_once(graph, rt):           # :274-333
    inp = graph.ensureGpuBuffer(Tensor.from2D([[2.0, 4.0]]))
    out = graph.newOutputBuffer(1, 2)
    graph.recordUnary(op.OP_SQRT, inp, out)
    result = graph.createOutputTensor(out)
    rt.downloadResult = [1.414, 2.0]
    graph.materialize(result)
    assert len(rt.flushCalls) == 1 and rt.downloads == [out.id]
    assert abs(result.data[0, 0] - 1.414) < 1e-3 and not out.cpuStale
    graph.materialize(result)
    assert len(rt.downloads) == 1
    graph.materialize(Tensor(2, 2))                                   # no GPU tag: no-op
    assert len(rt.downloads) == 1


def test_release_all_releases_resets_and_restarts_ids(graph, rt):     # :337-359,477-486
    t = Tensor.from2D([[1, 2]])
    graph.ensureGpuBuffer(t)
    graph.recordUnary(op.OP_NEG, graph.ensureGpuBuffer(t), graph.newOutputBuffer(1, 2))
    graph.releaseAll()
    assert len(rt.releaseCalls) == 1 and graph.isEmpty() and t.getGpuTag() is None
    assert graph.ensureGpuBuffer(Tensor.from2D([[9]])).id == 0
    g2 = ComputeGraph(RecordingRuntime())
    g2.releaseAll()
    assert not g2.runtime.releaseCalls


def test_release_all_materializes_stale_tracked_tensor(graph, rt):    # :392-408
    t = Tensor.from2D([[1.0]])
    buf = graph.ensureGpuBuffer(t)
    graph.flush()
    buf.cpuStale = True
    rt.downloadResult = [42.0]
    graph.releaseAll()
    assert t.data[0, 0] == 42.0 and t.getGpuTag() is None and not buf.cpuStale


def test_all_42_opcodes_are_distinct():                               # :362-390
    codes = list(op.REFERENCE_OPCODES.values())
    assert len(codes) == 42 and len(set(codes)) == 42 and sorted(codes) == list(range(1, 43))


def test_adamw_encodes_thirteen_ints(graph, rt):                      # :424-450
    w, g, mt, vt = (graph.newOutputBuffer(1, 4) for _ in range(4))
    graph.recordAdamWUpdate(w, g, mt, vt, 1e-3, 0.9, 0.999, 1e-8, 0.01, 0.9, 0.999, 4)
    graph.flush()
    stream, length = rt.flushCalls[0]
    assert length == 13
    assert list(stream) == [op.OP_ADAMW_UPDATE, w.id, g.id, mt.id, vt.id, bits(1e-3), bits(0.9), bits(0.999),
                            bits(1e-8), bits(0.01), bits(0.9), bits(0.999), 4]


def test_flush_marks_buffers_allocated_and_alloc_without_ops(graph, rt):   # :454-486
    t = Tensor.from2D([[1.0]])
    inp = graph.ensureGpuBuffer(t)
    out = graph.newOutputBuffer(1, 1)
    out_t = graph.createOutputTensor(out)
    assert not inp.allocatedOnGpu and not out.allocatedOnGpu
    graph.recordUnary(op.OP_NEG, inp, out)
    graph.flush()
    assert inp.allocatedOnGpu and out.allocatedOnGpu
    g2 = ComputeGraph(RecordingRuntime())
    g2.newOutputBuffer(2, 4)
    g2.flush()
    assert len(g2.runtime.allocCalls) == 1 and not g2.runtime.flushCalls
    del out_t


def test_orphaned_buffers_are_released_on_flush(graph, rt):           # :488-527
    t = Tensor.from2D([[1.0]])
    old = graph.ensureGpuBuffer(t)
    graph.flush()
    t.setGpuTag(graph.newOutputBuffer(1, 1))
    graph.flush()
    assert old.id in list(rt.releaseCalls[-1][0])
    t2 = Tensor.from2D([[2.0]])
    b2 = graph.ensureGpuBuffer(t2)
    graph.flush()
    t2.setGpuTag(None)
    n = len(rt.releaseCalls)
    graph.flush()
    assert len(rt.releaseCalls) == n + 1 and b2.id in list(rt.releaseCalls[-1][0])
    # a tensor that was garbage collected orphans its buffer too (WeakReference semantics)
    t3 = Tensor.from2D([[3.0]])
    b3 = graph.ensureGpuBuffer(t3).id
    graph.flush()
    del t3
    gc.collect()
    graph.flush()
    assert b3 in list(rt.releaseCalls[-1][0])


# ── HipBackend on top of the recording runtime: op -> stream mapping ─────────

def test_backend_records_reference_encodings(rt):
    be = HipBackend(rt)
    Tensor.setBackend(be)
    a, b = Tensor.from2D([[1, 2, 3], [4, 5, 6]]), Tensor.from2D([[7, 8], [9, 10], [11, 12]])
    c = be.matmul(a, b)
    d = c.multiplyScalar(0.5).addRowVector(Tensor.from2D([[1, 1]]))
    d.clamp(-1.0, 1.0)
    be.graph.flush()
    s = list(rt.flushCalls[0][0])
    ga, gb, gc_ = a.getGpuTag().id, b.getGpuTag().id, c.getGpuTag().id
    assert s[:7] == [op.OP_MATMUL, ga, gb, gc_, 2, 2, 3]              # [op,a,b,out,m,n,k]
    assert s[7] == op.OP_MULTIPLY_SCALAR and s[10] == bits(0.5) and s[11] == 4
    assert s[12] == op.OP_ADD_ROW_VECTOR and s[16:18] == [2, 2]
    assert s[18] == op.OP_CLAMP and s[21:24] == [bits(-1.0), bits(1.0), 4]


def test_backend_in_place_rebinds_to_new_buffer_and_releases_old(rt):  # MetalBackend.java:400-411
    be = HipBackend(rt)
    Tensor.setBackend(be)
    a, b = Tensor.from2D([[1.0, 2.0]]), Tensor.from2D([[3.0, 4.0]])
    be.graph.ensureGpuBuffer(a)
    old = a.getGpuTag().id
    a.addInPlace(b)
    assert a.getGpuTag().id != old and a.getGpuTag().cpuStale
    be.graph.flush()
    be.graph.flush()
    assert any(old in list(ids) for ids, _ in rt.releaseCalls)


def test_backend_shape_errors_before_recording(rt):                   # MetalBackendTest.java:80-86,271-276,315-323,364-372
    be = HipBackend(rt)
    Tensor.setBackend(be)
    with pytest.raises(ValueError, match="Shape mismatch"):
        be.matmul(Tensor(3, 4), Tensor(5, 2))
    with pytest.raises(ValueError, match="Shape mismatch"):
        be.softmaxBackward(Tensor(2, 3), Tensor(3, 2))
    with pytest.raises(ValueError, match="layerNormBackward: std"):
        be.layerNormBackward(Tensor(4, 8), Tensor(4, 8), Tensor(4, 2), 8)
    with pytest.raises(ValueError, match="targets length"):
        be.crossEntropyGradient(Tensor(4, 8), [0, 1, 2])
    assert be.graph.isEmpty()


def test_int_targets_travel_as_float_column(rt):                      # MetalBackend.java:43-54,531-539
    be = HipBackend(rt)
    Tensor.setBackend(be)
    be.crossEntropyGradient(Tensor(3, 5), [4, 0, 2])
    be.graph.flush()
    cols = [d for _, d in rt.uploads if d.size == 3]
    assert len(cols) == 1 and list(cols[0]) == [4.0, 0.0, 2.0]
    s = list(rt.flushCalls[0][0])
    assert s[0] == op.OP_CROSS_ENTROPY_GRADIENT and s[4:6] == [3, 5]
