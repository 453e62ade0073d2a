"""GPU-vs-CPU differential tests of the 42 primitive opcodes through HipBackend ->
ComputeGraph -> C ABI -> HIP kernels, against the CPU oracle on the same seeded inputs.
Shapes, seeds and tolerances follow the reference's own GPU test
src/test/java/io/github/kirstenali/deepj/tensor/metal/MetalBackendTest.java (cited per test);
where that test loosened a tolerance "because fast-math exp", this one does not have to."""
import numpy as np
import pytest

from deepj_amd import HipNative, Tensor
from deepj_amd import opcodes as op
from oracle import cpu_ref as ref
from gpu_util import assert_close, backend, rnd, tensor

pytestmark = pytest.mark.gpu


def test_native_is_available():                                       # :41-44
    assert HipNative.available()


def test_small_matmul_matches_expected_values():                      # :46-68
    with backend() as be:
        c = be.matmul(tensor([[1, 2, 3], [4, 5, 6]]), tensor([[7, 8], [9, 10], [11, 12]]))
        assert (c.rows, c.cols) == (2, 2)
        assert_close([[58, 64], [139, 154]], c, atol=1e-6, rtol=0)


@pytest.mark.parametrize("m,k,n", [(128, 192, 64), (1, 2048, 513), (65, 33, 127), (200, 513, 70), (3, 1, 5),
                                   (1100, 257, 2050), (1536, 64, 1537)])       # large enough for the 128 x 128 tile, ragged
def test_matmul_matches_cpu(m, k, n):                                 # :70-78 (+ ragged shapes)
    a, b = rnd(m, k, 1), rnd(k, n, 2)
    with backend() as be:
        assert_close(ref.matmul(a, b), be.matmul(tensor(a), tensor(b)), 1e-4, 1e-4, f"matmul {m}x{k}x{n}")


def test_matmul_rejects_shape_mismatch():                             # :80-86
    with backend() as be:
        with pytest.raises(ValueError, match="Shape mismatch"):
            be.matmul(tensor(rnd(3, 4, 3)), tensor(rnd(5, 2, 4)))


def test_elementwise_binary_ops():
    a, b = rnd(37, 53, 5), rnd(37, 53, 6) + 0.5
    with backend() as be:
        ta, tb = tensor(a), tensor(b)
        assert_close(ref.add(a, b), be.add(ta, tb), 1e-6, 1e-6)
        assert_close(ref.subtract(a, b), be.subtract(ta, tb), 1e-6, 1e-6)
        assert_close(ref.multiply(a, b), be.multiply(ta, tb), 1e-6, 1e-6)
        assert_close(ref.divide(a, b), be.divide(ta, tb), 1e-6, 1e-6)


def test_broadcast_and_scalar_ops_match_cpu():                        # :88-113
    a, row, col = rnd(8, 16, 100), rnd(1, 16, 101), rnd(8, 1, 102)
    with backend() as be:
        ta, tr, tc = tensor(a), tensor(row), tensor(col)
        assert_close(ref.add_row_vector(a, row), be.addRowVector(ta, tr))
        assert_close(ref.add_broadcast_cols(a, col), be.addBroadcastCols(ta, tc))
        assert_close(ref.subtract_broadcast_cols(a, col), be.subtractBroadcastCols(ta, tc))
        assert_close(ref.divide_broadcast_cols(a, col), be.divideBroadcastCols(ta, tc))
        assert_close(ref.multiply_broadcast_cols(a, col), be.multiplyBroadcastCols(ta, tc))
        assert_close(ref.multiply_broadcast_rows(a, row), be.multiplyBroadcastRows(ta, tr))
        assert_close(ref.add_scalar(a, 0.25), be.addScalar(ta, 0.25))
        assert_close(ref.divide_scalar(a, 1.5), be.divideScalar(ta, 1.5))
        assert_close(ref.multiply_scalar(a, -2.5), be.multiplyScalar(ta, -2.5))


@pytest.mark.parametrize("rows,cols", [(32, 24), (29, 513), (5, 2048), (1, 1)])
def test_reductions_and_transpose_match_cpu(rows, cols):              # :115-135 (+ wide rows :222-233)
    a = rnd(rows, cols, 111)
    with backend() as be:
        ta = tensor(a)
        assert_close(ref.transpose(a), be.transpose(ta))
        assert_close(ref.sum_rows(a), be.sumRows(ta))
        assert_close(ref.sum_along_rows(a), be.sumAlongRows(ta))
        assert_close(ref.sum_along_cols(a), be.sumAlongCols(ta))
        assert_close(ref.mean_along_rows(a), be.meanAlongRows(ta))
        assert_close(ref.variance_along_rows(a), be.varianceAlongRows(ta))
        assert_close(ref.max_along_rows(a), be.maxAlongRows(ta), 0, 0)
        # whole-tensor fp32 sums: the CPU's sequential sum itself carries ~n*eps relative error
        assert abs(ref.sum_(a) - be.sum(ta)) <= 1e-4 + 1e-5 * ref.sum_abs(a)
        assert abs(ref.sum_abs(a) - be.sumAbs(ta)) <= 1e-4 + 1e-5 * ref.sum_abs(a)


def test_unary_math_and_activations():
    a = rnd(19, 33, 7) * 10.0
    pos = np.abs(a) + 0.01
    with backend() as be:
        ta, tp = tensor(a), tensor(pos)
        assert_close(ref.sqrt(pos), be.sqrt(tp), 0, 1e-7)
        assert_close(ref.neg(a), be.neg(ta), 0, 0)
        assert_close(ref.exp(a), be.exp(ta), 0, 2e-7)
        assert_close(ref.log(pos), be.log(tp), 1e-7, 2e-7)
        assert_close(ref.tanh(a), be.tanh(ta), 1e-7, 2e-7)
        assert_close(ref.sigmoid(a), be.sigmoid(ta), 1e-7, 2e-7)
        assert_close(ref.relu(a), be.relu(ta), 0, 0)
        assert_close(ref.gelu(a), be.gelu(ta), 1e-6, 1e-6)
        g = rnd(19, 33, 8)
        assert_close(ref.relu_backward(a, g), be.reluBackward(ta, tensor(g)), 0, 0)
        assert_close(ref.gelu_backward(a, g), be.geluBackward(ta, tensor(g)), 1e-6, 1e-6)


def test_softmax_rows_matches_cpu_and_sums_to_one():
    for rows, cols, seed in [(32, 64, 11), (17, 769, 13), (3, 5000, 14)]:
        x = rnd(rows, cols, seed) * 20.0
        with backend() as be:
            p = be.softmaxRows(tensor(x)).numpy()
        assert_close(ref.softmax_rows(x), p, 1e-7, 1e-5)
        assert np.allclose(p.sum(1), 1.0, atol=1e-5)


def test_max_clamp_pow_and_scatter_add_rows_match_cpu():              # :137-172
    a = rnd(16, 20, 121)
    with backend() as be:
        ta = tensor(a)
        assert_close(ref.max_along_rows(a), be.maxAlongRows(ta))
        assert_close(ref.clamp(a, -0.25, 0.35), be.clamp(ta, -0.25, 0.35), 0, 0)
        assert_close(ref.pow_(a, 2.0), be.pow(ta, 2.0))
        for idx, ts, gs, tol in [([3, 1, 7, 2, 4, 5], 122, 123, 1e-4), ([3, 1, 7, 1, 4, 3], 124, 125, 1e-3)]:
            target_cpu = rnd(10, 8, ts)
            target_gpu = tensor(target_cpu)
            grad = rnd(6, 8, gs)
            ref.scatter_add_rows(target_cpu, idx, grad)
            Tensor.scatterAddRows(target_gpu, idx, tensor(grad))
            assert_close(target_cpu, target_gpu, tol, tol)


def test_scatter_add_rows_many_duplicates():                          # :174-197
    target_cpu = rnd(64, 32, 129)
    grad = rnd(128, 32, 130)
    idx = ref.JavaRandom(131).ints(128, 64)
    with backend():
        target_gpu = tensor(target_cpu)
        ref.scatter_add_rows(target_cpu, idx, grad)
        Tensor.scatterAddRows(target_gpu, list(idx), tensor(grad))
        assert_close(target_cpu, target_gpu, 1e-3, 1e-3)


def test_scalar_sum_abs_and_cross_entropy_loss_match_cpu():           # :199-238
    with backend() as be:
        a = rnd(23, 17, 126)
        assert abs(ref.sum_abs(a) - be.sumAbs(tensor(a))) <= 1e-4
        for rows, cols, ls, ts, tol in [(19, 31, 127, 128, 1e-4), (23, 777, 133, 134, 1e-3)]:
            logits = rnd(rows, cols, ls)
            targets = list(ref.JavaRandom(ts).ints(rows, cols))
            assert abs(ref.cross_entropy_loss(logits, targets) - be.crossEntropyLoss(tensor(logits), targets)) <= tol
        wide = rnd(29, 513, 132)
        assert abs(ref.sum_abs(wide) - be.sumAbs(tensor(wide))) <= 1e-3 + 1e-5 * ref.sum_abs(wide)


def test_softmax_backward_matches_cpu():                              # :240-266
    with backend() as be:
        for rows, cols, s1, s2 in [(32, 64, 10, 11), (17, 769, 12, 13)]:
            g, sm = rnd(rows, cols, s1), ref.softmax_rows(rnd(rows, cols, s2))
            assert_close(ref.softmax_backward(g, sm), be.softmaxBackward(tensor(g), tensor(sm)))
        with pytest.raises(ValueError, match="Shape mismatch"):       # :268-276
            be.softmaxBackward(tensor(rnd(2, 3, 21)), tensor(rnd(3, 2, 22)))


def test_layer_norm_backward_matches_cpu():                           # :278-323
    with backend() as be:
        for rows, cols, s1, s2 in [(16, 32, 31, 32), (11, 777, 33, 34)]:
            d, xh = rnd(rows, cols, s1), rnd(rows, cols, s2)
            std = (0.5 + np.abs(xh[:, :1])).astype(np.float32)
            assert_close(ref.layer_norm_backward(d, xh, std, cols),
                         be.layerNormBackward(tensor(d), tensor(xh), tensor(std), cols))
        with pytest.raises(ValueError, match="layerNormBackward: std"):
            be.layerNormBackward(tensor(rnd(4, 8, 41)), tensor(rnd(4, 8, 42)), tensor(rnd(4, 2, 43)), 8)


def test_cross_entropy_gradient_matches_cpu():                        # :325-372, at 1e-4 instead of 1e-3/1e-2
    with backend() as be:
        for rows, cols, ls, ts in [(32, 64, 51, 52), (17, 769, 53, 54)]:
            logits = rnd(rows, cols, ls)
            targets = list(ref.JavaRandom(ts).ints(rows, cols))
            assert_close(ref.cross_entropy_gradient(logits, targets),
                         be.crossEntropyGradient(tensor(logits), targets), 1e-6, 1e-4)
        with pytest.raises(ValueError, match="targets length"):
            be.crossEntropyGradient(tensor(rnd(4, 8, 61)), [0, 1, 2])


def test_cross_entropy_bad_target_gives_nan_not_a_fault():            # deepj_metal_jni.mm:472-476,497-503
    with backend() as be:
        g = be.crossEntropyGradient(tensor(rnd(2, 5, 1)), [1, 7]).numpy()
        assert np.all(np.isfinite(g[0])) and np.all(np.isnan(g[1]))


def test_adamw_update_matches_cpu_single_and_multiple_steps():        # :374-450
    lr, b1, b2, eps, wd = 1e-3, 0.9, 0.999, 1e-8, 0.01
    with backend() as be:
        w_cpu, g = rnd(32, 64, 71), rnd(32, 64, 72)
        mt_cpu, vt_cpu = np.zeros_like(w_cpu), np.zeros_like(w_cpu)
        w_gpu, mt_gpu, vt_gpu = tensor(w_cpu), Tensor(32, 64), Tensor(32, 64)
        ref.adamw_update(w_cpu, g, mt_cpu, vt_cpu, lr, b1, b2, eps, wd, 1 - b1, 1 - b2)
        be.adamWUpdate(w_gpu, tensor(g), mt_gpu, vt_gpu, lr, b1, b2, eps, wd, 1 - b1, 1 - b2)
        assert_close(w_cpu, w_gpu); assert_close(mt_cpu, mt_gpu); assert_close(vt_cpu, vt_gpu)

        w_cpu = rnd(16, 48, 81)
        mt_cpu, vt_cpu = np.zeros_like(w_cpu), np.zeros_like(w_cpu)
        w_gpu, mt_gpu, vt_gpu = tensor(w_cpu), Tensor(16, 48), Tensor(16, 48)
        for step in range(1, 6):
            g = rnd(16, 48, 90 + step)
            bc1 = np.float32(1.0) - np.float32(np.power(np.float64(np.float32(b1)), step))
            bc2 = np.float32(1.0) - np.float32(np.power(np.float64(np.float32(b2)), step))
            ref.adamw_update(w_cpu, g, mt_cpu, vt_cpu, lr, b1, b2, eps, wd, float(bc1), float(bc2))
            be.adamWUpdate(w_gpu, tensor(g), mt_gpu, vt_gpu, lr, b1, b2, eps, wd, float(bc1), float(bc2))
        assert_close(w_cpu, w_gpu); assert_close(mt_cpu, mt_gpu); assert_close(vt_cpu, vt_gpu)


def test_in_place_ops_and_chained_lazy_graph():
    a, b = rnd(9, 11, 200), rnd(9, 11, 201)
    with backend():
        t = tensor(a)
        t.addInPlace(tensor(b)).multiplyScalarInPlace(0.5).sigmoidInPlace().negInPlace()
        exp = ref.neg(ref.sigmoid(ref.multiply_scalar(ref.add(a, b), 0.5)))
        assert_close(exp, t, 1e-7, 1e-6)
        t.set(0, 0, 3.0)                       # host write -> re-upload on next use (Tensor.java:213-217)
        exp[0, 0] = 3.0
        assert_close(ref.add_scalar(exp, 1.0), t.addScalar(1.0), 1e-7, 1e-6)


def test_rmsnorm_composition_of_six_primitives():                     # RMSNorm1D.java:46-57 through primitive ops
    x, gamma = rnd(7, 256, 300), 1.0 + rnd(1, 256, 301)
    with backend():
        tx = tensor(x)
        rms = tx.multiply(tx).meanAlongRows().addScalar(1e-6).sqrt()
        out = tx.divideBroadcastCols(rms).multiplyBroadcastRows(tensor(gamma))
        assert_close(ref.rmsnorm(x, gamma), out, 1e-6, 1e-5)


# ── the boundary's failure behaviour, forced from the host ───────────────────

def test_native_errors_surface_as_exceptions_and_runtime_survives():
    HipNative.init(0)
    with pytest.raises(RuntimeError, match="Unknown op code in graph: 63"):    # deepj_metal_jni.mm:2120-2121
        HipNative.nativeFlushOps(np.array([63, 0, 0, 0], np.int32), 4)
    with pytest.raises(RuntimeError, match="Buffer not found for upload"):     # :1512-1516
        HipNative.nativeUploadBuffer(123456, np.zeros(4, np.float32))
    with pytest.raises(RuntimeError, match="Buffer not found for download"):   # :1528-1532
        HipNative.nativeDownloadBuffer(123456, np.zeros(4, np.float32))
    with pytest.raises(RuntimeError, match="missing GPU buffer id=999"):       # :1404-1410
        HipNative.nativeFlushOps(np.array([1, 999, 998, 997, 4], np.int32), 5)
    HipNative.nativeAllocBuffers([900001, 900002], [4, 2], 2)
    try:
        with pytest.raises(RuntimeError, match="holds 2 floats, op needs 4"):  # host-side bounds check
            HipNative.nativeFlushOps(np.array([8, 900001, 900002, 4], np.int32), 4)
        with pytest.raises(RuntimeError, match="truncated"):
            HipNative.nativeFlushOps(np.array([5, 900001, 900001], np.int32), 3)
        HipNative.nativeAllocBuffers([900001], [1 << 20], 1)                    # existing id: no-op (:1489)
        HipNative.nativeUploadBuffer(900001, np.arange(4, dtype=np.float32))
        out = np.zeros(4, np.float32)
        HipNative.nativeDownloadBuffer(900001, out)
        assert list(out) == [0, 1, 2, 3]
    finally:
        HipNative.nativeReleaseBuffers([900001, 900002, 424242], 3)             # unknown id ignored (:1545-1547)
    with backend() as be:                                                       # still works afterwards
        assert_close([[3.0]], be.add(tensor([[1.0]]), tensor([[2.0]])), 0, 0)


def test_graph_replay_is_refused_once_a_captured_buffer_or_the_workspace_is_gone():
    """A captured graph replays raw device addresses: after a buffer it names is released (or re-created elsewhere),
    or after the workspace it used was replaced by a larger one, a launch must fail and run nothing."""
    from deepj_amd.fused import DeviceBuffers, Stream
    HipNative.init(0)
    dev = DeviceBuffers()
    try:
        a, out = dev.upload(np.arange(8, dtype=np.float32)), dev.alloc(8)
        add = Stream().emit(op.OP_ADD_SCALAR, a, out, np.float32(1.0).view(np.int32), 8).array()
        g1 = HipNative.graphCapture(add)
        HipNative.graphLaunch(g1, 2)
        assert list(dev.download(out, (8,))) == [1, 2, 3, 4, 5, 6, 7, 8]
        dev.write(out, np.zeros(8, np.float32))
        dev.release(a)
        with pytest.raises(RuntimeError, match="released or reallocated"):
            HipNative.graphLaunch(g1, 1)
        assert not dev.download(out, (8,)).any(), "a refused replay must launch nothing"
        HipNative.graphDestroy(g1)
        # a graph that uses the workspace (normalised rows of an M > 1 Q8_LINEAR), then a stream that needs a larger one
        m, k, n = 8, 64, 4
        x, gm, w, o = dev.alloc(m * k), dev.alloc(k), dev.alloc(HipNative.q8Floats(k, n)), dev.alloc(m * n)
        Stream().fill(x, 0, m * k).fill(gm, 0, k).fill(w, 0, HipNative.q8Floats(k, n)).run()
        g2 = HipNative.graphCapture(Stream().q8_linear(x, w, o, m, k, n, gamma=gm).array())
        HipNative.graphLaunch(g2, 1)
        big_m, big_k = 16384, 8192                   # 128 Mi floats of normalised rows: more than any other test's stream needs
        bx, bg, bw, bo = (dev.alloc(big_m * big_k), dev.alloc(big_k), dev.alloc(HipNative.q8Floats(big_k, n)),
                          dev.alloc(big_m * n))
        Stream().fill(bx, 0, big_m * big_k).fill(bg, 0, big_k).fill(bw, 0, HipNative.q8Floats(big_k, n)).run()
        Stream().q8_linear(bx, bw, bo, big_m, big_k, n, gamma=bg).run()
        with pytest.raises(RuntimeError, match="workspace was reallocated"):
            HipNative.graphLaunch(g2, 1)
        HipNative.graphDestroy(g2)
        # opcode 82 once named an op that was withdrawn: it is an unknown opcode like any other
        with pytest.raises(RuntimeError, match="Unknown op code in graph: 82"):
            HipNative.nativeFlushOps(np.array([82, 2], np.int32), 2)
    finally:
        dev.release_all()


def test_released_buffers_are_recycled_without_new_driver_allocations():
    with backend() as be:
        t = tensor(rnd(64, 64, 1))
        for _ in range(3):
            t.addScalarInPlace(1.0)
            t.materialize()
        before = HipNative.poolStats()["driver_allocs"]
        for _ in range(50):
            t.addScalarInPlace(1.0)
            t.materialize()
        after = HipNative.poolStats()
        assert after["driver_allocs"] == before, "in-place rebinding must reuse pooled blocks"
