package io.github.kirstenali.deepj.tensor.hip;

import io.github.kirstenali.deepj.tensor.ComputeGraph;
import io.github.kirstenali.deepj.tensor.GpuBuffer;
import io.github.kirstenali.deepj.tensor.Tensor;
import io.github.kirstenali.deepj.tensor.TensorBackend;

import java.util.HashMap;
import java.util.Map;

import static io.github.kirstenali.deepj.tensor.ComputeGraph.*;

/**
 * TensorBackend for AMD MI355X (gfx950) GPUs.
 *
 * <p>Drop-in: {@code Tensor.setBackend(new HipBackend())}. Every operation is recorded lazily
 * into a private {@link ComputeGraph}; the graph is flushed to the HIP runtime as one int32
 * command stream when a tensor is materialised. Tensors stay resident in HBM between flushes.
 * "In-place" operations write a fresh buffer and rebind the tensor to it; the old buffer is
 * released by the graph's orphan scan and recycled by the native pool, so no device allocation
 * happens in steady state.
 */
public final class HipBackend implements TensorBackend {

    private final ComputeGraph graph;
    private final Map<Integer, Tensor> indexColumns = new HashMap<>();

    public HipBackend() {
        this.graph = new ComputeGraph(new HipGpuRuntime());
    }

    // ── plumbing ─────────────────────────────────────────────────────────

    private GpuBuffer in(Tensor t) {
        return graph.ensureGpuBuffer(t);
    }

    private GpuBuffer fresh(int rows, int cols) {
        return graph.newOutputBuffer(rows, cols);
    }

    private Tensor wrap(GpuBuffer out) {
        return graph.createOutputTensor(out);
    }

    private static void stale(GpuBuffer b) {
        b.cpuStale = true;
        b.needsUpload = false;
    }

    private static void rowVector(Tensor v, Tensor a) {
        if (v.rows != 1 || v.cols != a.cols)
            throw new IllegalArgumentException("Expected row vector 1x" + a.cols + " but got " + v.rows + "x" + v.cols);
    }

    private static void colVector(Tensor v, Tensor a) {
        if (v.rows != a.rows || v.cols != 1)
            throw new IllegalArgumentException("Expected col vector " + a.rows + "x1 but got " + v.rows + "x" + v.cols);
    }

    /** Integer targets / indices travel to the device as a float column tensor. */
    private Tensor indexColumn(int[] values) {
        Tensor t = indexColumns.computeIfAbsent(values.length, n -> new Tensor(n, 1));
        for (int i = 0; i < values.length; i++) t.data[i] = values[i];
        if (t.getGpuTag() instanceof GpuBuffer gb) {
            gb.needsUpload = true;
            gb.cpuStale = false;
        }
        return t;
    }

    // ── op families ──────────────────────────────────────────────────────

    private GpuBuffer binary(int op, String name, Tensor a, Tensor b) {
        Tensor.requireSameShape(a, b, name);
        GpuBuffer ga = in(a), gb = in(b), out = fresh(a.rows, a.cols);
        graph.recordBinary(op, ga, gb, out);
        return out;
    }

    private GpuBuffer unary(int op, Tensor a) {
        GpuBuffer ga = in(a), out = fresh(a.rows, a.cols);
        graph.recordUnary(op, ga, out);
        return out;
    }

    private GpuBuffer scalar(int op, Tensor a, float s) {
        GpuBuffer ga = in(a), out = fresh(a.rows, a.cols);
        if (op == OP_MULTIPLY_SCALAR) graph.recordMultiplyScalar(ga, out, s);
        else graph.recordScalarUnary(op, ga, out, s);
        return out;
    }

    private Tensor rowBroadcast(int op, Tensor a, Tensor v) {
        rowVector(v, a);
        GpuBuffer ga = in(a), gv = in(v), out = fresh(a.rows, a.cols);
        graph.recordRowBroadcast(op, ga, gv, out, a.rows, a.cols);
        return wrap(out);
    }

    private Tensor colBroadcast(int op, Tensor a, Tensor v) {
        colVector(v, a);
        GpuBuffer ga = in(a), gv = in(v), out = fresh(a.rows, a.cols);
        graph.recordColBroadcast(op, ga, gv, out, a.rows, a.cols);
        return wrap(out);
    }

    private Tensor reduce(int op, Tensor a, int outRows, int outCols) {
        GpuBuffer ga = in(a), out = fresh(outRows, outCols);
        graph.recordReduction(op, ga, out, a.rows, a.cols);
        return wrap(out);
    }

    private void rebind(Tensor target, GpuBuffer out) {
        graph.bindTensorToBuffer(target, out);
    }

    // ── TensorBackend ────────────────────────────────────────────────────

    @Override public void materializeTensor(Tensor t) { graph.materialize(t); }

    @Override public void releaseResources() { graph.releaseAll(); indexColumns.clear(); }

    @Override
    public Tensor matmul(Tensor a, Tensor b) {
        if (a.cols != b.rows)
            throw new IllegalArgumentException("Shape mismatch for matmul: " + a.rows + "x" + a.cols + " vs " + b.rows + "x" + b.cols);
        GpuBuffer ga = in(a), gb = in(b), out = fresh(a.rows, b.cols);
        graph.recordMatmul(ga, gb, out, a.rows, b.cols, a.cols);
        return wrap(out);
    }

    @Override public Tensor add(Tensor a, Tensor b)      { return wrap(binary(OP_ADD, "add", a, b)); }
    @Override public Tensor subtract(Tensor a, Tensor b) { return wrap(binary(OP_SUBTRACT, "subtract", a, b)); }
    @Override public Tensor multiply(Tensor a, Tensor b) { return wrap(binary(OP_MULTIPLY, "multiply", a, b)); }
    @Override public Tensor divide(Tensor a, Tensor b)   { return wrap(binary(OP_DIVIDE, "divide", a, b)); }

    @Override public Tensor addRowVector(Tensor a, Tensor v)          { return rowBroadcast(OP_ADD_ROW_VECTOR, a, v); }
    @Override public Tensor addBroadcastRows(Tensor a, Tensor v)      { return addRowVector(a, v); }
    @Override public Tensor multiplyBroadcastRows(Tensor a, Tensor v) { return rowBroadcast(OP_MULTIPLY_BROADCAST_ROWS, a, v); }
    @Override public Tensor addBroadcastCols(Tensor a, Tensor v)      { return colBroadcast(OP_ADD_BROADCAST_COLS, a, v); }
    @Override public Tensor subtractBroadcastCols(Tensor a, Tensor v) { return colBroadcast(OP_SUBTRACT_BROADCAST_COLS, a, v); }
    @Override public Tensor divideBroadcastCols(Tensor a, Tensor v)   { return colBroadcast(OP_DIVIDE_BROADCAST_COLS, a, v); }
    @Override public Tensor multiplyBroadcastCols(Tensor a, Tensor v) { return colBroadcast(OP_MULTIPLY_BROADCAST_COLS, a, v); }

    @Override public Tensor multiplyScalar(Tensor a, float s) { return wrap(scalar(OP_MULTIPLY_SCALAR, a, s)); }
    @Override public Tensor addScalar(Tensor a, float s)      { return wrap(scalar(OP_ADD_SCALAR, a, s)); }
    @Override public Tensor divideScalar(Tensor a, float s)   { return wrap(scalar(OP_DIVIDE_SCALAR, a, s)); }

    @Override public Tensor sumRows(Tensor a)           { return reduce(OP_SUM_ROWS, a, 1, a.cols); }
    @Override public Tensor sumAlongCols(Tensor a)      { return sumRows(a); }
    @Override public Tensor sumAlongRows(Tensor a)      { return reduce(OP_SUM_ALONG_ROWS, a, a.rows, 1); }
    @Override public Tensor meanAlongRows(Tensor a)     { return reduce(OP_MEAN_ALONG_ROWS, a, a.rows, 1); }
    @Override public Tensor varianceAlongRows(Tensor a) { return reduce(OP_VARIANCE_ALONG_ROWS, a, a.rows, 1); }
    @Override public Tensor maxAlongRows(Tensor a)      { return reduce(OP_MAX_ALONG_ROWS, a, a.rows, 1); }

    @Override
    public float sum(Tensor a) {
        GpuBuffer ga = in(a), out = fresh(1, 1);
        graph.recordSumScalar(ga, out, a.rows, a.cols);
        Tensor s = wrap(out);
        s.materialize();
        return s.data[0];
    }

    @Override
    public float sumAbs(Tensor a) {
        GpuBuffer ga = in(a), perRow = fresh(a.rows, 1);
        graph.recordSumAbs(ga, perRow, a.rows, a.cols);
        Tensor s = sumRows(wrap(perRow));
        s.materialize();
        return s.data[0];
    }

    @Override
    public Tensor transpose(Tensor a) {
        GpuBuffer ga = in(a), out = fresh(a.cols, a.rows);
        graph.recordTranspose(ga, out, a.rows, a.cols);
        return wrap(out);
    }

    @Override
    public Tensor clamp(Tensor a, float min, float max) {
        GpuBuffer ga = in(a), out = fresh(a.rows, a.cols);
        graph.recordClamp(ga, out, min, max);
        return wrap(out);
    }

    @Override
    public Tensor pow(Tensor a, float exponent) {
        GpuBuffer ga = in(a), out = fresh(a.rows, a.cols);
        graph.recordPow(ga, out, exponent);
        return wrap(out);
    }

    @Override public Tensor sqrt(Tensor a)    { return wrap(unary(OP_SQRT, a)); }
    @Override public Tensor neg(Tensor a)     { return wrap(unary(OP_NEG, a)); }
    @Override public Tensor exp(Tensor a)     { return wrap(unary(OP_EXP, a)); }
    @Override public Tensor log(Tensor a)     { return wrap(unary(OP_LOG, a)); }
    @Override public Tensor tanh(Tensor a)    { return wrap(unary(OP_TANH, a)); }
    @Override public Tensor sigmoid(Tensor a) { return wrap(unary(OP_SIGMOID, a)); }
    @Override public Tensor relu(Tensor a)    { return wrap(unary(OP_RELU, a)); }
    @Override public Tensor gelu(Tensor a)    { return wrap(unary(OP_GELU, a)); }

    @Override public Tensor reluBackward(Tensor x, Tensor g) { return wrap(binary(OP_RELU_BACKWARD, "reluBackward", x, g)); }
    @Override public Tensor geluBackward(Tensor x, Tensor g) { return wrap(binary(OP_GELU_BACKWARD, "geluBackward", x, g)); }

    @Override
    public Tensor softmaxRows(Tensor logits) {
        GpuBuffer ga = in(logits), out = fresh(logits.rows, logits.cols);
        graph.recordSoftmaxRows(ga, out, logits.rows, logits.cols);
        return wrap(out);
    }

    @Override
    public Tensor softmaxBackward(Tensor gradOutput, Tensor softmaxOut) {
        Tensor.requireSameShape(gradOutput, softmaxOut, "softmaxBackward");
        GpuBuffer gg = in(gradOutput), gs = in(softmaxOut), out = fresh(gradOutput.rows, gradOutput.cols);
        graph.recordSoftmaxBackward(gg, gs, out, gradOutput.rows, gradOutput.cols);
        return wrap(out);
    }

    // in-place family: compute into a new buffer, then point the tensor at it
    @Override public void addInPlace(Tensor a, Tensor b)      { rebind(a, binary(OP_ADD, "addInPlace", a, b)); }
    @Override public void subtractInPlace(Tensor a, Tensor b) { rebind(a, binary(OP_SUBTRACT, "subtractInPlace", a, b)); }
    @Override public void multiplyInPlace(Tensor a, Tensor b) { rebind(a, binary(OP_MULTIPLY, "multiplyInPlace", a, b)); }
    @Override public void divideInPlace(Tensor a, Tensor b)   { rebind(a, binary(OP_DIVIDE, "divideInPlace", a, b)); }
    @Override public void multiplyScalarInPlace(Tensor a, float s) { rebind(a, scalar(OP_MULTIPLY_SCALAR, a, s)); }
    @Override public void addScalarInPlace(Tensor a, float s)      { rebind(a, scalar(OP_ADD_SCALAR, a, s)); }
    @Override public void divideScalarInPlace(Tensor a, float s)   { rebind(a, scalar(OP_DIVIDE_SCALAR, a, s)); }
    @Override public void sqrtInPlace(Tensor a)    { rebind(a, unary(OP_SQRT, a)); }
    @Override public void negInPlace(Tensor a)     { rebind(a, unary(OP_NEG, a)); }
    @Override public void expInPlace(Tensor a)     { rebind(a, unary(OP_EXP, a)); }
    @Override public void logInPlace(Tensor a)     { rebind(a, unary(OP_LOG, a)); }
    @Override public void reluInPlace(Tensor a)    { rebind(a, unary(OP_RELU, a)); }
    @Override public void geluInPlace(Tensor a)    { rebind(a, unary(OP_GELU, a)); }
    @Override public void tanhInPlace(Tensor a)    { rebind(a, unary(OP_TANH, a)); }
    @Override public void sigmoidInPlace(Tensor a) { rebind(a, unary(OP_SIGMOID, a)); }

    @Override
    public Tensor crossEntropyGradient(Tensor logits, int[] targets) {
        Tensor.requireTargetsMatchRows(logits, targets);
        GpuBuffer gl = in(logits), gt = in(indexColumn(targets)), out = fresh(logits.rows, logits.cols);
        graph.recordCrossEntropyGradient(gl, gt, out, logits.rows, logits.cols);
        return wrap(out);
    }

    @Override
    public float crossEntropyLoss(Tensor logits, int[] targets) {
        Tensor.requireTargetsMatchRows(logits, targets);
        GpuBuffer gl = in(logits), gt = in(indexColumn(targets)), perRow = fresh(logits.rows, 1);
        graph.recordCrossEntropyLoss(gl, gt, perRow, logits.rows, logits.cols);
        Tensor mean = sumRows(wrap(perRow)).divideScalar(logits.rows);
        mean.materialize();
        return mean.data[0];
    }

    @Override
    public void adamWUpdate(Tensor w, Tensor g, Tensor mt, Tensor vt, float lr, float beta1, float beta2,
                            float eps, float weightDecay, float bc1, float bc2) {
        Tensor.requireSameShape(w, g, "adamWUpdate");
        Tensor.requireSameShape(w, mt, "adamWUpdate");
        Tensor.requireSameShape(w, vt, "adamWUpdate");
        GpuBuffer gw = in(w), gg = in(g), gm = in(mt), gv = in(vt);
        graph.recordAdamWUpdate(gw, gg, gm, gv, lr, beta1, beta2, eps, weightDecay, bc1, bc2, w.rows * w.cols);
        stale(gw);
        stale(gm);
        stale(gv);
    }

    @Override
    public Tensor layerNormBackward(Tensor dXHat, Tensor xHat, Tensor std, int dim) {
        Tensor.requireSameShape(dXHat, xHat, "layerNormBackward");
        if (dim != dXHat.cols)
            throw new IllegalArgumentException("layerNormBackward: dim=" + dim + " must equal tensor cols=" + dXHat.cols);
        if (std.rows != dXHat.rows || std.cols != 1)
            throw new IllegalArgumentException("layerNormBackward: std must be " + dXHat.rows + "x1 but got " + std.rows + "x" + std.cols);
        GpuBuffer gd = in(dXHat), gx = in(xHat), gs = in(std), out = fresh(dXHat.rows, dXHat.cols);
        graph.recordLayerNormBackward(gd, gx, gs, out, dXHat.rows, dXHat.cols);
        return wrap(out);
    }

    @Override
    public void scatterAddRows(Tensor target, int[] indices, Tensor grad) {
        if (indices.length != grad.rows)
            throw new IllegalArgumentException("scatterAddRows: indices length " + indices.length + " must match grad rows " + grad.rows);
        if (target.cols != grad.cols)
            throw new IllegalArgumentException("scatterAddRows: target cols " + target.cols + " must match grad cols " + grad.cols);
        if (indices.length == 0) return;
        GpuBuffer gt = in(target), gg = in(grad), gi = in(indexColumn(indices));
        graph.recordScatterAddRowsAtomic(gt, gi, gg, target.rows, target.cols, indices.length);
        stale(gt);
    }
}
