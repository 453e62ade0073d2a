"""HipBackend: the TensorBackend of this library, a structural twin of the reference's
MetalBackend (src/main/java/io/github/kirstenali/deepj/tensor/metal/MetalBackend.java:8-633):
every op is recorded into a private ComputeGraph and nothing runs until a tensor is
materialised.  In-place ops get a new output buffer and rebind the tensor
(MetalBackend.java:400-411); ops that return a scalar materialise at once
(:247-266,541-555); integer targets and indices travel as float column tensors (:43-54).

HipGpuRuntime is the five-call pass-through to the native library
(cf. MetalGpuRuntime.java:9-35).
"""
from __future__ import annotations

import numpy as np

from . import opcodes as op
from ._native import HipNative
from .compute_graph import ComputeGraph, GpuBuffer
from .tensor import Tensor


class HipGpuRuntime:
    def allocBuffers(self, ids, sizes, count): HipNative.nativeAllocBuffers(ids, sizes, count)
    def uploadBuffer(self, buf_id, data): HipNative.nativeUploadBuffer(buf_id, data)
    def downloadBuffer(self, buf_id, out): HipNative.nativeDownloadBuffer(buf_id, out)
    def releaseBuffers(self, ids, count): HipNative.nativeReleaseBuffers(ids, count)
    def flushOps(self, cmd_stream, length): HipNative.nativeFlushOps(cmd_stream[:length], length)


def _require_row_vector(v, target):
    if v.rows != 1 or v.cols != target.cols:
        raise ValueError(f"Expected row vector 1x{target.cols} but got {v.rows}x{v.cols}")


def _require_col_vector(v, target):
    if v.rows != target.rows or v.cols != 1:
        raise ValueError(f"Expected col vector {target.rows}x1 but got {v.rows}x{v.cols}")


class HipBackend:
    def __init__(self, runtime=None):
        self.graph = ComputeGraph(runtime if runtime is not None else HipGpuRuntime())
        self._int_column_scratch: dict[int, Tensor] = {}

    # ── lazy helpers ────────────────────────────────────────────────────────
    def _in(self, t): return self.graph.ensureGpuBuffer(t)
    def _out(self, buf): return self.graph.createOutputTensor(buf)

    def _int_column(self, values) -> Tensor:
        t = self._int_column_scratch.get(len(values))
        if t is None:
            t = Tensor(len(values), 1)
            self._int_column_scratch[len(values)] = t
        t.data[:, 0] = np.asarray(values, dtype=np.float32)
        if isinstance(t.getGpuTag(), GpuBuffer):
            t.getGpuTag().needsUpload = True
            t.getGpuTag().cpuStale = False
        return t

    def materializeTensor(self, t): self.graph.materialize(t)

    def releaseResources(self):
        self.graph.releaseAll()
        self._int_column_scratch.clear()

    # ── matmul / element-wise ───────────────────────────────────────────────
    def matmul(self, a, b):
        if a.cols != b.rows:
            raise ValueError(f"Shape mismatch for matmul: {a.rows}x{a.cols} vs {b.rows}x{b.cols}")
        ga, gb = self._in(a), self._in(b)
        out = self.graph.newOutputBuffer(a.rows, b.cols)
        self.graph.recordMatmul(ga, gb, out, a.rows, b.cols, a.cols)
        return self._out(out)

    def _binary(self, opcode, name, a, b):
        Tensor.requireSameShape(a, b, name)
        ga, gb = self._in(a), self._in(b)
        out = self.graph.newOutputBuffer(a.rows, a.cols)
        self.graph.recordBinary(opcode, ga, gb, out)
        return out

    def add(self, a, b): return self._out(self._binary(op.OP_ADD, "add", a, b))
    def subtract(self, a, b): return self._out(self._binary(op.OP_SUBTRACT, "subtract", a, b))
    def multiply(self, a, b): return self._out(self._binary(op.OP_MULTIPLY, "multiply", a, b))
    def divide(self, a, b): return self._out(self._binary(op.OP_DIVIDE, "divide", a, b))
    def reluBackward(self, x, g): return self._out(self._binary(op.OP_RELU_BACKWARD, "reluBackward", x, g))
    def geluBackward(self, x, g): return self._out(self._binary(op.OP_GELU_BACKWARD, "geluBackward", x, g))

    # ── broadcasts ──────────────────────────────────────────────────────────
    def _row_bcast(self, opcode, a, v):
        _require_row_vector(v, a)
        ga, gv = self._in(a), self._in(v)
        out = self.graph.newOutputBuffer(a.rows, a.cols)
        self.graph.recordRowBroadcast(opcode, ga, gv, out, a.rows, a.cols)
        return self._out(out)

    def _col_bcast(self, opcode, a, v):
        _require_col_vector(v, a)
        ga, gv = self._in(a), self._in(v)
        out = self.graph.newOutputBuffer(a.rows, a.cols)
        self.graph.recordColBroadcast(opcode, ga, gv, out, a.rows, a.cols)
        return self._out(out)

    def addRowVector(self, a, v): return self._row_bcast(op.OP_ADD_ROW_VECTOR, a, v)
    def addBroadcastRows(self, a, v): return self.addRowVector(a, v)
    def multiplyBroadcastRows(self, a, v): return self._row_bcast(op.OP_MULTIPLY_BROADCAST_ROWS, a, v)
    def addBroadcastCols(self, a, v): return self._col_bcast(op.OP_ADD_BROADCAST_COLS, a, v)
    def subtractBroadcastCols(self, a, v): return self._col_bcast(op.OP_SUBTRACT_BROADCAST_COLS, a, v)
    def divideBroadcastCols(self, a, v): return self._col_bcast(op.OP_DIVIDE_BROADCAST_COLS, a, v)
    def multiplyBroadcastCols(self, a, v): return self._col_bcast(op.OP_MULTIPLY_BROADCAST_COLS, a, v)

    # ── scalar ops ──────────────────────────────────────────────────────────
    def _scalar(self, opcode, a, s):
        ga = self._in(a)
        out = self.graph.newOutputBuffer(a.rows, a.cols)
        if opcode == op.OP_MULTIPLY_SCALAR:
            self.graph.recordMultiplyScalar(ga, out, s)
        else:
            self.graph.recordScalarUnary(opcode, ga, out, s)
        return out

    def multiplyScalar(self, a, s): return self._out(self._scalar(op.OP_MULTIPLY_SCALAR, a, s))
    def addScalar(self, a, s): return self._out(self._scalar(op.OP_ADD_SCALAR, a, s))
    def divideScalar(self, a, s): return self._out(self._scalar(op.OP_DIVIDE_SCALAR, a, s))

    # ── reductions ──────────────────────────────────────────────────────────
    def _reduce(self, opcode, a, out_rows, out_cols):
        ga = self._in(a)
        out = self.graph.newOutputBuffer(out_rows, out_cols)
        self.graph.recordReduction(opcode, ga, out, a.rows, a.cols)
        return self._out(out)

    def sumRows(self, a): return self._reduce(op.OP_SUM_ROWS, a, 1, a.cols)
    def sumAlongCols(self, a): return self.sumRows(a)
    def sumAlongRows(self, a): return self._reduce(op.OP_SUM_ALONG_ROWS, a, a.rows, 1)
    def meanAlongRows(self, a): return self._reduce(op.OP_MEAN_ALONG_ROWS, a, a.rows, 1)
    def varianceAlongRows(self, a): return self._reduce(op.OP_VARIANCE_ALONG_ROWS, a, a.rows, 1)
    def maxAlongRows(self, a): return self._reduce(op.OP_MAX_ALONG_ROWS, a, a.rows, 1)

    def sum(self, a) -> float:
        ga = self._in(a)
        out = self.graph.newOutputBuffer(1, 1)
        self.graph.recordSumScalar(ga, out, a.rows, a.cols)
        scalar = self._out(out)
        scalar.materialize()
        return float(scalar.data[0, 0])

    def sumAbs(self, a) -> float:
        ga = self._in(a)
        rows = self.graph.newOutputBuffer(a.rows, 1)
        self.graph.recordSumAbs(ga, rows, a.rows, a.cols)
        scalar = self.sumRows(self._out(rows))
        scalar.materialize()
        return float(scalar.data[0, 0])

    # ── unary ───────────────────────────────────────────────────────────────
    def transpose(self, a):
        ga = self._in(a)
        out = self.graph.newOutputBuffer(a.cols, a.rows)
        self.graph.recordTranspose(ga, out, a.rows, a.cols)
        return self._out(out)

    def clamp(self, a, lo, hi):
        ga = self._in(a)
        out = self.graph.newOutputBuffer(a.rows, a.cols)
        self.graph.recordClamp(ga, out, lo, hi)
        return self._out(out)

    def pow(self, a, exponent):
        ga = self._in(a)
        out = self.graph.newOutputBuffer(a.rows, a.cols)
        self.graph.recordPow(ga, out, exponent)
        return self._out(out)

    def _unary(self, opcode, a):
        ga = self._in(a)
        out = self.graph.newOutputBuffer(a.rows, a.cols)
        self.graph.recordUnary(opcode, ga, out)
        return out

    def sqrt(self, a): return self._out(self._unary(op.OP_SQRT, a))
    def neg(self, a): return self._out(self._unary(op.OP_NEG, a))
    def exp(self, a): return self._out(self._unary(op.OP_EXP, a))
    def log(self, a): return self._out(self._unary(op.OP_LOG, a))
    def tanh(self, a): return self._out(self._unary(op.OP_TANH, a))
    def sigmoid(self, a): return self._out(self._unary(op.OP_SIGMOID, a))
    def relu(self, a): return self._out(self._unary(op.OP_RELU, a))
    def gelu(self, a): return self._out(self._unary(op.OP_GELU, a))

    # ── softmax ─────────────────────────────────────────────────────────────
    def softmaxRows(self, logits):
        ga = self._in(logits)
        out = self.graph.newOutputBuffer(logits.rows, logits.cols)
        self.graph.recordSoftmaxRows(ga, out, logits.rows, logits.cols)
        return self._out(out)

    def softmaxBackward(self, grad, softmax):
        Tensor.requireSameShape(grad, softmax, "softmaxBackward")
        gg, gs = self._in(grad), self._in(softmax)
        out = self.graph.newOutputBuffer(grad.rows, grad.cols)
        self.graph.recordSoftmaxBackward(gg, gs, out, grad.rows, grad.cols)
        return self._out(out)

    # ── in-place: new buffer, rebind (MetalBackend.java:400-526) ────────────
    def addInPlace(self, a, b): self.graph.bindTensorToBuffer(a, self._binary(op.OP_ADD, "addInPlace", a, b))
    def subtractInPlace(self, a, b): self.graph.bindTensorToBuffer(a, self._binary(op.OP_SUBTRACT, "subtractInPlace", a, b))
    def multiplyInPlace(self, a, b): self.graph.bindTensorToBuffer(a, self._binary(op.OP_MULTIPLY, "multiplyInPlace", a, b))
    def divideInPlace(self, a, b): self.graph.bindTensorToBuffer(a, self._binary(op.OP_DIVIDE, "divideInPlace", a, b))
    def multiplyScalarInPlace(self, a, s): self.graph.bindTensorToBuffer(a, self._scalar(op.OP_MULTIPLY_SCALAR, a, s))
    def addScalarInPlace(self, a, s): self.graph.bindTensorToBuffer(a, self._scalar(op.OP_ADD_SCALAR, a, s))
    def divideScalarInPlace(self, a, s): self.graph.bindTensorToBuffer(a, self._scalar(op.OP_DIVIDE_SCALAR, a, s))
    def sqrtInPlace(self, a): self.graph.bindTensorToBuffer(a, self._unary(op.OP_SQRT, a))
    def negInPlace(self, a): self.graph.bindTensorToBuffer(a, self._unary(op.OP_NEG, a))
    def expInPlace(self, a): self.graph.bindTensorToBuffer(a, self._unary(op.OP_EXP, a))
    def logInPlace(self, a): self.graph.bindTensorToBuffer(a, self._unary(op.OP_LOG, a))
    def reluInPlace(self, a): self.graph.bindTensorToBuffer(a, self._unary(op.OP_RELU, a))
    def geluInPlace(self, a): self.graph.bindTensorToBuffer(a, self._unary(op.OP_GELU, a))
    def tanhInPlace(self, a): self.graph.bindTensorToBuffer(a, self._unary(op.OP_TANH, a))
    def sigmoidInPlace(self, a): self.graph.bindTensorToBuffer(a, self._unary(op.OP_SIGMOID, a))

    # ── fused ops ───────────────────────────────────────────────────────────
    def crossEntropyGradient(self, logits, targets):
        Tensor.requireTargetsMatchRows(logits, targets)
        tt = self._int_column(targets)
        gl, gt = self._in(logits), self._in(tt)
        out = self.graph.newOutputBuffer(logits.rows, logits.cols)
        self.graph.recordCrossEntropyGradient(gl, gt, out, logits.rows, logits.cols)
        return self._out(out)

    def crossEntropyLoss(self, logits, targets) -> float:
        Tensor.requireTargetsMatchRows(logits, targets)
        tt = self._int_column(targets)
        gl, gt = self._in(logits), self._in(tt)
        rows = self.graph.newOutputBuffer(logits.rows, 1)
        self.graph.recordCrossEntropyLoss(gl, gt, rows, logits.rows, logits.cols)
        scalar = self.sumRows(self._out(rows)).divideScalar(logits.rows)
        scalar.materialize()
        return float(scalar.data[0, 0])

    def adamWUpdate(self, w, g, mt, vt, lr, beta1, beta2, eps, weight_decay, bc1, bc2):
        for other in (g, mt, vt):
            Tensor.requireSameShape(w, other, "adamWUpdate")
        gw, gg, gmt, gvt = self._in(w), self._in(g), self._in(mt), self._in(vt)
        self.graph.recordAdamWUpdate(gw, gg, gmt, gvt, lr, beta1, beta2, eps, weight_decay, bc1, bc2,
                                     w.rows * w.cols)
        for b in (gw, gmt, gvt):
            b.cpuStale = True
            b.needsUpload = False

    def layerNormBackward(self, dxhat, xhat, std, dim):
        Tensor.requireSameShape(dxhat, xhat, "layerNormBackward")
        if dim != dxhat.cols:
            raise ValueError(f"layerNormBackward: dim={dim} must equal tensor cols={dxhat.cols}")
        if std.rows != dxhat.rows or std.cols != 1:
            raise ValueError(f"layerNormBackward: std must be {dxhat.rows}x1 but got {std.rows}x{std.cols}")
        gd, gx, gs = self._in(dxhat), self._in(xhat), self._in(std)
        out = self.graph.newOutputBuffer(dxhat.rows, dxhat.cols)
        self.graph.recordLayerNormBackward(gd, gx, gs, out, dxhat.rows, dxhat.cols)
        return self._out(out)

    def scatterAddRows(self, target, indices, grad):
        if len(indices) != grad.rows:
            raise ValueError(f"scatterAddRows: indices length {len(indices)} must match grad rows {grad.rows}")
        if target.cols != grad.cols:
            raise ValueError(f"scatterAddRows: target cols {target.cols} must match grad cols {grad.cols}")
        if len(indices) == 0:
            return
        it = self._int_column(indices)
        gt, gg, gi = self._in(target), self._in(grad), self._in(it)
        self.graph.recordScatterAddRowsAtomic(gt, gi, gg, target.rows, target.cols, len(indices))
        gt.cpuStale = True
        gt.needsUpload = False
