"""Host-side lazy graph: the Python twin of the reference's
src/main/java/io/github/kirstenali/deepj/tensor/{ComputeGraph,GpuBuffer,GpuRuntime,TensorAdapters}.java.

It records ops as a flat int32 command stream, assigns buffer ids, batches
allocations and uploads, flushes everything through a GpuRuntime (five calls)
and releases buffers no tensor points at any more.  In a JVM deployment the
reference's own ComputeGraph plays this part unchanged; this twin exists so that
the native library can be driven and tested from Python with exactly the
protocol the Java class speaks (same encodings, same call order).
"""
from __future__ import annotations

import struct
import weakref
from typing import Protocol

import numpy as np

from . import opcodes as op


class GpuRuntime(Protocol):
    """GpuRuntime.java:9-28."""

    def allocBuffers(self, ids, sizes, count: int) -> None: ...
    def uploadBuffer(self, buf_id: int, data: np.ndarray) -> None: ...
    def downloadBuffer(self, buf_id: int, out: np.ndarray) -> None: ...
    def releaseBuffers(self, ids, count: int) -> None: ...
    def flushOps(self, cmd_stream: np.ndarray, length: int) -> None: ...


class GpuBuffer:
    """GpuBuffer.java:9-32."""

    __slots__ = ("id", "rows", "cols", "needsUpload", "cpuStale", "allocatedOnGpu")

    def __init__(self, id: int, rows: int, cols: int, needs_upload: bool):
        self.id, self.rows, self.cols = id, rows, cols
        self.needsUpload = needs_upload
        self.cpuStale = False
        self.allocatedOnGpu = True

    def floatCount(self) -> int:
        return self.rows * self.cols


def float_bits(value: float) -> int:
    """Float.floatToRawIntBits as a signed int32."""
    return struct.unpack("<i", struct.pack("<f", np.float32(value)))[0]


# stride and buffer-id slots per opcode (ComputeGraph.java:89-147)
_OP_META: dict[int, tuple[int, tuple[int, ...]]] = {}
for _o in (op.OP_SQRT, op.OP_NEG, op.OP_EXP, op.OP_LOG, op.OP_TANH, op.OP_SIGMOID, op.OP_RELU, op.OP_GELU):
    _OP_META[_o] = (4, (1, 2))
for _o in (op.OP_ADD, op.OP_SUBTRACT, op.OP_MULTIPLY, op.OP_DIVIDE, op.OP_RELU_BACKWARD, op.OP_GELU_BACKWARD):
    _OP_META[_o] = (5, (1, 2, 3))
for _o in (op.OP_MULTIPLY_SCALAR, op.OP_ADD_SCALAR, op.OP_DIVIDE_SCALAR, op.OP_TRANSPOSE, op.OP_SUM_ROWS,
           op.OP_MEAN_ALONG_ROWS, op.OP_VARIANCE_ALONG_ROWS, op.OP_SUM_ALONG_ROWS, op.OP_MAX_ALONG_ROWS,
           op.OP_SOFTMAX_ROWS, op.OP_POW, op.OP_SUM_ABS, op.OP_SUM_SCALAR):
    _OP_META[_o] = (5, (1, 2))
_OP_META[op.OP_CLAMP] = (6, (1, 2))
for _o in (op.OP_SCATTER_ADD_ROWS, op.OP_SCATTER_ADD_ROWS_ATOMIC):
    _OP_META[_o] = (7, (1, 2, 3))
for _o in (op.OP_CROSS_ENTROPY_LOSS, op.OP_CROSS_ENTROPY_GRADIENT, op.OP_SOFTMAX_BACKWARD, op.OP_ADD_ROW_VECTOR,
           op.OP_ADD_BROADCAST_COLS, op.OP_SUBTRACT_BROADCAST_COLS, op.OP_DIVIDE_BROADCAST_COLS,
           op.OP_MULTIPLY_BROADCAST_ROWS, op.OP_MULTIPLY_BROADCAST_COLS):
    _OP_META[_o] = (6, (1, 2, 3))
_OP_META[op.OP_MATMUL] = (7, (1, 2, 3))
_OP_META[op.OP_LAYERNORM_BACKWARD] = (7, (1, 2, 3, 4))
_OP_META[op.OP_ADAMW_UPDATE] = (13, (1, 2, 3, 4))


class ComputeGraph:
    def __init__(self, runtime: GpuRuntime):
        if runtime is None:
            raise TypeError("runtime")          # Objects.requireNonNull
        self.runtime = runtime
        self._next_buf_id = 0
        self._cmd = np.zeros(4096, dtype=np.int32)
        self._pos = 0
        self._op_count = 0
        self._pending_allocs: list[tuple[int, int]] = []
        self._pending_uploads: list[tuple[int, np.ndarray]] = []
        self._buf_to_tensor: dict[int, weakref.ReferenceType] = {}

    # ── buffer management (ComputeGraph.java:172-234) ───────────────────────
    def ensureGpuBuffer(self, t) -> GpuBuffer:
        existing = t.getGpuTag()
        if isinstance(existing, GpuBuffer):
            self._track(existing.id, t)
            if existing.needsUpload:
                self._pending_uploads.append((existing.id, pack_f32(t)))
                existing.needsUpload = False
                existing.cpuStale = False
            return existing
        buf_id = self._next_buf_id
        self._next_buf_id += 1
        buf = GpuBuffer(buf_id, t.rows, t.cols, True)
        buf.allocatedOnGpu = False
        self._pending_allocs.append((buf_id, buf.floatCount()))
        self._pending_uploads.append((buf_id, pack_f32(t)))
        t.setGpuTag(buf)
        self._track(buf_id, t)
        return buf

    def _track(self, buf_id: int, t) -> None:
        self._buf_to_tensor[buf_id] = weakref.ref(t)

    def newOutputBuffer(self, rows: int, cols: int) -> GpuBuffer:
        buf_id = self._next_buf_id
        self._next_buf_id += 1
        buf = GpuBuffer(buf_id, rows, cols, False)
        buf.cpuStale = True
        buf.allocatedOnGpu = False
        self._pending_allocs.append((buf_id, buf.floatCount()))
        return buf

    def createOutputTensor(self, buf: GpuBuffer):
        from .tensor import Tensor
        t = Tensor(buf.rows, buf.cols)
        self.bindTensorToBuffer(t, buf)
        return t

    def bindTensorToBuffer(self, t, buf: GpuBuffer) -> None:
        t.setGpuTag(buf)
        self._track(buf.id, t)

    # ── op recording (ComputeGraph.java:238-518) ────────────────────────────
    def _emit(self, *words: int) -> None:
        n = len(words)
        if self._pos + n > self._cmd.size:
            grown = np.zeros(max(self._cmd.size * 2, self._pos + n), dtype=np.int32)
            grown[: self._pos] = self._cmd[: self._pos]
            self._cmd = grown
        self._cmd[self._pos: self._pos + n] = words
        self._pos += n
        self._op_count += 1

    def recordBinary(self, opcode, a, b, out): self._emit(opcode, a.id, b.id, out.id, out.floatCount())
    def recordMatmul(self, a, b, out, m, n, k): self._emit(op.OP_MATMUL, a.id, b.id, out.id, m, n, k)
    def recordUnary(self, opcode, inp, out): self._emit(opcode, inp.id, out.id, out.floatCount())

    def recordMultiplyScalar(self, inp, out, scalar):
        self._emit(op.OP_MULTIPLY_SCALAR, inp.id, out.id, float_bits(scalar), out.floatCount())

    def recordScalarUnary(self, opcode, inp, out, scalar):
        self._emit(opcode, inp.id, out.id, float_bits(scalar), out.floatCount())

    def recordPow(self, inp, out, exponent):
        self._emit(op.OP_POW, inp.id, out.id, float_bits(exponent), out.floatCount())

    def recordClamp(self, inp, out, lo, hi):
        self._emit(op.OP_CLAMP, inp.id, out.id, float_bits(lo), float_bits(hi), out.floatCount())

    def recordScatterAddRows(self, target, indices, grad, target_rows, target_cols, n_indices):
        self._emit(op.OP_SCATTER_ADD_ROWS, target.id, indices.id, grad.id, target_rows, target_cols, n_indices)

    def recordScatterAddRowsAtomic(self, target, indices, grad, target_rows, target_cols, n_indices):
        self._emit(op.OP_SCATTER_ADD_ROWS_ATOMIC, target.id, indices.id, grad.id, target_rows, target_cols, n_indices)

    def recordSumAbs(self, inp, out, rows, cols): self._emit(op.OP_SUM_ABS, inp.id, out.id, rows, cols)

    def recordCrossEntropyLoss(self, logits, targets, out, rows, cols):
        self._emit(op.OP_CROSS_ENTROPY_LOSS, logits.id, targets.id, out.id, rows, cols)

    def recordCrossEntropyGradient(self, logits, targets, out, rows, cols):
        self._emit(op.OP_CROSS_ENTROPY_GRADIENT, logits.id, targets.id, out.id, rows, cols)

    def recordSumScalar(self, inp, out, rows, cols): self._emit(op.OP_SUM_SCALAR, inp.id, out.id, rows, cols)
    def recordTranspose(self, inp, out, rows, cols): self._emit(op.OP_TRANSPOSE, inp.id, out.id, rows, cols)

    def recordRowBroadcast(self, opcode, a, row_vec, out, rows, cols):
        self._emit(opcode, a.id, row_vec.id, out.id, rows, cols)

    def recordColBroadcast(self, opcode, a, col_vec, out, rows, cols):
        self._emit(opcode, a.id, col_vec.id, out.id, rows, cols)

    def recordReduction(self, opcode, inp, out, rows, cols): self._emit(opcode, inp.id, out.id, rows, cols)
    def recordSoftmaxRows(self, inp, out, rows, cols): self._emit(op.OP_SOFTMAX_ROWS, inp.id, out.id, rows, cols)

    def recordSoftmaxBackward(self, grad, softmax, out, rows, cols):
        self._emit(op.OP_SOFTMAX_BACKWARD, grad.id, softmax.id, out.id, rows, cols)

    def recordLayerNormBackward(self, dxhat, xhat, std, out, rows, cols):
        self._emit(op.OP_LAYERNORM_BACKWARD, dxhat.id, xhat.id, std.id, out.id, rows, cols)

    def recordAdamWUpdate(self, w, g, mt, vt, lr, beta1, beta2, eps, weight_decay, bc1, bc2, n):
        self._emit(op.OP_ADAMW_UPDATE, w.id, g.id, mt.id, vt.id, float_bits(lr), float_bits(beta1),
                   float_bits(beta2), float_bits(eps), float_bits(weight_decay), float_bits(bc1), float_bits(bc2), n)

    def isEmpty(self) -> bool:
        return self._op_count == 0

    # ── flush (ComputeGraph.java:528-671) ───────────────────────────────────
    def flush(self) -> None:
        if self._op_count == 0 and not self._pending_allocs:
            self._release_orphans()
            return
        self._allocate_pending()
        self._upload_pending()
        self._execute_pending()
        self._release_orphans()

    def _allocate_pending(self) -> None:
        if not self._pending_allocs:
            return
        ids = np.array([a[0] for a in self._pending_allocs], dtype=np.int32)
        sizes = np.array([a[1] for a in self._pending_allocs], dtype=np.int32)
        self.runtime.allocBuffers(ids, sizes, len(ids))
        for ref in self._buf_to_tensor.values():
            t = ref()
            if t is not None and isinstance(t.getGpuTag(), GpuBuffer):
                t.getGpuTag().allocatedOnGpu = True
        self._pending_allocs.clear()

    def _upload_pending(self) -> None:
        for buf_id, data in self._pending_uploads:
            self.runtime.uploadBuffer(buf_id, data)
        self._pending_uploads.clear()

    def _execute_pending(self) -> None:
        if self._op_count > 0:
            self.runtime.flushOps(self._cmd, self._pos)
        self._pos = 0
        self._op_count = 0

    def _release_orphans(self) -> None:
        if not self._buf_to_tensor:
            return
        orphans = []
        for buf_id, ref in self._buf_to_tensor.items():
            t = ref()
            orphaned = t is None or not isinstance(t.getGpuTag(), GpuBuffer) or t.getGpuTag().id != buf_id
            if orphaned and not self._referenced_by_pending_ops(buf_id):
                orphans.append(buf_id)
        if not orphans:
            return
        for buf_id in orphans:
            self._pending_allocs = [a for a in self._pending_allocs if a[0] != buf_id]
            self._pending_uploads = [u for u in self._pending_uploads if u[0] != buf_id]
            del self._buf_to_tensor[buf_id]
        ids = np.array(orphans, dtype=np.int32)
        self.runtime.releaseBuffers(ids, len(ids))

    def _referenced_by_pending_ops(self, buf_id: int) -> bool:
        pos = 0
        while pos < self._pos:
            meta = _OP_META.get(int(self._cmd[pos]))
            if meta is None:
                return True                     # unknown op: be conservative
            stride, slots = meta
            if any(int(self._cmd[pos + s]) == buf_id for s in slots):
                return True
            pos += stride
        return False

    # ── materialize / release (ComputeGraph.java:676-740) ───────────────────
    def materialize(self, t) -> None:
        buf = t.getGpuTag()
        if not isinstance(buf, GpuBuffer) or not buf.cpuStale:
            return
        self.flush()
        flat = np.zeros(buf.floatCount(), dtype=np.float32)
        self.runtime.downloadBuffer(buf.id, flat)
        unpack_f32_into(flat, t)
        buf.cpuStale = False

    def releaseAll(self) -> None:
        self.flush()
        for ref in list(self._buf_to_tensor.values()):
            t = ref()
            if t is None:
                continue
            gb = t.getGpuTag()
            if not isinstance(gb, GpuBuffer) or not gb.cpuStale:
                continue
            flat = np.zeros(gb.floatCount(), dtype=np.float32)
            self.runtime.downloadBuffer(gb.id, flat)
            unpack_f32_into(flat, t)
            gb.cpuStale = False
            gb.needsUpload = False
        for ref in self._buf_to_tensor.values():
            t = ref()
            if t is not None:
                t.setGpuTag(None)
        if self._buf_to_tensor:
            ids = np.array(list(self._buf_to_tensor.keys()), dtype=np.int32)
            self.runtime.releaseBuffers(ids, len(ids))
        self._buf_to_tensor.clear()
        self._pending_allocs.clear()
        self._pending_uploads.clear()
        self._pos = 0
        self._op_count = 0
        self._next_buf_id = 0


# TensorAdapters.java:9-47
def pack_f32(t) -> np.ndarray:
    return np.array(t.data, dtype=np.float32, copy=True).reshape(-1)


def unpack_f32_into(src: np.ndarray, dst) -> None:
    if src.size != dst.data.size:
        raise ValueError(f"Size mismatch: src has {src.size} floats but tensor is {dst.rows}x{dst.cols}")
    dst.data.reshape(-1)[:] = src


def from_int_column(values) -> "object":
    from .tensor import Tensor
    t = Tensor(len(values), 1)
    t.data[:, 0] = np.asarray(values, dtype=np.float32)
    return t
