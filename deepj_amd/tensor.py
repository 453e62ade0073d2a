"""Tensor: the Python twin of src/main/java/io/github/kirstenali/deepj/tensor/Tensor.java.

A 2-D row-major fp32 matrix with a host copy (`data`, a numpy [rows x cols] array) and
an optional GPU handle.  Every op forwards to the active TensorBackend; host accessors
call materialize() first (Tensor.java:73-77,208-245).  There is no CPU compute backend
in this package: ops need a HipBackend, set with Tensor.setBackend.
"""
from __future__ import annotations

import numpy as np

from .compute_graph import GpuBuffer


class Tensor:
    _backend = None

    def __init__(self, rows: int, cols: int | None = None):
        if isinstance(rows, Tensor):                      # copy constructor (Tensor.java:50-59)
            src = rows
            src.materialize()
            self.rows, self.cols = src.rows, src.cols
            self.data = src.data.copy()
        else:
            self.rows, self.cols = int(rows), int(cols)
            self.data = np.zeros((self.rows, self.cols), dtype=np.float32)
        self._gpu_tag = None

    # ── backend switch (Tensor.java:24-41) ──────────────────────────────────
    @staticmethod
    def setBackend(backend) -> None:
        if backend is None:
            raise ValueError("backend cannot be null")
        Tensor._backend = backend

    @staticmethod
    def backend():
        if Tensor._backend is None:
            raise RuntimeError("no TensorBackend set: call Tensor.setBackend(HipBackend())")
        return Tensor._backend

    def getGpuTag(self): return self._gpu_tag
    def setGpuTag(self, tag): self._gpu_tag = tag

    def materialize(self) -> "Tensor":
        if self._gpu_tag is not None:
            Tensor.backend().materializeTensor(self)
        return self

    def _mark_needs_upload(self) -> None:
        if isinstance(self._gpu_tag, GpuBuffer):
            self._gpu_tag.needsUpload = True
            self._gpu_tag.cpuStale = False

    # ── factories ───────────────────────────────────────────────────────────
    @staticmethod
    def from2D(values) -> "Tensor":
        a = np.asarray(values, dtype=np.float32)
        if a.ndim != 2:
            raise ValueError("All rows must have the same length")
        t = Tensor(a.shape[0], a.shape[1])
        t.data[:] = a
        return t

    @staticmethod
    def zeros(rows, cols): return Tensor(rows, cols)

    @staticmethod
    def ones(rows, cols):
        t = Tensor(rows, cols)
        t.data.fill(1.0)
        return t

    @staticmethod
    def random(rows, cols, rnd) -> "Tensor":
        """Tensor.random(rows, cols, Random): (float)(nextGaussian()*0.1), row-major."""
        t = Tensor(rows, cols)
        t.data[:] = rnd.tensor(rows, cols)
        return t

    @staticmethod
    def causalMask(size) -> "Tensor":
        t = Tensor(size, size)
        t.data[:] = np.triu(np.full((size, size), -1e9, dtype=np.float32), 1)
        return t

    # ── shape checks (Tensor.java:253-267) ──────────────────────────────────
    @staticmethod
    def requireSameShape(a, b, name: str) -> None:
        if a.rows != b.rows or a.cols != b.cols:
            raise ValueError(f"Shape mismatch for {name}: {a.rows}x{a.cols} vs {b.rows}x{b.cols}")

    @staticmethod
    def requireTargetsMatchRows(logits, targets) -> None:
        if len(targets) != logits.rows:
            raise ValueError(f"targets length {len(targets)} must match logits rows {logits.rows}")

    # ── ops: forward to the backend (Tensor.java:80-205) ────────────────────
    def matmul(self, o): return Tensor.backend().matmul(self, o)
    def add(self, o): return Tensor.backend().add(self, o)
    def subtract(self, o): return Tensor.backend().subtract(self, o)
    def multiply(self, o): return Tensor.backend().multiply(self, o)
    def divide(self, o): return Tensor.backend().divide(self, o)
    def addRowVector(self, v): return Tensor.backend().addRowVector(self, v)
    def addBroadcastCols(self, v): return Tensor.backend().addBroadcastCols(self, v)
    def divideBroadcastCols(self, v): return Tensor.backend().divideBroadcastCols(self, v)
    def subtractBroadcastCols(self, v): return Tensor.backend().subtractBroadcastCols(self, v)
    def multiplyBroadcastCols(self, v): return Tensor.backend().multiplyBroadcastCols(self, v)
    def addBroadcastRows(self, v): return Tensor.backend().addBroadcastRows(self, v)
    def multiplyBroadcastRows(self, v): return Tensor.backend().multiplyBroadcastRows(self, v)
    def multiplyScalar(self, s): return Tensor.backend().multiplyScalar(self, s)
    def addScalar(self, s): return Tensor.backend().addScalar(self, s)
    def divideScalar(self, s): return Tensor.backend().divideScalar(self, s)
    def sumRows(self): return Tensor.backend().sumRows(self)
    def sumAlongRows(self): return Tensor.backend().sumAlongRows(self)
    def sumAlongCols(self): return Tensor.backend().sumAlongCols(self)
    def meanAlongRows(self): return Tensor.backend().meanAlongRows(self)
    def varianceAlongRows(self): return Tensor.backend().varianceAlongRows(self)
    def maxAlongRows(self): return Tensor.backend().maxAlongRows(self)
    def transpose(self): return Tensor.backend().transpose(self)
    def clamp(self, lo, hi): return Tensor.backend().clamp(self, lo, hi)
    def pow(self, e): return Tensor.backend().pow(self, e)
    def sqrt(self): return Tensor.backend().sqrt(self)
    def neg(self): return Tensor.backend().neg(self)
    def exp(self): return Tensor.backend().exp(self)
    def log(self): return Tensor.backend().log(self)
    def tanhActivation(self): return Tensor.backend().tanh(self)
    def sigmoidActivation(self): return Tensor.backend().sigmoid(self)
    def reluActivation(self): return Tensor.backend().relu(self)
    def reluBackward(self, g): return Tensor.backend().reluBackward(self, g)
    def geluActivation(self): return Tensor.backend().gelu(self)
    def geluBackward(self, g): return Tensor.backend().geluBackward(self, g)
    def softmaxRows(self): return Tensor.backend().softmaxRows(self)
    def softmaxBackward(self, s): return Tensor.backend().softmaxBackward(self, s)
    def crossEntropyGradient(self, targets): return Tensor.backend().crossEntropyGradient(self, targets)
    def crossEntropyLoss(self, targets): return Tensor.backend().crossEntropyLoss(self, targets)
    def sum(self): return Tensor.backend().sum(self)
    def sumAbs(self): return Tensor.backend().sumAbs(self)

    def addInPlace(self, b): Tensor.backend().addInPlace(self, b); return self
    def subtractInPlace(self, b): Tensor.backend().subtractInPlace(self, b); return self
    def multiplyInPlace(self, b): Tensor.backend().multiplyInPlace(self, b); return self
    def divideInPlace(self, b): Tensor.backend().divideInPlace(self, b); return self
    def multiplyScalarInPlace(self, s): Tensor.backend().multiplyScalarInPlace(self, s); return self
    def addScalarInPlace(self, s): Tensor.backend().addScalarInPlace(self, s); return self
    def divideScalarInPlace(self, s): Tensor.backend().divideScalarInPlace(self, s); return self
    def sqrtInPlace(self): Tensor.backend().sqrtInPlace(self); return self
    def negInPlace(self): Tensor.backend().negInPlace(self); return self
    def expInPlace(self): Tensor.backend().expInPlace(self); return self
    def logInPlace(self): Tensor.backend().logInPlace(self); return self
    def reluInPlace(self): Tensor.backend().reluInPlace(self); return self
    def geluInPlace(self): Tensor.backend().geluInPlace(self); return self
    def tanhInPlace(self): Tensor.backend().tanhInPlace(self); return self
    def sigmoidInPlace(self): Tensor.backend().sigmoidInPlace(self); return self

    @staticmethod
    def adamWUpdate(w, g, mt, vt, lr, beta1, beta2, eps, weight_decay, bc1, bc2):
        Tensor.backend().adamWUpdate(w, g, mt, vt, lr, beta1, beta2, eps, weight_decay, bc1, bc2)

    @staticmethod
    def layerNormBackward(dxhat, xhat, std, dim):
        return Tensor.backend().layerNormBackward(dxhat, xhat, std, dim)

    @staticmethod
    def scatterAddRows(target, indices, grad):
        Tensor.backend().scatterAddRows(target, indices, grad)

    # ── host accessors: materialize first (Tensor.java:208-245) ─────────────
    def get(self, r, c):
        self.materialize()
        return float(self.data[r, c])

    def set(self, r, c, value):
        self.materialize()
        self.data[r, c] = value
        self._mark_needs_upload()

    def getRow(self, row):
        self.materialize()
        t = Tensor(1, self.cols)
        t.data[0] = self.data[row]
        return t

    def setRow(self, row, source, src_row):
        self.materialize()
        source.materialize()
        self.data[row] = source.data[src_row]
        self._mark_needs_upload()

    def rowData(self, r):
        return self.data[r].copy()

    @staticmethod
    def sliceRows(t, row_indices, cols):
        t.materialize()
        out = Tensor(len(row_indices), cols)
        out.data[:] = t.data[np.asarray(row_indices, dtype=np.int64), :cols]
        return out

    def numpy(self) -> np.ndarray:
        """Materialised host copy."""
        self.materialize()
        return self.data
