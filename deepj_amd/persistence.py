"""Checkpoint files of the reference (ModelSerializer.java:18-98): big-endian int32 parameter count, then
per parameter big-endian int32 rows, int32 cols and rows*cols big-endian float64 values, parameters in
`model.parameters()` order.

For the decoder-only models that order is (DecoderOnlyModel.java:79-85, AbstractTransformerBlock.java:21-27,
sub-layers {ln1, ln2, attn, mlp}; Linear.java:54-56 = W then b):
    emb, per block [g1, g2, attention matrices, wg, bg, wu, bu, wd, bd], gf, wlm, blm
i.e. 12 parameters per Llama block and 14 per DeepSeek block - the names `parameter_names` returns.
GPTModel (GPTModel.java:64-69, LayerNorm1D.java:80-82 = gamma then beta, FNN = its Linears in order):
    emb, pos, per block [g1, be1, g2, be2, wq, wk, wv, wo, wg, bg, wd, bd], gf, bf, wlm, blm
"""
from __future__ import annotations

import os
import struct

import numpy as np

from .models import DeepSeekConfig, GPTConfig, LlamaConfig


def parameter_names(cfg) -> list[str]:
    if isinstance(cfg, GPTConfig):
        per = ["g1", "be1", "g2", "be2", "wq", "wk", "wv", "wo", "wg", "bg", "wd", "bd"]
        names = ["emb", "pos"]
        for l in range(cfg.nLayers):
            names += [f"L{l}.{w}" for w in per]
        return names + ["gf", "bf", "wlm", "blm"]
    attn = ["wdq", "wuq", "wdkv", "wuk", "wuv", "wo"] if isinstance(cfg, DeepSeekConfig) else ["wq", "wk", "wv", "wo"]
    per = ["g1", "g2"] + attn + ["wg", "bg", "wu", "bu", "wd", "bd"]
    names = ["emb"]
    for l in range(cfg.nLayers):
        names += [f"L{l}.{w}" for w in per]
    return names + ["gf", "wlm", "blm"]


def parameter_shapes(cfg) -> list[tuple[int, int]]:
    """(rows, cols) of every parameter, reference orientation (weights [dIn x dOut], vectors [1 x n])."""
    d, f, v = cfg.dModel, cfg.dFF, cfg.vocabSize
    if isinstance(cfg, GPTConfig):
        per = [(1, d)] * 4 + [(d, d)] * 4 + [(d, f), (1, f), (f, d), (1, d)]
        return [(v, d), (cfg.maxSeqLen, d)] + per * cfg.nLayers + [(1, d), (1, d), (d, v), (1, v)]
    if isinstance(cfg, DeepSeekConfig):
        q, k = cfg.qRank, cfg.kvRank
        attn = [(d, q), (q, d), (d, k), (k, d), (k, d), (d, d)]
    else:
        attn = [(d, d)] * 4
    per = [(1, d), (1, d)] + attn + [(d, f), (1, f), (d, f), (1, f), (f, d), (1, d)]
    return [(v, d)] + per * cfg.nLayers + [(1, d), (d, v), (1, v)]


class ModelSerializer:
    """save / load with the reference's file format and error messages (IOError where Java throws IOException)."""

    @staticmethod
    def save(params, path) -> None:
        if params is None:
            raise ValueError("params is null")                       # ModelSerializer.java:31-35
        parent = os.path.dirname(os.path.abspath(path))
        os.makedirs(parent, exist_ok=True)                           # ModelSerializer.java:37-42
        with open(path, "wb") as out:
            out.write(struct.pack(">i", len(params)))
            for p in params:
                a = np.asarray(p, dtype=np.float32)
                if a.ndim == 1:
                    a = a.reshape(1, -1)
                if a.ndim != 2:
                    raise ValueError("parameters are 2-D tensors")
                out.write(struct.pack(">ii", a.shape[0], a.shape[1]))
                a.astype(">f8").tofile(out)                          # float -> double is exact

    @staticmethod
    def read(path, expected_shapes=None):
        """Yields (index, float32 array) per parameter; validates count and shapes when given."""
        with open(path, "rb") as f:
            (count,) = struct.unpack(">i", _exactly(f, 4))
            if expected_shapes is not None and count != len(expected_shapes):
                raise IOError("Parameter count mismatch")            # ModelSerializer.java:81-87
            for i in range(count):
                rows, cols = struct.unpack(">ii", _exactly(f, 8))
                if expected_shapes is not None and (rows, cols) != tuple(expected_shapes[i]):
                    raise IOError(f"Shape mismatch at parameter {i}")    # ModelSerializer.java:89-95
                if rows < 0 or cols < 0:
                    raise IOError(f"Shape mismatch at parameter {i}")
                data = np.fromfile(f, dtype=">f8", count=rows * cols)
                if data.size != rows * cols:
                    raise EOFError("checkpoint file is truncated")
                yield i, data.astype(np.float32).reshape(rows, cols)     # (float) readDouble()

    @staticmethod
    def load_arrays(path, expected_shapes=None):
        return [a for _, a in ModelSerializer.read(path, expected_shapes)]

    @staticmethod
    def load(model, path) -> None:
        """Loads a checkpoint written by the reference (or by `save`) into a model created with seed=None,
        one parameter at a time (a parameter is quantised on the device as soon as it arrives), then finalizes it."""
        names = parameter_names(model.cfg)
        shapes = parameter_shapes(model.cfg)
        for i, a in ModelSerializer.read(path, shapes):
            model.setWeight(names[i], a)
        model.finalize()


def _exactly(f, n: int) -> bytes:
    b = f.read(n)
    if len(b) != n:
        raise EOFError("checkpoint file is truncated")
    return b
