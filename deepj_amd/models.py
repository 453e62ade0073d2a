"""Inference models on the native decode driver: Python faces of the reference's
LlamaConfig/LlamaModel, DeepSeekConfig/DeepSeekModel, GPTConfig/GPTModel and TextGenerator
(src/main/java/io/github/kirstenali/deepj/models/...) for the forward/generate path.

`forward(ids)` returns logits for every row like DecoderOnlyModel.forward
(DecoderOnlyModel.java:58-64); `TextGenerator.generate` works on token ids and runs
prefill + a device-resident greedy loop (topK = 1) or host-side sampling (any other
topK/temperature), drawing from a java.util.Random twin exactly as
TextGenerator.java:104-151 does.
"""
from __future__ import annotations

import ctypes as C
from dataclasses import dataclass

import numpy as np

from ._native import library

_i32p = C.POINTER(C.c_int32)
_f32p = C.POINTER(C.c_float)
_bound = False


def _lib():
    global _bound
    lib = library()
    if not _bound:
        lib.deepj_runner_create.argtypes = [_i32p, C.c_int32]
        lib.deepj_runner_create.restype = C.c_void_p
        lib.deepj_runner_destroy.argtypes = [C.c_void_p]
        lib.deepj_runner_last_error.argtypes = [C.c_void_p]
        lib.deepj_runner_last_error.restype = C.c_char_p
        lib.deepj_runner_set_weight.argtypes = [C.c_void_p, C.c_char_p, C.c_void_p, C.c_int32, C.c_int32]
        lib.deepj_runner_init_seeded.argtypes = [C.c_void_p, C.c_int64, C.c_int32]
        lib.deepj_runner_init_seeded_gpt.argtypes = [C.c_void_p, C.c_int64, C.c_float, C.c_int32]
        lib.deepj_runner_finalize.argtypes = [C.c_void_p]
        lib.deepj_runner_set_prepared_budget.argtypes = [C.c_void_p, C.c_int64]
        lib.deepj_runner_prepared_bytes.argtypes = [C.c_void_p]
        lib.deepj_runner_prepared_bytes.restype = C.c_int64
        lib.deepj_runner_reset.argtypes = [C.c_void_p]
        lib.deepj_runner_prefill.argtypes = [C.c_void_p, _i32p, C.c_int32, C.c_void_p, C.c_int32]
        lib.deepj_runner_decode.argtypes = [C.c_void_p, C.c_int32, C.c_int32]
        lib.deepj_runner_step.argtypes = [C.c_void_p, C.c_int32]
        lib.deepj_runner_last_logits.argtypes = [C.c_void_p, C.c_void_p]
        lib.deepj_runner_tokens.argtypes = [C.c_void_p, _i32p, C.c_int32, _i32p]
        lib.deepj_runner_generate.argtypes = [C.c_void_p, _i32p, C.c_int32, C.c_int32, C.c_float, C.c_int32,
                                              C.c_int64, C.c_int32, _i32p]
        lib.deepj_runner_decode_stream.argtypes = [C.c_void_p, _i32p, C.c_int32, _i32p]
        lib.deepj_runner_prefill_stream.argtypes = [C.c_void_p, C.c_int32, _i32p, C.c_int32, _i32p]
        lib.deepj_host_random_create.argtypes = [C.c_int64]
        lib.deepj_host_random_create.restype = C.c_void_p
        lib.deepj_host_random_destroy.argtypes = [C.c_void_p]
        lib.deepj_host_random_fill.argtypes = [C.c_void_p, C.c_void_p, C.c_int64, C.c_double, C.c_int32]
        lib.deepj_host_random_next_gaussian.argtypes = [C.c_void_p]
        lib.deepj_host_random_next_gaussian.restype = C.c_double
        lib.deepj_host_random_next_int.argtypes = [C.c_void_p, C.c_int32]
        lib.deepj_host_random_next_int.restype = C.c_int32
        lib.deepj_host_random_next_float.argtypes = [C.c_void_p]
        lib.deepj_host_random_next_float.restype = C.c_float
        _bound = True
    return lib


class JavaRandom:
    """java.util.Random (host library's twin; Tensor.random draws through it)."""

    def __init__(self, seed: int):
        self._h = _lib().deepj_host_random_create(seed)

    def __del__(self):
        if getattr(self, "_h", None):
            _lib().deepj_host_random_destroy(self._h)
            self._h = None

    def nextGaussian(self) -> float: return _lib().deepj_host_random_next_gaussian(self._h)
    def nextFloat(self) -> float: return _lib().deepj_host_random_next_float(self._h)

    def nextInt(self, bound: int | None = None) -> int:
        if bound is not None and bound <= 0:
            raise ValueError("bound must be positive")
        return _lib().deepj_host_random_next_int(self._h, 0 if bound is None else bound)

    def ints(self, n: int, bound: int) -> np.ndarray:
        return np.array([self.nextInt(bound) for _ in range(n)], dtype=np.int32)

    def tensor(self, rows: int, cols: int, scale: float = 0.1, threads: int = 0) -> np.ndarray:
        out = np.empty((rows, cols), dtype=np.float32)
        _lib().deepj_host_random_fill(self._h, out.ctypes.data, rows * cols, scale, threads)
        return out


@dataclass(frozen=True)
class LlamaConfig:
    """LlamaConfig.java:8-27."""
    vocabSize: int
    maxSeqLen: int
    dModel: int
    nHeads: int
    nLayers: int
    dFF: int

    @staticmethod
    def defaultDFF(d_model: int) -> int:
        raw = int(round(8.0 / 3 * d_model))
        return (raw + 63) // 64 * 64


@dataclass(frozen=True)
class DeepSeekConfig:
    """DeepSeekConfig.java:14-36 (qRank and kvRank are required)."""
    vocabSize: int
    maxSeqLen: int
    dModel: int
    nHeads: int
    nLayers: int
    dFF: int
    qRank: int
    kvRank: int


@dataclass(frozen=True)
class GPTConfig:
    """GPTConfig.java:8-27: initScale multiplies every parameter after init, gradClipNorm is a training knob."""
    vocabSize: int
    maxSeqLen: int
    dModel: int
    nHeads: int
    nLayers: int
    dFF: int
    initScale: float = 0.2
    gradClipNorm: float = 1.0

    def __post_init__(self):
        _validate(self, head_dims=False)
        if not np.isfinite(self.initScale) or self.initScale <= 0.0:
            raise ValueError("initScale must be finite and > 0")
        if not np.isfinite(self.gradClipNorm) or self.gradClipNorm <= 0.0:
            raise ValueError("gradClipNorm must be finite and > 0")


def _validate(cfg, head_dims: bool = True) -> None:
    # TransformerConfig.validateCommon (TransformerConfig.java:19-31)
    for name in ("vocabSize", "maxSeqLen", "dModel", "nHeads", "nLayers", "dFF"):
        if getattr(cfg, name) <= 0:
            raise ValueError(f"{name} must be > 0")
    if cfg.dModel % cfg.nHeads != 0:
        raise ValueError("dModel must be divisible by nHeads")
    if isinstance(cfg, DeepSeekConfig):
        if cfg.qRank <= 0:
            raise ValueError("qRank must be > 0")
        if cfg.kvRank <= 0:
            raise ValueError("kvRank must be > 0")
    if head_dims and cfg.dModel // cfg.nHeads not in (32, 64, 128):
        raise ValueError("this backend supports head dims 32, 64 and 128")


_next_id_base = [1 << 29]


class _DecoderOnlyModel:
    def __init__(self, cfg, seed: int | None, threads: int = 0, latent_cache: bool = False):
        _validate(cfg)
        self.cfg = cfg
        kind = 1 if isinstance(cfg, DeepSeekConfig) else (2 if isinstance(cfg, GPTConfig) else 0)
        if latent_cache and kind != 1:
            raise ValueError("the latent KV cache belongs to the DeepSeek (MLA) model")
        arr = (C.c_int32 * 9)(3 if latent_cache else kind, cfg.vocabSize, cfg.maxSeqLen, cfg.dModel, cfg.nHeads, cfg.nLayers, cfg.dFF,
                              getattr(cfg, "qRank", 0), getattr(cfg, "kvRank", 0))
        base = _next_id_base[0]
        _next_id_base[0] += 1 << 20
        self._h = _lib().deepj_runner_create(arr, base)
        if not self._h:
            raise ValueError("invalid model configuration")
        if seed is not None:
            if kind == 2:
                self._check(_lib().deepj_runner_init_seeded_gpt(self._h, seed, cfg.initScale, threads))
            else:
                self._check(_lib().deepj_runner_init_seeded(self._h, seed, threads))
            self._check(_lib().deepj_runner_finalize(self._h))

    def _check(self, rc: int) -> None:
        if rc != 0:
            msg = _lib().deepj_runner_last_error(self._h).decode("utf-8", "replace")
            if msg.startswith("Token id out of range") or "exceeds maxSeqLen" in msg or "must be" in msg:
                raise ValueError(msg)
            raise RuntimeError(msg)

    def close(self) -> None:
        if getattr(self, "_h", None):
            _lib().deepj_runner_destroy(self._h)
            self._h = None

    def __del__(self):
        try:
            self.close()
        except Exception:  # noqa: BLE001 - interpreter shutdown
            pass

    # weights ------------------------------------------------------------------
    def setWeight(self, name: str, value) -> None:
        a = np.ascontiguousarray(np.asarray(value, dtype=np.float32))
        if a.ndim == 1:
            a = a.reshape(1, -1)
        self._check(_lib().deepj_runner_set_weight(self._h, name.encode(), a.ctypes.data, a.shape[0], a.shape[1]))

    def finalize(self) -> None:
        self._check(_lib().deepj_runner_finalize(self._h))

    def setPreparedBudget(self, nbytes: int | None) -> None:
        """Bytes the model may spend on fp16 copies of its weights for the prompt GEMM (2 bytes per weight when every
        layer has one): None = no limit, 0 = none (every call converts), otherwise layers in order while it lasts.
        Same results whatever the budget."""
        self._check(_lib().deepj_runner_set_prepared_budget(self._h, -1 if nbytes is None else int(nbytes)))

    def preparedBytes(self) -> int:
        return int(_lib().deepj_runner_prepared_bytes(self._h))

    # inference ----------------------------------------------------------------
    def reset(self) -> None:
        self._check(_lib().deepj_runner_reset(self._h))

    def forward(self, ids) -> np.ndarray:
        """Logits [len(ids) x vocab] of a fresh sequence (DecoderOnlyModel.forward)."""
        ids = np.ascontiguousarray(np.asarray(ids, dtype=np.int32))
        self.reset()
        out = np.empty((len(ids), self.cfg.vocabSize), dtype=np.float32)
        self._check(_lib().deepj_runner_prefill(self._h, ids.ctypes.data_as(_i32p), len(ids), out.ctypes.data, 0))
        return out

    def prefill(self, ids, choose_next: bool = True) -> None:
        ids = np.ascontiguousarray(np.asarray(ids, dtype=np.int32))
        self._check(_lib().deepj_runner_prefill(self._h, ids.ctypes.data_as(_i32p), len(ids), None,
                                                1 if choose_next else 0))

    def _mode(self, use_graph) -> int:
        """0 eager per-token stream, 1 the stream as a replayed HIP graph (default)."""
        return 0 if use_graph is False else 1

    def decode(self, steps: int, use_graph: bool | None = None) -> None:
        self._check(_lib().deepj_runner_decode(self._h, steps, self._mode(use_graph)))

    def step(self, token: int) -> None:
        """Feed one caller-chosen token through the single-row (cached) path; see lastLogits()."""
        self._check(_lib().deepj_runner_step(self._h, int(token)))

    def lastLogits(self) -> np.ndarray:
        out = np.empty(self.cfg.vocabSize, dtype=np.float32)
        self._check(_lib().deepj_runner_last_logits(self._h, out.ctypes.data))
        return out

    def tokens(self) -> np.ndarray:
        out = np.empty(self.cfg.maxSeqLen, dtype=np.int32)
        n = C.c_int32()
        self._check(_lib().deepj_runner_tokens(self._h, out.ctypes.data_as(_i32p), out.size, C.byref(n)))
        return out[: n.value].copy()

    def prefillStream(self, n: int) -> np.ndarray:
        """The command stream of an n-token prompt at the current position (ids: those of the last prefill)."""
        ln = C.c_int32()
        self._check(_lib().deepj_runner_prefill_stream(self._h, n, None, 0, C.byref(ln)))
        out = np.empty(ln.value, dtype=np.int32)
        self._check(_lib().deepj_runner_prefill_stream(self._h, n, out.ctypes.data_as(_i32p), out.size, C.byref(ln)))
        return out

    def decodeStream(self) -> np.ndarray:
        n = C.c_int32()
        self._check(_lib().deepj_runner_decode_stream(self._h, None, 0, C.byref(n)))
        out = np.empty(n.value, dtype=np.int32)
        self._check(_lib().deepj_runner_decode_stream(self._h, out.ctypes.data_as(_i32p), out.size, C.byref(n)))
        return out


class LlamaModel(_DecoderOnlyModel):
    """new LlamaModel(cfg, seed) (LlamaModel.java:27-42); seed=None leaves the weights to setWeight."""

    def __init__(self, cfg: LlamaConfig, seed: int | None = 42, threads: int = 0):
        super().__init__(cfg, seed, threads)


class DeepSeekModel(_DecoderOnlyModel):
    """new DeepSeekModel(cfg, seed) (DeepSeekModel.java:29-46).  latent_cache: keep cKV (kvRank floats per token and
    layer) instead of the rotated K and V (2 * dModel) and re-expand it every step - eight times less cache at the
    README's ranks, at the price of a [context x kvRank] x [kvRank x 2 dModel] product per layer and token."""

    def __init__(self, cfg: DeepSeekConfig, seed: int | None = 42, threads: int = 0, latent_cache: bool = False):
        super().__init__(cfg, seed, threads, latent_cache)


class GPTModel(_DecoderOnlyModel):
    """new GPTModel(cfg, seed) (GPTModel.java:27-46): LayerNorm blocks with a GELU feed-forward, learned
    positions, every parameter scaled by cfg.initScale."""

    def __init__(self, cfg: GPTConfig, seed: int | None = 42, threads: int = 0):
        super().__init__(cfg, seed, threads)

    def gradClipNorm(self) -> float:
        return self.cfg.gradClipNorm


class TextGenerator:
    """TextGenerator.generate on token ids (TextGenerator.java:66-87)."""

    @staticmethod
    def generate(model: _DecoderOnlyModel, prompt_ids, max_new_tokens: int, temperature: float = 1.0,
                 top_k: int = 1, seed: int = 0, use_graph: bool | None = None) -> np.ndarray:
        prompt = np.ascontiguousarray(np.asarray(prompt_ids, dtype=np.int32))
        out = np.empty(len(prompt) + max(max_new_tokens, 0), dtype=np.int32)
        model._check(_lib().deepj_runner_generate(model._h, prompt.ctypes.data_as(_i32p), len(prompt),
                                                  max_new_tokens, temperature, top_k, seed,
                                                  model._mode(use_graph), out.ctypes.data_as(_i32p)))
        return out
