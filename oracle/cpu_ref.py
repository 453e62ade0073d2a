"""TEST INFRASTRUCTURE ONLY: ctypes/numpy front end of the CPU oracle (liboracle.so).

The oracle is a plain-C restatement of the reference's CpuBackend and inference
layers (see cpu_backend.h / model_ref.h for the file:line map).  Only tests,
the smoke check and the benchmark's CPU-baseline leg may import this module;
the shipped package never does.
"""
from __future__ import annotations

import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "liboracle.so")

f32p = C.POINTER(C.c_float)
i32p = C.POINTER(C.c_int32)
i8p = C.POINTER(C.c_int8)


def build(force: bool = False) -> str:
    """Compile liboracle.so with the Makefile next to this file."""
    if force or not os.path.exists(_LIB_PATH):
        subprocess.check_call(["make", "-C", _HERE, "-B", "liboracle.so"], stdout=subprocess.DEVNULL)
    return _LIB_PATH


def _load() -> C.CDLL:
    if not os.path.exists(_LIB_PATH):
        build()
    return C.CDLL(_LIB_PATH)


lib = _load()


def _fp(a: np.ndarray):
    assert a.dtype == np.float32 and a.flags["C_CONTIGUOUS"], (a.dtype, a.flags)
    return a.ctypes.data_as(f32p)


def _ip(a: np.ndarray):
    assert a.dtype == np.int32 and a.flags["C_CONTIGUOUS"]
    return a.ctypes.data_as(i32p)


def f32(a) -> np.ndarray:
    return np.ascontiguousarray(np.asarray(a, dtype=np.float32))


def i32(a) -> np.ndarray:
    return np.ascontiguousarray(np.asarray(a, dtype=np.int32))


# ── java.util.Random ────────────────────────────────────────────────────────

class _JR(C.Structure):
    _fields_ = [("seed", C.c_uint64), ("have_next", C.c_int), ("next_next", C.c_double)]


lib.jr_init.argtypes = [C.POINTER(_JR), C.c_int64]
lib.jr_next_int.argtypes = [C.POINTER(_JR)]
lib.jr_next_int.restype = C.c_int32
lib.jr_next_int_bound.argtypes = [C.POINTER(_JR), C.c_int32]
lib.jr_next_int_bound.restype = C.c_int32
lib.jr_next_float.argtypes = [C.POINTER(_JR)]
lib.jr_next_float.restype = C.c_float
lib.jr_next_double.argtypes = [C.POINTER(_JR)]
lib.jr_next_double.restype = C.c_double
lib.jr_next_gaussian.argtypes = [C.POINTER(_JR)]
lib.jr_next_gaussian.restype = C.c_double
lib.fdlibm_log.argtypes = [C.c_double]
lib.fdlibm_log.restype = C.c_double
lib.ref_random.argtypes = [f32p, C.c_int64, C.POINTER(_JR)]


class JavaRandom:
    """java.util.Random (JDK specification)."""

    def __init__(self, seed: int):
        self._r = _JR()
        lib.jr_init(C.byref(self._r), seed)

    def next_int(self, bound: int | None = None) -> int:
        if bound is None:
            return lib.jr_next_int(C.byref(self._r))
        if bound <= 0:
            raise ValueError("bound must be positive")
        return lib.jr_next_int_bound(C.byref(self._r), bound)

    def next_float(self) -> float:
        return lib.jr_next_float(C.byref(self._r))

    def next_double(self) -> float:
        return lib.jr_next_double(C.byref(self._r))

    def next_gaussian(self) -> float:
        return lib.jr_next_gaussian(C.byref(self._r))

    def ints(self, n: int, bound: int) -> np.ndarray:
        return np.array([self.next_int(bound) for _ in range(n)], dtype=np.int32)

    def tensor(self, rows: int, cols: int) -> np.ndarray:
        """Tensor.random(rows, cols, this): (float)(nextGaussian()*0.1), row-major."""
        out = np.empty((rows, cols), dtype=np.float32)
        lib.ref_random(_fp(out), rows * cols, C.byref(self._r))
        return out

    def gaussians_f32(self, rows: int, cols: int, scale: float = 1.0) -> np.ndarray:
        """(float)(nextGaussian()*scale) with the product formed in f64, like the reference."""
        g = np.array([self.next_gaussian() for _ in range(rows * cols)], dtype=np.float64)
        return (g * scale).astype(np.float32).reshape(rows, cols)


def random_tensor(rows: int, cols: int, seed: int) -> np.ndarray:
    return JavaRandom(seed).tensor(rows, cols)


# ── threading knobs ─────────────────────────────────────────────────────────
lib.ref_set_threads.argtypes = [C.c_int]
lib.ref_get_threads.restype = C.c_int
lib.ref_default_threads.restype = C.c_int
lib.ref_set_column_parallel.argtypes = [C.c_int]


def set_threads(n: int) -> None:
    lib.ref_set_threads(n)


def default_threads() -> int:
    return lib.ref_default_threads()


def set_column_parallel(on: bool) -> None:
    lib.ref_set_column_parallel(1 if on else 0)


# ── CpuBackend ops ──────────────────────────────────────────────────────────

def _sig(name, *argtypes, restype=None):
    fn = getattr(lib, name)
    fn.argtypes = list(argtypes)
    fn.restype = restype
    return fn


_I = C.c_int
_F = C.c_float
for _n in ("add", "subtract", "multiply", "divide", "relu_backward", "gelu_backward",
           "add_row_vector", "multiply_broadcast_rows", "add_broadcast_cols",
           "subtract_broadcast_cols", "multiply_broadcast_cols", "divide_broadcast_cols",
           "softmax_backward"):
    _sig("ref_" + _n, f32p, f32p, f32p, _I, _I)
for _n in ("multiply_scalar", "add_scalar", "divide_scalar", "pow"):
    _sig("ref_" + _n, f32p, _F, f32p, _I, _I)
for _n in ("sum_rows", "sum_along_rows", "mean_along_rows", "variance_along_rows", "max_along_rows",
           "transpose", "sqrt", "neg", "exp", "log", "tanh", "sigmoid", "relu", "gelu", "softmax_rows",
           "silu"):
    _sig("ref_" + _n, f32p, f32p, _I, _I)
_sig("ref_matmul", f32p, f32p, f32p, _I, _I, _I)
_sig("ref_clamp", f32p, _F, _F, f32p, _I, _I)
_sig("ref_sum", f32p, C.c_int64, restype=_F)
_sig("ref_sum_abs", f32p, C.c_int64, restype=_F)
_sig("ref_causal_mask", f32p, _I)
_sig("ref_cross_entropy_loss", f32p, i32p, _I, _I, restype=_F)
_sig("ref_cross_entropy_gradient", f32p, i32p, f32p, _I, _I)
_sig("ref_adamw_update", f32p, f32p, f32p, f32p, C.c_int64, _F, _F, _F, _F, _F, _F, _F)
_sig("ref_layer_norm_backward", f32p, f32p, f32p, f32p, _I, _I)
_sig("ref_scatter_add_rows", f32p, i32p, _I, f32p, _I)
_sig("ref_slice_rows", f32p, i32p, _I, _I, f32p)


def _shape_err(op, a, b):
    return ValueError(f"Shape mismatch for {op}: {a.shape[0]}x{a.shape[1]} vs {b.shape[0]}x{b.shape[1]}")


def _binary(name, a, b):
    a, b = f32(a), f32(b)
    if a.shape != b.shape:
        raise _shape_err(name, a, b)
    out = np.empty_like(a)
    getattr(lib, "ref_" + name)(_fp(a), _fp(b), _fp(out), a.shape[0], a.shape[1])
    return out


def add(a, b): return _binary("add", a, b)
def subtract(a, b): return _binary("subtract", a, b)
def multiply(a, b): return _binary("multiply", a, b)
def divide(a, b): return _binary("divide", a, b)
def relu_backward(x, g): return _binary("relu_backward", x, g)
def gelu_backward(x, g): return _binary("gelu_backward", x, g)
def softmax_backward(g, s): return _binary("softmax_backward", g, s)


def matmul(a, b):
    a, b = f32(a), f32(b)
    if a.shape[1] != b.shape[0]:
        raise ValueError(f"Shape mismatch for matmul: {a.shape[0]}x{a.shape[1]} cannot be multiplied by "
                         f"{b.shape[0]}x{b.shape[1]}")
    out = np.empty((a.shape[0], b.shape[1]), dtype=np.float32)
    lib.ref_matmul(_fp(a), _fp(b), _fp(out), a.shape[0], b.shape[1], a.shape[1])
    return out


def _row_bcast(name, a, rv):
    a, rv = f32(a), f32(rv)
    if rv.shape != (1, a.shape[1]):
        raise ValueError(f"rowVector must be 1x{a.shape[1]}")
    out = np.empty_like(a)
    getattr(lib, "ref_" + name)(_fp(a), _fp(rv), _fp(out), a.shape[0], a.shape[1])
    return out


def _col_bcast(name, a, cv):
    a, cv = f32(a), f32(cv)
    if cv.shape != (a.shape[0], 1):
        raise ValueError(f"colVector must be {a.shape[0]}x1")
    out = np.empty_like(a)
    getattr(lib, "ref_" + name)(_fp(a), _fp(cv), _fp(out), a.shape[0], a.shape[1])
    return out


def add_row_vector(a, rv): return _row_bcast("add_row_vector", a, rv)
def add_broadcast_rows(a, rv): return add_row_vector(a, rv)
def multiply_broadcast_rows(a, rv): return _row_bcast("multiply_broadcast_rows", a, rv)
def add_broadcast_cols(a, cv): return _col_bcast("add_broadcast_cols", a, cv)
def subtract_broadcast_cols(a, cv): return _col_bcast("subtract_broadcast_cols", a, cv)
def multiply_broadcast_cols(a, cv): return _col_bcast("multiply_broadcast_cols", a, cv)
def divide_broadcast_cols(a, cv): return _col_bcast("divide_broadcast_cols", a, cv)


def _scalar(name, a, s):
    a = f32(a)
    out = np.empty_like(a)
    getattr(lib, "ref_" + name)(_fp(a), float(s), _fp(out), a.shape[0], a.shape[1])
    return out


def multiply_scalar(a, s): return _scalar("multiply_scalar", a, s)
def add_scalar(a, s): return _scalar("add_scalar", a, s)
def divide_scalar(a, s): return _scalar("divide_scalar", a, s)
def pow_(a, e): return _scalar("pow", a, e)


def _unary(name, a):
    a = f32(a)
    out = np.empty_like(a)
    getattr(lib, "ref_" + name)(_fp(a), _fp(out), a.shape[0], a.shape[1])
    return out


def sqrt(a): return _unary("sqrt", a)
def neg(a): return _unary("neg", a)
def exp(a): return _unary("exp", a)
def log(a): return _unary("log", a)
def tanh(a): return _unary("tanh", a)
def sigmoid(a): return _unary("sigmoid", a)
def relu(a): return _unary("relu", a)
def gelu(a): return _unary("gelu", a)
def softmax_rows(a): return _unary("softmax_rows", a)
def silu(a): return _unary("silu", a)


def _reduce(name, a, out_shape):
    a = f32(a)
    out = np.empty(out_shape, dtype=np.float32)
    getattr(lib, "ref_" + name)(_fp(a), _fp(out), a.shape[0], a.shape[1])
    return out


def sum_rows(a): a = f32(a); return _reduce("sum_rows", a, (1, a.shape[1]))
def sum_along_cols(a): return sum_rows(a)
def sum_along_rows(a): a = f32(a); return _reduce("sum_along_rows", a, (a.shape[0], 1))
def mean_along_rows(a): a = f32(a); return _reduce("mean_along_rows", a, (a.shape[0], 1))
def variance_along_rows(a): a = f32(a); return _reduce("variance_along_rows", a, (a.shape[0], 1))
def max_along_rows(a): a = f32(a); return _reduce("max_along_rows", a, (a.shape[0], 1))


def transpose(a):
    a = f32(a)
    out = np.empty((a.shape[1], a.shape[0]), dtype=np.float32)
    lib.ref_transpose(_fp(a), _fp(out), a.shape[0], a.shape[1])
    return out


def clamp(a, lo, hi):
    a = f32(a)
    out = np.empty_like(a)
    lib.ref_clamp(_fp(a), float(lo), float(hi), _fp(out), a.shape[0], a.shape[1])
    return out


def sum_(a): a = f32(a); return float(lib.ref_sum(_fp(a), a.size))
def sum_abs(a): a = f32(a); return float(lib.ref_sum_abs(_fp(a), a.size))


def causal_mask(size):
    out = np.empty((size, size), dtype=np.float32)
    lib.ref_causal_mask(_fp(out), size)
    return out


def _check_targets(logits, targets):
    if len(targets) != logits.shape[0]:
        raise ValueError(f"targets length {len(targets)} must match logits rows {logits.shape[0]}")


def cross_entropy_loss(logits, targets):
    logits, targets = f32(logits), i32(targets)
    _check_targets(logits, targets)
    return float(lib.ref_cross_entropy_loss(_fp(logits), _ip(targets), logits.shape[0], logits.shape[1]))


def cross_entropy_gradient(logits, targets):
    logits, targets = f32(logits), i32(targets)
    _check_targets(logits, targets)
    out = np.empty_like(logits)
    lib.ref_cross_entropy_gradient(_fp(logits), _ip(targets), _fp(out), logits.shape[0], logits.shape[1])
    return out


def adamw_update(w, g, mt, vt, lr, beta1, beta2, eps, weight_decay, bc1, bc2):
    """In place on w, mt, vt (float32 C-contiguous arrays)."""
    lib.ref_adamw_update(_fp(w), _fp(f32(g)), _fp(mt), _fp(vt), w.size,
                         lr, beta1, beta2, eps, weight_decay, bc1, bc2)


def layer_norm_backward(dxhat, xhat, std, dim):
    dxhat, xhat, std = f32(dxhat), f32(xhat), f32(std)
    out = np.empty_like(dxhat)
    lib.ref_layer_norm_backward(_fp(dxhat), _fp(xhat), _fp(std), _fp(out), dxhat.shape[0], dim)
    return out


def scatter_add_rows(target, indices, grad):
    """In place on target."""
    indices, grad = i32(indices), f32(grad)
    lib.ref_scatter_add_rows(_fp(target), _ip(indices), len(indices), _fp(grad), target.shape[1])


def slice_rows(t, idx):
    t, idx = f32(t), i32(idx)
    out = np.empty((len(idx), t.shape[1]), dtype=np.float32)
    lib.ref_slice_rows(_fp(t), _ip(idx), len(idx), t.shape[1], _fp(out))
    return out


# ── layers ──────────────────────────────────────────────────────────────────
_sig("ref_linear", f32p, f32p, f32p, f32p, _I, _I, _I)
_sig("ref_rmsnorm", f32p, f32p, f32p, _I, _I)
_sig("ref_layernorm", f32p, f32p, f32p, f32p, _I, _I)
_sig("ref_swiglu", f32p, f32p, f32p, f32p, f32p, f32p, f32p, f32p, _I, _I, _I)
_sig("ref_rope_tables", _I, _I, f32p, f32p)
_sig("ref_rope_apply", f32p, f32p, _I, _I, _I, f32p, f32p, _I)
_sig("ref_split_heads", f32p, f32p, _I, _I, _I)
_sig("ref_merge_heads", f32p, f32p, _I, _I, _I)
_sig("ref_attention_heads", f32p, f32p, f32p, f32p, _I, _I, _I, _I)
_sig("ref_mhsa_forward", f32p, f32p, f32p, f32p, f32p, f32p, _I, _I, _I, f32p, f32p, _I)
_sig("ref_mla_forward", f32p, f32p, f32p, f32p, f32p, f32p, f32p, f32p, _I, _I, _I, _I, _I, f32p, f32p)
_sig("ref_q8_padded_k", _I, restype=_I)
_sig("ref_q8_quantize", f32p, _I, _I, i8p, f32p)
_sig("ref_q8_dequantize", i8p, f32p, _I, _I, f32p)

RMS_EPS = 1e-6
Q8_GROUP = 32


def linear(x, w, b):
    x, w, b = f32(x), f32(w), f32(b).reshape(1, -1)
    out = np.empty((x.shape[0], w.shape[1]), dtype=np.float32)
    lib.ref_linear(_fp(x), _fp(w), _fp(b), _fp(out), x.shape[0], w.shape[0], w.shape[1])
    return out


def rmsnorm(x, gamma):
    x, gamma = f32(x), f32(gamma).reshape(1, -1)
    out = np.empty_like(x)
    lib.ref_rmsnorm(_fp(x), _fp(gamma), _fp(out), x.shape[0], x.shape[1])
    return out


def layernorm(x, gamma, beta):
    x, gamma, beta = f32(x), f32(gamma).reshape(1, -1), f32(beta).reshape(1, -1)
    out = np.empty_like(x)
    lib.ref_layernorm(_fp(x), _fp(gamma), _fp(beta), _fp(out), x.shape[0], x.shape[1])
    return out


def swiglu(x, wg, bg, wu, bu, wd, bd):
    x, wg, bg, wu, bu, wd, bd = (f32(t) for t in (x, wg, bg, wu, bu, wd, bd))
    out = np.empty((x.shape[0], wd.shape[1]), dtype=np.float32)
    lib.ref_swiglu(_fp(x), _fp(wg), _fp(bg), _fp(wu), _fp(bu), _fp(wd), _fp(bd), _fp(out),
                   x.shape[0], wg.shape[0], wg.shape[1])
    return out


def rope_tables(head_dim, max_seq):
    cos = np.empty((max_seq, head_dim // 2), dtype=np.float32)
    sin = np.empty_like(cos)
    lib.ref_rope_tables(head_dim, max_seq, _fp(cos), _fp(sin))
    return cos, sin


def rope_apply(t, seq, n_heads, cos, sin, pos0=0):
    t = f32(t)
    out = np.empty_like(t)
    lib.ref_rope_apply(_fp(t), _fp(out), seq, n_heads, t.shape[1], _fp(cos), _fp(sin), pos0)
    return out


def split_heads(t, n_heads):
    t = f32(t)
    seq, d = t.shape
    out = np.empty((n_heads * seq, d // n_heads), dtype=np.float32)
    lib.ref_split_heads(_fp(t), _fp(out), seq, n_heads, d // n_heads)
    return out


def merge_heads(t, n_heads):
    t = f32(t)
    seq, hd = t.shape[0] // n_heads, t.shape[1]
    out = np.empty((seq, n_heads * hd), dtype=np.float32)
    lib.ref_merge_heads(_fp(t), _fp(out), seq, n_heads, hd)
    return out


def attention_heads(qh, kh, vh, n_heads, causal=True):
    qh, kh, vh = f32(qh), f32(kh), f32(vh)
    out = np.empty_like(qh)
    lib.ref_attention_heads(_fp(qh), _fp(kh), _fp(vh), _fp(out), qh.shape[0] // n_heads, n_heads,
                            qh.shape[1], 1 if causal else 0)
    return out


def mhsa_forward(x, wq, wk, wv, wo, n_heads, cos=None, sin=None, causal=True):
    x, wq, wk, wv, wo = (f32(t) for t in (x, wq, wk, wv, wo))
    out = np.empty_like(x)
    lib.ref_mhsa_forward(_fp(x), _fp(wq), _fp(wk), _fp(wv), _fp(wo), _fp(out), x.shape[0], x.shape[1],
                         n_heads, _fp(cos) if cos is not None else None,
                         _fp(sin) if sin is not None else None, 1 if causal else 0)
    return out


def mla_forward(x, wdq, wuq, wdkv, wuk, wuv, wo, n_heads, cos, sin):
    x, wdq, wuq, wdkv, wuk, wuv, wo = (f32(t) for t in (x, wdq, wuq, wdkv, wuk, wuv, wo))
    out = np.empty_like(x)
    lib.ref_mla_forward(_fp(x), _fp(wdq), _fp(wuq), _fp(wdkv), _fp(wuk), _fp(wuv), _fp(wo), _fp(out),
                        x.shape[0], x.shape[1], n_heads, wdq.shape[1], wdkv.shape[1], _fp(cos), _fp(sin))
    return out


def q8_quantize(w):
    """w [K x N] fp32 -> (q [N x Kp] int8, scales [N x Kp/32] fp32)."""
    w = f32(w)
    k, n = w.shape
    kp = lib.ref_q8_padded_k(k)
    q = np.empty((n, kp), dtype=np.int8)
    s = np.empty((n, kp // Q8_GROUP), dtype=np.float32)
    lib.ref_q8_quantize(_fp(w), k, n, q.ctypes.data_as(i8p), _fp(s))
    return q, s


def q8_dequantize(q, s, k):
    n = q.shape[0]
    out = np.empty((k, n), dtype=np.float32)
    lib.ref_q8_dequantize(np.ascontiguousarray(q).ctypes.data_as(i8p), _fp(f32(s)), k, n, _fp(out))
    return out


def q8_roundtrip(w):
    q, s = q8_quantize(w)
    return q8_dequantize(q, s, np.asarray(w).shape[0])


# ── models ──────────────────────────────────────────────────────────────────

class _Cfg(C.Structure):
    _fields_ = [("kind", _I), ("vocab", _I), ("max_seq", _I), ("d", _I), ("heads", _I), ("layers", _I),
                ("dff", _I), ("q_rank", _I), ("kv_rank", _I), ("init_scale", _F)]


lib.ref_set_fast_fill.argtypes = [_I]
lib.ref_set_fast_fill.restype = None
lib.ref_model_create.argtypes = [C.POINTER(_Cfg), C.c_int64]
lib.ref_model_create.restype = C.c_void_p
lib.ref_model_free.argtypes = [C.c_void_p]
lib.ref_model_q8_roundtrip.argtypes = [C.c_void_p]
lib.ref_model_weight.argtypes = [C.c_void_p, C.c_char_p, C.POINTER(_I), C.POINTER(_I)]
lib.ref_model_weight.restype = f32p
lib.ref_model_forward.argtypes = [C.c_void_p, i32p, _I, f32p]
lib.ref_model_forward.restype = _I
lib.ref_model_hidden.argtypes = [C.c_void_p, i32p, _I, _I, f32p]
lib.ref_model_hidden.restype = _I
lib.ref_model_reset_cache.argtypes = [C.c_void_p]
lib.ref_model_forward_cached.argtypes = [C.c_void_p, i32p, _I, f32p, _I]
lib.ref_model_forward_cached.restype = _I
lib.ref_sample_from_logits.argtypes = [f32p, _I, _F, _I, C.POINTER(_JR)]
lib.ref_sample_from_logits.restype = C.c_int32
lib.ref_generate.argtypes = [C.c_void_p, i32p, _I, _I, _F, _I, C.c_int64, _I, i32p, f32p]
lib.ref_generate.restype = _I


class Model:
    """LlamaModel / DeepSeekModel / GPTModel of the reference, seeded init included."""

    def __init__(self, *, vocab, max_seq, d, heads, layers, dff, seed, q_rank=0, kv_rank=0, timing_only_fill=False,
                 gpt=False, init_scale=0.2):
        """timing_only_fill: weights from a cheap hash instead of the seeded Gaussian stream - same
        sizes and arithmetic, different values; only for measuring the CPU path's speed.
        gpt: GPTModel (LayerNorm, GELU FNN, learned positions), every parameter times init_scale
        (GPTConfig.java default 0.2)."""
        self.kind = 2 if gpt else (1 if q_rank else 0)
        if gpt and q_rank:
            raise ValueError("a GPT model has no latent ranks")
        if vocab <= 0 or max_seq <= 0 or d <= 0 or heads <= 0 or layers <= 0 or dff <= 0:
            raise ValueError("config values must be > 0")
        if d % heads != 0:
            raise ValueError("dModel must be divisible by nHeads")
        self.cfg = _Cfg(self.kind, vocab, max_seq, d, heads, layers, dff, q_rank, kv_rank, init_scale)
        self.init_scale = init_scale
        self.vocab, self.max_seq, self.d, self.heads, self.layers, self.dff = vocab, max_seq, d, heads, layers, dff
        self.q_rank, self.kv_rank = q_rank, kv_rank
        lib.ref_set_fast_fill(1 if timing_only_fill else 0)
        try:
            self._h = lib.ref_model_create(C.byref(self.cfg), seed)
        finally:
            lib.ref_set_fast_fill(0)

    def close(self):
        if self._h:
            lib.ref_model_free(self._h)
            self._h = None

    def __del__(self):
        self.close()

    def q8_roundtrip(self):
        lib.ref_model_q8_roundtrip(self._h)

    def weight(self, name: str) -> np.ndarray:
        """View (no copy) of a weight: 'emb','gf','wlm','blm','L3.wq', ..."""
        r, c = _I(), _I()
        p = lib.ref_model_weight(self._h, name.encode(), C.byref(r), C.byref(c))
        if not p:
            raise KeyError(name)
        return np.ctypeslib.as_array(p, shape=(r.value, c.value))

    def weight_names(self):
        if self.kind == 2:      # GPTModel parameter order: tokEmb, posEmb, blocks {ln1, ln2, attn, mlp}, normF, lmHead
            names = ["emb", "pos"]
            per = ["g1", "be1", "g2", "be2", "wq", "wk", "wv", "wo", "wg", "bg", "wd", "bd"]
            tail = ["gf", "bf", "wlm", "blm"]
        else:
            names = ["emb"]
            per = (["g1", "g2", "wq", "wk", "wv", "wo"] if self.kind == 0 else
                   ["g1", "g2", "wdq", "wuq", "wdkv", "wuk", "wuv", "wo"]) + ["wg", "bg", "wu", "bu", "wd", "bd"]
            tail = ["gf", "wlm", "blm"]
        for l in range(self.layers):
            names += [f"L{l}.{w}" for w in per]
        return names + tail

    def forward(self, ids) -> np.ndarray:
        ids = i32(ids)
        out = np.empty((len(ids), self.vocab), dtype=np.float32)
        rc = lib.ref_model_forward(self._h, _ip(ids), len(ids), _fp(out))
        if rc == -2:
            raise ValueError(f"seqLen {len(ids)} exceeds maxSeq {self.max_seq}")
        if rc != 0:
            raise ValueError("Token id out of range")
        return out

    def hidden(self, ids, n_layers: int) -> np.ndarray:
        """The block stack's state after its first n_layers blocks, [len(ids) x d]: the input of block n_layers."""
        ids = i32(ids)
        out = np.empty((len(ids), self.d), dtype=np.float32)
        rc = lib.ref_model_hidden(self._h, _ip(ids), len(ids), n_layers, _fp(out))
        if rc != 0:
            raise ValueError(f"hidden failed rc={rc}")
        return out

    def reset_cache(self):
        lib.ref_model_reset_cache(self._h)

    def forward_cached(self, ids, last_only=False) -> np.ndarray:
        ids = i32(ids)
        out = np.empty((1 if last_only else len(ids), self.vocab), dtype=np.float32)
        rc = lib.ref_model_forward_cached(self._h, _ip(ids), len(ids), _fp(out), 1 if last_only else 0)
        if rc == -1:
            raise ValueError("Token id out of range")
        if rc != 0:
            raise ValueError("context exceeds maxSeqLen")
        return out

    def generate(self, prompt, max_new, temperature=1.0, top_k=1, seed=0, use_cache=False, return_logits=False):
        prompt = i32(prompt)
        out = np.empty(len(prompt) + max_new, dtype=np.int32)
        logits = np.empty((max_new, self.vocab), dtype=np.float32) if return_logits else None
        rc = lib.ref_generate(self._h, _ip(prompt), len(prompt), max_new, temperature, top_k, seed,
                              1 if use_cache else 0, _ip(out), _fp(logits) if return_logits else None)
        if rc != 0:
            raise ValueError(f"generate failed rc={rc}")
        return (out, logits) if return_logits else out


def sample_from_logits(logits, temperature, top_k, rnd: JavaRandom) -> int:
    logits = f32(logits).reshape(-1)
    return lib.ref_sample_from_logits(_fp(logits), logits.size, temperature, top_k, C.byref(rnd._r))
