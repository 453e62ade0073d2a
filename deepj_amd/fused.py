"""Direct access to the native runtime for the fused inference opcodes: buffer ids in a
range of their own (so they never collide with the ids a ComputeGraph hands out, which
restart at 0 after releaseAll - ComputeGraph.java:739 in the reference) and a small
encoder for the opcodes the reference's ComputeGraph has no record* method for.

The encodings are the ones include/deepj_hip.h documents; the native decode driver
emits exactly the same words.
"""
from __future__ import annotations

import numpy as np

from . import opcodes as op
from ._native import HipNative

FUSED_ID_BASE = 1 << 28


class DeviceBuffers:
    """Id allocator + upload/download helpers on top of the five GpuRuntime calls."""

    def __init__(self, base: int = FUSED_ID_BASE):
        self._next = base
        self._sizes: dict[int, int] = {}

    def alloc(self, floats: int) -> int:
        buf_id = self._next
        self._next += 1
        HipNative.nativeAllocBuffers([buf_id], [int(floats)], 1)
        self._sizes[buf_id] = int(floats)
        return buf_id

    def upload(self, array) -> int:
        a = np.ascontiguousarray(array)
        if a.dtype not in (np.float32, np.int32):
            a = a.astype(np.float32)
        buf_id = self.alloc(a.size)
        HipNative.nativeUploadBuffer(buf_id, a.reshape(-1))
        return buf_id

    def write(self, buf_id: int, array) -> None:
        a = np.ascontiguousarray(array)
        HipNative.nativeUploadBuffer(buf_id, a.reshape(-1))

    def download(self, buf_id: int, shape, dtype=np.float32) -> np.ndarray:
        out = np.empty(int(np.prod(shape)), dtype=dtype)
        HipNative.nativeDownloadBuffer(buf_id, out)
        return out.reshape(shape)

    def size(self, buf_id: int) -> int:
        return self._sizes[buf_id]

    def release(self, *ids: int) -> None:
        ids = [i for i in ids if i in self._sizes]
        for i in ids:
            del self._sizes[i]
        if ids:
            HipNative.nativeReleaseBuffers(ids, len(ids))

    def release_all(self) -> None:
        self.release(*list(self._sizes))


class Stream:
    """Accumulates command words; run() hands them to flushOps."""

    def __init__(self):
        self.words: list[int] = []

    def emit(self, *w: int) -> "Stream":
        self.words.extend(int(x) for x in w)
        return self

    # fused opcodes -----------------------------------------------------------
    def q8_quantize(self, src, dst, k, n, row_off=0, row_step=1, total_rows=None):
        return self.emit(op.OP_Q8_QUANTIZE, src, dst, k, n, row_off, row_step, n if total_rows is None else total_rows)

    def q8_dequantize(self, src, dst, k, n, row_off=0, row_step=1, total_rows=None):
        return self.emit(op.OP_Q8_DEQUANTIZE, src, dst, k, n, row_off, row_step, n if total_rows is None else total_rows)

    def q8_linear(self, x, w, out, m, k, n, *, gamma=-1, bias=-1, bias2=-1, residual=-1, swiglu=False, beta=-1,
                  gelu=False, attn_merge_hd=0):
        """beta >= 0 turns the gamma prologue into LayerNorm (beta travels in the bias2 word); attn_merge_hd > 0:
        x is the records buffer of attn_decode_records and the prologue merges it (head dim in the gamma word)."""
        if attn_merge_hd:
            flags = op.LIN_ATTN_MERGE | (op.LIN_BIAS if bias >= 0 else 0) | (op.LIN_RESIDUAL if residual >= 0 else 0)
            return self.emit(op.OP_Q8_LINEAR, x, w, out, m, k, n, flags, attn_merge_hd, bias, -1, residual)
        layernorm = beta >= 0
        if layernorm and swiglu:
            raise ValueError("LayerNorm prologue and SwiGLU share the bias2 word")
        flags = ((op.LIN_LAYERNORM if layernorm else (op.LIN_RMSNORM if gamma >= 0 else 0)) |
                 (op.LIN_BIAS if bias >= 0 else 0) | (op.LIN_RESIDUAL if residual >= 0 else 0) |
                 (op.LIN_SWIGLU if swiglu else 0) | (op.LIN_GELU if gelu else 0))
        return self.emit(op.OP_Q8_LINEAR, x, w, out, m, k, n, flags, gamma, bias, beta if layernorm else bias2, residual)

    def layernorm(self, x, gamma, beta, out, rows, cols):
        return self.emit(op.OP_LAYERNORM, x, gamma, beta, out, rows, cols)

    def add_positions(self, x, table, state, rows, d, max_seq):
        return self.emit(op.OP_ADD_POSITIONS, x, table, state, rows, d, max_seq)

    def rmsnorm(self, x, gamma, out, rows, cols): return self.emit(op.OP_RMSNORM, x, gamma, out, rows, cols)
    def silu_mul(self, gate, up, out, n): return self.emit(op.OP_SILU_MUL, gate, up, out, n)

    def embed_gather(self, table, ids, out, n_ids, d, vocab, ids_off=0):
        return self.emit(op.OP_EMBED_GATHER, table, ids, out, n_ids, d, vocab, ids_off)

    def rope_kv_store(self, qkv, q_out, k_cache, v_cache, state, cos, sin, S, H, hd, max_seq, layer):
        return self.emit(op.OP_ROPE_KV_STORE, qkv, q_out, k_cache, v_cache, state, cos, sin, S, H, hd, max_seq, layer)

    def rope_rows(self, x, out, state, cos, sin, rows, H, hd, max_seq, pos_from_row, row_stride=0, live_extra=-1):
        return self.emit(op.OP_ROPE_ROWS, x, out, state, cos, sin, rows, H, hd, max_seq, 1 if pos_from_row else 0,
                         row_stride, live_extra)

    def attention(self, q, k_cache, v_cache, out, state, scratch, S, H, hd, max_seq, layer):
        return self.emit(op.OP_ATTENTION, q, k_cache, v_cache, out, state, scratch, S, H, hd, max_seq, layer)

    def attention_kv(self, q, k, v, out, state, scratch, S, H, hd, max_seq, tok_stride=0, v_off=0):
        return self.emit(op.OP_ATTENTION_KV, q, k, v, out, state, scratch, S, H, hd, max_seq, 0, tok_stride, v_off)

    def argmax_rows(self, logits, out, rows, cols): return self.emit(op.OP_ARGMAX_ROWS, logits, out, rows, cols)

    def decode_advance(self, state, token, tokens, capacity, n_pos=1):
        return self.emit(op.OP_DECODE_ADVANCE, state, token, tokens, capacity, n_pos)

    def decode_next(self, logits, state, tokens, capacity, table, x, vocab, d, n_pos=1):
        return self.emit(op.OP_DECODE_NEXT, logits, state, tokens, capacity, table, x, vocab, d, n_pos)

    def attn_decode(self, qkv, k_cache, v_cache, out, state, scratch, cos, sin, H, hd, max_seq, layer):
        return self.emit(op.OP_ATTN_DECODE, qkv, k_cache, v_cache, out, state, scratch, cos, sin, H, hd, max_seq, layer)

    def attn_decode_records(self, qkv, k_cache, v_cache, records, state, cos, sin, H, hd, max_seq, layer):
        return self.emit(op.OP_ATTN_DECODE_RECORDS, qkv, k_cache, v_cache, records, state, cos, sin, H, hd, max_seq, layer)

    def append_rows(self, src, dst, state, rows, row_floats, max_rows, dst_off=0):
        return self.emit(op.OP_APPEND_ROWS, src, dst, state, rows, row_floats, max_rows, dst_off)

    def q8_linear_dyn(self, x, w, out, m_max, k, n, state, extra_rows, x_off=0):
        return self.emit(op.OP_Q8_LINEAR_DYN, x, w, out, m_max, k, n, state, extra_rows, x_off)

    def copy(self, src, dst, n, src_off=0, dst_off=0): return self.emit(op.OP_COPY, src, dst, n, src_off, dst_off)
    def fill(self, dst, bits, n): return self.emit(op.OP_FILL, dst, bits, n)
    def stream_read(self, src, sink, n): return self.emit(op.OP_STREAM_READ, src, sink, n)
    def nop(self, grid=1): return self.emit(op.OP_NOP, grid)
    def q8_prepare(self, w, prepared, k, rows): return self.emit(op.OP_Q8_PREPARE, w, prepared, k, rows)

    def q8_linear_rope(self, x, w, q_out, m, k, d, k_cache, v_cache, state, cos, sin, H, hd, max_seq, layer, *, gamma=-1,
                       bias=-1, beta=-1):
        """The q | k | v projection (weight rows 3 d) with ROPE_KV_STORE as its epilogue (HipNative.q8LinearRopeOk says
        for which shapes)."""
        layernorm = beta >= 0
        flags = ((op.LIN_LAYERNORM if layernorm else (op.LIN_RMSNORM if gamma >= 0 else 0)) | (op.LIN_BIAS if bias >= 0 else 0))
        return self.emit(op.OP_Q8_LINEAR_ROPE, x, w, q_out, m, k, d, flags, gamma, bias, beta, k_cache, v_cache, state, cos, sin,
                         H, hd, max_seq, layer)
    def matmul(self, a, b, out, m, n, k): return self.emit(op.OP_MATMUL, a, b, out, m, n, k)

    # execution -----------------------------------------------------------------
    def array(self) -> np.ndarray:
        return np.asarray(self.words, dtype=np.int32)

    def run(self) -> None:
        a = self.array()
        HipNative.nativeFlushOps(a, a.size)

    def profile(self, iters: int) -> np.ndarray:
        """Mean kernel duration of every op in microseconds (events on each op's own dispatch)."""
        return HipNative.profileOps(self.array(), iters)

    def time(self, iters: int) -> float:
        """Milliseconds for `iters` back-to-back executions (HIP events on the library's stream)."""
        return HipNative.timeOps(self.array(), iters)


def attn_decode_scratch_floats(H: int, hd: int) -> int:
    """Floats of the scratch buffer the fused ATTN_DECODE op needs (no initialisation required)."""
    return H * max(1, min(16, 512 // H)) * (hd + 4)


def attn_record_floats(H: int, hd: int) -> int:
    """Floats of the records buffer ATTN_DECODE_RECORDS writes and the ATTN_MERGE prologue reads."""
    return H * HipNative.attnRecordSplits() * (hd + 4)


def attention_scratch_floats(H: int, hd: int, max_seq: int = 0) -> int:
    """Floats a scratch buffer of ATTENTION / ATTENTION_KV must hold to serve any S (one row and short prompts of up to
    32 rows use it)."""
    return max(HipNative.attentionScratchFloats(S, H, hd, max_seq) for S in range(1, 34))
