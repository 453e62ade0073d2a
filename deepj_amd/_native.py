"""ctypes binding of libdeepj_hip.so - the Python twin of the reference's
MetalNative (src/main/java/io/github/kirstenali/deepj/tensor/metal/MetalNative.java:10-57):
five calls into the native library plus the runtime-control extras.

The HIP library is the product: if it is missing or fails to load, every entry
point raises; there is no CPU fallback.
"""
from __future__ import annotations

import ctypes as C
import os

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
# DEEPJ_HIP_LIBRARY: another build of the library (python -m deepj_amd.build --no-kernarg-preload writes one for runs
# under a counter-collecting profiler); a relative path is taken from the package's parent directory
LIB_PATH = os.environ.get("DEEPJ_HIP_LIBRARY") or os.path.join(_HERE, "libdeepj_hip.so")
if not os.path.isabs(LIB_PATH):
    LIB_PATH = os.path.join(os.path.dirname(_HERE), LIB_PATH)

_i32p = C.POINTER(C.c_int32)
_f32p = C.POINTER(C.c_float)

_lib = None
_load_error: Exception | None = None


def _bind(lib: C.CDLL) -> None:
    lib.deepj_hip_init.argtypes = [C.c_int32]
    lib.deepj_hip_alloc_buffers.argtypes = [_i32p, _i32p, C.c_int32]
    lib.deepj_hip_upload.argtypes = [C.c_int32, C.c_void_p, C.c_int64]
    lib.deepj_hip_download.argtypes = [C.c_int32, C.c_void_p, C.c_int64]
    lib.deepj_hip_release.argtypes = [_i32p, C.c_int32]
    lib.deepj_hip_flush_ops.argtypes = [_i32p, C.c_int32]
    lib.deepj_hip_flush_ops_noalloc.argtypes = [_i32p, C.c_int32]
    lib.deepj_hip_last_error.restype = C.c_char_p
    lib.deepj_hip_pool_stats.argtypes = [C.POINTER(C.c_int64)]
    lib.deepj_hip_stream.restype = C.c_void_p
    lib.deepj_hip_attn_record_splits.restype = C.c_int32
    lib.deepj_hip_attention_scratch_floats.argtypes = [C.c_int32, C.c_int32, C.c_int32, C.c_int32]
    lib.deepj_hip_attention_scratch_floats.restype = C.c_int64
    lib.deepj_hip_q8_floats.argtypes = [C.c_int32, C.c_int32]
    lib.deepj_hip_q8_floats.restype = C.c_int64
    lib.deepj_hip_q8_prepared_floats.argtypes = [C.c_int32, C.c_int32]
    lib.deepj_hip_q8_prepared_floats.restype = C.c_int64
    lib.deepj_hip_q8_gemm_path.argtypes = [C.c_int32, C.c_int32, C.c_int32]
    lib.deepj_hip_q8_gemm_path.restype = C.c_int32
    lib.deepj_hip_q8_gemm_tile.argtypes = [C.c_int32, C.c_int32, C.c_int32, _i32p, _i32p, _i32p]
    lib.deepj_hip_q8_gemm_tile.restype = None
    lib.deepj_hip_q8_gemm_tile_prepared.argtypes = [C.c_int32, C.c_int32, C.c_int32, _i32p, _i32p, _i32p]
    lib.deepj_hip_q8_gemm_tile_prepared.restype = None
    lib.deepj_hip_q8_linear_rope_ok.argtypes = [C.c_int32, C.c_int32, C.c_int32]
    lib.deepj_hip_q8_linear_rope_ok.restype = C.c_int32
    lib.deepj_hip_clock_probe.argtypes = [_i32p, C.c_int32, C.c_int32, C.c_int32, C.c_int32, C.POINTER(C.c_uint64), C.POINTER(C.c_uint64)]
    lib.deepj_hip_clock_probe.restype = C.c_int
    lib.deepj_hip_q8_gemm_f16_extents.argtypes = [C.c_int32, C.c_int32, C.c_int32, C.c_int32, C.c_int32, C.POINTER(C.c_int64), C.POINTER(C.c_int64)]
    lib.deepj_hip_q8_gemm_f16_extents.restype = C.c_int32
    lib.deepj_hip_time_ops.argtypes = [_i32p, C.c_int32, C.c_int32, _f32p]
    lib.deepj_hip_profile_ops.argtypes = [_i32p, C.c_int32, C.c_int32, _f32p, C.c_int32, _i32p, _f32p, _i32p]
    lib.deepj_hip_graph_capture.argtypes = [_i32p, C.c_int32, _i32p]
    lib.deepj_hip_graph_launch.argtypes = [C.c_int32, C.c_int32]
    lib.deepj_hip_graph_destroy.argtypes = [C.c_int32]
    for name in ("deepj_hip_init", "deepj_hip_alloc_buffers", "deepj_hip_upload", "deepj_hip_download",
                 "deepj_hip_release", "deepj_hip_flush_ops", "deepj_hip_flush_ops_noalloc", "deepj_hip_synchronize", "deepj_hip_shutdown",
                 "deepj_hip_trim", "deepj_hip_pool_stats", "deepj_hip_time_ops", "deepj_hip_profile_ops", "deepj_hip_graph_capture",
                 "deepj_hip_graph_launch", "deepj_hip_graph_destroy"):
        getattr(lib, name).restype = C.c_int


def library() -> C.CDLL:
    """The loaded native library; raises RuntimeError when it is not there."""
    global _lib, _load_error
    if _lib is not None:
        return _lib
    if _load_error is None:
        try:
            if not os.path.exists(LIB_PATH):
                raise FileNotFoundError(f"{LIB_PATH} is not built (run: python -m deepj_amd.build)")
            lib = C.CDLL(LIB_PATH)
            _bind(lib)
            _lib = lib
            return lib
        except Exception as exc:  # noqa: BLE001 - remembered and re-raised on every use
            _load_error = exc
    raise RuntimeError(f"[DeepJ/HIP] native library unavailable: {_load_error}")


def _check(rc: int) -> None:
    if rc != 0:
        raise RuntimeError(library().deepj_hip_last_error().decode("utf-8", "replace"))


def _ids(a) -> np.ndarray:
    return np.ascontiguousarray(np.asarray(a, dtype=np.int32))


class HipNative:
    """Static facade, one method per native entry point (names as in MetalNative)."""

    @staticmethod
    def available() -> bool:
        try:
            library()
            return True
        except RuntimeError:
            return False

    @staticmethod
    def nativeAllocBuffers(ids, sizes, count: int) -> None:
        ids, sizes = _ids(ids), _ids(sizes)
        _check(library().deepj_hip_alloc_buffers(ids.ctypes.data_as(_i32p), sizes.ctypes.data_as(_i32p), count))

    @staticmethod
    def nativeUploadBuffer(buf_id: int, data: np.ndarray) -> None:
        data = np.ascontiguousarray(data)
        assert data.dtype.itemsize == 4, "buffers hold 32-bit words"
        _check(library().deepj_hip_upload(buf_id, data.ctypes.data, data.size))

    @staticmethod
    def nativeDownloadBuffer(buf_id: int, out: np.ndarray) -> None:
        assert out.flags["C_CONTIGUOUS"] and out.dtype.itemsize == 4
        _check(library().deepj_hip_download(buf_id, out.ctypes.data, out.size))

    @staticmethod
    def nativeReleaseBuffers(ids, count: int) -> None:
        ids = _ids(ids)
        _check(library().deepj_hip_release(ids.ctypes.data_as(_i32p), count))

    @staticmethod
    def nativeFlushOps(cmd_stream, length: int) -> None:
        cmd = _ids(cmd_stream)
        _check(library().deepj_hip_flush_ops(cmd.ctypes.data_as(_i32p), length))

    @staticmethod
    def flushOpsNoAlloc(cmd_stream, length: int) -> None:
        """flushOps over the library's static scratch array: no device allocation on this path."""
        cmd = _ids(cmd_stream)
        _check(library().deepj_hip_flush_ops_noalloc(cmd.ctypes.data_as(_i32p), length))

    # ── runtime control ─────────────────────────────────────────────────────
    @staticmethod
    def init(device: int = 0) -> None:
        _check(library().deepj_hip_init(device))

    @staticmethod
    def synchronize() -> None:
        _check(library().deepj_hip_synchronize())

    @staticmethod
    def shutdown() -> None:
        _check(library().deepj_hip_shutdown())

    @staticmethod
    def trim() -> None:
        _check(library().deepj_hip_trim())

    @staticmethod
    def poolStats() -> dict:
        out = (C.c_int64 * 4)()
        _check(library().deepj_hip_pool_stats(out))
        return {"live_buffers": out[0], "live_bytes": out[1], "cached_bytes": out[2], "driver_allocs": out[3]}

    @staticmethod
    def q8Floats(k: int, rows: int) -> int:
        return int(library().deepj_hip_q8_floats(k, rows))

    @staticmethod
    def attentionScratchFloats(S: int, H: int, hd: int, max_seq: int) -> int:
        return int(library().deepj_hip_attention_scratch_floats(S, H, hd, max_seq))

    @staticmethod
    def attnRecordSplits() -> int:
        return int(library().deepj_hip_attn_record_splits())

    @staticmethod
    def q8PreparedFloats(k: int, rows: int) -> int:
        """Floats of the buffer OP_Q8_PREPARE fills for a Q8 weight of `rows` rows over k inputs."""
        return int(library().deepj_hip_q8_prepared_floats(k, rows))

    @staticmethod
    def q8GemmTile(m: int, k: int, rows: int):
        """(tile rows, tile columns, workgroups sharing a tile's K) of the fp16 GEMM for this problem; rows 0: not taken."""
        r, c, s = C.c_int32(), C.c_int32(), C.c_int32()
        library().deepj_hip_q8_gemm_tile(m, k, rows, C.byref(r), C.byref(c), C.byref(s))
        return r.value, c.value, s.value

    @staticmethod
    def q8GemmTilePrepared(m: int, k: int, rows: int):
        """The same for a weight already in the fp16 GEMM's layout (OP_Q8_PREPARE): taken from 16 rows on."""
        r, c, s = C.c_int32(), C.c_int32(), C.c_int32()
        library().deepj_hip_q8_gemm_tile_prepared(m, k, rows, C.byref(r), C.byref(c), C.byref(s))
        return r.value, c.value, s.value

    @staticmethod
    def q8GemmF16Extents(m: int, k: int, rows: int, tile_rows: int = 0, tile_cols: int = 0):
        """(verdict, reach, size): bytes the fp16 GEMM's direct loads reach in (planes, fp16 weights, scales) against the
        bytes those hold; verdict 1 inside, 0 outside, -1 not a shape of these kernels.  Host arithmetic, no GPU call."""
        reach, size = (C.c_int64 * 3)(), (C.c_int64 * 3)()
        ok = int(library().deepj_hip_q8_gemm_f16_extents(m, k, rows, tile_rows, tile_cols, reach, size))
        return ok, list(reach), list(size)

    @staticmethod
    def q8LinearRopeOk(m: int, k: int, d: int) -> bool:
        """Whether OP_Q8_LINEAR_ROPE takes a projection of m rows over k inputs to 3 d outputs."""
        return bool(library().deepj_hip_q8_linear_rope_ok(m, k, d))

    @staticmethod
    def q8GemmPath(m: int, k: int, rows: int) -> int:
        """128 or 64 (rows per workgroup tile) when a Q8_LINEAR of m rows over such a weight runs on the fp16 direct-load
        GEMM, 0 when it runs on the bf16 kernels or the matvec."""
        return int(library().deepj_hip_q8_gemm_path(m, k, rows))

    @staticmethod
    def timeOps(cmd_stream, iters: int) -> float:
        cmd = _ids(cmd_stream)
        ms = C.c_float()
        _check(library().deepj_hip_time_ops(cmd.ctypes.data_as(_i32p), cmd.size, iters, C.byref(ms)))
        return float(ms.value)

    @staticmethod
    def profileOps(cmd_stream, iters: int, max_ops: int = 4096, detail: bool = False):
        """Mean kernel time (microseconds) of every op of the stream: a start and a stop event on each of the op's
        dispatches, summed per op.  detail=True also returns the op's longest dispatch (its main kernel) and its
        number of dispatches."""
        cmd = _ids(cmd_stream)
        out = np.empty(max_ops, dtype=np.float32)
        top = np.empty(max_ops, dtype=np.float32)
        cnt = np.empty(max_ops, dtype=np.int32)
        n = C.c_int32()
        _check(library().deepj_hip_profile_ops(cmd.ctypes.data_as(_i32p), cmd.size, iters,
                                               out.ctypes.data_as(_f32p), max_ops, C.byref(n),
                                               top.ctypes.data_as(_f32p), cnt.ctypes.data_as(_i32p)))
        if detail:
            return out[: n.value].copy(), top[: n.value].copy(), cnt[: n.value].copy()
        return out[: n.value].copy()

    @staticmethod
    def clockProbe(cmd_stream, iters: int, samples: int, sleep_reps: int = 1):
        """Runs the stream `iters` times while a one-wavefront kernel on a second stream samples the shader clock.
        Returns (MHz per sampling interval, wall time of each interval's end in microseconds from the first sample,
        (begin, end) of the stream's runs on the same time axis)."""
        cmd = _ids(cmd_stream)
        pairs = np.zeros(2 * samples, dtype=np.uint64)
        window = np.zeros(2, dtype=np.uint64)
        _check(library().deepj_hip_clock_probe(cmd.ctypes.data_as(_i32p), cmd.size, iters, samples, sleep_reps,
                                               pairs.ctypes.data_as(C.POINTER(C.c_uint64)), window.ctypes.data_as(C.POINTER(C.c_uint64))))
        clk, wall = pairs[0::2].astype(np.int64), pairs[1::2].astype(np.int64)
        dw = np.maximum(np.diff(wall), 1)
        mhz = np.diff(clk) / dw * 100.0
        t = (wall[1:] - wall[0]) / 100.0
        win = ((int(window[0]) - int(wall[0])) / 100.0, (int(window[1]) - int(wall[0])) / 100.0)
        return mhz, t, win

    @staticmethod
    def graphCapture(cmd_stream) -> int:
        cmd = _ids(cmd_stream)
        h = C.c_int32()
        _check(library().deepj_hip_graph_capture(cmd.ctypes.data_as(_i32p), cmd.size, C.byref(h)))
        return int(h.value)

    @staticmethod
    def graphLaunch(handle: int, times: int = 1) -> None:
        _check(library().deepj_hip_graph_launch(handle, times))

    @staticmethod
    def graphDestroy(handle: int) -> None:
        _check(library().deepj_hip_graph_destroy(handle))
