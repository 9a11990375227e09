"""ctypes host layer over the C ABI of ``libfastnn_hip.so`` (include/fastnn_hip.h).

Loading never falls back to a CPU path: if the shared library is missing or a GPU entry
point fails, an exception is raised.
"""
from __future__ import annotations

import ctypes as C
import os
from dataclasses import dataclass
from typing import Optional

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libfastnn_hip.so")

DT_I8, DT_I4, DT_U8, DT_U4, DT_F8, DT_F8R, DT_F4, DT_I4CB = range(8)
ACT_NONE, ACT_RELU, ACT_GELU, ACT_SILU = range(4)
FLAG_DEVICE_PTRS = 1
FLAG_I4CB_AS_WRITTEN = 2
FLAG_ACT_F16_SINGLE = 4
FLAG_FORCE_GENERIC = 8
FLAG_PREFER_FMA = 16
FLAG_ACT_QUANT = 32
OPT_CODEBOOK_CACHE = 1
OPT_GEMV_ROW_TILES = 2
OPT_ROWS16_ROW_TILES = 3
OPT_ROWS16_MIN_M = 4
OPT_TILE_SHAPE = 5
OPT_TILE_SPLIT = 6
OPT_TILE_STAGES = 7
OPT_TILE_MIN_M = 8
OPT_GEMV_INT8 = 9
OPT_GEMM_INT8 = 10
OPT_GEMM_INT8_MIN_M = 11
OPT_CODEBOOK_EXPANDED = 12
OPT_GEMV_INT8_MAX_M = 13
OPT_CONV_EPILOGUE = 14
OPT_CONV_RANGES = 15
OPT_CONV_IMPLICIT = 16
OPT_FUSE_RESIDUAL = 17
OPT_FUSE_PREP = 18
OPT_STREAM_MIN_M = 19
OPT_STREAM_MAX_M = 20
OPT_STREAM_SHAPE = 21
OPT_DIGIT_PLANES = 22
OPT_GEMV_TILE_MAJOR = 23

STATUS_NAMES = {0: "Ok", 1: "Dispatch", 2: "Memory", 3: "UnsupportedOp", 4: "Compilation"}

# every symbol include/fastnn_hip.h declares
EXPORTED_SYMBOLS = [
    "fnn_hip_device_count", "fnn_hip_create", "fnn_hip_destroy", "fnn_hip_last_error", "fnn_hip_sync", "fnn_hip_set_option", "fnn_hip_get_option", "fnn_hip_stream",
    "fnn_hip_malloc", "fnn_hip_free", "fnn_hip_upload", "fnn_hip_download",
    "fnn_hip_weight_register", "fnn_hip_weight_lookup", "fnn_hip_weight_release", "fnn_hip_dequant",
    "fnn_hip_qmatmul", "fnn_hip_qmatmul_static", "fnn_hip_quantize_activations", "fnn_hip_dequantize_activations", "fnn_hip_quantize_activations_per_channel", "fnn_hip_dequantize_activations_per_channel", "fnn_hip_qmatmul_i8act", "fnn_hip_qconv2d", "fnn_hip_qconv2d_i8act",
    "fnn_hip_timer_start", "fnn_hip_timer_stop",
    "fnn_hip_graph_begin", "fnn_hip_graph_end", "fnn_hip_graph_launch", "fnn_hip_graph_destroy",
    "fnn_hip_workspace_epoch",
    "fnn_packed_words", "fnn_quantize_weights", "fnn_transpose_kn_to_nk", "fnn_hip_version",
]
# every symbol include/fastnn_hip_backend.h declares
BACKEND_SYMBOLS = [
    "fnn_backend_create", "fnn_backend_destroy", "fnn_backend_name", "fnn_backend_last_error",
    "fnn_backend_set_kernel_flags", "fnn_backend_set_graph_replay", "fnn_backend_set_option",
    "fnn_backend_allocate_arena", "fnn_backend_write_arena", "fnn_backend_read_arena",
    "fnn_plan_create", "fnn_plan_destroy", "fnn_plan_add_write_const", "fnn_plan_add_fill",
    "fnn_plan_add_memcopy", "fnn_plan_add_call_kernel", "fnn_plan_len", "fnn_plan_replayed", "fnn_plan_ranges_used", "fnn_plan_residuals_fused", "fnn_plan_operands_handed", "fnn_plan_arena_size",
    "fnn_plan_set_param_dims", "fnn_plan_from_bincode", "fnn_plan_to_bincode", "fnn_plan_describe",
    "fnn_backend_dispatch", "fnn_backend_dispatch_env", "fnn_backend_dispatch_from", "fnn_backend_dispatch_profile",
    "fnn_backend_dispatch_profile_env",
    "fnn_hip_elementwise", "fnn_hip_fill_f32", "fnn_hip_copy",
    "fnn_hip_copy2d_f32", "fnn_hip_concat_f32", "fnn_hip_maxpool2d_f32", "fnn_hip_avgpool2d_f32", "fnn_hip_upsample_nearest2d_f32",
]


class FnnError(RuntimeError):
    """A non-zero fnn_status; mirrors fastnn's BackendError variants."""

    def __init__(self, status: int, message: str):
        super().__init__(f"{STATUS_NAMES.get(status, status)} error: {message}")
        self.status = status
        self.kind = STATUS_NAMES.get(status, str(status))
        self.message = message


_lib = None


def load_library(path: Optional[str] = None):
    """Load libfastnn_hip.so; raises if it has not been built (no fallback)."""
    global _lib
    if _lib is not None and path is None:
        return _lib
    p = path or LIB_PATH
    if not os.path.exists(p):
        raise FileNotFoundError(
            f"{p} not found: build it with `python -m fastnn_amd.build` (hipcc, gfx950). "
            "There is no CPU fallback.")
    lib = C.CDLL(p)
    _prototype(lib)
    if path is None:
        _lib = lib
    return lib


_vp = C.c_void_p
_i64 = C.c_int64
_u64 = C.c_uint64
_sz = C.c_size_t


class Slice(C.Structure):
    """fnn_slice: BufferSlice {offset, size} in bytes."""
    _fields_ = [("offset", C.c_uint64), ("size", C.c_uint64)]


class DimExpr(C.Structure):
    """fnn_dim_expr: kind 0 Known(value), 1 Symbol(symbol), 2 Bounded{sym: symbol, max: value}."""
    _fields_ = [("kind", C.c_uint32), ("value", C.c_uint64), ("symbol", C.c_char_p)]


class WeightMeta(C.Structure):
    """fnn_weight_meta: QuantizedWeightMeta."""
    _fields_ = [("bit_width", C.c_uint64), ("scales", _vp), ("n_scales", C.c_uint64),
                ("zero_points", _vp), ("n_zero_points", C.c_uint64), ("shape", _vp), ("n_shape", C.c_uint64),
                ("quant_block_size", C.c_uint64), ("codebooks", _vp), ("n_codebooks", C.c_uint64)]


def _prototype(l):
    l.fnn_hip_device_count.restype = C.c_int
    l.fnn_hip_create.argtypes = [C.c_int, C.POINTER(_vp)]
    l.fnn_hip_destroy.argtypes = [_vp]
    l.fnn_hip_destroy.restype = None
    l.fnn_hip_last_error.argtypes = [_vp]
    l.fnn_hip_last_error.restype = C.c_char_p
    l.fnn_hip_sync.argtypes = [_vp]
    l.fnn_hip_set_option.argtypes = [_vp, C.c_int, _i64]
    l.fnn_hip_get_option.argtypes = [_vp, C.c_int, C.POINTER(_i64)]
    l.fnn_hip_stream.argtypes = [_vp]
    l.fnn_hip_stream.restype = _vp
    l.fnn_hip_malloc.argtypes = [_vp, _sz, C.POINTER(_vp)]
    l.fnn_hip_free.argtypes = [_vp, _vp]
    l.fnn_hip_upload.argtypes = [_vp, _vp, _vp, _sz]
    l.fnn_hip_download.argtypes = [_vp, _vp, _vp, _sz]
    l.fnn_hip_weight_register.argtypes = [_vp, C.c_uint64, C.c_int, _vp, _sz, _i64, _i64, _vp, _sz, _vp, _sz,
                                          C.c_int, _vp, C.POINTER(_vp)]
    l.fnn_hip_weight_lookup.argtypes = [_vp, C.c_uint64, C.POINTER(_vp)]
    l.fnn_hip_weight_release.argtypes = [_vp, _vp]
    l.fnn_hip_dequant.argtypes = [_vp, _vp, _vp, C.c_int]
    l.fnn_hip_qmatmul.argtypes = [_vp, _vp, _vp, _i64, _vp, C.c_int, _vp, C.c_int]
    l.fnn_hip_qmatmul_static.argtypes = [_vp, _vp, _vp, _i64, _vp, C.c_int, _vp, C.c_int]
    l.fnn_hip_quantize_activations.argtypes = [_vp, _vp, _i64, C.c_float, C.c_float, _vp, C.c_int]
    l.fnn_hip_quantize_activations_per_channel.argtypes = [_vp, _vp, C.c_uint64, C.c_uint64, C.c_uint32, _vp, _vp, _vp, C.c_uint64]
    l.fnn_hip_dequantize_activations_per_channel.argtypes = [_vp, _vp, C.c_uint64, _vp, C.c_uint64]
    l.fnn_hip_qmatmul_i8act.argtypes = [_vp, _vp, _vp, _i64, _vp, _vp, C.c_int]
    l.fnn_hip_qconv2d.argtypes = [_vp, _vp, _vp, _i64, _i64, _i64, _i64, C.c_int, C.c_int, C.c_int, C.c_int,
                                  C.c_int, C.c_int, _vp, C.c_int, _vp, _vp, C.c_int]
    l.fnn_hip_qconv2d_i8act.argtypes = [_vp, _vp, _vp, _i64, _i64, _i64, _i64, C.c_int, C.c_int, C.c_int, C.c_int,
                                        C.c_int, C.c_int, _vp, C.c_int, _vp, C.c_int]
    l.fnn_hip_timer_start.argtypes = [_vp]
    l.fnn_hip_timer_stop.argtypes = [_vp, C.POINTER(C.c_float)]
    l.fnn_hip_graph_begin.argtypes = [_vp]
    l.fnn_hip_graph_end.argtypes = [_vp, C.POINTER(_vp)]
    l.fnn_hip_graph_launch.argtypes = [_vp, _vp]
    l.fnn_hip_graph_destroy.argtypes = [_vp, _vp]
    l.fnn_hip_workspace_epoch.argtypes = [_vp]
    l.fnn_hip_workspace_epoch.restype = _u64
    l.fnn_packed_words.argtypes = [C.c_int, _i64, _i64]
    l.fnn_packed_words.restype = _sz
    l.fnn_quantize_weights.argtypes = [C.c_int, _vp, _i64, _i64, C.c_int, _vp, _vp, _vp, _vp]
    l.fnn_transpose_kn_to_nk.argtypes = [_vp, _i64, _i64, _vp]
    l.fnn_transpose_kn_to_nk.restype = None
    l.fnn_hip_version.restype = C.c_char_p
    l.fnn_backend_create.argtypes = [C.c_int, C.POINTER(_vp)]
    l.fnn_backend_destroy.argtypes = [_vp]
    l.fnn_backend_destroy.restype = None
    l.fnn_backend_name.argtypes = [_vp]
    l.fnn_backend_name.restype = C.c_char_p
    l.fnn_backend_set_kernel_flags.argtypes = [_vp, C.c_int]
    l.fnn_backend_set_graph_replay.argtypes = [_vp, C.c_int]
    l.fnn_backend_set_option.argtypes = [_vp, C.c_int, _i64]
    l.fnn_backend_last_error.argtypes = [_vp]
    l.fnn_backend_last_error.restype = C.c_char_p
    l.fnn_backend_allocate_arena.argtypes = [_vp, _u64]
    l.fnn_backend_write_arena.argtypes = [_vp, _u64, _vp, _u64]
    l.fnn_backend_read_arena.argtypes = [_vp, _u64, _vp, _u64]
    l.fnn_plan_create.argtypes = [_u64, C.POINTER(_vp)]
    l.fnn_plan_destroy.argtypes = [_vp]
    l.fnn_plan_destroy.restype = None
    l.fnn_plan_add_write_const.argtypes = [_vp, Slice, _vp, _u64]
    l.fnn_plan_add_fill.argtypes = [_vp, Slice, C.c_float]
    l.fnn_plan_add_memcopy.argtypes = [_vp, Slice, Slice]
    l.fnn_plan_add_call_kernel.argtypes = [_vp, C.c_char_p, C.POINTER(Slice), _u64, Slice, C.POINTER(Slice),
                                           C.POINTER(_u64), _u64, C.POINTER(WeightMeta)]
    l.fnn_plan_len.argtypes = [_vp]
    l.fnn_plan_len.restype = _u64
    l.fnn_plan_replayed.argtypes = [_vp]
    l.fnn_plan_replayed.restype = C.c_int
    l.fnn_plan_ranges_used.argtypes = [_vp]
    l.fnn_plan_ranges_used.restype = C.c_uint64
    l.fnn_plan_residuals_fused.argtypes = [_vp]
    l.fnn_plan_residuals_fused.restype = C.c_uint64
    l.fnn_plan_operands_handed.argtypes = [_vp]
    l.fnn_plan_operands_handed.restype = C.c_uint64
    l.fnn_backend_dispatch.argtypes = [_vp, _vp]
    l.fnn_backend_dispatch_env.argtypes = [_vp, _vp, C.POINTER(C.c_char_p), C.POINTER(_u64), _u64]
    l.fnn_backend_dispatch_from.argtypes = [_vp, _vp, C.POINTER(C.c_char_p), C.POINTER(_u64), _u64, _u64, C.POINTER(_u64)]
    l.fnn_plan_arena_size.argtypes = [_vp]
    l.fnn_plan_arena_size.restype = _u64
    l.fnn_plan_set_param_dims.argtypes = [_vp, _u64, C.POINTER(DimExpr), _u64]
    l.fnn_plan_from_bincode.argtypes = [_vp, _u64, C.POINTER(_vp)]
    l.fnn_plan_to_bincode.argtypes = [_vp, _vp, _u64, C.POINTER(_u64)]
    l.fnn_plan_describe.argtypes = [_vp, _u64, C.c_char_p, _u64]
    l.fnn_backend_dispatch_profile.argtypes = [_vp, _vp, C.POINTER(_u64), _u64]
    l.fnn_backend_dispatch_profile_env.argtypes = [_vp, _vp, C.POINTER(C.c_char_p), C.POINTER(_u64), _u64, C.POINTER(_u64), _u64]
    l.fnn_hip_elementwise.argtypes = [_vp, C.c_int, _vp, _vp, _u64, _vp, _u64]
    l.fnn_hip_fill_f32.argtypes = [_vp, _vp, _u64, C.c_float]
    l.fnn_hip_copy.argtypes = [_vp, _vp, _vp, _u64]
    l.fnn_hip_copy2d_f32.argtypes = [_vp, _vp, _u64, _u64, _vp, _u64, _u64, _u64, _u64]
    l.fnn_hip_concat_f32.argtypes = [_vp, _vp, _u64, _u64, _u64, _vp, _vp, _vp, _u64]
    l.fnn_hip_maxpool2d_f32.argtypes = [_vp, _vp, _u64, _vp, _u64, _u64, _u64, _u64, _u64, _u64, _u64, _u64, _vp, _u64]
    l.fnn_hip_avgpool2d_f32.argtypes = [_vp, _vp, _u64, _vp, _u64, _u64, _u64, _u64, _u64, _u64, _u64, _u64]
    l.fnn_hip_upsample_nearest2d_f32.argtypes = [_vp, _vp, _vp, _u64, _u64, _u64, _u64, _u64]


def _np_ptr(a: Optional[np.ndarray]):
    return None if a is None else a.ctypes.data_as(_vp)


def _as_ptr(x):
    """numpy array -> host pointer; int -> raw (device) pointer; None -> NULL."""
    if x is None:
        return None
    if isinstance(x, np.ndarray):
        return x.ctypes.data_as(_vp)
    return _vp(int(x))


@dataclass
class PackedWeight:
    """Host image of a quantised weight: what fastnn's pass stores in the constant's bytes
    plus QuantizedWeightMeta (src/backend/mod.rs:42-58)."""
    dtype: int
    rows: int                      # N (or OC)
    inner: int                     # K (or IC/g*KH*KW)
    words: np.ndarray              # uint32
    scales: np.ndarray             # float32
    zeros: np.ndarray              # float32 (empty for I4CB)
    qblock: int = 0
    codebook: Optional[np.ndarray] = None

    @property
    def bit_width(self) -> int:
        return 8 if self.dtype in (DT_I8, DT_U8, DT_F8, DT_F8R) else 4

    def packed_bytes(self) -> int:
        items = 32 // self.bit_width
        return self.rows * (-(-self.inner // items)) * 4


def quantize_weights(dtype: int, w_nk: np.ndarray, qblock: int = 32) -> PackedWeight:
    """Quantise a transposed [N,K] f32 matrix with fastnn's packer for `dtype` (host, no GPU)."""
    l = load_library()
    w = np.ascontiguousarray(w_nk, dtype=np.float32)
    if w.ndim != 2:
        raise FnnError(4, "quantize_weights expects a 2-D [N,K] matrix")
    rows, inner = w.shape
    words = np.zeros(l.fnn_packed_words(dtype, rows, inner), np.uint32)
    if dtype == DT_I4CB:
        bpr = -(-inner // qblock)
        scales = np.zeros(rows * bpr, np.float32)
        zeros = np.zeros(0, np.float32)
        cb = np.zeros(16, np.float32)
    else:
        scales = np.zeros(rows, np.float32)
        zeros = np.zeros(rows, np.float32)
        cb = None
    rc = l.fnn_quantize_weights(dtype, _np_ptr(w), rows, inner, qblock if dtype == DT_I4CB else 0,
                                _np_ptr(words), _np_ptr(scales), _np_ptr(zeros) if zeros.size else None,
                                _np_ptr(cb))
    if rc:
        raise FnnError(rc, f"fnn_quantize_weights failed for dtype {dtype} (NaN in a codebook weight?)")
    return PackedWeight(dtype, rows, inner, words, scales, zeros, qblock if dtype == DT_I4CB else 0, cb)


def quantize_weights_kn(dtype: int, w_kn: np.ndarray, qblock: int = 32) -> PackedWeight:
    """Logical [K,N] weight (as a graph holds it) -> transposed -> packed [N,K]."""
    l = load_library()
    w = np.ascontiguousarray(w_kn, dtype=np.float32)
    k, n = w.shape
    t = np.empty((n, k), np.float32)
    l.fnn_transpose_kn_to_nk(_np_ptr(w), k, n, _np_ptr(t))
    return quantize_weights(dtype, t, qblock)


class DeviceBuffer:
    """A device allocation owned by a HipContext."""

    def __init__(self, ctx: "HipContext", nbytes: int):
        self.ctx = ctx
        self.nbytes = nbytes
        p = _vp()
        ctx._check(ctx.lib.fnn_hip_malloc(ctx.handle, nbytes, C.byref(p)))
        self.ptr = p.value

    def upload(self, arr: np.ndarray, offset: int = 0):
        a = np.ascontiguousarray(arr)
        assert offset + a.nbytes <= self.nbytes
        self.ctx._check(self.ctx.lib.fnn_hip_upload(self.ctx.handle, _vp(self.ptr + offset), _np_ptr(a), a.nbytes))
        return self

    def download(self, dtype, count: int, offset: int = 0) -> np.ndarray:
        out = np.empty(count, dtype=dtype)
        assert offset + out.nbytes <= self.nbytes
        self.ctx._check(self.ctx.lib.fnn_hip_download(self.ctx.handle, _np_ptr(out), _vp(self.ptr + offset), out.nbytes))
        return out

    def free(self):
        if self.ptr:
            self.ctx.lib.fnn_hip_free(self.ctx.handle, _vp(self.ptr))
            self.ptr = 0


class HipContext:
    """One device + one HIP stream (fnn_hip_ctx)."""

    def __init__(self, device: int = 0):
        self.lib = load_library()
        h = _vp()
        rc = self.lib.fnn_hip_create(device, C.byref(h))
        if rc:
            raise FnnError(rc, self.lib.fnn_hip_last_error(None).decode())
        self.handle = h
        self._next_key = 1

    def close(self):
        if self.handle:
            self.lib.fnn_hip_destroy(self.handle)
            self.handle = None

    def __enter__(self):
        return self

    def __exit__(self, *a):
        self.close()

    def _check(self, rc: int):
        if rc:
            raise FnnError(rc, self.lib.fnn_hip_last_error(self.handle).decode())

    def sync(self):
        self._check(self.lib.fnn_hip_sync(self.handle))

    def set_option(self, option: int, value: int):
        """fnn_hip_set_option: per-context kernel selection (OPT_* constants)."""
        self._check(self.lib.fnn_hip_set_option(self.handle, option, value))

    def get_option(self, option: int) -> int:
        v = _i64()
        self._check(self.lib.fnn_hip_get_option(self.handle, option, C.byref(v)))
        return v.value

    def alloc(self, nbytes: int) -> DeviceBuffer:
        return DeviceBuffer(self, nbytes)

    def to_device(self, arr: np.ndarray) -> DeviceBuffer:
        a = np.ascontiguousarray(arr)
        return DeviceBuffer(self, max(a.nbytes, 16)).upload(a)

    # ---- weights ----
    def register(self, pw: PackedWeight, key: Optional[int] = None):
        if key is None:
            key = self._next_key
            self._next_key += 1
        h = _vp()
        self._check(self.lib.fnn_hip_weight_register(
            self.handle, key, pw.dtype, _np_ptr(pw.words), pw.words.size, pw.rows, pw.inner,
            _np_ptr(pw.scales) if pw.scales.size else None, pw.scales.size,
            _np_ptr(pw.zeros) if pw.zeros.size else None, pw.zeros.size, pw.qblock,
            _np_ptr(pw.codebook) if pw.codebook is not None else None, C.byref(h)))
        return h

    def release(self, wh):
        self._check(self.lib.fnn_hip_weight_release(self.handle, wh))

    def dequant(self, wh, rows: int, inner: int) -> np.ndarray:
        out = np.empty((rows, inner), np.float32)
        self._check(self.lib.fnn_hip_dequant(self.handle, wh, _np_ptr(out), 0))
        return out

    # ---- MatMul ----
    def qmatmul(self, wh, a: np.ndarray, n: int, bias: Optional[np.ndarray] = None, act: int = ACT_NONE,
                flags: int = 0) -> np.ndarray:
        """Host-pointer call: copies in, runs, copies out, synchronises."""
        a = np.ascontiguousarray(a, dtype=np.float32)
        m = a.shape[0]
        out = np.empty((m, n), np.float32)
        b = None if bias is None else np.ascontiguousarray(bias, dtype=np.float32)
        self._check(self.lib.fnn_hip_qmatmul(self.handle, wh, _np_ptr(a), m, _np_ptr(b), act, _np_ptr(out), flags))
        return out

    def qmatmul_dev(self, wh, a_ptr: int, m: int, out_ptr: int, bias_ptr: int = 0, act: int = ACT_NONE,
                    flags: int = 0):
        """Device-pointer call: only enqueues on the context's stream."""
        self._check(self.lib.fnn_hip_qmatmul(self.handle, wh, _vp(a_ptr), m, _vp(bias_ptr) if bias_ptr else None, act,
                                             _vp(out_ptr), flags | FLAG_DEVICE_PTRS))

    def qmatmul_static(self, wh, a_ptr: int, m: int, out_ptr: int, bias_ptr: int = 0, act: int = ACT_NONE,
                       flags: int = 0):
        """fnn_hip_qmatmul_static: the device-pointer MatMul that allocates nothing (static workspace)."""
        self._check(self.lib.fnn_hip_qmatmul_static(self.handle, wh, _vp(a_ptr), m, _vp(bias_ptr) if bias_ptr else None,
                                                    act, _vp(out_ptr), flags))

    def quantize_activations(self, x: np.ndarray, scale: float = 0.0, zp: float = 0.0) -> np.ndarray:
        x = np.ascontiguousarray(x, dtype=np.float32).reshape(-1)
        payload = np.zeros(8 + x.size, np.uint8)
        self._check(self.lib.fnn_hip_quantize_activations(self.handle, _np_ptr(x), x.size, scale, zp,
                                                          _np_ptr(payload), 0))
        return payload

    def quantize_activations_per_channel(self, x: np.ndarray, numel: int, scales, zero_points, payload: np.ndarray) -> np.ndarray:
        """Per-channel "quantize_activations" over the f32 values `x` (all of them readable: x_len = x.size) into a copy
        of `payload` (its bytes beyond what the kernel writes stay as passed in); returns the payload bytes."""
        x = np.ascontiguousarray(x, dtype=np.float32).reshape(-1)
        sc = np.ascontiguousarray(scales, dtype=np.float32)
        zp = np.ascontiguousarray(zero_points, dtype=np.float32)
        assert sc.size == zp.size
        payload = np.ascontiguousarray(payload, dtype=np.uint8)
        dx, dp = self.to_device(x), self.to_device(payload)
        try:
            self._check(self.lib.fnn_hip_quantize_activations_per_channel(self.handle, _vp(dx.ptr), x.size, numel, sc.size, _np_ptr(sc),
                                                                          _np_ptr(zp), _vp(dp.ptr), payload.size))
            self.sync()
            return dp.download(np.uint8, payload.size)
        finally:
            dx.free()
            dp.free()

    def dequantize_activations_per_channel(self, payload: np.ndarray, out: np.ndarray) -> np.ndarray:
        """Per-channel "dequantize_activations" of `payload` over a copy of the f32 array `out` (values the kernel does
        not write stay as passed in)."""
        payload = np.ascontiguousarray(payload, dtype=np.uint8)
        out = np.ascontiguousarray(out, dtype=np.float32).reshape(-1)
        dp, do = self.to_device(payload), self.to_device(out)
        try:
            self._check(self.lib.fnn_hip_dequantize_activations_per_channel(self.handle, _vp(dp.ptr), payload.size, _vp(do.ptr), out.size))
            self.sync()
            return do.download(np.float32, out.size)
        finally:
            dp.free()
            do.free()

    def qmatmul_i8act(self, wh, payload: np.ndarray, m: int, n: int, want_acc: bool = False, flags: int = 0):
        payload = np.ascontiguousarray(payload, dtype=np.uint8)
        out = np.empty((m, n), np.float32)
        acc = np.zeros((m, n), np.int32) if want_acc else None
        self._check(self.lib.fnn_hip_qmatmul_i8act(self.handle, wh, _np_ptr(payload), m, _np_ptr(out), _np_ptr(acc),
                                                   flags))
        return (out, acc) if want_acc else out

    def qconv2d(self, wh, x: np.ndarray, oc: int, kh: int, kw: int, stride: int, pad: int, dil: int, groups: int,
                bias: Optional[np.ndarray] = None, act: int = ACT_NONE, want_acc: bool = False, flags: int = 0):
        x = np.ascontiguousarray(x, dtype=np.float32)
        b, c, h, w = x.shape

        def osz(i, k):
            dk = (k - 1) * dil + 1
            return (i + 2 * pad - dk) // stride + 1 if i + 2 * pad >= dk else 0
        ho, wo = osz(h, kh), osz(w, kw)
        y = np.zeros((b, oc, ho, wo), np.float32)
        acc = np.zeros((b, oc, ho, wo), np.int32) if want_acc else None
        bb = None if bias is None else np.ascontiguousarray(bias, dtype=np.float32)
        self._check(self.lib.fnn_hip_qconv2d(self.handle, wh, _np_ptr(x), b, c, h, w, kh, kw, stride, pad, dil, groups,
                                             _np_ptr(bb), act, _np_ptr(y), _np_ptr(acc), flags))
        return (y, acc) if want_acc else y

    def qconv2d_i8act(self, wh, payload: np.ndarray, shape, oc: int, kh: int, kw: int, stride: int, pad: int, dil: int,
                      groups: int, bias: Optional[np.ndarray] = None, act: int = ACT_NONE, flags: int = 0):
        """conv2d_i8_i8 / conv2d_i4_i8: `payload` = [scale][zero][int8 NCHW of `shape`]."""
        payload = np.ascontiguousarray(payload, dtype=np.uint8)
        b, c, h, w = shape
        if payload.size != 8 + b * c * h * w:
            raise ValueError(f"payload holds {payload.size} bytes, 8 + B*C*H*W = {8 + b * c * h * w}")

        def osz(i, k):
            dk = (k - 1) * dil + 1
            return (i + 2 * pad - dk) // stride + 1 if i + 2 * pad >= dk else 0
        y = np.zeros((b, oc, osz(h, kh), osz(w, kw)), np.float32)
        bb = None if bias is None else np.ascontiguousarray(bias, dtype=np.float32)
        self._check(self.lib.fnn_hip_qconv2d_i8act(self.handle, wh, _np_ptr(payload), b, c, h, w, kh, kw, stride, pad,
                                                   dil, groups, _np_ptr(bb), act, _np_ptr(y), flags))
        return y

    # ---- timing / graphs ----
    def stream(self) -> int:
        """The context's hipStream_t as an integer (fnn_hip_stream)."""
        return self.lib.fnn_hip_stream(self.handle) or 0

    def timer_start(self):
        self._check(self.lib.fnn_hip_timer_start(self.handle))

    def timer_stop(self) -> float:
        ms = C.c_float()
        self._check(self.lib.fnn_hip_timer_stop(self.handle, C.byref(ms)))
        return ms.value

    def graph_begin(self):
        self._check(self.lib.fnn_hip_graph_begin(self.handle))

    def graph_end(self):
        g = _vp()
        self._check(self.lib.fnn_hip_graph_end(self.handle, C.byref(g)))
        return g

    def graph_launch(self, g):
        self._check(self.lib.fnn_hip_graph_launch(self.handle, g))

    def graph_destroy(self, g):
        self.lib.fnn_hip_graph_destroy(self.handle, g)
