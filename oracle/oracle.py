"""ctypes binding of the CPU oracle (``libfnn_oracle.so``).

TEST INFRASTRUCTURE ONLY.  Only ``tests/``, ``__graft_entry__.smoke()`` and the
``cpu_baseline`` leg of ``bench.py`` may import this module; the shipped package
never does.  It is the checker, not the thing measured or shipped.
"""
from __future__ import annotations

import ctypes as C
import os
import subprocess
from dataclasses import dataclass, field
from typing import Optional

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "libfnn_oracle.so")

I8, I4, U8, U4, F8, F8R, F4, I4CB = range(8)
ACT_NONE, ACT_RELU, ACT_GELU, ACT_SILU = range(4)
DT_NAMES = {I8: "i8", I4: "i4", U8: "u8", U4: "u4", F8: "f8", F8R: "f8r", F4: "f4", I4CB: "i4cb"}
MARGIN = 16


_BASE_SO = os.path.join(_HERE, "libfnn_cpu_baseline.so")


def build(force: bool = False) -> str:
    """Compile the oracle and the tuned CPU baseline with gcc (flags live in the Makefile)."""
    for so, src in ((_SO, "fnn_oracle.c"), (_BASE_SO, "fnn_cpu_baseline.c")):
        if force or not os.path.exists(so) or os.path.getmtime(so) < os.path.getmtime(os.path.join(_HERE, src)):
            subprocess.run(["make", "-C", _HERE, "-B", os.path.basename(so)], check=True, stdout=subprocess.DEVNULL)
    return _SO


_base_lib = None


def cpu_qgemm(p: "Packed", a, bias=None, act: int = 0, threads: int = 1) -> np.ndarray:
    """The tuned CPU baseline (fnn_cpu_baseline.c): AVX2 unpack + FMA dots, weight rows over `threads` threads.
    I8 and I4 per-channel weights only; raises for other types or on a CPU without AVX2/FMA."""
    global _base_lib
    if _base_lib is None:
        if not os.path.exists(_BASE_SO):
            build()
        _base_lib = C.CDLL(_BASE_SO)
        _base_lib.fnn_cpu_qgemm.argtypes = [C.c_int, C.c_void_p, C.c_int64, C.c_int64, C.c_void_p, C.c_void_p, C.c_void_p,
                                            C.c_int64, C.c_void_p, C.c_int, C.c_void_p, C.c_int]
    a = _f32(a)
    m, k = a.shape
    assert k == p.inner
    out = np.zeros((m, p.rows), np.float32)
    b = None if bias is None else _f32(bias)
    zeros = p.zeros if p.zeros.size == p.rows else None
    rc = _base_lib.fnn_cpu_qgemm(p.dt, p.words.ctypes.data_as(C.c_void_p), p.rows, k, p.scales.ctypes.data_as(C.c_void_p),
                                 None if zeros is None else zeros.ctypes.data_as(C.c_void_p), a.ctypes.data_as(C.c_void_p), m,
                                 None if b is None else b.ctypes.data_as(C.c_void_p), act, out.ctypes.data_as(C.c_void_p), threads)
    if rc:
        raise ValueError(f"fnn_cpu_qgemm rc={rc}")
    return out


_lib = None


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_SO):
            build()
        _lib = C.CDLL(_SO)
        _proto(_lib)
    return _lib


_f32p = np.ctypeslib.ndpointer(dtype=np.float32, flags="C_CONTIGUOUS")
_u32p = np.ctypeslib.ndpointer(dtype=np.uint32, flags="C_CONTIGUOUS")
_u8p = np.ctypeslib.ndpointer(dtype=np.uint8, flags="C_CONTIGUOUS")
_i32p = np.ctypeslib.ndpointer(dtype=np.int32, flags="C_CONTIGUOUS")
_sz = C.c_size_t


def _proto(l):
    l.fnn_or_items.argtypes = [C.c_int]
    l.fnn_or_unpack_word.argtypes = [C.c_int, C.c_uint32, _f32p]
    l.fnn_or_pack_word.argtypes = [C.c_int, _f32p]
    l.fnn_or_pack_word.restype = C.c_uint32
    for n in ("e4m3", "e5m2"):
        getattr(l, f"fnn_or_{n}_to_f32").argtypes = [C.c_uint8]
        getattr(l, f"fnn_or_{n}_to_f32").restype = C.c_float
        getattr(l, f"fnn_or_f32_to_{n}").argtypes = [C.c_float]
        getattr(l, f"fnn_or_f32_to_{n}").restype = C.c_uint8
    l.fnn_or_fp4_to_f32.argtypes = [C.c_uint8]
    l.fnn_or_fp4_to_f32.restype = C.c_float
    l.fnn_or_f32_to_fp4.argtypes = [C.c_float]
    l.fnn_or_f32_to_fp4.restype = C.c_uint8
    for n in ("i8x4_dot", "i4x8_dot", "f4x8_dot"):
        getattr(l, f"fnn_or_{n}").argtypes = [C.c_uint32, C.c_uint32]
        getattr(l, f"fnn_or_{n}").restype = C.c_int32
    for n in ("i8x4_sum", "i4x8_sum"):
        getattr(l, f"fnn_or_{n}").argtypes = [C.c_uint32]
        getattr(l, f"fnn_or_{n}").restype = C.c_int32
    l.fnn_or_packed_words.argtypes = [C.c_int, _sz, _sz]
    l.fnn_or_packed_words.restype = _sz
    l.fnn_or_from_f32_slice.argtypes = [C.c_int, _f32p, _sz, _sz, C.c_float, C.c_float, _u32p]
    l.fnn_or_quant_per_channel_asym.argtypes = [C.c_int, _f32p, _sz, _sz, _u32p, _f32p, _f32p]
    l.fnn_or_quant_per_channel_sym.argtypes = [C.c_int, _f32p, _sz, _sz, _u32p, _f32p, _f32p]
    l.fnn_or_kmeans16.argtypes = [_f32p, _sz, C.c_int, _f32p]
    l.fnn_or_quant_codebook.argtypes = [_f32p, _sz, _sz, _sz, _u32p, _f32p, _f32p]
    l.fnn_or_transpose.argtypes = [_f32p, _sz, _sz, _f32p]
    l.fnn_or_dequant.argtypes = [C.c_int, _u32p, _sz, _sz, C.c_void_p, _sz, C.c_void_p, _sz, _sz,
                                 C.c_void_p, _f32p]
    l.fnn_or_qmatmul.argtypes = [C.c_int, _u32p, _sz, _sz, C.c_void_p, _sz, C.c_void_p, _sz, _sz,
                                 C.c_void_p, _f32p, _sz, _f32p, C.c_int, _sz, C.c_int]
    l.fnn_or_bias_act.argtypes = [_f32p, _sz, _sz, C.c_void_p, C.c_int]
    l.fnn_or_act.argtypes = [C.c_float, C.c_int]
    l.fnn_or_act.restype = C.c_float
    l.fnn_or_quantize_activations.argtypes = [_f32p, _sz, _u8p]
    l.fnn_or_dequantize_activations.argtypes = [_u8p, _sz, _f32p, _sz]
    l.fnn_or_quantize_activations_calibrated.argtypes = [_f32p, _sz, C.c_float, C.c_float, _u8p]
    l.fnn_or_quantize_activations_per_channel.argtypes = [_f32p, _sz, _sz, _sz, _f32p, _f32p, _u8p, _sz]
    l.fnn_or_quantize_activations_per_channel.restype = C.c_int
    l.fnn_or_dequantize_activations_per_channel.argtypes = [_u8p, _sz, _f32p, _sz]
    l.fnn_or_dequantize_activations_per_channel.restype = C.c_int
    l.fnn_or_qmatmul_i8act.argtypes = [C.c_int, _u32p, _sz, _sz, C.c_void_p, _sz, C.c_void_p, _sz,
                                       _u8p, _sz, _sz, _f32p, C.c_void_p]
    l.fnn_or_conv_out_size.argtypes = [_sz] * 5
    l.fnn_or_conv_out_size.restype = _sz
    l.fnn_or_qconv2d_i8.argtypes = [_f32p, _sz, _sz, _sz, _sz, _u32p, _sz, C.c_void_p, _sz,
                                    C.c_void_p, _sz, C.c_void_p, _sz, _sz, _sz, _sz, _sz, _sz,
                                    C.c_int, _f32p, C.c_void_p, C.c_void_p, C.c_void_p]
    l.fnn_or_qconv2d_i4.argtypes = l.fnn_or_qconv2d_i8.argtypes
    l.fnn_or_qconv2d_i8payload.argtypes = [C.c_int, _u8p, _sz, _sz, _sz, _sz, _u32p, _sz, C.c_void_p, _sz, C.c_void_p,
                                           _sz, C.c_void_p, _sz, _sz, _sz, _sz, _sz, _sz, C.c_int, _f32p]
    l.fnn_or_qconv2d_float.argtypes = [C.c_int, _f32p, _sz, _sz, _sz, _sz, _u32p, _sz, C.c_void_p, _sz,
                                       C.c_void_p, _sz, _sz, C.c_void_p, C.c_void_p, _sz, _sz, _sz, _sz,
                                       _sz, _sz, C.c_int, _f32p]
    l.fnn_or_concat.argtypes = [C.c_void_p, C.c_void_p, _sz, _sz, _f32p, _sz]
    l.fnn_or_concat.restype = _sz
    l.fnn_or_slice.argtypes = [_f32p, _sz, _sz, _sz, _sz, _f32p, _sz]
    l.fnn_or_maxpool2d.argtypes = [_f32p, _sz, _sz, _sz, _sz, _sz, _sz, _sz, _sz, _f32p, _sz, C.c_void_p, _sz]
    l.fnn_or_avgpool2d.argtypes = [_f32p, _sz, _sz, _sz, _sz, _sz, _sz, _sz, _sz, _f32p, _sz]
    l.fnn_or_upsample_nearest2d.argtypes = [_f32p, _sz, _sz, _sz, _sz, _sz, _f32p]
    l.fnn_or_seeded_values.argtypes = [C.c_uint64, _sz, _f32p]


def _ptr(a: Optional[np.ndarray]):
    return None if a is None else a.ctypes.data_as(C.c_void_p)


def _f32(a) -> np.ndarray:
    return np.ascontiguousarray(a, dtype=np.float32)


@dataclass
class Packed:
    """A packed weight as fastnn's PackedTensor holds it (packed_tensor.rs:95-126)."""
    dt: int
    rows: int
    inner: int
    words: np.ndarray                   # uint32, rows*ceil(inner/ITEMS) + 16
    scales: np.ndarray                  # float32
    zeros: np.ndarray                   # float32 (empty for the codebook type)
    qblock: int = 0
    codebook: Optional[np.ndarray] = None
    extra: dict = field(default_factory=dict)

    @property
    def items(self) -> int:
        return items(self.dt)

    @property
    def words_per_row(self) -> int:
        return -(-self.inner // self.items)


def items(dt: int) -> int:
    return lib().fnn_or_items(dt)


def unpack_word(dt: int, w: int) -> np.ndarray:
    out = np.zeros(8, np.float32)
    lib().fnn_or_unpack_word(dt, w & 0xFFFFFFFF, out)
    return out[: items(dt)]


def pack_word(dt: int, vals) -> int:
    v = np.zeros(8, np.float32)
    v[: len(vals)] = vals
    return int(lib().fnn_or_pack_word(dt, v))


def seeded_values(seed: int, n: int) -> np.ndarray:
    out = np.zeros(n, np.float32)
    lib().fnn_or_seeded_values(seed, n, out)
    return out


def from_f32_slice(dt: int, data, rows: int, inner: int, scale: float, zero: float) -> Packed:
    data = _f32(data).reshape(-1)
    words = np.zeros(lib().fnn_or_packed_words(dt, rows, inner), np.uint32)
    lib().fnn_or_from_f32_slice(dt, data, rows, inner, scale, zero, words)
    return Packed(dt, rows, inner, words, np.array([scale], np.float32),
                  np.array([zero], np.float32))


def quantize(dt: int, w_nk, qblock: int = 32) -> Packed:
    """Quantise an [N,K] f32 matrix the way the reference's pass does for `dt`
    (quantization.rs:170-260 integer types, :281-495 float/codebook types)."""
    w = _f32(w_nk)
    rows, inner = w.shape
    flat = w.reshape(-1)
    words = np.zeros(lib().fnn_or_packed_words(dt, rows, inner), np.uint32)
    if dt == I4CB:
        bpr = -(-inner // qblock)
        scales = np.zeros(rows * bpr, np.float32)
        cb = np.zeros(16, np.float32)
        rc = lib().fnn_or_quant_codebook(flat, rows, inner, qblock, words, scales, cb)
        if rc:
            raise ValueError(f"codebook quantiser failed rc={rc}")
        return Packed(dt, rows, inner, words, scales, np.zeros(0, np.float32), qblock, cb)
    scales = np.zeros(rows, np.float32)
    zeros = np.zeros(rows, np.float32)
    if dt in (F8, F8R):
        lib().fnn_or_quant_per_channel_sym(dt, flat, rows, inner, words, scales, zeros)
    else:
        lib().fnn_or_quant_per_channel_asym(dt, flat, rows, inner, words, scales, zeros)
    return Packed(dt, rows, inner, words, scales, zeros)


def quantize_kn(dt: int, w_kn, qblock: int = 32) -> Packed:
    """Logical [K,N] weight -> transposed [N,K] -> packed (quantization.rs:144-156)."""
    w = _f32(w_kn)
    k, n = w.shape
    t = np.zeros((n, k), np.float32)
    lib().fnn_or_transpose(w.reshape(-1), k, n, t.reshape(-1))
    return quantize(dt, t, qblock)


def kmeans16(values, iters: int = 30) -> np.ndarray:
    v = _f32(values).reshape(-1)
    out = np.zeros(16, np.float32)
    rc = lib().fnn_or_kmeans16(v, v.size, iters, out)
    if rc:
        raise ValueError(f"kmeans16 rc={rc}")
    return out


def dequant(p: Packed) -> np.ndarray:
    out = np.zeros((p.rows, p.inner), np.float32)
    rc = lib().fnn_or_dequant(p.dt, p.words, p.rows, p.inner, _ptr(p.scales), p.scales.size,
                              _ptr(p.zeros) if p.zeros.size else None, p.zeros.size, p.qblock,
                              _ptr(p.codebook), out.reshape(-1))
    if rc:
        raise ValueError(f"dequant rc={rc}")
    return out


def qmatmul(p: Packed, a, order: int = 2, k_tile: int = 0, bias=None, act: int = ACT_NONE,
            i4cb_as_written: bool = False) -> np.ndarray:
    """out[M,N] = act(A . deq(W)^T + bias); order 0 scalar f32, 1 AVX2-order f32, 2 f64 accumulate."""
    a = _f32(a)
    m, k = a.shape
    assert k == p.inner
    out = np.zeros((m, p.rows), np.float32)
    rc = lib().fnn_or_qmatmul(p.dt, p.words, p.rows, k, _ptr(p.scales), p.scales.size,
                              _ptr(p.zeros) if p.zeros.size else None, p.zeros.size, p.qblock,
                              _ptr(p.codebook), a.reshape(-1), m, out.reshape(-1), order, k_tile,
                              int(i4cb_as_written))
    if rc:
        raise ValueError(f"qmatmul rc={rc}")
    if bias is not None or act != ACT_NONE:
        b = None if bias is None else _f32(bias)
        lib().fnn_or_bias_act(out.reshape(-1), m, p.rows, _ptr(b), act)
    return out


def act_fn(x: np.ndarray, act: int) -> np.ndarray:
    x = _f32(x).copy()
    lib().fnn_or_bias_act(x.reshape(-1), 1, x.size, None, act)
    return x


def quantize_activations(x, scale: Optional[float] = None, zp: float = 0.0) -> np.ndarray:
    x = _f32(x).reshape(-1)
    payload = np.zeros(8 + x.size, np.uint8)
    if scale is None:
        lib().fnn_or_quantize_activations(x, x.size, payload)
    else:
        lib().fnn_or_quantize_activations_calibrated(x, x.size, scale, zp, payload)
    return payload


def dequantize_activations(payload, n: int) -> np.ndarray:
    payload = np.ascontiguousarray(payload, np.uint8)
    out = np.zeros(n, np.float32)
    lib().fnn_or_dequantize_activations(payload, payload.size, out, n)
    return out


def quantize_activations_per_channel(x, numel: int, scales, zero_points, payload) -> np.ndarray:
    """The per-channel loops over a copy of `payload` (bytes they do not reach keep their value); ValueError where
    the reference would panic on a slice index."""
    x = _f32(x).reshape(-1)
    sc, zp = _f32(scales).reshape(-1), _f32(zero_points).reshape(-1)
    assert sc.size == zp.size
    payload = np.ascontiguousarray(payload, np.uint8).copy()
    if lib().fnn_or_quantize_activations_per_channel(x, x.size, numel, sc.size, sc, zp, payload, payload.size) != 0:
        raise ValueError("quantize_activations (per channel): the header does not fit the payload")
    return payload


def dequantize_activations_per_channel(payload, out) -> np.ndarray:
    payload = np.ascontiguousarray(payload, np.uint8)
    out = _f32(out).reshape(-1).copy()
    if lib().fnn_or_dequantize_activations_per_channel(payload, payload.size, out, out.size) != 0:
        raise ValueError("dequantize_activations (per channel): the header does not fit the payload")
    return out


def make_payload(scale: float, zp: float, q_i8) -> np.ndarray:
    q = np.asarray(q_i8, dtype=np.int8).reshape(-1)
    payload = np.zeros(8 + q.size, np.uint8)
    payload[0:4] = np.frombuffer(np.float32(scale).tobytes(), np.uint8)
    payload[4:8] = np.frombuffer(np.float32(zp).tobytes(), np.uint8)
    payload[8:] = q.view(np.uint8)
    return payload


def qmatmul_i8act(p: Packed, payload: np.ndarray, m: int, want_acc: bool = False):
    out = np.zeros((m, p.rows), np.float32)
    acc = np.zeros((m, p.rows), np.int32) if want_acc else None
    rc = lib().fnn_or_qmatmul_i8act(p.dt, p.words, p.rows, p.inner, _ptr(p.scales), p.scales.size,
                                    _ptr(p.zeros) if p.zeros.size else None, p.zeros.size,
                                    payload, payload.size, m, out.reshape(-1), _ptr(acc))
    if rc:
        raise ValueError(f"qmatmul_i8act rc={rc}")
    return (out, acc) if want_acc else out


def conv_out_size(inp, kernel, stride, pad, dil) -> int:
    return int(lib().fnn_or_conv_out_size(inp, kernel, stride, pad, dil))


def qconv2d_i8(x, p: Packed, kh: int, kw: int, stride: int, pad: int, dil: int, groups: int,
               bias=None, act: int = ACT_NONE, want_acc: bool = False):
    """x NCHW f32; p packed [OC, C/g*KH*KW] I8 weights (or I4 weights: the 16-level variant)."""
    x = _f32(x)
    b, c, h, w = x.shape
    oc = p.rows
    ho, wo = conv_out_size(h, kh, stride, pad, dil), conv_out_size(w, kw, stride, pad, dil)
    y = np.zeros((b, oc, ho, wo), np.float32)
    acc = np.zeros((b, oc, ho, wo), np.int32) if want_acc else None
    sa = np.zeros(b * groups, np.float32)
    za = np.zeros(b * groups, np.float32)
    bb = None if bias is None else _f32(bias)
    fn = lib().fnn_or_qconv2d_i4 if p.dt == I4 else lib().fnn_or_qconv2d_i8
    rc = fn(x.reshape(-1), b, c, h, w, p.words, oc, _ptr(p.scales),
            p.scales.size, _ptr(p.zeros), p.zeros.size, _ptr(bb), kh, kw,
            stride, pad, dil, groups, act, y.reshape(-1), _ptr(acc), _ptr(sa), _ptr(za))
    if rc:
        raise ValueError(f"qconv2d_i8 rc={rc}")
    if want_acc:
        return y, acc, sa, za
    return y


def qconv2d_float(x, p: Packed, kh: int, kw: int, stride: int, pad: int, dil: int, groups: int,
                  bias=None, act: int = ACT_NONE) -> np.ndarray:
    """Conv2d of the weight types without an integer kernel: f32 convolution with dequantised weights."""
    x = _f32(x)
    b, c, h, w = x.shape
    oc = p.rows
    ho, wo = conv_out_size(h, kh, stride, pad, dil), conv_out_size(w, kw, stride, pad, dil)
    y = np.zeros((b, oc, ho, wo), np.float32)
    bb = None if bias is None else _f32(bias)
    rc = lib().fnn_or_qconv2d_float(p.dt, x.reshape(-1), b, c, h, w, p.words, oc, _ptr(p.scales), p.scales.size,
                                    _ptr(p.zeros) if p.zeros.size else None, p.zeros.size, p.qblock,
                                    _ptr(p.codebook), _ptr(bb), kh, kw, stride, pad, dil, groups, act,
                                    y.reshape(-1))
    if rc:
        raise ValueError(f"qconv2d_float rc={rc}")
    return y


def concat(inputs, outer_count: int, out_len: int) -> np.ndarray:
    """The "concat" kernel: params [axis, inner_stride, outer_count]; inputs are flat f32 arrays."""
    arrs = [_f32(a).reshape(-1) for a in inputs]
    ptrs = (C.c_void_p * len(arrs))(*[a.ctypes.data for a in arrs])
    lens = (C.c_size_t * len(arrs))(*[a.size for a in arrs])
    out = np.zeros(out_len, np.float32)
    lib().fnn_or_concat(ptrs, lens, len(arrs), outer_count, out, out_len)
    return out


def slice_f32(x, start: int, end: int, stride: int, out_len: int) -> np.ndarray:
    """The "slice_f32" kernel: params [dim, start, end, stride = elements per index of the sliced dim]."""
    x = _f32(x).reshape(-1)
    out = np.zeros(out_len, np.float32)
    lib().fnn_or_slice(x, x.size, start, end, stride, out, out_len)
    return out


def maxpool2d(x, kernel: int, stride: int, pad: int, return_indices: bool = False):
    """"pool_f32" with is_max = 1; with return_indices also the i64 secondary output (kh*kernel + kw per window)."""
    x = _f32(x)
    n, c, h, w = x.shape
    ho = max(h + 2 * pad - kernel, 0) // stride + 1
    wo = max(w + 2 * pad - kernel, 0) // stride + 1
    out = np.zeros((n, c, ho, wo), np.float32)
    idx = np.zeros((n, c, ho, wo), np.int64) if return_indices else None
    lib().fnn_or_maxpool2d(x.reshape(-1), x.size, n, c, h, w, kernel, stride, pad, out.reshape(-1), out.size,
                           None if idx is None else idx.ctypes.data_as(C.c_void_p), 0 if idx is None else idx.size)
    return (out, idx) if return_indices else out


def avgpool2d(x, kernel: int, stride: int, pad: int) -> np.ndarray:
    x = _f32(x)
    n, c, h, w = x.shape
    ho = max(h + 2 * pad - kernel, 0) // stride + 1
    wo = max(w + 2 * pad - kernel, 0) // stride + 1
    out = np.zeros((n, c, ho, wo), np.float32)
    lib().fnn_or_avgpool2d(x.reshape(-1), x.size, n, c, h, w, kernel, stride, pad, out.reshape(-1), out.size)
    return out


def upsample_nearest2d(x, sh: int, sw: int) -> np.ndarray:
    x = _f32(x)
    n, c, h, w = x.shape
    out = np.zeros((n, c, h * sh, w * sw), np.float32)
    lib().fnn_or_upsample_nearest2d(x.reshape(-1), n * c, h, w, sh, sw, out.reshape(-1))
    return out


def qconv2d_i8payload(payload, shape, p: Packed, kh: int, kw: int, stride: int, pad: int, dil: int, groups: int,
                      bias=None, act: int = ACT_NONE) -> np.ndarray:
    """conv2d_i8_i8 / conv2d_i4_i8: `payload` = [scale][zero][B*C*H*W int8] of an NCHW tensor of `shape`."""
    payload = np.ascontiguousarray(payload, np.uint8)
    b, c, h, w = shape
    oc = p.rows
    ho, wo = conv_out_size(h, kh, stride, pad, dil), conv_out_size(w, kw, stride, pad, dil)
    y = np.zeros((b, oc, ho, wo), np.float32)
    bb = None if bias is None else _f32(bias)
    rc = lib().fnn_or_qconv2d_i8payload(p.dt, payload, payload.size, c, h, w, p.words, oc, _ptr(p.scales), p.scales.size,
                                        _ptr(p.zeros), p.zeros.size, _ptr(bb), kh, kw, stride, pad, dil, groups, act,
                                        y.reshape(-1))
    if rc:
        raise ValueError(f"qconv2d_i8payload rc={rc}")
    return y
