"""Python view of the host-side HipBackend (include/fastnn_hip_backend.h).

Mirrors fastnn's ``Backend`` trait surface for the quantised-MatMul path
(src/backend/mod.rs:133-255): ``ExecutablePlan`` holds ``Instruction``s over one byte
arena, ``HipBackend.dispatch`` runs them on the GPU.  Instruction and argument meaning
follow CpuBackend::dispatch (src/backend/cpu/mod.rs:2644-2683); a kernel without a GPU
implementation raises ``FnnError`` of kind ``UnsupportedOp`` whose message is the kernel
name.
"""
from __future__ import annotations

import ctypes as C
from typing import Optional, Sequence

import numpy as np

from . import lib as _l
import json

from .lib import DimExpr, FnnError, Slice, WeightMeta

BITS_OF = {_l.DT_I8: 8, _l.DT_I4: 4, _l.DT_U8: 8, _l.DT_U4: 4, _l.DT_F8: 8, _l.DT_F8R: 8, _l.DT_F4: 4, _l.DT_I4CB: 4}
KERNEL_OF = {_l.DT_I8: "matmul_i8", _l.DT_I4: "matmul_i4", _l.DT_U8: "matmul_u8", _l.DT_U4: "matmul_u4",
             _l.DT_F8: "matmul_f8", _l.DT_F8R: "matmul_f8r", _l.DT_F4: "matmul_f4", _l.DT_I4CB: "matmul_i4"}


def meta_of(pw: "_l.PackedWeight", shape: Optional[Sequence[int]] = None):
    """QuantizedWeightMeta of a packed weight (src/backend/mod.rs:40-58) as plain fields."""
    return dict(bit_width=BITS_OF[pw.dtype], scales=np.ascontiguousarray(pw.scales, np.float32),
                zero_points=np.ascontiguousarray(pw.zeros, np.float32),
                shape=list(shape) if shape is not None else [pw.rows, pw.inner],
                quant_block_size=pw.qblock if pw.dtype == _l.DT_I4CB else 0,
                codebooks=None if pw.codebook is None else np.ascontiguousarray(pw.codebook, np.float32).reshape(1, 16))


class ExecutablePlan:
    """ExecutablePlan {instructions, arena_size} (src/backend/mod.rs:109-131)."""

    def __init__(self, arena_size: int, _handle=None):
        self.lib = _l.load_library()
        if _handle is None:
            h = C.c_void_p()
            rc = self.lib.fnn_plan_create(arena_size, C.byref(h))
            if rc:
                raise FnnError(rc, "fnn_plan_create failed")
            _handle = h
        self.handle = _handle
        self.arena_size = arena_size

    @classmethod
    def load(cls, path_or_bytes) -> "ExecutablePlan":
        """ExecutablePlan::load (src/backend/mod.rs:124-130): a plan saved by fastnn with bincode."""
        data = path_or_bytes if isinstance(path_or_bytes, (bytes, bytearray)) else open(path_or_bytes, "rb").read()
        lib = _l.load_library()
        h = C.c_void_p()
        buf = (C.c_uint8 * max(len(data), 1)).from_buffer_copy(bytes(data) if data else b"\0")
        rc = lib.fnn_plan_from_bincode(buf, len(data), C.byref(h))
        if rc:
            msg = lib.fnn_backend_last_error(None)
            raise FnnError(rc, msg.decode() if msg else "fnn_plan_from_bincode failed")
        return cls(int(lib.fnn_plan_arena_size(h)), _handle=h)

    def to_bytes(self) -> bytes:
        """ExecutablePlan::save (src/backend/mod.rs:117-122) into memory."""
        need = C.c_uint64()
        self._ok(self.lib.fnn_plan_to_bincode(self.handle, None, 0, C.byref(need)), "save")
        buf = (C.c_uint8 * max(need.value, 1))()
        self._ok(self.lib.fnn_plan_to_bincode(self.handle, buf, need.value, C.byref(need)), "save")
        return bytes(buf[: need.value])

    def save(self, path: str):
        with open(path, "wb") as f:
            f.write(self.to_bytes())

    def describe(self, index: int) -> dict:
        """One instruction as a dict (fnn_plan_describe)."""
        buf = C.create_string_buffer(1 << 16)
        self._ok(self.lib.fnn_plan_describe(self.handle, index, buf, len(buf)), "describe")
        return json.loads(buf.value.decode())

    def set_param_dims(self, index: int, dims) -> "ExecutablePlan":
        """CallKernel.param_dims of instruction `index`: ints (Known), str (Symbol) or (str, max) (Bounded)."""
        arr = (DimExpr * max(len(dims), 1))()
        for i, d in enumerate(dims):
            if isinstance(d, str):
                arr[i] = DimExpr(1, 0, d.encode())
            elif isinstance(d, tuple):
                arr[i] = DimExpr(2, int(d[1]), d[0].encode())
            else:
                arr[i] = DimExpr(0, int(d), None)
        self._ok(self.lib.fnn_plan_set_param_dims(self.handle, index, arr, len(dims)), "param_dims")
        return self

    def __len__(self):
        return int(self.lib.fnn_plan_len(self.handle))

    @property
    def replayed(self) -> bool:
        """True when the last dispatch of this plan ran as a HIP-graph replay."""
        return bool(self.lib.fnn_plan_replayed(self.handle))

    @property
    def ranges_used(self) -> int:
        """Quantised Conv2d instructions that took their activation ranges from the instruction before them."""
        return int(self.lib.fnn_plan_ranges_used(self.handle))

    @property
    def residuals_fused(self) -> int:
        """add_f32 instructions whose sum the MatMul or Conv2d before them stored (no launch of their own)."""
        return int(self.lib.fnn_plan_residuals_fused(self.handle))

    @property
    def operands_handed(self) -> int:
        """MatMul instructions whose activation operand the MatMul before them prepared."""
        return int(self.lib.fnn_plan_operands_handed(self.handle))

    def _ok(self, rc, what):
        if rc:
            msg = self.lib.fnn_backend_last_error(None)
            raise FnnError(rc, f"{what}: {msg.decode() if msg else 'malformed instruction'}")

    def write_const(self, offset: int, data) -> "ExecutablePlan":
        buf = np.ascontiguousarray(data).view(np.uint8).reshape(-1)
        self._ok(self.lib.fnn_plan_add_write_const(self.handle, Slice(offset, buf.nbytes), buf.ctypes.data_as(C.c_void_p),
                                                   buf.nbytes), "WriteConst")
        return self

    def fill(self, offset: int, size: int, value: float) -> "ExecutablePlan":
        self._ok(self.lib.fnn_plan_add_fill(self.handle, Slice(offset, size), value), "Fill")
        return self

    def memcopy(self, dst, src) -> "ExecutablePlan":
        self._ok(self.lib.fnn_plan_add_memcopy(self.handle, Slice(*dst), Slice(*src)), "MemCopy")
        return self

    def call_kernel(self, kernel_name: str, inputs, output, params=(), meta: Optional[dict] = None,
                    secondary_output=None) -> "ExecutablePlan":
        """Instruction::CallKernel.  meta["codebooks"]: [n, 16] f32 (QuantizedWeightMeta.codebooks) or None;
        secondary_output: (offset, size) of CallKernel.secondary_output_slice or None."""
        ins = (Slice * max(len(inputs), 1))(*[Slice(o, s) for o, s in inputs])
        par = (C.c_uint64 * max(len(params), 1))(*[int(p) for p in params])
        mp = None
        keep = []
        if meta is not None:
            sc = np.ascontiguousarray(meta["scales"], np.float32)
            zp = np.ascontiguousarray(meta["zero_points"], np.float32)
            sh = np.ascontiguousarray(meta["shape"], np.uint64)
            cb = meta.get("codebooks")
            cb = None if cb is None else np.ascontiguousarray(cb, np.float32).reshape(-1, 16)
            keep = [sc, zp, sh, cb]
            m = WeightMeta(int(meta["bit_width"]), sc.ctypes.data_as(C.c_void_p), sc.size,
                           zp.ctypes.data_as(C.c_void_p), zp.size, sh.ctypes.data_as(C.c_void_p), sh.size,
                           int(meta.get("quant_block_size", 0)), None if cb is None else cb.ctypes.data_as(C.c_void_p),
                           0 if cb is None else cb.shape[0])
            mp = C.byref(m)
        sec = None if secondary_output is None else C.byref(Slice(*secondary_output))
        self._ok(self.lib.fnn_plan_add_call_kernel(self.handle, kernel_name.encode(), ins, len(inputs), Slice(*output), sec,
                                                   par, len(params), mp), kernel_name)
        del keep
        return self

    def close(self):
        if self.handle:
            self.lib.fnn_plan_destroy(self.handle)
            self.handle = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


class HipBackend:
    """Backend (src/backend/mod.rs:133-255): name / allocate_arena / write_arena / read_arena / dispatch."""

    def __init__(self, device: int = 0):
        self.lib = _l.load_library()
        h = C.c_void_p()
        rc = self.lib.fnn_backend_create(device, C.byref(h))
        if rc:
            msg = self.lib.fnn_backend_last_error(None)
            raise FnnError(rc, msg.decode() if msg else "fnn_backend_create failed")
        self.handle = h

    def _check(self, rc):
        if rc:
            raise FnnError(rc, self.lib.fnn_backend_last_error(self.handle).decode())

    @property
    def name(self) -> str:
        return self.lib.fnn_backend_name(self.handle).decode()

    def allocate_arena(self, total_bytes: int):
        self._check(self.lib.fnn_backend_allocate_arena(self.handle, total_bytes))

    def write_arena(self, offset: int, data):
        buf = np.ascontiguousarray(data).view(np.uint8).reshape(-1)
        self._check(self.lib.fnn_backend_write_arena(self.handle, offset, buf.ctypes.data_as(C.c_void_p), buf.nbytes))

    def read_arena(self, offset: int, size: int, dtype=np.uint8) -> np.ndarray:
        out = np.empty(size, np.uint8)
        self._check(self.lib.fnn_backend_read_arena(self.handle, offset, out.ctypes.data_as(C.c_void_p), size))
        return out.view(dtype)

    def set_kernel_flags(self, flags: int):
        """Extra FNN_FLAG_* bits for every MatMul / Conv2d call (e.g. lib.FLAG_ACT_F16_SINGLE)."""
        self._check(self.lib.fnn_backend_set_kernel_flags(self.handle, flags))

    def set_graph_replay(self, enabled: bool):
        """Resident plans replay as one HIP graph (default) or run instruction by instruction."""
        self._check(self.lib.fnn_backend_set_graph_replay(self.handle, 1 if enabled else 0))

    def set_option(self, option: int, value: int):
        """fnn_hip_set_option on the backend's context (lib.OPT_* constants)."""
        self._check(self.lib.fnn_backend_set_option(self.handle, option, value))

    def dispatch(self, plan: ExecutablePlan, shape_env: Optional[dict] = None):
        """Backend::dispatch; shape_env = {symbol: value} is the call's ShapeEnv (empty when omitted)."""
        if not shape_env:
            self._check(self.lib.fnn_backend_dispatch(self.handle, plan.handle))
            return
        names = (C.c_char_p * len(shape_env))(*[k.encode() for k in shape_env])
        values = (C.c_uint64 * len(shape_env))(*[int(v) for v in shape_env.values()])
        self._check(self.lib.fnn_backend_dispatch_env(self.handle, plan.handle, names, values, len(shape_env)))

    def dispatch_from(self, plan: ExecutablePlan, first: int = 0, shape_env: Optional[dict] = None):
        """One segment of a dispatch (fnn_backend_dispatch_from): returns None when the end of the plan was reached,
        else the index of the instruction whose kernel has no GPU implementation (run it elsewhere, resume behind it)."""
        env = shape_env or {}
        names = (C.c_char_p * max(len(env), 1))(*[k.encode() for k in env])
        values = (C.c_uint64 * max(len(env), 1))(*[int(v) for v in env.values()])
        stopped = C.c_uint64()
        rc = self.lib.fnn_backend_dispatch_from(self.handle, plan.handle, names, values, len(env), first, C.byref(stopped))
        if rc == 3:
            return int(stopped.value)
        self._check(rc)
        return None

    def dispatch_profile(self, plan: ExecutablePlan, shape_env: Optional[dict] = None):
        """Backend::dispatch_profile: nanoseconds per instruction, under the call's ShapeEnv (empty when omitted)."""
        n = len(plan)
        t = (C.c_uint64 * max(n, 1))()
        if not shape_env:
            self._check(self.lib.fnn_backend_dispatch_profile(self.handle, plan.handle, t, n))
        else:
            names = (C.c_char_p * len(shape_env))(*[k.encode() for k in shape_env])
            values = (C.c_uint64 * len(shape_env))(*[int(v) for v in shape_env.values()])
            self._check(self.lib.fnn_backend_dispatch_profile_env(self.handle, plan.handle, names, values, len(shape_env), t, n))
        return [int(t[i]) for i in range(n)]

    def close(self):
        if self.handle:
            self.lib.fnn_backend_destroy(self.handle)
            self.handle = None

    def __enter__(self):
        return self

    def __exit__(self, *a):
        self.close()
