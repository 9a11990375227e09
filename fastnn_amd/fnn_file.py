"""Reader / writer of fastnn's `.fnn` state-dict files (src/io/serialize.rs:113-281), host only.

Layout: magic "FNN\\0", u32 version, u64 count, then per parameter
  v3: u64 len + name (utf-8) | u64 byte-len + shape (i64 each) | u8 dtype tag | u64 len + data bytes
  v2: the same without the dtype tag (f32)
  v1: u64 len + name | u64 rank + rank x i64 | u64 element count + f32 data
all little endian.  Dtype tags (serialize.rs:225-245): 0 F32, 1 F64, 2 I32, 3 I64, 4 Bool, 5 F16, 6 BF16, 7 I4,
8 I8Scaled, 9 F8, 10 F8R, 11 F4.  The loader's consistency rule is followed as written: len(data) / DType::size()
(src/storage.rs:137-151; 1 for every packed type) must equal the product of the shape.  A packed tensor's scales and
zero points are not in the file (they live in the graph's node metadata), so packed payloads come back as raw bytes.

`AotExecutor(params=...)` takes the f32 entries of such a file as they are.
"""
from __future__ import annotations

import struct
from typing import Dict, Tuple

import numpy as np

MAGIC = b"FNN\x00"
FORMAT_VERSION = 3
DTYPE_OF_TAG = {0: np.float32, 1: np.float64, 2: np.int32, 3: np.int64, 4: np.bool_, 5: np.float16}
ELEM_SIZE = {0: 4, 1: 8, 2: 4, 3: 8, 4: 1, 5: 2, 6: 2, 7: 1, 8: 1, 9: 1, 10: 1, 11: 1}
TAG_NAMES = {0: "F32", 1: "F64", 2: "I32", 3: "I64", 4: "Bool", 5: "F16", 6: "BF16", 7: "I4", 8: "I8Scaled", 9: "F8",
             10: "F8R", 11: "F4"}


class FnnFormatError(ValueError):
    """FastnnError::Serialization"""


class _Reader:
    def __init__(self, data: bytes):
        self.d, self.i = data, 0

    def take(self, n: int) -> bytes:
        if n < 0 or self.i + n > len(self.d):
            raise FnnFormatError(f"unexpected end of file at byte {self.i} (wanted {n} more)")
        b = self.d[self.i:self.i + n]
        self.i += n
        return b

    def u64(self) -> int:
        return struct.unpack("<Q", self.take(8))[0]

    def prefixed(self) -> bytes:
        return self.take(self.u64())


def load_state_dict(path_or_bytes) -> Dict[str, Tuple[int, Tuple[int, ...], np.ndarray]]:
    """{name: (dtype tag, shape, array)}; arrays of tags 0-5 have their numpy dtype and shape, BF16 comes back as
    uint16 words, packed types (tags 7-11) as a flat uint8 array of the stored bytes."""
    data = path_or_bytes if isinstance(path_or_bytes, (bytes, bytearray)) else open(path_or_bytes, "rb").read()
    r = _Reader(bytes(data))
    magic = r.take(4)
    if magic != MAGIC:
        raise FnnFormatError(f"Invalid file format: expected magic bytes {list(MAGIC)}, got {list(magic)}")
    version = struct.unpack("<I", r.take(4))[0]
    if version > FORMAT_VERSION:
        raise FnnFormatError(f"Unsupported format version: {version}. Maximum supported version is {FORMAT_VERSION}")
    out = {}
    for _ in range(r.u64()):
        if version == 1:
            name = r.prefixed().decode("utf-8")
            shape = tuple(struct.unpack("<q", r.take(8))[0] & 0xffffffff for _ in range(r.u64()))   # `as u32` in the reader
            n = r.u64()
            arr = np.frombuffer(r.take(n * 4), "<f4").copy()
            out[name] = (0, shape, arr.reshape(shape) if int(np.prod(shape, dtype=np.int64)) == n else arr)
            continue
        name = r.prefixed().decode("utf-8")
        sb = r.prefixed()
        shape = tuple(struct.unpack(f"<{len(sb) // 8}q", sb[: len(sb) // 8 * 8]))
        tag = r.take(1)[0] if version >= 3 else 0
        if tag not in ELEM_SIZE:
            raise FnnFormatError(f"Unknown dtype tag {tag} for parameter '{name}'")
        payload = r.prefixed()
        numel = 1
        for d in shape:
            numel *= d
        if numel != len(payload) // ELEM_SIZE[tag]:
            raise FnnFormatError(f"Shape mismatch for parameter '{name}': shape {list(shape)} expects {numel} elements of "
                                 f"{TAG_NAMES[tag]}, but data has {len(payload) // ELEM_SIZE[tag]} elements")
        if tag in DTYPE_OF_TAG:
            arr = np.frombuffer(payload, np.dtype(DTYPE_OF_TAG[tag]).newbyteorder("<")).reshape(shape).copy()
        elif tag == 6:
            arr = np.frombuffer(payload, "<u2").reshape(shape).copy()
        else:
            arr = np.frombuffer(payload, np.uint8).copy()
        out[name] = (tag, shape, arr)
    return out


def save_state_dict(state: Dict[str, np.ndarray], path: str):
    """save_state_dict (serialize.rs:113-141), version 3, for arrays of the plain dtypes (tags 0-5)."""
    tag_of = {np.dtype(v): k for k, v in DTYPE_OF_TAG.items()}
    with open(path, "wb") as f:
        f.write(MAGIC + struct.pack("<IQ", FORMAT_VERSION, len(state)))
        for name, arr in state.items():
            a = np.ascontiguousarray(arr)
            if a.dtype not in tag_of:
                raise FnnFormatError(f"dtype {a.dtype} of '{name}' has no .fnn tag among the plain types")
            nb = name.encode("utf-8")
            f.write(struct.pack("<Q", len(nb)) + nb)
            f.write(struct.pack("<Q", 8 * a.ndim) + struct.pack(f"<{a.ndim}q", *a.shape))
            f.write(bytes([tag_of[a.dtype]]))
            raw = a.astype(a.dtype.newbyteorder("<"), copy=False).tobytes()
            f.write(struct.pack("<Q", len(raw)) + raw)


def f32_params(path_or_bytes) -> Dict[str, np.ndarray]:
    """The f32 entries of a `.fnn` file as {name: array}: what AotExecutor(params=...) takes."""
    return {k: v[2] for k, v in load_state_dict(path_or_bytes).items() if v[0] == 0}
