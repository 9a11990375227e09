#!/usr/bin/env python3
"""Hand-assembles the byte image of a saved fastnn ExecutablePlan (tests/golden/executable_plan.bin) and an annotated
listing of it (executable_plan.txt).

No file written by fastnn itself exists in this environment (no Rust toolchain to run ExecutablePlan::save), so the
image is put together field by field from the serde-derived layout of the reference's types under bincode 1.3 with its
default options (Cargo.lock pins bincode 1.3.3): little endian, usize/u64 as 8 bytes, enum variant index as u32,
Vec/String length as u64, Option as one tag byte, f32 as 4 bytes, [f32; 16] without a length, Arc<T> as T.
Types (paths relative to the fastnn tree): ExecutablePlan src/backend/mod.rs:100-107, Instruction :60-98 (variant
order CallKernel, MemCopy, Fill, WriteConst), BufferSlice :27-31, QuantizedWeightMeta :40-58, DimExpr
src/ir/node.rs:163-167 (variant order Known, Symbol, Bounded), NodeId = usize src/ir/node.rs:8.

Every emit() call below is one field; the listing records offset, bytes and meaning.  Run from the repository root:
    python tests/golden/make_plan_fixture.py
"""
import os
import struct

HERE = os.path.dirname(os.path.abspath(__file__))
out = bytearray()
listing = []


def emit(fmt, value, what):
    b = struct.pack("<" + fmt, *value) if isinstance(value, tuple) else struct.pack("<" + fmt, value)
    listing.append(f"{len(out):5d}  {b.hex():<34s} {what}")
    out.extend(b)


def emit_bytes(b, what):
    listing.append(f"{len(out):5d}  {bytes(b[:12]).hex()}{'..' if len(b) > 12 else '':<10s} {what} ({len(b)} bytes)")
    out.extend(b)


def usize(v, what): emit("Q", v, what + ": usize")
def slice_(off, size, what):
    usize(off, what + ".offset")
    usize(size, what + ".size")
def string(s, what):
    usize(len(s), what + " length")
    emit_bytes(s.encode(), what + " utf-8")
def f32s(vals, what):
    usize(len(vals), what + " length")
    for i, v in enumerate(vals):
        emit("f", v, f"{what}[{i}]: f32")
def usizes(vals, what):
    usize(len(vals), what + " length")
    for i, v in enumerate(vals):
        usize(v, f"{what}[{i}]")


# I8 weight [N=4, K=8]: row r = bytes (two u32 words per row, lane i of a word at bits [8i, 8i+8))
W_ROWS = [[1, -1, 2, -2, 3, -3, 4, -4], [5, 6, 7, 8, -5, -6, -7, -8], [127, -128, 0, 1, -1, 64, -64, 10], [0, 0, 0, 9, 0, 0, -9, 0]]
W_BYTES = b"".join(struct.pack("<8b", *r) for r in W_ROWS)
BIAS = [0.5, -0.25, 1.0, 0.0]
# I4 codebook weight [N=2, K=32]: 4 words per row, nibble i of a word at bits [4i, 4i+4)
CB_IDX = [[(3 * k + r) % 16 for k in range(32)] for r in range(2)]
CB_BYTES = b"".join(struct.pack("<I", sum(n << (4 * i) for i, n in enumerate(row[w * 8:(w + 1) * 8]))) for row in CB_IDX for w in range(4))
CODEBOOK = [(-1.0 + 2.0 * i / 15.0) for i in range(16)]

usize(8, "ExecutablePlan.instructions length")

emit("I", 3, "[0] Instruction variant 3 = WriteConst")
slice_(128, 32, "[0] dst")
usize(len(W_BYTES), "[0] data length")
emit_bytes(W_BYTES, "[0] data: I8x4 words of the [4, 8] weight")

emit("I", 3, "[1] Instruction variant 3 = WriteConst")
slice_(192, 16, "[1] dst")
usize(16, "[1] data length")
emit_bytes(struct.pack("<4f", *BIAS), "[1] data: bias [4] f32")

emit("I", 2, "[2] Instruction variant 2 = Fill")
slice_(256, 32, "[2] dst")
emit("f", 0.5, "[2] value: f32")

emit("I", 0, "[3] Instruction variant 0 = CallKernel")
string("matmul_i8_relu", "[3] kernel_name")
usize(3, "[3] input_slices length")
slice_(0, 64, "[3] input_slices[0] (activations [B, 8] f32, room for B = 2)")
slice_(128, 32, "[3] input_slices[1] (weight words)")
slice_(192, 16, "[3] input_slices[2] (bias)")
slice_(256, 32, "[3] output_slice")
emit("B", 0, "[3] secondary_output_slice: None")
usizes([2, 8, 4], "[3] params [M, K, N]")
emit("B", 1, "[3] node_id: Some")
usize(7, "[3] node_id value")
emit("B", 1, "[3] param_dims: Some")
usize(3, "[3] param_dims length")
emit("I", 1, "[3] param_dims[0] DimExpr variant 1 = Symbol")
string("B", "[3] param_dims[0] symbol")
emit("I", 0, "[3] param_dims[1] DimExpr variant 0 = Known")
emit("Q", 8, "[3] param_dims[1] value: u64")
emit("I", 0, "[3] param_dims[2] DimExpr variant 0 = Known")
emit("Q", 4, "[3] param_dims[2] value: u64")
emit("B", 1, "[3] weight_meta: Some(Arc<QuantizedWeightMeta>)")
usize(8, "[3] weight_meta.bit_width")
f32s([0.5, 0.25, 1.0, 2.0], "[3] weight_meta.scales")
f32s([0.0, 0.5, -1.0, 0.0], "[3] weight_meta.zero_points")
usizes([4, 8], "[3] weight_meta.shape")
usize(0, "[3] weight_meta.quant_block_size")
usize(0, "[3] weight_meta.codebooks length")

emit("I", 1, "[4] Instruction variant 1 = MemCopy")
slice_(320, 32, "[4] dst")
slice_(256, 32, "[4] src")

emit("I", 0, "[5] Instruction variant 0 = CallKernel")
string("pool_f32", "[5] kernel_name")
usize(1, "[5] input_slices length")
slice_(320, 32, "[5] input_slices[0] ([1, 2, 2, 2] f32)")
slice_(384, 8, "[5] output_slice ([1, 2, 1, 1] f32)")
emit("B", 1, "[5] secondary_output_slice: Some")
slice_(392, 16, "[5] secondary_output_slice (i64 window positions)")
usizes([2, 2, 0, 1, 1, 2, 2, 2], "[5] params [kernel, stride, padding, is_max, N, C, H, W]")
emit("B", 0, "[5] node_id: None")
emit("B", 0, "[5] param_dims: None")
emit("B", 0, "[5] weight_meta: None")

emit("I", 3, "[6] Instruction variant 3 = WriteConst")
slice_(512, 32, "[6] dst")
usize(len(CB_BYTES), "[6] data length")
emit_bytes(CB_BYTES, "[6] data: I4x8 codebook indices of the [2, 32] weight")

emit("I", 0, "[7] Instruction variant 0 = CallKernel")
string("matmul_i4", "[7] kernel_name")
usize(2, "[7] input_slices length")
slice_(576, 512, "[7] input_slices[0] (activations [B, 32] f32, room for B = 4)")
slice_(512, 32, "[7] input_slices[1] (codebook indices)")
slice_(1152, 32, "[7] output_slice ([B, 2] f32, room for B = 4)")
emit("B", 0, "[7] secondary_output_slice: None")
usizes([4, 32, 2], "[7] params [M, K, N]")
emit("B", 0, "[7] node_id: None")
emit("B", 1, "[7] param_dims: Some")
usize(3, "[7] param_dims length")
emit("I", 2, "[7] param_dims[0] DimExpr variant 2 = Bounded")
string("B", "[7] param_dims[0] sym")
emit("Q", 4, "[7] param_dims[0] max: u64")
emit("I", 0, "[7] param_dims[1] DimExpr variant 0 = Known")
emit("Q", 32, "[7] param_dims[1] value: u64")
emit("I", 0, "[7] param_dims[2] DimExpr variant 0 = Known")
emit("Q", 2, "[7] param_dims[2] value: u64")
emit("B", 1, "[7] weight_meta: Some(Arc<QuantizedWeightMeta>)")
usize(4, "[7] weight_meta.bit_width")
f32s([0.75, 1.5], "[7] weight_meta.scales (one per block of 32: [2 rows x 1 block])")
f32s([], "[7] weight_meta.zero_points")
usizes([2, 32], "[7] weight_meta.shape")
usize(32, "[7] weight_meta.quant_block_size")
usize(1, "[7] weight_meta.codebooks length")
for i, v in enumerate(CODEBOOK):
    emit("f", v, f"[7] weight_meta.codebooks[0][{i}]: f32 (array element, no length)")

usize(1280, "ExecutablePlan.arena_size")
usizes([0, 0, 0, 1, 2, 3, 0, 1], "ExecutablePlan.levels")

with open(os.path.join(HERE, "executable_plan.bin"), "wb") as f:
    f.write(out)
with open(os.path.join(HERE, "executable_plan.txt"), "w") as f:
    f.write("offset  bytes (little endian)              field\n")
    f.write("\n".join(listing) + "\n")
print(len(out), "bytes")
