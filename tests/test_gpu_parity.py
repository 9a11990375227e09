"""GPU parity tests: the HIP path, called through the C ABI, against the CPU oracle on the
same seeded inputs.  Bit-exact for packing, unpacking, codebook lookup, integer
accumulators and quantised activations; float outputs within the tolerance stated at each
test (max |d| / max |ref| and element-wise |d| <= tol*|ref| + tol*max|ref|)."""
import numpy as np
import pytest

import fastnn_amd
from fastnn_amd import lib as flib
from gpu_common import NAMES, assert_close, rel_err, slice_rows, to_oracle

pytestmark = pytest.mark.gpu

ALL_DT = list(range(8))
# f32-accumulate kernels (FMA GEMV, generic): stated tolerance 2e-5 of max|ref| vs the f64 oracle
TOL_F32 = 2e-5
# north-star bound for every f32-accumulate path
TOL_NORTH_STAR = 1e-3


@pytest.fixture(scope="module")
def ctx():
    c = fastnn_amd.HipContext(0)
    yield c
    c.close()


def _weights(rng, n, k, dist="normal"):
    if dist == "laplace":
        w = np.where(rng.random((n, k)) < 0.9, rng.laplace(0, 0.02, (n, k)), rng.laplace(0, 0.1, (n, k)))
    else:
        w = rng.standard_normal((n, k)) * 0.02
        w[rng.random((n, k)) < 0.001] *= 8
    return w.astype(np.float32)


# --------------------------------------------------------------------------- decode
def test_fp8_fp4_decode_tables_bit_exact(ctx, orc):
    """Every F8/F8R byte and F4 nibble at every lane position decodes to the reference value
    (NaN for all exponent-15 E4M3 bytes, +0.0 for FP4 nibble 0x8)."""
    for dt, bits in ((flib.DT_F8, 8), (flib.DT_F8R, 8), (flib.DT_F4, 4)):
        items = 32 // bits
        ncodes = 1 << bits
        # row r: code (r + lane) mod ncodes at every lane -> all codes at all positions
        words = np.zeros(ncodes + 16, np.uint32)
        for r in range(ncodes):
            w = 0
            for i in range(items):
                w |= ((r + i) % ncodes) << (bits * i)
            words[r] = w
        pw = fastnn_amd.PackedWeight(dt, ncodes, items, words, np.ones(ncodes, np.float32),
                                     np.zeros(ncodes, np.float32))
        h = ctx.register(pw)
        got = ctx.dequant(h, ncodes, items)
        want = orc.dequant(to_oracle(orc, pw))
        assert np.array_equal(np.isnan(got), np.isnan(want)), NAMES[dt]
        ok = ~np.isnan(want)
        assert np.array_equal(got[ok].view(np.uint32), want[ok].view(np.uint32)), NAMES[dt]
        ctx.release(h)


@pytest.mark.parametrize("dt", ALL_DT)
@pytest.mark.parametrize("shape", [(64, 128), (33, 77), (5, 3), (256, 4096)])
def test_dequant_bit_exact(ctx, orc, dt, shape):
    """unpack*scale+zero (one multiply, one add) and scales[blk]*codebook[nibble] are bit-exact."""
    rng = np.random.default_rng(2000 + dt)
    n, k = shape
    pw = fastnn_amd.quantize_weights(dt, _weights(rng, n, k, "laplace" if dt == 7 else "normal"))
    h = ctx.register(pw)
    got = ctx.dequant(h, n, k)
    want = orc.dequant(to_oracle(orc, pw))
    assert got.tobytes() == want.tobytes()
    ctx.release(h)
    if dt != flib.DT_I4CB:  # raw random words: every code incl. NaN bytes, random scales/zeros
        items = 32 // pw.bit_width
        kp = -(-k // items)
        words = rng.integers(0, 2 ** 32, n * kp + 16, dtype=np.uint64).astype(np.uint32)
        pr = fastnn_amd.PackedWeight(dt, n, k, words, rng.uniform(0.01, 2, n).astype(np.float32),
                                     rng.uniform(-1, 1, n).astype(np.float32))
        h = ctx.register(pr)
        got = ctx.dequant(h, n, k)
        want = orc.dequant(to_oracle(orc, pr))
        assert np.array_equal(np.isnan(got), np.isnan(want))
        ok = ~np.isnan(want)
        assert np.array_equal(got[ok].view(np.uint32), want[ok].view(np.uint32))
        ctx.release(h)


def test_grouped_and_scalar_scales(ctx, orc):
    rng = np.random.default_rng(3)
    n, k = 12, 40
    words = rng.integers(0, 2 ** 32, n * 10 + 16, dtype=np.uint64).astype(np.uint32)
    for ns in (1, 3, 12):
        pw = fastnn_amd.PackedWeight(flib.DT_I8, n, k, words, rng.uniform(0.5, 1.5, ns).astype(np.float32),
                                     rng.uniform(-1, 1, ns).astype(np.float32))
        h = ctx.register(pw)
        assert ctx.dequant(h, n, k).tobytes() == orc.dequant(to_oracle(orc, pw)).tobytes()
        a = rng.standard_normal((2, k)).astype(np.float32)
        assert_close(ctx.qmatmul(h, a, n), orc.qmatmul(to_oracle(orc, pw), a), TOL_F32)
        ctx.release(h)
    # zero_points omitted (FP8 metadata): treated as zeros
    pw = fastnn_amd.PackedWeight(flib.DT_F8, n, k, words & np.uint32(0x77777777),
                                 rng.uniform(0.5, 1.5, n).astype(np.float32), np.zeros(0, np.float32))
    h = ctx.register(pw)
    po = orc.Packed(orc.F8, n, k, pw.words, pw.scales, np.zeros(n, np.float32))
    assert ctx.dequant(h, n, k).tobytes() == orc.dequant(po).tobytes()
    ctx.release(h)


# --------------------------------------------------------------------------- f32-activation MatMul
GEMV_SHAPES = [(1, 256, 64), (1, 1024, 100), (2, 512, 48), (3, 2048, 33), (4, 4096, 128), (1, 8192, 16)]
# matrix-core shapes: every M-tile count, several K-chunks, ragged N, K not a multiple of the tile
MFMA_SHAPES = [(5, 512, 64), (16, 4096, 48), (17, 1024, 100), (33, 2048, 40), (64, 8192, 32), (100, 640, 72),
               (256, 1024, 130), (8, 96, 16), (12, 12288, 24)]
RAGGED_SHAPES = [(1, 7, 5), (3, 9, 4), (2, 100, 17), (5, 61, 130), (9, 333, 20), (17, 4100, 12), (1, 48, 8)]
# one-launch kernels for 2..16 rows: several row tiles per workgroup (wide N), 4- and 8-wave workgroups (K <= 2048 or
# more), K with a partial last slice and more than one round of 4096
ROW_TILE_SHAPES = [(2, 1024, 8500), (4, 4096, 8500), (7, 1024, 8500), (8, 2048, 4400), (6, 8200, 40), (13, 4096, 8500),
                   (16, 1024, 4400), (9, 520, 40), (11, 8200, 24), (16, 4096, 16)]


@pytest.mark.parametrize("dt", ALL_DT)
@pytest.mark.parametrize("m,k,n", GEMV_SHAPES + RAGGED_SHAPES + MFMA_SHAPES)
def test_qmatmul_matches_oracle(ctx, orc, dt, m, k, n):
    rng = np.random.default_rng(3000 + dt * 17 + k)
    pw = fastnn_amd.quantize_weights(dt, _weights(rng, n, k, "laplace" if dt == 7 else "normal"))
    a = rng.standard_normal((m, k)).astype(np.float32)
    h = ctx.register(pw)
    want = orc.qmatmul(to_oracle(orc, pw), a, order=2)
    got = ctx.qmatmul(h, a, n)
    assert_close(got, want, TOL_F32, f"{NAMES[dt]} {m}x{k}x{n}")
    gen = ctx.qmatmul(h, a, n, flags=flib.FLAG_FORCE_GENERIC)
    assert_close(gen, want, TOL_F32, f"generic {NAMES[dt]} {m}x{k}x{n}")
    fma = ctx.qmatmul(h, a, n, flags=flib.FLAG_PREFER_FMA)
    assert_close(fma, want, TOL_F32, f"fma {NAMES[dt]} {m}x{k}x{n}")
    if dt in (0, 1, 3) and m <= 4:     # default route: int8 matrix cores; the f16 GEMV kernel takes them when asked
        ctx.set_option(flib.OPT_GEMV_INT8, 0)
        try:
            assert_close(ctx.qmatmul(h, a, n), want, TOL_F32, f"f16 gemv {NAMES[dt]} {m}x{k}x{n}")
        finally:
            ctx.set_option(flib.OPT_GEMV_INT8, 1)
    # the reference's own f32 summation orders sit inside the same band
    assert rel_err(orc.qmatmul(to_oracle(orc, pw), a, order=1), want) <= TOL_F32 * 5
    ctx.release(h)


@pytest.mark.parametrize("dt", ALL_DT)
@pytest.mark.parametrize("m,k,n", [(1, 512, 48), (20, 200, 37)])
def test_oracle_packed_weights_through_the_device(ctx, orc, dt, m, k, n):
    """The words, scales, zeros and codebook the ORACLE's quantiser produces, registered and multiplied on the device:
    the product's host packer (which every other test here feeds to both sides) has to produce the same bytes, and
    the device has to agree with the oracle on a weight image the product did not write."""
    rng = np.random.default_rng(3300 + dt * 13 + k)
    w = _weights(rng, n, k, "laplace" if dt == 7 else "normal")
    w[1] = 0.0
    w[2] = 0.015
    po = orc.quantize(dt, w)
    pw = fastnn_amd.quantize_weights(dt, w)
    assert np.array_equal(pw.words, po.words) and pw.scales.tobytes() == po.scales.tobytes() and pw.zeros.tobytes() == po.zeros.tobytes()
    if dt == 7:
        assert pw.codebook.tobytes() == po.codebook.tobytes() and pw.qblock == po.qblock
    theirs = flib.PackedWeight(po.dt, po.rows, po.inner, po.words, po.scales, po.zeros, po.qblock, po.codebook)
    a = rng.standard_normal((m, k)).astype(np.float32)
    h = ctx.register(theirs)
    assert_close(ctx.qmatmul(h, a, n), orc.qmatmul(po, a, order=2), TOL_F32, f"{NAMES[dt]} {m}x{k}x{n}")
    assert ctx.dequant(h, n, k).tobytes() == orc.dequant(po).tobytes()
    ctx.release(h)


@pytest.mark.parametrize("dt", [0, 1, 2, 3, 4, 5, 6])
@pytest.mark.parametrize("m,k,n", ROW_TILE_SHAPES)
def test_qmatmul_row_tile_kernels(ctx, orc, dt, m, k, n):
    """M <= 8 (hi / lo operand rows of one MFMA) and 9 <= M <= 16 (activation rows = operand rows), with bias and
    activation, both activation modes; f32 accumulation, stated bounds 2e-5 / 1e-3 of max|ref|."""
    rng = np.random.default_rng(3500 + dt * 31 + m)
    pw = fastnn_amd.quantize_weights(dt, _weights(rng, n, k))
    a = rng.standard_normal((m, k)).astype(np.float32)
    bias = (rng.standard_normal(n) * 0.01).astype(np.float32)
    h = ctx.register(pw)
    want = orc.qmatmul(to_oracle(orc, pw), a, order=2, bias=bias, act=3)
    assert_close(ctx.qmatmul(h, a, n, bias=bias, act=3), want, TOL_F32, f"{NAMES[dt]} {m}x{k}x{n}")
    assert_close(ctx.qmatmul(h, a, n, bias=bias, act=3, flags=flib.FLAG_ACT_F16_SINGLE), want, TOL_NORTH_STAR,
                 f"f16x1 {NAMES[dt]} {m}x{k}x{n}")
    ctx.release(h)


# int8 GEMV: wide N, partial last slice, two slices per wave (K > 4096), four-wave workgroups (K <= 2048), a single
# tile, ragged N, every row count
INT8_GEMV_SHAPES = [(1, 4096, 8500), (2, 1024, 8500), (3, 520, 4200), (4, 8200, 72), (1, 2048, 16), (4, 4096, 4400), (1, 11008, 4096),
                    (2, 64, 40), (5, 4096, 4400), (7, 520, 300), (8, 2048, 8500), (11, 1032, 200), (16, 4096, 1100)]


@pytest.mark.parametrize("dt", [0, 1, 3])
@pytest.mark.parametrize("m,k,n", INT8_GEMV_SHAPES)
def test_int8_gemv_kernel(ctx, orc, dt, m, k, n):
    """M <= 16 with I8 / I4 / U4 weights on the int8 matrix cores (the default for these weights up to M = 8; chunks of
    four activation rows against the same packed bytes beyond M = 4): the activations enter as four
    exact base-256 digits (30 bits below the maximum of their 512 k-values) and the sums are exact integers, so the
    result sits well inside the 2e-5 MatMul bound (asserted: 4e-6 of max|ref|, measured 4e-8 .. 2e-6); bias + SiLU
    epilogue."""
    rng = np.random.default_rng(3700 + dt * 13 + m + k)
    pw = fastnn_amd.quantize_weights(dt, _weights(rng, n, k))
    a = rng.standard_normal((m, k)).astype(np.float32)
    a[:, ::97] *= 300.0                                  # wide dynamic range inside a slice
    bias = (rng.standard_normal(n) * 0.01).astype(np.float32)
    h = ctx.register(pw)
    want = orc.qmatmul(to_oracle(orc, pw), a, order=2, bias=bias, act=3)
    ctx.set_option(flib.OPT_GEMV_INT8_MAX_M, 16)
    ctx.set_option(flib.OPT_STREAM_MAX_M, 0)   # (a long K over few columns would go to the streaming kernel from M = 5 or 9)
    try:
        got = ctx.qmatmul(h, a, n, bias=bias, act=3)
        assert_close(got, want, 4e-6, f"int8 gemv {NAMES[dt]} {m}x{k}x{n}")
        for rt in (1, 2, 3):               # any number of row tiles per workgroup gives the same bits
            ctx.set_option(flib.OPT_GEMV_ROW_TILES, rt)
            assert np.array_equal(ctx.qmatmul(h, a, n, bias=bias, act=3), got), f"{rt} row tiles"
            # ... and so does either layout of the packed words (the tile-major copy, default where the rows are whole
            # 64-byte blocks, and the row-major words)
            ctx.set_option(flib.OPT_GEMV_TILE_MAJOR, 0)
            assert np.array_equal(ctx.qmatmul(h, a, n, bias=bias, act=3), got), f"{rt} row tiles, row-major words"
            ctx.set_option(flib.OPT_GEMV_TILE_MAJOR, 1)
    finally:
        ctx.set_option(flib.OPT_GEMV_ROW_TILES, 0)
        ctx.set_option(flib.OPT_GEMV_INT8, 1)
        ctx.set_option(flib.OPT_GEMV_INT8_MAX_M, 8)
        ctx.set_option(flib.OPT_GEMV_TILE_MAJOR, 1)
        ctx.set_option(flib.OPT_STREAM_MAX_M, 32)
    ctx.release(h)


@pytest.mark.parametrize("m", [3, 7])
def test_int8_gemv_propagates_non_finite_activations(ctx, orc, m):
    """The integer digits cannot carry a NaN or an infinity: the slice scale does, so the affected output rows are NaN
    (the float path gives NaN or inf there) and the other rows are untouched."""
    rng = np.random.default_rng(3800)
    k, n = 1024, 64
    pw = fastnn_amd.quantize_weights(flib.DT_I8, _weights(rng, n, k))
    a = rng.standard_normal((m, k)).astype(np.float32)
    h = ctx.register(pw)
    clean = ctx.qmatmul(h, a, n)
    a[0, 700] = np.nan
    a[m - 1, 3] = np.inf
    got = ctx.qmatmul(h, a, n)
    assert np.isnan(got[0]).all() and np.isnan(got[m - 1]).all()
    assert np.array_equal(got[1:m - 1], clean[1:m - 1])
    ctx.release(h)


DIGIT_GEMM_SHAPES = [(17, 4096, 1100), (40, 1000, 300), (64, 200, 4400), (130, 2048, 260), (256, 4096, 1408), (300, 520, 96),
                     (1024, 1024, 512)]


@pytest.mark.parametrize("planes", [4, 3])
@pytest.mark.parametrize("dt", [0, 1, 3])
@pytest.mark.parametrize("m,k,n", DIGIT_GEMM_SHAPES)
def test_int8_digit_plane_gemm(ctx, orc, dt, m, k, n, planes):
    """M >= 17 with I8 / I4 / U4 weights on the int8 matrix cores (the default for these weights): activation rows as
    exact base-256 digit planes, exact integer sums per plane, f32 recombination (the single-rounding mode stays on
    the f16 tiles).  Four planes: rint at 2^-30 of the row maximum, 4e-6 of max|ref| stated; three planes (what the
    default takes wherever it is faster): rint at 2^-22, 2e-5 stated, on rows with a 200x dynamic range.  Ragged K
    and N, every tile shape, K split on and off; bias + GELU epilogue."""
    rng = np.random.default_rng(4700 + dt * 13 + m + k)
    pw = fastnn_amd.quantize_weights(dt, _weights(rng, n, k))
    a = rng.standard_normal((m, k)).astype(np.float32)
    a[:, ::89] *= 200.0                                  # wide dynamic range inside a row
    a[m // 2] = 0.0                                      # an all-zero row
    bias = (rng.standard_normal(n) * 0.01).astype(np.float32)
    h = ctx.register(pw)
    want = orc.qmatmul(to_oracle(orc, pw), a, order=2, bias=bias, act=2)
    tol = 4e-6 if planes == 4 else TOL_F32
    try:
        ctx.set_option(flib.OPT_STREAM_MAX_M, 0)         # (M <= 32 would go to the one-launch kernel, tested on its own)
        ctx.set_option(flib.OPT_DIGIT_PLANES, planes)
        got = ctx.qmatmul(h, a, n, bias=bias, act=2)
        int8_default = not (planes == 4 and dt == 0 and m >= 768)   # 8-bit weights at four planes: the f16 tiles take M >= 768
        assert_close(got, want, tol if int8_default else TOL_F32, f"digit gemm {NAMES[dt]} {m}x{k}x{n}")
        err = rel_err(got, want)
        assert rel_err(ctx.qmatmul(h, a, n, bias=bias, act=2, flags=flib.FLAG_ACT_F16_SINGLE), want) <= TOL_NORTH_STAR
        for shape in (0, 1, 2, 3, 4):
            for split in (1, 3):
                ctx.set_option(flib.OPT_TILE_SHAPE, shape)
                ctx.set_option(flib.OPT_TILE_SPLIT, split)
                assert_close(ctx.qmatmul(h, a, n, bias=bias, act=2), want, tol, f"shape {shape} split {split}")
        ctx.set_option(flib.OPT_TILE_SHAPE, -1)
        ctx.set_option(flib.OPT_TILE_SPLIT, 0)
        ctx.set_option(flib.OPT_GEMM_INT8, 0)            # the f16 tiles take the same call
        f16 = ctx.qmatmul(h, a, n, bias=bias, act=2)
        assert_close(f16, want, TOL_F32)
        assert np.array_equal(f16, got) != int8_default
        print(f"planes {planes} {NAMES[dt]} {m}x{k}x{n}: {err:.2e}", flush=True)
    finally:
        ctx.set_option(flib.OPT_TILE_SHAPE, -1)
        ctx.set_option(flib.OPT_TILE_SPLIT, 0)
        ctx.set_option(flib.OPT_GEMM_INT8, 1)
        ctx.set_option(flib.OPT_DIGIT_PLANES, 0)
        ctx.set_option(flib.OPT_STREAM_MAX_M, 32)
    ctx.release(h)


# one-launch streaming kernel: one and two activation blocks, ragged N and K (K % 512 != 0, K < 256), wide N (several
# column tiles), long K (many splits), a single k chunk
STREAM_SHAPES = [(17, 4096, 1100), (32, 2048, 4100), (24, 520, 300), (31, 8192, 136), (20, 64, 40), (32, 1160, 4096), (9, 4096, 520),
                 (16, 2048, 2048)]
# (splits << 8) | (row tiles per wave << 4) | (k per round / 256); 0 = by rule
STREAM_FORMS = [0, 0x11, 0x12, 0x21, 0x22, 0x112, 0x211, 0x322, 0x512]


@pytest.mark.parametrize("dt", [0, 1, 2, 3, 4, 5, 6])
@pytest.mark.parametrize("m,k,n", STREAM_SHAPES)
def test_streaming_matmul_kernel(ctx, orc, dt, m, k, n):
    """17 <= M <= 32 (9 <= M by option) in one launch: weights straight into the matrix-core operand registers,
    activations converted in the kernel (three exact digit planes of rint(x 2^-e), |v| < 2^22 per row and round, for
    I8 / I4 / U4 weights; f16 hi + lo for U8 / F8 / F8R / F4), K split over workgroups and added in split order by the
    last one to arrive.  Every launch form gives the oracle's result within 2e-5 of max|ref| (rows with a 200x dynamic
    range, an all-zero row, bias + SiLU), a given form gives the same bits on every call, and a call that the rule
    declines (K % 64 != 0 for the f16 types, too many workgroups) still comes out right through the other kernels."""
    rng = np.random.default_rng(5100 + dt * 7 + m + k)
    pw = fastnn_amd.quantize_weights(dt, _weights(rng, n, k))
    a = rng.standard_normal((m, k)).astype(np.float32)
    a[:, ::89] *= 200.0
    a[m // 2] = 0.0
    bias = (rng.standard_normal(n) * 0.01).astype(np.float32)
    h = ctx.register(pw)
    want = orc.qmatmul(to_oracle(orc, pw), a, order=2, bias=bias, act=3)
    try:
        ctx.set_option(flib.OPT_STREAM_MIN_M, 9)
        ctx.set_option(flib.OPT_ROWS16_MIN_M, 17)
        for form in STREAM_FORMS:
            ctx.set_option(flib.OPT_STREAM_SHAPE, form)
            got = ctx.qmatmul(h, a, n, bias=bias, act=3)
            assert_close(got, want, TOL_F32, f"stream {NAMES[dt]} {m}x{k}x{n} form {form:#x}")
            again = ctx.qmatmul(h, a, n, bias=bias, act=3)
            assert np.array_equal(got, again), f"form {form:#x}: two calls differ"
    finally:
        ctx.set_option(flib.OPT_STREAM_SHAPE, 0)
        ctx.set_option(flib.OPT_STREAM_MIN_M, 17)
        ctx.set_option(flib.OPT_ROWS16_MIN_M, 9)
    ctx.release(h)


def test_streaming_matmul_takes_the_default_route_and_propagates_non_finite_rows(ctx, orc):
    """By default M = 17..32 on a shape the rule accepts runs in the streaming kernel: its result differs in the last
    bits from the digit-plane / tiled path's (another summation), both within bounds.  A row holding a NaN or an
    infinity gives a NaN row with integer weights (the digits cannot carry it; the float path gives NaN or inf) and
    non-finite values with float weights; the other rows are untouched."""
    rng = np.random.default_rng(5200)
    m, k, n = 32, 2048, 1024
    for dt in (flib.DT_I8, flib.DT_F8):
        pw = fastnn_amd.quantize_weights(dt, _weights(rng, n, k))
        a = rng.standard_normal((m, k)).astype(np.float32)
        h = ctx.register(pw)
        want = orc.qmatmul(to_oracle(orc, pw), a, order=2)
        clean = ctx.qmatmul(h, a, n)
        ctx.set_option(flib.OPT_STREAM_MAX_M, 0)
        try:
            other = ctx.qmatmul(h, a, n)
        finally:
            ctx.set_option(flib.OPT_STREAM_MAX_M, 32)
        assert_close(clean, want, TOL_F32)
        assert_close(other, want, TOL_F32)
        assert not np.array_equal(clean, other)
        ctx.set_option(flib.OPT_GEMV_TILE_MAJOR, 0)   # the same kernel on the row-major words: the same bits
        try:
            assert np.array_equal(ctx.qmatmul(h, a, n), clean)
        finally:
            ctx.set_option(flib.OPT_GEMV_TILE_MAJOR, 1)
        a[0, 700] = np.nan
        a[20, 3] = np.inf
        a[31, 2047] = -np.inf
        got = ctx.qmatmul(h, a, n)
        for r in (0, 20, 31):
            assert not np.isfinite(got[r]).any()
            if dt == flib.DT_I8:
                assert np.isnan(got[r]).all()
        keep = [r for r in range(m) if r not in (0, 20, 31)]
        assert np.array_equal(got[keep], clean[keep])
        ctx.release(h)


@pytest.mark.parametrize("dt", [flib.DT_I8, flib.DT_I4, flib.DT_U8, flib.DT_F8, flib.DT_F4])
@pytest.mark.parametrize("m,k,n", [(5, 8192, 512), (8, 16384, 256), (12, 8192, 2048), (16, 4096, 768), (9, 8192, 4000), (16, 4096, 2040), (8, 4096, 1000)])
def test_streaming_matmul_narrow_outputs_from_m5(ctx, orc, dt, m, k, n):
    """A long K over few output columns: the streaming kernel takes 9 <= M <= 16 where K >= 4 N (K >= 2 N from K = 8192
    on) and 5 <= M <= 8 where N <= 2048, K >= 4 N and K >= 8192 (16384 for the types of the int8 GEMV): the one-launch
    kernels for those M give a workgroup whole rows, few workgroups here, each converting all activations.  Against the
    oracle with bias + SiLU, the same bits on two calls, and another kernel than the one that runs with the streaming
    kernel off exactly where the rule says so."""
    rng = np.random.default_rng(5500 + dt * 11 + m)
    pw = fastnn_amd.quantize_weights(dt, _weights(rng, n, k))
    a = rng.standard_normal((m, k)).astype(np.float32)
    a[:, ::97] *= 150.0
    a[m // 2] = 0.0
    bias = (rng.standard_normal(n) * 0.01).astype(np.float32)
    h = ctx.register(pw)
    want = orc.qmatmul(to_oracle(orc, pw), a, order=2, bias=bias, act=3)
    got = ctx.qmatmul(h, a, n, bias=bias, act=3)
    assert_close(got, want, TOL_F32, f"narrow {NAMES[dt]} {m}x{k}x{n}")
    assert np.array_equal(got, ctx.qmatmul(h, a, n, bias=bias, act=3))
    ctx.set_option(flib.OPT_STREAM_MAX_M, 0)
    try:
        other = ctx.qmatmul(h, a, n, bias=bias, act=3)
    finally:
        ctx.set_option(flib.OPT_STREAM_MAX_M, 32)
    assert_close(other, want, TOL_F32)
    int_type = dt in (flib.DT_I8, flib.DT_I4)
    takes = (m >= 9 and (k >= 4 * n or (k >= 2 * n and k >= 8192))) or (n <= 2048 and k >= 4 * n and k >= (16384 if int_type else 8192))
    assert np.array_equal(got, other) != takes, "the streaming kernel " + ("did not take" if takes else "took") + " the call"
    ctx.release(h)


@pytest.mark.parametrize("m,k,n", [(5, 4096, 520), (16, 1024, 300), (17, 2048, 1100), (32, 4096, 2048), (33, 1536, 260), (48, 2048, 1100),
                                   (64, 4096, 1024), (64, 128, 4400), (50, 2048, 5000)])
def test_streaming_matmul_codebook_weights(ctx, orc, m, k, n):
    """Codebook weights with blocks of 32 at 5 <= M <= 64 (K % 128 == 0) run in the streaming kernel: a matrix-core step
    is one block (the lane loads are transposed across the k groups), its sum is folded with the block scale -- the
    reference's association.  Every launch form within the MatMul bound of the oracle (rows with a 200x dynamic range,
    an all-zero row, ragged N, bias + SiLU), the same bits on every call and on either layout of the words, and another
    kernel than the tiled path's (which FNN_OPT_CODEBOOK_EXPANDED = 2 selects)."""
    rng = np.random.default_rng(5400 + m + k)
    pw = fastnn_amd.quantize_weights(flib.DT_I4CB, _weights(rng, n, k, "laplace"))
    a = rng.standard_normal((m, k)).astype(np.float32)
    a[:, ::89] *= 200.0
    a[m // 2] = 0.0
    bias = (rng.standard_normal(n) * 0.01).astype(np.float32)
    h = ctx.register(pw)
    want = orc.qmatmul(to_oracle(orc, pw), a, order=2, bias=bias, act=3)
    try:
        for form in STREAM_FORMS:
            ctx.set_option(flib.OPT_STREAM_SHAPE, form)
            got = ctx.qmatmul(h, a, n, bias=bias, act=3)
            assert_close(got, want, TOL_F32, f"stream codebook {m}x{k}x{n} form {form:#x}")
            assert np.array_equal(got, ctx.qmatmul(h, a, n, bias=bias, act=3)), f"form {form:#x}: two calls differ"
            if form in (0, 0x112):
                ctx.set_option(flib.OPT_GEMV_TILE_MAJOR, 0)
                assert np.array_equal(got, ctx.qmatmul(h, a, n, bias=bias, act=3)), f"form {form:#x}: the layouts differ"
                ctx.set_option(flib.OPT_GEMV_TILE_MAJOR, 1)
        ctx.set_option(flib.OPT_STREAM_SHAPE, 0)
        by_rule = ctx.qmatmul(h, a, n, bias=bias, act=3)
        ctx.set_option(flib.OPT_CODEBOOK_EXPANDED, 2)
        tiled = ctx.qmatmul(h, a, n, bias=bias, act=3)
        assert_close(tiled, want, TOL_F32)
        if n * ((k + 511) // 512) <= 320 * 128:      # (the rule declines launches of more than 320 workgroups)
            assert not np.array_equal(by_rule, tiled)
    finally:
        ctx.set_option(flib.OPT_STREAM_SHAPE, 0)
        ctx.set_option(flib.OPT_GEMV_TILE_MAJOR, 1)
        ctx.set_option(flib.OPT_CODEBOOK_EXPANDED, 0)
    ctx.release(h)


@pytest.mark.parametrize("dt", [flib.DT_I4, flib.DT_I8, flib.DT_F4])
@pytest.mark.parametrize("m,k,n", [(20, 4096, 5200), (32, 2048, 10500), (17, 1536, 11008)])
def test_streaming_matmul_wide_outputs(ctx, orc, dt, m, k, n):
    """Wide outputs (more than 320 workgroups with one row tile per wave) run in the streaming kernel on two row tiles
    per wave and one to three rounds per workgroup, picked by rule: against the oracle on a sample of output rows
    (the first, a ragged last column tile, some in between), with bias and activation, and against the tiled path."""
    rng = np.random.default_rng(5300 + dt + n)
    pw = fastnn_amd.quantize_weights(dt, _weights(rng, n, k))
    a = rng.standard_normal((m, k)).astype(np.float32)
    bias = (rng.standard_normal(n) * 0.01).astype(np.float32)
    h = ctx.register(pw)
    got = ctx.qmatmul(h, a, n, bias=bias, act=2)
    ctx.set_option(flib.OPT_STREAM_MAX_M, 0)
    try:
        other = ctx.qmatmul(h, a, n, bias=bias, act=2)
    finally:
        ctx.set_option(flib.OPT_STREAM_MAX_M, 32)
    assert not np.array_equal(got, other)          # (another kernel, another summation order)
    assert_close(got, other, 2 * TOL_F32)
    rows = np.unique(np.concatenate([np.arange(0, 40), np.arange(n - 300, n), rng.integers(0, n, 200)]))
    want = orc.qmatmul(to_oracle(orc, slice_rows(pw, rows)), a, order=2, bias=bias[rows], act=2)
    assert_close(got[:, rows], want, TOL_F32, f"{NAMES[dt]} {m}x{k}x{n}")
    ctx.release(h)


@pytest.mark.parametrize("dt", [flib.DT_I8, flib.DT_I4, flib.DT_U4, flib.DT_U8, flib.DT_F8, flib.DT_F8R, flib.DT_F4])
@pytest.mark.parametrize("m,k,n", [(1, 2048, 300), (6, 4096, 1000), (12, 2048, 1100), (16, 8192, 72), (24, 2048, 1100), (40, 2048, 300), (200, 1024, 520)])
def test_tile_major_copy_of_the_words_gives_the_same_bits(ctx, orc, dt, m, k, n):
    """The kernels that read the packed words from the tile-major copy (blocks of 16 rows x 64 bytes: the GEMV kernels,
    the streaming kernel, the tile kernels of the weight types with 64 bytes per row and stage) against the same
    kernels on the row-major words: identical outputs, ragged N (a partial last row block), and the oracle's bound."""
    rng = np.random.default_rng(6100 + dt * 7 + m)
    pw = fastnn_amd.quantize_weights(dt, _weights(rng, n, k))
    a = rng.standard_normal((m, k)).astype(np.float32)
    bias = (rng.standard_normal(n) * 0.01).astype(np.float32)
    h = ctx.register(pw)
    got = ctx.qmatmul(h, a, n, bias=bias, act=1)
    ctx.set_option(flib.OPT_GEMV_TILE_MAJOR, 0)
    try:
        assert np.array_equal(ctx.qmatmul(h, a, n, bias=bias, act=1), got)
    finally:
        ctx.set_option(flib.OPT_GEMV_TILE_MAJOR, 1)
    assert_close(got, orc.qmatmul(to_oracle(orc, pw), a, order=2, bias=bias, act=1), TOL_F32, f"{NAMES[dt]} {m}x{k}x{n}")
    ctx.release(h)


def test_int8_digit_plane_gemm_non_finite_rows(ctx, orc):
    """A row holding a NaN or an infinity cannot be written as integer digits: its exponent entry carries a flag and
    the whole output row is NaN (the float path gives NaN or inf there); the other rows are untouched."""
    rng = np.random.default_rng(4800)
    m, k, n = 33, 1024, 200
    pw = fastnn_amd.quantize_weights(flib.DT_I4, _weights(rng, n, k))
    a = rng.standard_normal((m, k)).astype(np.float32)
    h = ctx.register(pw)
    ctx.set_option(flib.OPT_DIGIT_PLANES, 3)   # (weights this small go to the f16 tiles by rule)
    try:
        clean = ctx.qmatmul(h, a, n)
        a[0, 700] = np.nan
        a[20, 3] = np.inf
        a[32, 1023] = -np.inf
        got = ctx.qmatmul(h, a, n)
    finally:
        ctx.set_option(flib.OPT_DIGIT_PLANES, 0)
    for r in (0, 20, 32):
        assert np.isnan(got[r]).all()
    keep = [r for r in range(m) if r not in (0, 20, 32)]
    assert np.array_equal(got[keep], clean[keep])
    ctx.release(h)


@pytest.mark.parametrize("dt", [0, 1, 4, 6, 7])
@pytest.mark.parametrize("act", [0, 1, 2, 3])
@pytest.mark.parametrize("m,k,n", [(1, 512, 96), (3, 130, 50)])
def test_fused_bias_activation(ctx, orc, dt, act, m, k, n):
    """act(matmul + bias) equals the unfused chain matmul_q -> add -> act."""
    rng = np.random.default_rng(4000 + dt + act)
    pw = fastnn_amd.quantize_weights(dt, _weights(rng, n, k, "laplace" if dt == 7 else "normal"))
    a = rng.standard_normal((m, k)).astype(np.float32)
    bias = (rng.standard_normal(n) * 0.01).astype(np.float32)
    h = ctx.register(pw)
    want = orc.qmatmul(to_oracle(orc, pw), a, order=2, bias=bias, act=act)
    assert_close(ctx.qmatmul(h, a, n, bias=bias, act=act), want, TOL_F32)
    want_nb = orc.qmatmul(to_oracle(orc, pw), a, order=2, act=act)
    assert_close(ctx.qmatmul(h, a, n, act=act), want_nb, TOL_F32)
    ctx.release(h)


def test_reference_literal_cases_on_gpu(ctx, orc, golden):
    g = golden["gemm_f32act"]["asymmetric_zero_is_per_input_sum"]
    po = orc.from_f32_slice(orc.I8, g["weights_f32"], g["n"], g["k"], g["w_scale"], g["w_zero"])
    pw = fastnn_amd.PackedWeight(flib.DT_I8, g["n"], g["k"], po.words, po.scales, po.zeros)
    h = ctx.register(pw)
    a = np.array(g["input"], np.float32).reshape(g["m"], g["k"])
    assert np.allclose(ctx.qmatmul(h, a, g["n"]).reshape(-1), g["expected"], atol=g["abs_tol"])
    ctx.release(h)
    dts = {"i4": 1, "i8": 0, "f8": 4, "f8r": 5}
    for c in golden["seeded_end_to_end"]["cases"]:
        if c["quantize"] not in dts:
            continue
        m, k, n = c["m"], c["k"], c["n"]
        a = orc.seeded_values(c["seed"], m * k).reshape(m, k)
        w = orc.seeded_values(c["seed"] + 1, k * n).reshape(k, n)
        pw = fastnn_amd.quantize_weights_kn(dts[c["quantize"]], w)
        h = ctx.register(pw)
        got = ctx.qmatmul(h, a, n)
        expected = (a.astype(np.float64) @ w.astype(np.float64))
        allowed = np.maximum(c["abs_tol"], np.abs(expected) * c["rel_tol"])
        assert np.all(np.abs(got - expected) <= allowed), c
        ctx.release(h)


@pytest.mark.parametrize("m,k,n", [(5, 4096, 520), (16, 1056, 300), (40, 2048, 260), (64, 200, 4400), (130, 992, 96), (256, 4096, 256),
                                   (600, 1024, 384)])
def test_codebook_gemm_decoded_in_kernel_and_expanded(ctx, orc, m, k, n):
    """Codebook weights at M >= 5: nibbles looked up inside the tiled GEMM (per-block accumulators folded with the
    block scale, the reference's association) and the expanded f16 hi + lo operand are both within the MatMul bound
    of the oracle, in both activation modes; ragged K (blocks of 32 that do not fill a 64-value stage, rows that are
    not a multiple of 16 bytes) and ragged N; bias + SiLU."""
    rng = np.random.default_rng(5100 + m + k)
    pw = fastnn_amd.quantize_weights(flib.DT_I4CB, _weights(rng, n, k, "laplace"))
    a = rng.standard_normal((m, k)).astype(np.float32)
    a[:, ::61] *= 50.0
    bias = (rng.standard_normal(n) * 0.01).astype(np.float32)
    h = ctx.register(pw)
    want = orc.qmatmul(to_oracle(orc, pw), a, order=2, bias=bias, act=3)
    try:
        outs = {}
        for mode in (2, 1, 0):
            ctx.set_option(flib.OPT_CODEBOOK_EXPANDED, mode)
            outs[mode] = ctx.qmatmul(h, a, n, bias=bias, act=3)
            assert_close(outs[mode], want, TOL_F32, f"codebook mode {mode} {m}x{k}x{n}")
            assert rel_err(ctx.qmatmul(h, a, n, bias=bias, act=3, flags=flib.FLAG_ACT_F16_SINGLE), want) <= TOL_NORTH_STAR
        assert not np.array_equal(outs[2], outs[1])      # two different kernels
        for split in (1, 2, 5):
            ctx.set_option(flib.OPT_CODEBOOK_EXPANDED, 2)
            ctx.set_option(flib.OPT_TILE_SPLIT, split)
            for shape in (0, 1, 2):
                ctx.set_option(flib.OPT_TILE_SHAPE, shape)
                assert_close(ctx.qmatmul(h, a, n, bias=bias, act=3), want, TOL_F32, f"split {split} shape {shape}")
    finally:
        ctx.set_option(flib.OPT_CODEBOOK_EXPANDED, 0)
        ctx.set_option(flib.OPT_TILE_SPLIT, 0)
        ctx.set_option(flib.OPT_TILE_SHAPE, -1)
    ctx.release(h)


def test_i4cb_as_written_variant(ctx, orc):
    rng = np.random.default_rng(8)
    n = k = 64
    pw = fastnn_amd.quantize_weights(flib.DT_I4CB, _weights(rng, n, k, "laplace"))
    a = rng.standard_normal((3, k)).astype(np.float32)
    h = ctx.register(pw)
    want = orc.qmatmul(to_oracle(orc, pw), a, order=2, i4cb_as_written=True)
    assert_close(ctx.qmatmul(h, a, n, flags=flib.FLAG_I4CB_AS_WRITTEN), want, TOL_F32)
    ctx.release(h)


def test_device_pointer_calls_and_graph_replay(ctx, orc):
    rng = np.random.default_rng(9)
    n, k, m = 256, 1024, 1
    pw = fastnn_amd.quantize_weights(flib.DT_I4, _weights(rng, n, k))
    h = ctx.register(pw)
    a = rng.standard_normal((m, k)).astype(np.float32)
    bias = (rng.standard_normal(n) * 0.01).astype(np.float32)
    da, db, dout = ctx.to_device(a), ctx.to_device(bias), ctx.alloc(m * n * 4)
    want = orc.qmatmul(to_oracle(orc, pw), a, order=2, bias=bias, act=3)
    ctx.qmatmul_dev(h, da.ptr, m, dout.ptr, db.ptr, act=3)
    ctx.sync()
    eager = dout.download(np.float32, m * n).reshape(m, n)
    assert_close(eager, want, TOL_F32)
    ctx.graph_begin()
    ctx.qmatmul_dev(h, da.ptr, m, dout.ptr, db.ptr, act=3)
    g = ctx.graph_end()
    for rep in range(3):  # every replay, with eager work and syncs in between, equals the eager result
        dout.upload(np.zeros(m * n, np.float32))
        ctx.graph_launch(g)
        ctx.sync()
        assert dout.download(np.float32, m * n).tobytes() == eager.tobytes(), rep
        a2 = rng.standard_normal((m, k)).astype(np.float32)
        ctx.qmatmul(h, a2, n)
    ctx.graph_destroy(g)
    for b in (da, db, dout):
        b.free()
    ctx.release(h)


# --------------------------------------------------------------------------- I8 activations
@pytest.mark.parametrize("numel", [1, 7, 256, 4099, 100000])
def test_quantize_activations_bit_exact(ctx, orc, numel):
    rng = np.random.default_rng(10 + numel)
    x = (rng.standard_normal(numel) * 3).astype(np.float32)
    assert ctx.quantize_activations(x).tobytes() == orc.quantize_activations(x).tobytes()
    assert ctx.quantize_activations(x, 0.05, 0.25).tobytes() == orc.quantize_activations(x, 0.05, 0.25).tobytes()
    z = np.zeros(numel, np.float32)
    assert ctx.quantize_activations(z).tobytes() == orc.quantize_activations(z).tobytes()


@pytest.mark.parametrize("nc,numel", [(1, 1), (1, 300), (3, 100), (8, 8 * 4096), (300, 300 * 37 + 5), (64, 40), (5, 100003)])
def test_per_channel_activation_payloads_bit_exact(ctx, orc, nc, numel):
    """The per-channel "quantize_activations" / "dequantize_activations" payloads, byte for byte what the reference's
    loops leave behind (src/backend/cpu/mod.rs:6941-6975, 7026-7061): whole inputs, an input view shorter than numel,
    a payload that ends inside the code block, zero scales, non-finite values, more channels than one header launch
    carries, fewer elements than channels (chunk = 0); bytes and values the loops do not reach keep what they held."""
    rng = np.random.default_rng(900 + nc + numel)
    x = (rng.standard_normal(numel) * 3).astype(np.float32)
    if numel > 8:
        x[[1, 3, 5]] = [np.nan, np.inf, -np.inf]
    sc = rng.uniform(0.01, 0.1, nc).astype(np.float32)
    zp = rng.uniform(-1, 1, nc).astype(np.float32)
    if nc > 2:
        sc[nc // 2] = 0.0
    chunk = numel // nc
    header = 8 + 8 * nc
    fill = rng.integers(0, 256, header + chunk + 13).astype(np.uint8)
    cases = [(x, fill), (x, fill[:header + chunk // 2]), (x, fill[:header])]
    if numel > nc:
        cases += [(x[:numel - chunk // 2 - 1], fill), (x[:max(1, chunk // 3)], fill)]
    for xv, pl in cases:
        want = orc.quantize_activations_per_channel(xv, numel, sc, zp, pl)
        got = ctx.quantize_activations_per_channel(xv, numel, sc, zp, pl)
        assert got.tobytes() == want.tobytes(), (xv.size, pl.size)
    # the last channel under a zero scale: every code is 0
    sc0 = sc.copy()
    sc0[-1] = 0.0
    assert ctx.quantize_activations_per_channel(x, numel, sc0, zp, fill).tobytes() == orc.quantize_activations_per_channel(x, numel, sc0, zp, fill).tobytes()
    payload = orc.quantize_activations_per_channel(x, numel, sc, zp, fill)
    old = rng.standard_normal(numel + 9).astype(np.float32)
    for pl, out in [(payload, old), (payload, old[:max(1, numel - chunk // 2 - 1)]), (payload[:header + chunk // 2], old), (payload[:header], old)]:
        want = orc.dequantize_activations_per_channel(pl, out)
        got = ctx.dequantize_activations_per_channel(pl, out)
        assert got.tobytes() == want.tobytes(), (pl.size, out.size)
    with pytest.raises(flib.FnnError):   # the header does not fit: the reference panics
        ctx.quantize_activations_per_channel(x, numel, sc, zp, fill[:header - 1])
    # a header that claims more channels than the payload holds: nothing is written
    bad = payload.copy()
    bad[:4] = np.array([payload.size], np.uint32).view(np.uint8)
    assert ctx.dequantize_activations_per_channel(bad, old).tobytes() == old.tobytes()


@pytest.mark.parametrize("dt", [0, 1])
@pytest.mark.parametrize("m,k,n", [(1, 64, 32), (3, 61, 10), (16, 256, 64), (40, 1000, 72), (128, 512, 256)])
@pytest.mark.parametrize("zp", [0.0, 0.375])
def test_i8act_matmul_integer_exact(ctx, orc, dt, m, k, n, zp):
    rng = np.random.default_rng(5000 + dt + k)
    pw = fastnn_amd.quantize_weights(dt, _weights(rng, n, k))
    x = rng.standard_normal((m, k)).astype(np.float32)
    payload = orc.quantize_activations(x) if zp == 0.0 else orc.quantize_activations(x, 0.03, zp)
    h = ctx.register(pw)
    want, want_acc = orc.qmatmul_i8act(to_oracle(orc, pw), payload, m, want_acc=True)
    for flags in (0, flib.FLAG_FORCE_GENERIC):
        got, acc = ctx.qmatmul_i8act(h, payload, m, n, want_acc=True, flags=flags)
        if zp == 0.0:
            assert np.array_equal(acc, want_acc)          # i32 accumulators bit-exact
            assert_close(got, want, 1e-6)                  # same f32 formula on identical integers
        else:
            assert_close(got, want, TOL_F32)               # per-lane f32 path, summation order differs
    ctx.release(h)


@pytest.mark.parametrize("dt", [0, 1])
@pytest.mark.parametrize("m,k,n", [(200, 1000, 130), (256, 512, 264), (300, 2048, 72)])
def test_i8act_matmul_tile_forms(ctx, orc, dt, m, k, n):
    """The three tile forms of the int8 matrix-core GEMM behind matmul_i8_i8 / matmul_i4_i8 (128 x 128 on four waves, on
    eight waves, 256 x 128 on eight waves) and K splits of 1, 2 and 4: exact integer accumulators whatever the form,
    with ragged N and K, row counts that are and are not whole 256-row tiles, bias and activation in the epilogue's
    four-column groups (n % 4 != 0 included)."""
    rng = np.random.default_rng(5100 + dt + k)
    pw = fastnn_amd.quantize_weights(dt, _weights(rng, n, k))
    x = rng.standard_normal((m, k)).astype(np.float32)
    payload = orc.quantize_activations(x)
    h = ctx.register(pw)
    want, want_acc = orc.qmatmul_i8act(to_oracle(orc, pw), payload, m, want_acc=True)
    try:
        for form in (0, 1, 2):
            for split in (0, 1, 2, 4):
                ctx.set_option(flib.OPT_TILE_SHAPE, form)
                ctx.set_option(flib.OPT_TILE_SPLIT, split)
                got, acc = ctx.qmatmul_i8act(h, payload, m, n, want_acc=True)
                assert np.array_equal(acc, want_acc), (form, split)
                assert_close(got, want, 1e-6, f"form {form} split {split}")
    finally:
        ctx.set_option(flib.OPT_TILE_SHAPE, -1)
        ctx.set_option(flib.OPT_TILE_SPLIT, 0)
    ctx.release(h)


def test_i8act_literals_on_gpu(ctx, orc, golden):
    dts = {"i8": 0, "i4": 1}
    for c in golden["gemm_i8act"]["cases"]:
        po = orc.from_f32_slice(dts[c["dt"]], c["weights_f32"], c["n"], c["k"], c["w_scale"], c["w_zero"])
        pw = fastnn_amd.PackedWeight(dts[c["dt"]], c["n"], c["k"], po.words, po.scales, po.zeros)
        h = ctx.register(pw)
        payload = orc.make_payload(c["act_scale"], c["act_zp"], c["act_i8"])
        got = ctx.qmatmul_i8act(h, payload, c["m"], c["n"]).reshape(-1)
        want = np.array(c["expected"]) if "expected" in c else orc.qmatmul_i8act(po, payload, c["m"]).reshape(-1)
        assert np.allclose(got, want, atol=c["abs_tol"]), c["name"]
        ctx.release(h)


# --------------------------------------------------------------------------- quantised Conv2d
CONVS = [
    dict(b=2, c=3, h=20, w=24, oc=16, kh=3, kw=3, stride=2, pad=1, dil=1, groups=1),
    dict(b=1, c=16, h=12, w=12, oc=32, kh=1, kw=1, stride=1, pad=0, dil=1, groups=1),
    dict(b=1, c=8, h=10, w=7, oc=6, kh=3, kw=2, stride=1, pad=2, dil=2, groups=2),
    dict(b=3, c=5, h=9, w=9, oc=7, kh=3, kw=3, stride=1, pad=1, dil=1, groups=1),
    dict(b=1, c=32, h=16, w=16, oc=64, kh=3, kw=3, stride=1, pad=1, dil=1, groups=1),
    dict(b=2, c=12, h=13, w=14, oc=160, kh=3, kw=3, stride=1, pad=1, dil=1, groups=1),   # two column tiles, rows past a row tile
    dict(b=2, c=32, h=11, w=12, oc=32, kh=3, kw=3, stride=1, pad=1, dil=1, groups=32),   # depthwise: every group in one launch of the direct kernel
    dict(b=1, c=32, h=9, w=10, oc=48, kh=3, kw=3, stride=2, pad=1, dil=1, groups=16),
]


@pytest.fixture
def conv_epilogue(ctx, request):
    """Where the conv epilogue runs: 0 = by size, 2 = a kernel of its own, 3 = inside the GEMM kernel on 128-row tiles
    (0 takes the 64-row tiles at these sizes)."""
    ctx.set_option(flib.OPT_CONV_EPILOGUE, request.param)
    yield request.param
    ctx.set_option(flib.OPT_CONV_EPILOGUE, 0)


@pytest.mark.parametrize("cfg", CONVS)
@pytest.mark.parametrize("act", [0, 1, 3, 2])
@pytest.mark.parametrize("wdt", [flib.DT_I8, flib.DT_I4])
@pytest.mark.parametrize("conv_epilogue", [0, 2, 3], indirect=True)
def test_qconv2d_i8(ctx, orc, cfg, act, wdt, conv_epilogue):
    """I8 weights: conv2d_packed_i8x4; I4 weights: conv2d_packed_i4x8 (activations quantised to 16 levels)."""
    rng = np.random.default_rng(6000 + cfg["c"])
    kk = cfg["c"] // cfg["groups"] * cfg["kh"] * cfg["kw"]
    x = rng.uniform(0, 1, (cfg["b"], cfg["c"], cfg["h"], cfg["w"])).astype(np.float32)
    wt = (rng.standard_normal((cfg["oc"], kk)) * np.sqrt(2.0 / kk)).astype(np.float32)
    bias = (rng.standard_normal(cfg["oc"]) * 0.05).astype(np.float32)
    pw = fastnn_amd.quantize_weights(wdt, wt)
    h = ctx.register(pw)
    args = (cfg["kh"], cfg["kw"], cfg["stride"], cfg["pad"], cfg["dil"], cfg["groups"])
    want, want_acc, _, _ = orc.qconv2d_i8(x, to_oracle(orc, pw), *args, bias=bias, act=act, want_acc=True)
    got, acc = ctx.qconv2d(h, x, cfg["oc"], *args, bias=bias, act=act, want_acc=True)
    assert np.array_equal(acc, want_acc)   # i32 accumulators (incl. bias_q) bit-exact
    assert_close(got, want, 1e-5)          # same f32 formula; expf/tanhf differ in the last ulp
    got_nb = ctx.qconv2d(h, x, cfg["oc"], *args, act=act)
    assert_close(got_nb, orc.qconv2d_i8(x, to_oracle(orc, pw), *args, act=act), 1e-5)
    # the direct kernel (no im2col operand, no matrix cores) gives the same accumulators
    got_d, acc_d = ctx.qconv2d(h, x, cfg["oc"], *args, bias=bias, act=act, want_acc=True, flags=flib.FLAG_FORCE_GENERIC)
    assert np.array_equal(acc_d, want_acc)
    assert_close(got_d, want, 1e-5)
    ctx.release(h)


IMPLICIT_CONVS = CONVS + [
    dict(b=2, c=8, h=40, w=40, oc=24, kh=3, kw=3, stride=1, pad=1, dil=1, groups=1),     # taken by shape; one k slice
    dict(b=1, c=20, h=30, w=33, oc=40, kh=3, kw=3, stride=2, pad=1, dil=1, groups=1),    # two k slices, odd pixel count
    dict(b=3, c=64, h=7, w=9, oc=70, kh=3, kw=3, stride=1, pad=1, dil=1, groups=1),      # four k slices, blocks over three images
    dict(b=2, c=6, h=50, w=46, oc=12, kh=5, kw=5, stride=1, pad=2, dil=1, groups=2),     # groups, K past a step's end
    dict(b=1, c=230, h=12, w=14, oc=20, kh=3, kw=3, stride=1, pad=1, dil=1, groups=1),   # K = 2070: more taps than the geometry table holds
    dict(b=2, c=16, h=36, w=34, oc=16, kh=3, kw=3, stride=1, pad=0, dil=2, groups=1),    # no padding: every tap of every pixel inside the image
    dict(b=2, c=96, h=13, w=11, oc=300, kh=3, kw=3, stride=1, pad=1, dil=1, groups=1),   # many channels: ten blocks of 32 (fused: two per wave), K = 864
    dict(b=3, c=128, h=10, w=10, oc=136, kh=1, kw=1, stride=1, pad=0, dil=1, groups=1),  # 1x1, a ragged last channel block, blocks over two images
    dict(b=1, c=140, h=9, w=9, oc=72, kh=3, kw=3, stride=1, pad=1, dil=1, groups=1),     # K = 1260: the most steps the fused kernel holds in LDS
]


@pytest.mark.parametrize("cfg", IMPLICIT_CONVS)
@pytest.mark.parametrize("act", [0, 3])
@pytest.mark.parametrize("wdt", [flib.DT_I8, flib.DT_I4])
@pytest.mark.parametrize("mode", [0, 1, 3])
def test_qconv2d_implicit_gemm(ctx, orc, cfg, act, wdt, mode):
    """The kernels that fetch and quantise the im2col taps themselves (no int8 operand in memory): the same
    accumulators as conv2d_packed_i8x4 / conv2d_packed_i4x8, bit for bit.  mode 1: the implicit kernel (taps straight
    into the MFMA operand registers, a pass over the pixels per channel block) wherever it can run; mode 3: the fused
    kernel (a workgroup quantises 32 pixels once into LDS and runs all channels against them) wherever it can run;
    mode 0: what the library picks by shape."""
    ctx.set_option(flib.OPT_CONV_IMPLICIT, mode)
    try:
        rng = np.random.default_rng(6100 + cfg["c"])
        kk = cfg["c"] // cfg["groups"] * cfg["kh"] * cfg["kw"]
        x = rng.uniform(-0.3, 1, (cfg["b"], cfg["c"], cfg["h"], cfg["w"])).astype(np.float32)
        x[1 % cfg["b"]] *= 3.0   # images with different ranges
        wt = (rng.standard_normal((cfg["oc"], kk)) * np.sqrt(2.0 / kk)).astype(np.float32)
        bias = (rng.standard_normal(cfg["oc"]) * 0.05).astype(np.float32)
        pw = fastnn_amd.quantize_weights(wdt, wt)
        h = ctx.register(pw)
        args = (cfg["kh"], cfg["kw"], cfg["stride"], cfg["pad"], cfg["dil"], cfg["groups"])
        want, want_acc, _, _ = orc.qconv2d_i8(x, to_oracle(orc, pw), *args, bias=bias, act=act, want_acc=True)
        got, acc = ctx.qconv2d(h, x, cfg["oc"], *args, bias=bias, act=act, want_acc=True)
        assert np.array_equal(acc, want_acc)
        assert_close(got, want, 1e-5)
        got_nb = ctx.qconv2d(h, x, cfg["oc"], *args, act=act)
        assert_close(got_nb, orc.qconv2d_i8(x, to_oracle(orc, pw), *args, act=act), 1e-5)
        ctx.release(h)
    finally:
        ctx.set_option(flib.OPT_CONV_IMPLICIT, 0)


@pytest.mark.parametrize("wdt", [flib.DT_I8, flib.DT_I4])
def test_qconv2d_constant_and_empty(ctx, orc, wdt):
    x = np.full((1, 2, 4, 4), 0.5, np.float32)
    pw = fastnn_amd.quantize_weights(wdt, np.array([[-0.2, 0.1], [0.1, 0.1]], np.float32))
    h = ctx.register(pw)
    got = ctx.qconv2d(h, x, 2, 1, 1, 1, 0, 1, 1)
    assert_close(got, orc.qconv2d_i8(x, to_oracle(orc, pw), 1, 1, 1, 0, 1, 1), 1e-6)
    # kernel larger than the padded input: empty output, no launch
    y = ctx.qconv2d(h, np.zeros((1, 2, 1, 1), np.float32)[:, :, :1, :1], 2, 1, 1, 1, 0, 1, 1)
    assert y.shape == (1, 2, 1, 1)
    ctx.release(h)


@pytest.mark.parametrize("cfg", CONVS)
@pytest.mark.parametrize("wdt", [flib.DT_I8, flib.DT_I4])
@pytest.mark.parametrize("za", [0.0, 0.37])
def test_qconv2d_on_i8_payload(ctx, orc, cfg, wdt, za):
    """conv2d_i8_i8 / conv2d_i4_i8: int8 NCHW payload in, im2col on the integers (padding = 0),
    integer GEMM, then the 4-term formula with integer bias (I8) or the matmul_i4_i8 formula with
    an f32 bias (I4).  With za == 0 and no bias/activation the result is an exact function of
    the integer accumulators, so it must match the oracle to the last f32 operation (1e-6)."""
    rng = np.random.default_rng(6200 + cfg["c"])
    kk = cfg["c"] // cfg["groups"] * cfg["kh"] * cfg["kw"]
    shape = (cfg["b"], cfg["c"], cfg["h"], cfg["w"])
    q = rng.integers(-128, 128, shape).astype(np.int8)
    payload = orc.make_payload(0.0123, za, q.reshape(-1))
    wt = (rng.standard_normal((cfg["oc"], kk)) * np.sqrt(2.0 / kk)).astype(np.float32)
    bias = (rng.standard_normal(cfg["oc"]) * 0.05).astype(np.float32)
    pw = fastnn_amd.quantize_weights(wdt, wt)
    h = ctx.register(pw)
    args = (cfg["kh"], cfg["kw"], cfg["stride"], cfg["pad"], cfg["dil"], cfg["groups"])
    tol = 1e-6 if za == 0.0 else 2e-5
    assert_close(ctx.qconv2d_i8act(h, payload, shape, cfg["oc"], *args),
                 orc.qconv2d_i8payload(payload, shape, to_oracle(orc, pw), *args), tol, "plain")
    for act in (0, 1, 2, 3):
        want = orc.qconv2d_i8payload(payload, shape, to_oracle(orc, pw), *args, bias=bias, act=act)
        got = ctx.qconv2d_i8act(h, payload, shape, cfg["oc"], *args, bias=bias, act=act)
        assert_close(got, want, max(tol, 1e-5), f"act {act}")
    ctx.release(h)


def test_qconv2d_on_i8_payload_rejects_other_weight_types(ctx):
    pw = fastnn_amd.quantize_weights(flib.DT_U8, np.ones((2, 2), np.float32))
    h = ctx.register(pw)
    with pytest.raises(fastnn_amd.FnnError) as e:
        ctx.qconv2d_i8act(h, np.zeros(8 + 2 * 16, np.uint8), (1, 2, 4, 4), 2, 1, 1, 1, 0, 1, 1)
    assert e.value.kind == "UnsupportedOp"
    ctx.release(h)


FLOAT_CONVS = [
    dict(b=2, c=4, h=20, w=24, oc=16, kh=3, kw=3, stride=2, pad=1, dil=1, groups=1),
    dict(b=1, c=32, h=12, w=12, oc=48, kh=1, kw=1, stride=1, pad=0, dil=1, groups=1),
    dict(b=1, c=8, h=10, w=7, oc=6, kh=3, kw=2, stride=1, pad=2, dil=2, groups=2),
    dict(b=3, c=32, h=9, w=9, oc=40, kh=3, kw=3, stride=1, pad=1, dil=1, groups=1),
]


@pytest.mark.parametrize("cfg", FLOAT_CONVS)
@pytest.mark.parametrize("wdt", [flib.DT_U8, flib.DT_U4, flib.DT_F8, flib.DT_F8R, flib.DT_F4, flib.DT_I4CB])
def test_qconv2d_float_weight_types(ctx, orc, cfg, wdt):
    """Weight types without an integer conv kernel: f32 convolution with the dequantised weights
    (im2col rows + fused-dequant MatMul + NCHW turn on the GPU); f32 accumulation, stated bound 2e-5."""
    rng = np.random.default_rng(6100 + cfg["c"] + wdt)
    kk = cfg["c"] // cfg["groups"] * cfg["kh"] * cfg["kw"]
    x = rng.standard_normal((cfg["b"], cfg["c"], cfg["h"], cfg["w"])).astype(np.float32)
    wt = (rng.standard_normal((cfg["oc"], kk)) * np.sqrt(2.0 / kk)).astype(np.float32)
    bias = (rng.standard_normal(cfg["oc"]) * 0.05).astype(np.float32)
    pw = fastnn_amd.quantize_weights(wdt, wt)
    h = ctx.register(pw)
    args = (cfg["kh"], cfg["kw"], cfg["stride"], cfg["pad"], cfg["dil"], cfg["groups"])
    for act in (0, 1, 2, 3):
        want = orc.qconv2d_float(x, to_oracle(orc, pw), *args, bias=bias, act=act)
        got = ctx.qconv2d(h, x, cfg["oc"], *args, bias=bias, act=act)
        assert_close(got, want, 2e-5, f"act {act}")
    assert_close(ctx.qconv2d(h, x, cfg["oc"], *args), orc.qconv2d_float(x, to_oracle(orc, pw), *args), 2e-5, "no bias")
    got_g = ctx.qconv2d(h, x, cfg["oc"], *args, bias=bias, act=3, flags=flib.FLAG_FORCE_GENERIC)
    assert_close(got_g, orc.qconv2d_float(x, to_oracle(orc, pw), *args, bias=bias, act=3), 2e-5, "shape-agnostic kernel")
    with pytest.raises(fastnn_amd.FnnError) as e:      # no integer accumulators on this path
        ctx.qconv2d(h, x, cfg["oc"], *args, want_acc=True)
    assert e.value.kind == "Dispatch"
    ctx.release(h)


# --------------------------------------------------------------------------- error behaviour
def test_error_paths_mirror_reference_messages(ctx):
    rng = np.random.default_rng(11)
    pw = fastnn_amd.quantize_weights(flib.DT_I8, rng.standard_normal((8, 16)).astype(np.float32))
    bad = fastnn_amd.PackedWeight(pw.dtype, 8, 16, pw.words, np.zeros(0, np.float32), pw.zeros)
    with pytest.raises(fastnn_amd.FnnError) as e:
        ctx.register(bad)
    assert e.value.kind == "Dispatch" and "scale" in e.value.message  # public_error_paths.rs:42-118
    bad = fastnn_amd.PackedWeight(pw.dtype, 8, 16, pw.words, pw.scales[:3].copy(), pw.zeros[:3].copy())
    with pytest.raises(fastnn_amd.FnnError) as e:
        ctx.register(bad)
    assert "incompatible with shape" in e.value.message
    bad = fastnn_amd.PackedWeight(pw.dtype, 8, 16, pw.words[:10].copy(), pw.scales, pw.zeros)
    with pytest.raises(fastnn_amd.FnnError) as e:
        ctx.register(bad)
    assert "payload too short" in e.value.message
    bad = fastnn_amd.PackedWeight(pw.dtype, 8, 16, pw.words, pw.scales, pw.zeros[:4].copy())
    with pytest.raises(fastnn_amd.FnnError) as e:
        ctx.register(bad)
    assert "length mismatch" in e.value.message
    with pytest.raises(fastnn_amd.FnnError) as e:
        ctx.register(fastnn_amd.PackedWeight(42, 8, 16, pw.words, pw.scales, pw.zeros))
    assert e.value.kind == "UnsupportedOp"
    h = ctx.register(pw, key=777)
    with pytest.raises(fastnn_amd.FnnError):
        ctx.register(pw, key=777)
    with pytest.raises(fastnn_amd.FnnError) as e:
        ctx.qmatmul(h, np.zeros((1, 16), np.float32), 8, act=9)
    assert e.value.kind == "UnsupportedOp"
    f8 = ctx.register(fastnn_amd.quantize_weights(flib.DT_F8, rng.standard_normal((8, 16)).astype(np.float32)))
    with pytest.raises(fastnn_amd.FnnError) as e:
        ctx.qmatmul_i8act(f8, np.zeros(8 + 16, np.uint8), 1, 8)
    assert e.value.kind == "UnsupportedOp"
    with pytest.raises(fastnn_amd.FnnError) as e:
        ctx.qconv2d(h, np.zeros((1, 4, 4, 4), np.float32), 8, 2, 2, 1, 0, 1, 0)
    assert "groups" in e.value.message
    out = ctx.qmatmul(h, np.zeros((0, 16), np.float32), 8)   # empty batch is a no-op
    assert out.shape == (0, 8)
    ctx.release(h)
    ctx.release(f8)


# --------------------------------------------------------------------------- matrix-core specifics
@pytest.mark.parametrize("dt", [0, 1, 4, 6])
@pytest.mark.parametrize("mag", [1e-30, 1e-6, 1.0, 3e4, 1e9, 1e30])
@pytest.mark.parametrize("m", [3, 6, 14, 40])
def test_mfma_activation_range_is_f32(ctx, orc, dt, mag, m):
    """Activations far outside f16 range: the power-of-two scaling (per row, or per row and K slice) keeps f32
    accuracy in every kernel of the M range (GEMV kernels, 16-row kernel, tiled GEMMs)."""
    rng = np.random.default_rng(7000 + dt)
    k, n = 2048, 48
    pw = fastnn_amd.quantize_weights(dt, _weights(rng, n, k))
    a = (rng.standard_normal((m, k)) * mag).astype(np.float32)
    a[1] *= 1e-3          # rows of very different magnitude
    a[2, :100] *= 1e3     # and a wide spread inside one row
    h = ctx.register(pw)
    want = orc.qmatmul(to_oracle(orc, pw), a, order=2)
    got = ctx.qmatmul(h, a, n)
    for r in range(m):    # row-wise: each row is held to the tolerance on its own scale
        assert_close(got[r], want[r], TOL_F32, f"row {r} mag {mag}")
    ctx.release(h)


@pytest.mark.parametrize("dt", [0, 1, 2, 3, 4, 5, 6])
def test_mfma_single_f16_rounding_meets_north_star_tolerance(ctx, orc, dt):
    """FNN_FLAG_ACT_F16_SINGLE (opt-in) rounds activations to f16 once.  Stated tolerance:
    1e-3 of max|ref| for every type; for the asymmetric integer formats the kernel removes the
    first-order effect of the rounding on the row's mean lane value (|mean q| up to ~60),
    without which the error would be ~1.5e-3."""
    rng = np.random.default_rng(7100 + dt)
    m, k, n = 64, 4096, 96
    pw = fastnn_amd.quantize_weights(dt, _weights(rng, n, k))
    a = rng.standard_normal((m, k)).astype(np.float32)
    h = ctx.register(pw)
    want = orc.qmatmul(to_oracle(orc, pw), a, order=2)
    got = ctx.qmatmul(h, a, n, flags=flib.FLAG_ACT_F16_SINGLE)
    assert rel_err(got, want) <= TOL_NORTH_STAR
    assert_close(ctx.qmatmul(h, a, n), want, TOL_F32)
    ctx.release(h)


@pytest.mark.parametrize("name,dt,k,n,ms", [("c1", 0, 4096, 4096, (1, 32)), ("c2", 1, 4096, 11008, (1, 16, 128, 256)),
                                           ("c3", 7, 4096, 4096, (1, 64, 256)),
                                           ("c4_f8_up", 4, 2048, 8192, (64,)), ("c4_f8_down", 4, 8192, 2048, (64,)),
                                           ("c4_f4_up", 6, 2048, 8192, (64,)), ("c4_f4_down", 6, 8192, 2048, (64,))])
def test_full_size_configs_on_row_sample(ctx, orc, name, dt, k, n, ms):
    """BASELINE shapes at full size; the oracle checks a random sample of output columns
    (weight rows are independent), plus linearity in the activations as a whole-tensor property.
    The codebook weight is also dequantised whole, bit for bit."""
    rng = np.random.default_rng(8000 + dt + k // 1024)
    if name in ("c1", "c2"):
        w = _weights(rng, n, k)
    elif name == "c3":
        w = _weights(rng, n, k, "laplace")
    else:
        w = (rng.standard_normal((n, k)) / np.sqrt(k)).astype(np.float32)
    pw = fastnn_amd.quantize_weights(dt, w)
    bias = (rng.standard_normal(n) * 0.01).astype(np.float32)
    h = ctx.register(pw)
    if name == "c3":
        assert ctx.dequant(h, n, k).tobytes() == orc.dequant(to_oracle(orc, pw)).tobytes()
    rows = np.sort(rng.choice(n, 48, replace=False))
    sub = to_oracle(orc, slice_rows(pw, rows))
    for m in ms:
        a = rng.standard_normal((m, k)).astype(np.float32)
        got = ctx.qmatmul(h, a, n, bias=bias, act=flib.ACT_SILU)
        want = orc.qmatmul(sub, a, order=2, bias=bias[rows], act=orc.ACT_SILU)
        assert_close(got[:, rows], want, TOL_F32, f"{name} M={m}")
        # linearity without epilogue: f(a1 + a2) == f(a1) + f(a2) up to rounding
        a2 = rng.standard_normal((m, k)).astype(np.float32)
        lhs = ctx.qmatmul(h, a + a2, n)
        rhs = ctx.qmatmul(h, a, n).astype(np.float64) + ctx.qmatmul(h, a2, n).astype(np.float64)
        assert rel_err(lhs, rhs) <= 1e-5
    ctx.release(h)


# --------------------------------------------------------------------------- FNN_FLAG_ACT_QUANT (opt-in fast mode)
@pytest.mark.parametrize("dt", [flib.DT_I8, flib.DT_I4])
@pytest.mark.parametrize("m,k,n", [(1, 256, 64), (7, 1000, 72), (64, 2048, 300), (256, 4096, 512)])
def test_act_quant_mode_is_the_reference_i8_activation_chain(ctx, orc, dt, m, k, n):
    """FNN_FLAG_ACT_QUANT with I8 / I4 weights = quantize_activations (dynamic scale max|x| / 127, zero 0) ->
    matmul_i8_i8 / matmul_i4_i8 -> + bias -> activation.  Without bias and activation the call gives, bit for bit,
    what the two entry points of that chain give one after the other (whose payload and integer accumulators are
    bit-exact against the oracle in their own tests); with them it matches the oracle's chain to 1e-6 (same f32
    formula; the activation's exponential differs in the last place).  It is NOT the result of matmul_i8: against the
    f32-activation oracle the difference is the 8-bit activation rounding, a few 1e-3 of max|ref|."""
    rng = np.random.default_rng(6100 + dt + m + k)
    pw = fastnn_amd.quantize_weights(dt, _weights(rng, n, k))
    a = rng.standard_normal((m, k)).astype(np.float32)
    bias = (rng.standard_normal(n) * 0.01).astype(np.float32)
    h = ctx.register(pw)
    po = to_oracle(orc, pw)
    got = ctx.qmatmul(h, a, n, flags=flib.FLAG_ACT_QUANT)
    payload = ctx.quantize_activations(a)
    assert payload.tobytes() == orc.quantize_activations(a).tobytes()
    two_calls = ctx.qmatmul_i8act(h, payload, m, n)
    two_calls = two_calls[0] if isinstance(two_calls, tuple) else two_calls
    assert np.array_equal(got, two_calls)
    want = orc.qmatmul_i8act(po, orc.quantize_activations(a), m)
    assert_close(got, want, 1e-6, f"act-quant {NAMES[dt]} {m}x{k}x{n}")
    for act in (1, 3):
        got_e = ctx.qmatmul(h, a, n, bias=bias, act=act, flags=flib.FLAG_ACT_QUANT)
        assert_close(got_e, orc.act_fn((want + bias).astype(np.float32), act), 1e-6, f"epilogue {act}")
        gen = ctx.qmatmul(h, a, n, bias=bias, act=act, flags=flib.FLAG_ACT_QUANT | flib.FLAG_FORCE_GENERIC)
        assert_close(gen, got_e, 1e-6, "shape-agnostic kernel")
    exact = orc.qmatmul(po, a, order=2)
    err = rel_err(got, exact)
    assert 1e-5 < err < 2e-2, err        # a different function from matmul_i8 / matmul_i4, close to it
    ctx.release(h)


@pytest.mark.parametrize("m,k,n", [(3, 256, 64), (64, 2048, 300), (256, 4096, 512), (130, 1024, 1100)])
def test_act_quant_mode_fp8_matrix_cores(ctx, orc, m, k, n):
    """FNN_FLAG_ACT_QUANT with F8 weights: each activation row is scaled by a power of two (row maximum into
    [128, 256)) and rounded to nearest-even E4M3, v_mfma_f32_32x32x16_fp8_fp8 multiplies the E4M3 bytes of both
    operands exactly and accumulates in f32.  Checked against the same computation in numpy (activations rounded to
    E4M3 through torch's float8_e4m3fn, f64 product with the dequantised weights): 1e-4 of max|ref| (measured 2e-5,
    spread evenly over the outputs: the fp8 matrix core aligns the products of a step with fewer guard bits than a
    chain of f32 fused multiply-adds; a wrong scale, byte order or rounding mode would show as 1e-2); against the
    f32-activation oracle the 3-bit mantissa of the activations shows: below 5e-2 of max|ref| (stated tolerance of
    the mode).  Other weight types refuse the flag."""
    import torch
    rng = np.random.default_rng(6200 + m + k)
    pw = fastnn_amd.quantize_weights(flib.DT_F8, _weights(rng, n, k))
    a = rng.standard_normal((m, k)).astype(np.float32)
    a[0] *= 1e-3
    a[m - 1] *= 3e4
    bias = (rng.standard_normal(n) * 0.01).astype(np.float32)
    h = ctx.register(pw)
    po = to_oracle(orc, pw)
    got = ctx.qmatmul(h, a, n, bias=bias, act=1, flags=flib.FLAG_ACT_QUANT)
    mx = np.abs(a).max(axis=1)
    ex = np.where(mx > 0, np.floor(np.log2(np.maximum(mx, 1e-300))) - 7, 0.0)
    scaled = (a / (2.0 ** ex)[:, None]).astype(np.float32)
    a8 = torch.from_numpy(scaled).to(torch.float8_e4m3fn).to(torch.float32).numpy().astype(np.float64) * (2.0 ** ex)[:, None]
    deq = orc.dequant(po).astype(np.float64)
    want = np.maximum(a8 @ deq.T + bias, 0.0)
    assert_close(got, want, 1e-4, f"fp8 act-quant {m}x{k}x{n}")
    exact = orc.qmatmul(po, a, order=2, bias=bias, act=1)
    assert rel_err(got, exact) < 5e-2
    ctx.release(h)
    for dt in (flib.DT_U8, flib.DT_F4, flib.DT_I4CB):
        pw2 = fastnn_amd.quantize_weights(dt, _weights(rng, 32, 64))
        h2 = ctx.register(pw2)
        with pytest.raises(flib.FnnError) as e:
            ctx.qmatmul(h2, a[:, :64].copy(), 32, flags=flib.FLAG_ACT_QUANT)
        assert e.value.kind == "UnsupportedOp"
        ctx.release(h2)
