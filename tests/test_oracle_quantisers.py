"""Pins the oracle's weight quantisers and dequantiser: the reference's literal fixtures,
invariants the reference itself asserts (|deq - x| <= scale), closed forms, float64
re-derivations, and brute-force argmin checks."""
import numpy as np
import pytest


def _unpack_np(dt, words, rows, inner):
    """Independent vectorised unpack of raw lane integers (no decode tables)."""
    bits = 8 if dt in (0, 2, 4, 5) else 4
    items = 32 // bits
    kp = -(-inner // items)
    w = words[: rows * kp].reshape(rows, kp).astype(np.uint64)
    lanes = np.stack([(w >> np.uint64(bits * i)) & np.uint64((1 << bits) - 1) for i in range(items)], axis=-1)
    return lanes.reshape(rows, kp * items)[:, :inner].astype(np.int64)


@pytest.mark.parametrize("dt,bits", [(0, 8), (1, 4)])
def test_asym_int_quantiser_f64_rederivation(orc, dt, bits):
    rng = np.random.default_rng(10)
    w = (rng.standard_normal((9, 77)) * 0.02).astype(np.float32)
    w[3] = 0.125  # zero-range row -> (1, 0)
    p = orc.quantize(dt, w)
    U, B = 2 ** bits - 1, 2 ** (bits - 1)
    for r in range(w.shape[0]):
        mn, mx = np.float32(w[r].min()), np.float32(w[r].max())
        if mx == mn:
            assert p.scales[r] == 1.0 and p.zeros[r] == 0.0
            continue
        # same formula evaluated in f32 step by step (numpy scalars round every op)
        init = np.float32(mx - mn) / np.float32(U)
        lo, hi = np.float32(mn - init), np.float32(mx + init)
        scale = np.float32(hi - lo) / np.float32(U)
        zero = np.float32(lo + np.float32(B) * scale)
        assert p.scales[r] == scale and p.zeros[r] == zero
        # f64 meaning: the range [mn-init, mx+init] is cut into U steps, zero sits B steps above lo
        assert abs(float(scale) - (float(mx) - float(mn)) * (1 + 2 / U) / U) < 1e-9 + 1e-6 * float(scale)
    q = _unpack_np(dt, p.words, *w.shape)
    q = np.where(q >= B, q - 2 * B, q)
    deq = orc.dequant(p)
    assert np.array_equal(deq, (q.astype(np.float32) * p.scales[:, None] + p.zeros[:, None]).astype(np.float32))
    # the reference's own debug assertion (packed_tensor.rs:1009-1036)
    assert np.all(np.abs(deq - w) <= p.scales[:, None])
    # each lane is the nearest code: |x - deq| <= scale/2 (+ rounding slack) unless clamped
    inner = (q > -B) & (q < B - 1)
    assert np.all(np.abs(deq - w)[inner] <= 0.5 * np.broadcast_to(p.scales[:, None], w.shape)[inner] * (1 + 1e-3))
    # margin words and tail lanes are zero
    assert np.all(p.words[-16:] == 0)
    assert p.words.size == w.shape[0] * p.words_per_row + 16


def test_tail_lanes_are_packed_from_zero(orc):
    w = np.full((2, 5), 3.0, np.float32)
    w[0, 0] = -1.0
    p = orc.quantize(orc.I8, w)
    lanes = _unpack_np(orc.I8, p.words, 2, 8)
    # row 0: tail value 0.0 goes through pack_from_f32 directly (lane integer 0), not (0-zp)/s
    assert np.all(lanes[0, 5:] == 0)


def test_fp4_quantiser_literals(orc, golden):
    g = golden["fp4_quantiser"]["per_channel_scale_zp"]
    i = np.arange(64, dtype=np.float32)
    data = np.stack([np.float32(-5.0) + i * np.float32(10.0) / np.float32(63.0),
                     np.float32(1.0) + i * np.float32(4.0) / np.float32(63.0)])
    p = orc.quantize(orc.F4, data)
    assert abs(p.scales[0] - g["expected_scale"][0]) < g["abs_tol"]
    assert abs(p.scales[1] - g["expected_scale"][1]) < g["abs_tol"]
    assert abs(p.zeros[0] - g["expected_zero_row0"]) < g["abs_tol"]
    assert abs(p.zeros[1] - 3.0) < 1e-5  # mean of the uniform ramp 1..5
    r = golden["fp4_quantiser"]["per_channel_roundtrip"]
    ramp = (np.float32(-6.0) + i * np.float32(12.0) / np.float32(63.0)).reshape(1, 64)
    p = orc.quantize(orc.F4, ramp)
    assert np.all(np.abs(orc.dequant(p) - ramp) <= p.scales[0] + 1e-6)


def test_fp4_quantiser_formula(orc):
    rng = np.random.default_rng(11)
    w = rng.standard_normal((6, 50)).astype(np.float32)
    w[2] = -0.5
    p = orc.quantize(orc.F4, w)
    for r in range(6):
        if w[r].max() == w[r].min():
            assert p.scales[r] == 1.0 and p.zeros[r] == 0.0
            continue
        s = np.float32(0)
        for v in w[r]:
            s = np.float32(s + v)
        mean = np.float32(s / np.float32(50))
        dev = max(abs(np.float32(mean - w[r].min())), abs(np.float32(w[r].max() - mean)))
        assert p.zeros[r] == mean and p.scales[r] == np.float32(dev / np.float32(4))
    deq = orc.dequant(p)
    # codes live in [-4, 4]: error bounded by half the widest code gap in that range (1.0) * scale
    assert np.all(np.abs(deq - w) <= 0.5 * p.scales[:, None] * (1 + 1e-4) + 1e-7)


def test_fp8_quantiser_closed_form(orc):
    rng = np.random.default_rng(12)
    w = (rng.standard_normal((5, 33)) * 3).astype(np.float32)
    w[4] = 0
    p = orc.quantize(orc.F8, w)
    for r in range(4):
        assert p.scales[r] == np.float32(np.abs(w[r]).max()) / np.float32(240.0)
        codes = _unpack_np(orc.F8, p.words, 5, 33)[r]
        am = int(np.argmax(np.abs(w[r])))
        assert codes[am] & 0x7F == 0x77  # the row maximum encodes to +-240
    assert p.scales[4] == 1.0 and np.all(p.zeros == 0)
    deq = orc.dequant(p)
    assert np.all(np.abs(deq - w)[:4] <= np.abs(w[:4]) * 2 ** -4 + p.scales[:4, None] * 2 ** -9 * 1.01)


def test_codebook_fixture_and_invariants(orc, golden):
    g = golden["codebook_fixture"]
    data = np.array(g["data"], np.float32).reshape(g["rows"], g["inner"])
    p = orc.quantize(orc.I4CB, data, qblock=g["qblock"])
    assert p.scales.size == g["n_scales"] and p.codebook.shape == (16,)
    deq = orc.dequant(p)
    assert np.abs(deq - data).max() < g["max_err_below"]
    blocks = data.reshape(-1, g["qblock"])
    assert np.array_equal(p.scales, np.abs(blocks).max(axis=1))
    assert np.all(np.diff(p.codebook) >= 0)


@pytest.mark.parametrize("shape,qblock", [((8, 64), 32), ((5, 70), 32), ((3, 40), 8)])
def test_codebook_nibbles_are_argmin(orc, shape, qblock):
    rng = np.random.default_rng(13)
    w = rng.laplace(0, 0.02, shape).astype(np.float32)
    w[1, :qblock] = 0  # an all-zero block: scale 0, normalised values 0
    p = orc.quantize(orc.I4CB, w, qblock=qblock)
    rows, inner = shape
    bpr = -(-inner // qblock)
    nib = _unpack_np(orc.I4CB, p.words, rows, inner)
    for r in range(rows):
        for c in range(inner):
            s = p.scales[r * bpr + c // qblock]
            inv = np.float32(1.0) / s if s > 0 else np.float32(0)
            v = np.float32(w[r, c] * inv)
            d = np.abs(v - p.codebook)
            assert nib[r, c] == int(np.argmin(d))  # lowest index on ties
    assert p.scales[1 * bpr] == 0.0
    deq = orc.dequant(p)
    sc = np.repeat(p.scales.reshape(rows, bpr), qblock, axis=1)[:, :inner]
    assert np.array_equal(deq, (sc * p.codebook[nib]).astype(np.float32))
    assert p.zeros.size == 0


def test_kmeans16_closed_forms(orc):
    # n == 1 -> all centroids equal the value; empty -> zeros
    assert np.all(orc.kmeans16([0.25]) == 0.25)
    # 16 well separated tight clusters: Lloyd converges to the cluster means
    rng = np.random.default_rng(14)
    centres = np.linspace(-1, 1, 16)
    pts = (centres[:, None] + rng.uniform(-0.01, 0.01, (16, 40))).astype(np.float32)
    vals = pts.reshape(-1).copy()
    rng.shuffle(vals)
    cb = orc.kmeans16(vals)
    assert np.allclose(cb, pts.astype(np.float64).mean(axis=1), atol=1e-6)
    # fixed point: with the final codebook every centroid is the mean of its members
    data = rng.standard_normal(3000).astype(np.float32)
    cb = orc.kmeans16(data, iters=200)
    a = np.argmin(np.abs(data[:, None] - cb[None, :]), axis=1)
    for c in range(16):
        if np.any(a == c):
            assert abs(cb[c] - data[a == c].astype(np.float64).mean()) < 1e-4
    # percentile initialisation: with 0 iterations the centroids are order statistics
    cb0 = orc.kmeans16(data, iters=0)
    srt = np.sort(data)
    n = data.size
    want = [srt[min(int(np.float32((np.float32(i) + np.float32(0.5)) / np.float32(16)) * np.float32(n)), n - 1)]
            for i in range(16)]
    assert np.array_equal(cb0, np.array(want, np.float32))
    with pytest.raises(ValueError):
        orc.kmeans16([0.0, float("nan"), 1.0])


def test_i4_small_k_fixture(orc, golden):
    g = golden["i4_small_k"]
    data = np.array(g["data"], np.float32)
    scale = np.float32(np.abs(data).max()) / np.float32(7.0)
    p = orc.from_f32_slice(orc.I4, data, g["rows"], g["inner"], float(scale), 0.0)
    deq = orc.dequant(p).reshape(-1)
    assert np.all(np.abs(deq - data) <= scale + 0.01)
    assert p.words.size == 2 * 1 + 16  # one word per row of 4 elements


@pytest.mark.parametrize("dt", [0, 1, 2, 3, 4, 5, 6])
def test_dequant_is_one_multiply_add(orc, dt):
    rng = np.random.default_rng(15 + dt)
    rows, inner = 7, 37
    items = orc.items(dt)
    kp = -(-inner // items)
    words = rng.integers(0, 2 ** 32, rows * kp + 16, dtype=np.uint64).astype(np.uint32)
    scales = rng.uniform(0.01, 2, rows).astype(np.float32)
    zeros = rng.uniform(-1, 1, rows).astype(np.float32)
    p = orc.Packed(dt, rows, inner, words, scales, zeros)
    raw = np.stack([np.concatenate([orc.unpack_word(dt, int(w)) for w in words[r * kp:(r + 1) * kp]])[:inner]
                    for r in range(rows)])
    want = (raw * scales[:, None] + zeros[:, None]).astype(np.float32)
    got = orc.dequant(p)
    assert np.array_equal(np.isnan(got), np.isnan(want))
    assert np.array_equal(got[~np.isnan(got)], want[~np.isnan(want)])
    # grouped scales (fewer scales than rows) and single scale
    p1 = orc.Packed(dt, rows, inner, words, scales[:1].copy(), zeros[:1].copy())
    w1 = (raw * scales[0] + zeros[0]).astype(np.float32)
    g1 = orc.dequant(p1)
    assert np.array_equal(g1[~np.isnan(g1)], w1[~np.isnan(w1)])


def test_kmeans16_f32_sums_run_in_data_order(orc):
    """The Lloyd step adds each cluster's members into an f32 sum in data order (packed_tensor.rs:49-63);
    that order decides the last bit of the codebook.  Independent re-derivation: assignment by argmin
    (lowest index on ties), per-cluster running f32 sum via cumsum (sequential in numpy), one f32 divide.
    The case is order-sensitive: the same iteration with f64 means gives a different codebook."""
    rng = np.random.default_rng(77)
    data = np.concatenate([rng.uniform(-1, 1, 30000), rng.uniform(-1e-3, 1e-3, 10000)]).astype(np.float32)
    rng.shuffle(data)
    n = data.size
    srt = np.sort(data)
    c = np.array([srt[min(int(np.float32((np.float32(i) + np.float32(0.5)) / np.float32(16)) * np.float32(n)), n - 1)]
                  for i in range(16)], np.float32)
    c64 = c.copy()
    iters = 4
    for _ in range(iters):
        a = np.argmin(np.abs(data[:, None] - c[None, :]), axis=1)
        for ci in range(16):
            mem = data[a == ci]
            if mem.size:
                c[ci] = np.cumsum(mem, dtype=np.float32)[-1] / np.float32(mem.size)
        a64 = np.argmin(np.abs(data[:, None] - c64[None, :]), axis=1)
        for ci in range(16):
            mem = data[a64 == ci]
            if mem.size:
                c64[ci] = np.float32(mem.astype(np.float64).sum() / mem.size)
    got = orc.kmeans16(data, iters=iters)
    assert np.array_equal(got, np.sort(c))
    assert not np.array_equal(got, np.sort(c64))     # a pairwise / f64 sum would not pass the line above
