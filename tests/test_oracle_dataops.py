"""Pins the oracle's restatement of the f32 data-movement kernels that sit between quantised
convolutions (concat, slice_f32, pool_f32 max and average, upsample_nearest2d) against numpy / torch."""
import numpy as np
import pytest
import torch
import torch.nn.functional as F


@pytest.mark.parametrize("axis", [0, 1, 2, 3])
def test_concat_is_numpy_concatenate(orc, axis):
    rng = np.random.default_rng(1)
    shapes = [[2, 3, 4, 5], [2, 3, 4, 5], [2, 3, 4, 5]]
    shapes[1][axis] += 2
    shapes[2][axis] = 1
    xs = [rng.standard_normal(s).astype(np.float32) for s in shapes]
    want = np.concatenate(xs, axis=axis)
    outer = int(np.prod(shapes[0][:axis]))          # params[2] = product of the dims before the axis
    got = orc.concat(xs, outer, want.size)
    assert np.array_equal(got, want.reshape(-1))


def test_concat_clamps_to_the_output(orc):
    a, b = np.arange(6, dtype=np.float32), np.arange(10, 14, dtype=np.float32)
    got = orc.concat([a, b], 1, 8)                  # room for 8 of the 10 values
    assert np.array_equal(got, np.concatenate([a, b])[:8])


@pytest.mark.parametrize("dim,start,end", [(1, 0, 4), (1, 4, 8), (2, 1, 3), (3, 2, 5), (0, 1, 2)])
def test_slice_is_numpy_slicing(orc, dim, start, end):
    rng = np.random.default_rng(2)
    x = rng.standard_normal((2, 8, 4, 6)).astype(np.float32)
    idx = [slice(None)] * 4
    idx[dim] = slice(start, end)
    want = x[tuple(idx)]
    stride = int(np.prod(x.shape[dim + 1:]))        # elements per index of the sliced dimension
    got = orc.slice_f32(x, start, end, stride, want.size)
    assert np.array_equal(got, want.reshape(-1))


@pytest.mark.parametrize("k,s,p", [(5, 1, 2), (2, 2, 0), (3, 2, 1), (3, 1, 0)])
def test_maxpool_is_torch_max_pool2d(orc, k, s, p):
    rng = np.random.default_rng(3)
    x = rng.standard_normal((2, 3, 11, 9)).astype(np.float32)
    want = F.max_pool2d(torch.from_numpy(x), k, s, p).numpy()
    got = orc.maxpool2d(x, k, s, p)
    assert got.shape == want.shape and np.array_equal(got, want)


@pytest.mark.parametrize("k,s,p", [(5, 1, 2), (2, 2, 0), (3, 2, 1), (3, 1, 0)])
def test_maxpool_indices_are_window_positions_of_torchs_argmax(orc, k, s, p):
    """The secondary output holds kh*kernel + kw of the maximum inside its window.  torch returns the flat position
    in the input plane instead: converted here (distinct random values, so the argmax is unique)."""
    rng = np.random.default_rng(4)
    x = rng.permutation(2 * 3 * 11 * 9).astype(np.float32).reshape(2, 3, 11, 9)
    want_v, flat = F.max_pool2d(torch.from_numpy(x), k, s, p, return_indices=True)
    got_v, got_i = orc.maxpool2d(x, k, s, p, return_indices=True)
    assert np.array_equal(got_v, want_v.numpy())
    flat = flat.numpy()
    hh = np.arange(flat.shape[2]).reshape(1, 1, -1, 1)
    ww = np.arange(flat.shape[3]).reshape(1, 1, 1, -1)
    kh = flat // 9 - (hh * s - p)
    kw = flat % 9 - (ww * s - p)
    assert got_i.dtype == np.int64 and np.array_equal(got_i, kh * k + kw)


def test_maxpool_indices_on_ties_and_empty_windows(orc):
    """Strict `>`: among equal values the first tap in (kh, kw) order stays; a window that sees only padding
    reports position 0."""
    x = np.zeros((1, 1, 4, 4), np.float32)
    x[0, 0, 1, 1] = x[0, 0, 1, 2] = x[0, 0, 2, 1] = 5.0
    v, i = orc.maxpool2d(x, 3, 1, 0, return_indices=True)        # 2x2 windows over the 4x4 plane
    assert np.array_equal(v, np.full((1, 1, 2, 2), 5.0, np.float32))
    assert i[0, 0].tolist() == [[1 * 3 + 1, 1 * 3 + 0], [0 * 3 + 1, 0 * 3 + 0]]
    v, i = orc.maxpool2d(np.ones((1, 1, 2, 2), np.float32), 1, 1, 1, return_indices=True)
    assert np.isneginf(v[0, 0, 0, 0]) and i[0, 0, 0, 0] == 0 and i[0, 0, 1, 1] == 0


def test_maxpool_window_in_the_padding_only_is_minus_inf(orc):
    x = np.ones((1, 1, 2, 2), np.float32)
    got = orc.maxpool2d(x, 1, 1, 1)                 # 4x4 output, the border windows see padding only
    assert got.shape == (1, 1, 4, 4)
    assert np.all(np.isneginf(got[0, 0, 0])) and got[0, 0, 1, 1] == 1.0


@pytest.mark.parametrize("k,s,p", [(5, 1, 2), (2, 2, 0), (3, 2, 1), (3, 1, 0)])
def test_avgpool_is_torch_avg_pool2d_without_padding_in_the_count(orc, k, s, p):
    """Mean over the taps inside the image: torch's avg_pool2d(count_include_pad=False), evaluated in
    f64 (the f32 window sum is within 1e-6 of it); on integer-valued input with a power-of-two tap
    count the result is exact."""
    rng = np.random.default_rng(5)
    x = rng.standard_normal((2, 3, 11, 9)).astype(np.float32)
    want = F.avg_pool2d(torch.from_numpy(x).double(), k, s, p, count_include_pad=False).numpy()
    got = orc.avgpool2d(x, k, s, p)
    assert got.shape == want.shape and np.abs(got - want).max() <= 1e-6
    xi = rng.integers(-50, 50, (1, 2, 8, 8)).astype(np.float32)
    want = F.avg_pool2d(torch.from_numpy(xi).double(), 2, 2, 0).numpy()
    assert np.array_equal(orc.avgpool2d(xi, 2, 2, 0), want.astype(np.float32))


def test_avgpool_window_in_the_padding_only_is_zero(orc):
    x = np.ones((1, 1, 2, 2), np.float32)
    got = orc.avgpool2d(x, 1, 1, 1)
    assert got.shape == (1, 1, 4, 4) and np.all(got[0, 0, 0] == 0.0) and got[0, 0, 1, 1] == 1.0


@pytest.mark.parametrize("sh,sw", [(2, 2), (1, 3), (3, 1)])
def test_upsample_is_numpy_repeat(orc, sh, sw):
    rng = np.random.default_rng(4)
    x = rng.standard_normal((2, 3, 5, 4)).astype(np.float32)
    want = np.repeat(np.repeat(x, sh, axis=2), sw, axis=3)
    assert np.array_equal(orc.upsample_nearest2d(x, sh, sw), want)
    if sh == sw:
        t = F.interpolate(torch.from_numpy(x), scale_factor=sh, mode="nearest").numpy()
        assert np.array_equal(want, t)


def test_dequantize_activations_inverts_the_payload(orc):
    """q*scale + zp with two f32 roundings (numpy does the same two operations); a quantise ->
    dequantise round trip stays within half a step; a payload that ends early reads as q = 0."""
    rng = np.random.default_rng(9)
    q = rng.integers(-128, 128, 300).astype(np.int8)
    scale, zp = np.float32(0.0371), np.float32(-0.42)
    payload = orc.make_payload(scale, zp, q)
    got = orc.dequantize_activations(payload, 300)
    assert np.array_equal(got, q.astype(np.float32) * scale + zp)
    x = rng.standard_normal(500).astype(np.float32)
    pl = orc.quantize_activations(x)
    s = pl[:4].view(np.float32)[0]
    assert np.abs(orc.dequantize_activations(pl, 500) - x).max() <= 0.5 * s * (1 + 1e-6)
    short = orc.dequantize_activations(payload[:8 + 100], 120)
    assert np.array_equal(short[:100], got[:100]) and np.all(short[100:] == zp)


def _pc_payload_image(nc, chunk, scales, zps, codes, tail=b""):
    """[nc u32][chunk u32][scales][zero points][codes] written out by hand"""
    return np.concatenate([np.array([nc, chunk], np.uint32).view(np.uint8), np.asarray(scales, np.float32).view(np.uint8),
                           np.asarray(zps, np.float32).view(np.uint8), np.asarray(codes, np.int8).view(np.uint8),
                           np.frombuffer(tail, np.uint8)])


def test_per_channel_activation_payloads_as_the_reference_loops_write_them(orc):
    """src/backend/cpu/mod.rs:6941-6975, 7026-7061: every channel's codes start at the first byte behind the header,
    channels in ascending order, so the block ends as the codes of the last channel in range.  Byte images worked out
    by hand; the closed form against the per-tensor quantiser on the last chunk; one channel = the per-tensor pair."""
    x = np.array([1.0, 2.0, 3.0, 10.0, 20.0, 30.0], np.float32)
    fill = np.full(24 + 6, 0xAA, np.uint8)
    got = orc.quantize_activations_per_channel(x, 6, [1.0, 5.0], [0.0, 0.0], fill)
    assert np.array_equal(got, _pc_payload_image(2, 3, [1.0, 5.0], [0.0, 0.0], [2, 4, 6], b"\xaa\xaa\xaa"))
    # an input view one value short of numel: channel 1 reaches positions 0 and 1 only, position 2 keeps channel 0's code
    got = orc.quantize_activations_per_channel(x[:5], 6, [1.0, 5.0], [0.0, 0.0], fill)
    assert np.array_equal(got, _pc_payload_image(2, 3, [1.0, 5.0], [0.0, 0.0], [2, 4, 3], b"\xaa\xaa\xaa"))
    # a zero scale gives code 0, a zero point shifts before the division, the clamp saturates; a payload that ends
    # inside the block is filled as far as it goes
    got = orc.quantize_activations_per_channel(x, 6, [1.0, 0.0], [0.0, 0.0], fill)
    assert np.array_equal(got[24:27].view(np.int8), [0, 0, 0])
    got = orc.quantize_activations_per_channel(x, 6, [1.0, 0.1], [0.0, 9.0], fill[:26])
    assert np.array_equal(got, _pc_payload_image(2, 3, [1.0, 0.1], [0.0, 9.0], [10, 110]))
    with pytest.raises(ValueError):
        orc.quantize_activations_per_channel(x, 6, [1.0, 5.0], [0.0, 0.0], fill[:23])
    # dequantiser: every channel reads the same block
    img = _pc_payload_image(2, 3, [1.0, 5.0], [0.5, -1.0], [2, 4, 6])
    out = orc.dequantize_activations_per_channel(img, np.full(7, 99.0, np.float32))
    assert np.array_equal(out, [2.5, 4.5, 6.5, 9.0, 19.0, 29.0, 99.0])
    out = orc.dequantize_activations_per_channel(img, np.full(5, 99.0, np.float32))
    assert np.array_equal(out, [2.5, 4.5, 6.5, 9.0, 19.0])
    out = orc.dequantize_activations_per_channel(img[:26], np.full(6, 99.0, np.float32))   # codes past the payload read as 0
    assert np.array_equal(out, [2.5, 4.5, 0.5, 9.0, 19.0, -1.0])
    with pytest.raises(ValueError):
        orc.dequantize_activations_per_channel(img[:20], np.zeros(6, np.float32))
    # closed form on random data
    rng = np.random.default_rng(77)
    for nc, numel in [(1, 64), (3, 100), (7, 7 * 33), (16, 16 * 5 + 3)]:
        xr = (rng.standard_normal(numel) * 3).astype(np.float32)
        sc = rng.uniform(0.01, 0.1, nc).astype(np.float32)
        zp = rng.uniform(-1, 1, nc).astype(np.float32)
        chunk = numel // nc
        pl = orc.quantize_activations_per_channel(xr, numel, sc, zp, np.zeros(8 + 8 * nc + chunk, np.uint8))
        last = xr[(nc - 1) * chunk:nc * chunk]
        assert np.array_equal(pl[8 + 8 * nc:], orc.quantize_activations(last, float(sc[-1]), float(zp[-1]))[8:])
        deq = orc.dequantize_activations_per_channel(pl, np.full(numel, 7.0, np.float32))
        q = pl[8 + 8 * nc:].view(np.int8).astype(np.float32)
        for ch in range(nc):
            assert np.array_equal(deq[ch * chunk:(ch + 1) * chunk], q * sc[ch] + zp[ch])
        assert np.all(deq[nc * chunk:] == 7.0)
        if nc == 1:
            assert np.array_equal(deq, orc.dequantize_activations(orc.quantize_activations(xr, float(sc[0]), float(zp[0])), numel))
