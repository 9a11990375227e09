"""Pins the oracle's quantised Conv2d lowering: equals a float64 convolution of the
dequantised operands, integer accumulators equal an exact integer convolution, and the
im2col index formula is checked against torch's unfold."""
import numpy as np
import pytest
import torch
import torch.nn.functional as F


def _qw(p, k, bits=8):
    if bits == 4:
        kp = -(-k // 8)
        words = p.words[: p.rows * kp].reshape(p.rows, kp)
        nib = (words[:, :, None] >> (4 * np.arange(8, dtype=np.uint32))) & 0xF
        nib = nib.astype(np.int64).reshape(p.rows, kp * 8)[:, :k]
        return np.where(nib >= 8, nib - 16, nib)
    kp = -(-k // 4)
    w = p.words[: p.rows * kp].view(np.int8).reshape(p.rows, kp * 4)[:, :k]
    return w.astype(np.int64)


@pytest.mark.parametrize("cfg", [
    dict(b=2, c=3, h=9, w=11, oc=4, kh=3, kw=3, stride=2, pad=1, dil=1, groups=1),
    dict(b=1, c=4, h=8, w=8, oc=6, kh=1, kw=1, stride=1, pad=0, dil=1, groups=1),
    dict(b=1, c=4, h=10, w=7, oc=4, kh=3, kw=2, stride=1, pad=2, dil=2, groups=2),
    dict(b=1, c=5, h=6, w=6, oc=3, kh=3, kw=3, stride=1, pad=1, dil=1, groups=1),
])
@pytest.mark.parametrize("act", [0, 1, 3])
@pytest.mark.parametrize("bits", [8, 4])
def test_conv_matches_float_conv_of_dequantised(orc, cfg, act, bits):
    """bits=8: conv2d_packed_i8x4; bits=4: conv2d_packed_i4x8 (16 activation levels, 4-bit weights)."""
    rng = np.random.default_rng(300)
    levels, half, qlo, qhi = (255.0, 128.0, -128, 127) if bits == 8 else (15.0, 8.0, -8, 7)
    b, c, h, w, oc, kh, kw = (cfg[x] for x in ("b", "c", "h", "w", "oc", "kh", "kw"))
    stride, pad, dil, groups = cfg["stride"], cfg["pad"], cfg["dil"], cfg["groups"]
    cg = c // groups
    kk = cg * kh * kw
    x = rng.uniform(0, 1, (b, c, h, w)).astype(np.float32)
    wt = (rng.standard_normal((oc, kk)) * 0.1).astype(np.float32)
    bias = (rng.standard_normal(oc) * 0.05).astype(np.float32)
    p = orc.quantize(orc.I8 if bits == 8 else orc.I4, wt)
    y, acc, sa, za = orc.qconv2d_i8(x, p, kh, kw, stride, pad, dil, groups, bias=bias, act=act, want_acc=True)
    qw = _qw(p, kk, bits)
    ocg = oc // groups
    for n in range(b):
        for g in range(groups):
            xs = torch.from_numpy(x[n:n + 1, g * cg:(g + 1) * cg].astype(np.float64))
            col = F.unfold(xs, (kh, kw), dilation=dil, padding=pad, stride=stride)[0].numpy().T  # [P, K]
            mn, mx = np.float32(col.min()), np.float32(col.max())
            s = sa[n * groups + g]
            z = za[n * groups + g]
            assert s == np.float32(mx - mn) / np.float32(levels)
            assert z == np.float32(mn + np.float32(half) * s)
            inv = np.float32(1.0) / s
            t = (col.astype(np.float32) - z) * inv
            qa = np.clip(np.sign(t) * np.floor(np.abs(t) + np.float32(0.5)), qlo, qhi).astype(np.int64)
            for f in range(ocg):
                ch = g * ocg + f
                sab = np.float32(s * p.scales[ch])
                bq = int(np.sign(bias[ch] / sab) * np.floor(abs(np.float32(bias[ch] / sab)) + 0.5))
                want_acc = qa @ qw[ch] + bq
                assert np.array_equal(acc[n, ch].reshape(-1), want_acc.astype(np.int32))
                # float meaning: conv of dequantised operands + dequantised bias
                da = qa * float(s) + float(z)
                dw = qw[ch] * float(p.scales[ch]) + float(p.zeros[ch])
                val = da @ dw + bq * float(sab)
                if act == 1:
                    val = np.maximum(val, 0)
                elif act == 3:
                    val = val / (1 + np.exp(-val))
                got = y[n, ch].reshape(-1)
                assert np.abs(got - val).max() <= 1e-4 * (np.abs(val).max() + 1), (cfg, ch)


def test_conv_out_size(orc):
    for (i, k, s, p, d) in [(640, 3, 2, 1, 1), (7, 3, 1, 0, 1), (5, 3, 1, 0, 3), (2, 5, 1, 0, 1), (8, 1, 1, 0, 1)]:
        dk = (k - 1) * d + 1
        want = (i + 2 * p - dk) // s + 1 if i + 2 * p >= dk else 0
        assert orc.conv_out_size(i, k, s, p, d) == want


def test_conv_constant_input_has_unit_scale(orc):
    x = np.full((1, 2, 4, 4), 0.5, np.float32)
    wt = np.ones((2, 2), np.float32) * 0.1
    wt[0, 0] = -0.2
    p = orc.quantize(orc.I8, wt)
    y, acc, sa, za = orc.qconv2d_i8(x, p, 1, 1, 1, 0, 1, 1, want_acc=True)
    assert sa[0] == 1.0 and za[0] == 0.0  # zero range -> scale 1, zero 0; 0.5 rounds to 1
    deq = orc.dequant(p)
    assert np.allclose(y[0, :, 0, 0], deq.sum(axis=1), atol=1e-5)


def test_conv_i4_constant_input_keeps_its_zero_point(orc):
    """The 4-bit activation quantiser forms zero = min + 8*scale also for a flat input
    (packed_conv.rs:260-263): 0.5 everywhere -> scale 1, zero 8.5, q = clamp(round(-8), -8, 7) = -8,
    dequantised back to exactly 0.5."""
    x = np.full((1, 2, 4, 4), 0.5, np.float32)
    wt = np.ones((2, 2), np.float32) * 0.1
    wt[0, 0] = -0.2
    p = orc.quantize(orc.I4, wt)
    y, acc, sa, za = orc.qconv2d_i8(x, p, 1, 1, 1, 0, 1, 1, want_acc=True)
    assert sa[0] == 1.0 and za[0] == 8.5
    qw = _qw(p, 2, 4)
    assert np.array_equal(acc[0, :, 0, 0], -8 * qw.sum(axis=1))
    deq = orc.dequant(p)
    assert np.allclose(y[0, :, 0, 0], 0.5 * deq.sum(axis=1), atol=1e-5)


@pytest.mark.parametrize("dt", ["U8", "U4", "F8", "F8R", "F4", "I4CB"])
@pytest.mark.parametrize("cfg", [
    dict(b=2, c=4, h=9, w=11, oc=6, kh=3, kw=3, stride=2, pad=1, dil=1, groups=1),
    dict(b=1, c=8, h=10, w=7, oc=4, kh=3, kw=2, stride=1, pad=2, dil=2, groups=2),
    dict(b=1, c=32, h=5, w=5, oc=8, kh=1, kw=1, stride=1, pad=0, dil=1, groups=1),
])
def test_float_conv_equals_torch_conv_of_dequantised_weights(orc, dt, cfg):
    """The weight types without an integer conv kernel: an ordinary convolution with the dequantised
    weights, bias added after the sum, then the activation (checked against torch.nn.functional.conv2d
    in float64, an independent implementation)."""
    rng = np.random.default_rng(77)
    b, c, h, w, oc, kh, kw = (cfg[x] for x in ("b", "c", "h", "w", "oc", "kh", "kw"))
    stride, pad, dil, groups = cfg["stride"], cfg["pad"], cfg["dil"], cfg["groups"]
    kk = c // groups * kh * kw
    x = rng.standard_normal((b, c, h, w)).astype(np.float32)
    wt = (rng.standard_normal((oc, kk)) * 0.2).astype(np.float32)
    bias = (rng.standard_normal(oc) * 0.1).astype(np.float32)
    code = getattr(orc, dt)
    if dt == "I4CB":
        p = orc.quantize(code, wt, qblock=32)
    else:
        p = orc.quantize(code, wt)
    deq = orc.dequant(p).astype(np.float64).reshape(oc, c // groups, kh, kw)
    for act in (0, 1, 2, 3):
        got = orc.qconv2d_float(x, p, kh, kw, stride, pad, dil, groups, bias=bias, act=act)
        ref = F.conv2d(torch.from_numpy(x.astype(np.float64)), torch.from_numpy(deq), torch.from_numpy(bias.astype(np.float64)),
                       stride=stride, padding=pad, dilation=dil, groups=groups).numpy()
        if act == 1:
            ref = np.maximum(ref, 0)
        elif act == 2:
            ref = 0.5 * ref * (1 + np.tanh(0.7978846 * (ref + 0.044715 * ref ** 3)))
        elif act == 3:
            ref = ref / (1 + np.exp(-ref))
        assert got.shape == ref.shape
        assert np.abs(got - ref).max() <= 2e-6 * (np.abs(ref).max() + 1), (dt, cfg, act)
    nb = orc.qconv2d_float(x, p, kh, kw, stride, pad, dil, groups)
    ref = F.conv2d(torch.from_numpy(x.astype(np.float64)), torch.from_numpy(deq), None, stride=stride, padding=pad,
                   dilation=dil, groups=groups).numpy()
    assert np.abs(nb - ref).max() <= 2e-6 * (np.abs(ref).max() + 1)


@pytest.mark.parametrize("cfg", [
    dict(b=2, c=3, h=9, w=11, oc=4, kh=3, kw=3, stride=2, pad=1, dil=1, groups=1),
    dict(b=1, c=4, h=10, w=7, oc=4, kh=3, kw=2, stride=1, pad=2, dil=2, groups=2),
    dict(b=1, c=8, h=6, w=6, oc=3, kh=1, kw=1, stride=1, pad=0, dil=1, groups=1),
])
@pytest.mark.parametrize("act", [0, 1, 2, 3])
@pytest.mark.parametrize("bits", [8, 4])
@pytest.mark.parametrize("zero_act", [True, False])
def test_conv_on_i8_payload_matches_float_conv(orc, cfg, act, bits, zero_act):
    """conv2d_i8_i8 / conv2d_i4_i8: the float meaning is a convolution of the dequantised int8
    activations (padding taps are the integer 0, i.e. the value `za`) with the dequantised
    weights; the 8-bit form adds the bias rounded to the accumulator grid, the 4-bit form
    adds it in f32."""
    rng = np.random.default_rng(310)
    b, c, h, w, oc, kh, kw = (cfg[x] for x in ("b", "c", "h", "w", "oc", "kh", "kw"))
    stride, pad, dil, groups = cfg["stride"], cfg["pad"], cfg["dil"], cfg["groups"]
    cg, ocg = c // groups, oc // groups
    kk = cg * kh * kw
    q = rng.integers(-128, 128, (b, c, h, w)).astype(np.int8)
    sa, za = np.float32(0.0123), np.float32(0.0 if zero_act else 0.37)
    payload = np.concatenate([np.array([sa, za], np.float32).view(np.uint8), q.view(np.uint8).reshape(-1)])
    wt = (rng.standard_normal((oc, kk)) * 0.1).astype(np.float32)
    bias = (rng.standard_normal(oc) * 0.05).astype(np.float32)
    p = orc.quantize(orc.I8 if bits == 8 else orc.I4, wt)
    y = orc.qconv2d_i8payload(payload, (b, c, h, w), p, kh, kw, stride, pad, dil, groups, bias=bias, act=act)
    qw = _qw(p, kk, bits)
    for n in range(b):
        for g in range(groups):
            xs = torch.from_numpy(q[n:n + 1, g * cg:(g + 1) * cg].astype(np.float64))
            col = F.unfold(xs, (kh, kw), dilation=dil, padding=pad, stride=stride)[0].numpy().T  # exact ints
            da = col * float(sa) + float(za)
            for f in range(ocg):
                ch = g * ocg + f
                dw = qw[ch] * float(p.scales[ch]) + float(p.zeros[ch])
                if bits == 8:
                    sab = np.float32(sa * p.scales[ch])
                    r = np.float32(bias[ch] / sab)
                    bq = int(np.sign(r) * np.floor(abs(r) + np.float32(0.5)))
                    val = da @ dw + bq * float(sab)
                else:
                    val = da @ dw + float(bias[ch])
                if act == 1:
                    val = np.maximum(val, 0)
                elif act == 2:
                    val = 0.5 * val * (1 + np.tanh(0.7978845608 * (val + 0.044715 * val ** 3)))
                elif act == 3:
                    val = val / (1 + np.exp(-val))
                got = y[n, ch].reshape(-1)
                assert np.abs(got - val).max() <= 2e-5 * (np.abs(val).max() + 1), (cfg, ch)
