"""Pins the oracle's quantised MatMul (f32 and I8 activations): closed-form literals of the
reference's microkernel tests, its seeded end-to-end bounds, and the identity
(sum a*q)*s + z*sum(a) == sum a*(q*s+z) evaluated in float64."""
import numpy as np
import pytest

DT = {"i8": 0, "i4": 1, "u8": 2, "u4": 3, "f8": 4, "f8r": 5, "f4": 6, "i4cb": 7}


def test_f32act_asymmetric_zero_literal(orc, golden):
    g = golden["gemm_f32act"]["asymmetric_zero_is_per_input_sum"]
    p = orc.from_f32_slice(DT[g["dt"]], g["weights_f32"], g["n"], g["k"], g["w_scale"], g["w_zero"])
    a = np.array(g["input"], np.float32).reshape(g["m"], g["k"])
    for order in (0, 1, 2):
        out = orc.qmatmul(p, a, order=order)
        assert np.allclose(out.reshape(-1), g["expected"], atol=g["abs_tol"])


def test_i8act_literals(orc, golden):
    g = golden["gemm_i8act"]
    for c in g["cases"]:
        p = orc.from_f32_slice(DT[c["dt"]], c["weights_f32"], c["n"], c["k"], c["w_scale"], c["w_zero"])
        payload = orc.make_payload(c["act_scale"], c["act_zp"], c["act_i8"])
        out = orc.qmatmul_i8act(p, payload, c["m"]).reshape(-1)
        if "expected" in c:
            want = np.array(c["expected"], np.float64)
        else:
            deq = orc.dequant(p).astype(np.float64)
            a = np.array(c["act_i8"], np.float64) * c["act_scale"] + c["act_zp"]
            want = deq @ a
        assert np.allclose(out, want, atol=c["abs_tol"]), c["name"]
    c = g["with_scale"]
    w = np.arange(c["n"] * c["k"], dtype=np.float32)
    p = orc.from_f32_slice(0, w, c["n"], c["k"], c["w_scale"], 0.0)
    a = np.arange(c["k"], dtype=np.float32) * 0.5
    qa = np.clip(np.sign(a / c["act_scale"]) * np.floor(np.abs(a / c["act_scale"]) + 0.5), -128, 127).astype(np.int8)
    qw = np.clip(np.floor(w / c["w_scale"] + 0.5), -128, 127).reshape(c["n"], c["k"])
    out = orc.qmatmul_i8act(p, orc.make_payload(c["act_scale"], 0.0, qa), 1).reshape(-1)
    assert np.allclose(out, (qw @ qa.astype(np.float64)) * c["w_scale"] * c["act_scale"], atol=c["abs_tol"])
    c = g["batched_matches_f32_path"]
    w = (np.arange(c["n"] * c["k"]) % 4).astype(np.float32) - 1.5
    p = orc.from_f32_slice(0, w, c["n"], c["k"], 1.0, 0.0)
    qa = np.array(c["act_i8"], np.int8)
    out = orc.qmatmul_i8act(p, orc.make_payload(1.0, 0.0, qa), c["m"])
    ref = orc.qmatmul(p, qa.astype(np.float32).reshape(c["m"], c["k"]), order=0)
    assert np.allclose(out, ref, atol=c["abs_tol"])
    c = g["i4_signed_nibbles"]
    p = orc.from_f32_slice(1, c["weights_f32"], c["n"], c["k"], 1.0, 0.0)
    qa = np.array(c["act_i8"], np.int8)
    out = orc.qmatmul_i8act(p, orc.make_payload(1.0, 0.0, qa), c["m"])
    ref = orc.qmatmul(p, qa.astype(np.float32).reshape(c["m"], c["k"]), order=0)
    assert np.allclose(out, ref, atol=c["abs_tol"])


def test_seeded_end_to_end_bounds(orc, golden):
    """Same seeds, shapes and tolerances as the reference's cpu_reference_oracle tests."""
    for c in golden["seeded_end_to_end"]["cases"]:
        m, k, n = c["m"], c["k"], c["n"]
        a = orc.seeded_values(c["seed"], m * k).reshape(m, k)
        w = orc.seeded_values(c["seed"] + 1, k * n).reshape(k, n)
        q = c["quantize"]
        if q == "f4_sym":  # the reference's FP tests pack with from_f32_per_channel (symmetric)
            wt = np.ascontiguousarray(w.T)
            words = np.zeros(orc.lib().fnn_or_packed_words(6, n, k), np.uint32)
            sc, zr = np.zeros(n, np.float32), np.zeros(n, np.float32)
            orc.lib().fnn_or_quant_per_channel_sym(6, wt.reshape(-1), n, k, words, sc, zr)
            p = orc.Packed(6, n, k, words, sc, zr)
        else:
            p = orc.quantize_kn(DT[q], w)
        expected = np.zeros((m, n), np.float32)
        for i in range(m):
            for j in range(n):
                acc = np.float32(0)
                for d in range(k):
                    acc = np.float32(acc + a[i, d] * w[d, j])
                expected[i, j] = acc
        for order in (0, 1, 2):
            got = orc.qmatmul(p, a, order=order)
            allowed = np.maximum(c["abs_tol"], np.abs(expected) * c["rel_tol"])
            assert np.all(np.abs(got - expected) <= allowed), (c, order)


@pytest.mark.parametrize("dt", [0, 1, 2, 3, 4, 6, 7])
@pytest.mark.parametrize("m,k,n", [(1, 64, 48), (3, 100, 17), (5, 7, 9), (2, 4100, 6)])
def test_qmatmul_equals_f64_product_of_dequantised(orc, dt, m, k, n):
    rng = np.random.default_rng(100 + dt)
    w = (rng.standard_normal((n, k)) * 0.05).astype(np.float32)
    a = rng.standard_normal((m, k)).astype(np.float32)
    p = orc.quantize(dt, w)
    deq = orc.dequant(p).astype(np.float64)
    want = a.astype(np.float64) @ deq.T
    scale = np.abs(want).max() + 1e-30
    got64 = orc.qmatmul(p, a, order=2)
    assert np.abs(got64 - want).max() <= 2e-6 * scale
    for order, ktile in ((0, 0), (1, 0), (0, 4096), (1, 4096)):
        got = orc.qmatmul(p, a, order=order, k_tile=ktile)
        assert np.abs(got - want).max() <= 1e-4 * scale + 1e-5, (order, ktile)


def test_qmatmul_i4cb_as_written_is_reshape_not_transpose(orc):
    rng = np.random.default_rng(7)
    n = k = 32
    w = rng.laplace(0, 0.02, (n, k)).astype(np.float32)
    a = rng.standard_normal((2, k)).astype(np.float32)
    p = orc.quantize(orc.I4CB, w)
    deq = orc.dequant(p).astype(np.float64)
    intended = orc.qmatmul(p, a, order=2)
    written = orc.qmatmul(p, a, order=2, i4cb_as_written=True)
    assert np.allclose(intended, a @ deq.T, atol=1e-6)
    assert np.allclose(written, a @ deq.reshape(k, n), atol=1e-6)


@pytest.mark.parametrize("act", [1, 2, 3])
def test_epilogue_formulas_f64(orc, act):
    x = np.linspace(-6, 6, 481).astype(np.float32)
    got = orc.act_fn(x, act).astype(np.float64)
    xd = x.astype(np.float64)
    if act == 1:
        want = np.maximum(xd, 0)
    elif act == 2:
        want = 0.5 * xd * (1 + np.tanh(0.7978846 * (xd + 0.044715 * xd ** 3)))
    else:
        want = xd / (1 + np.exp(-xd))
    assert np.abs(got - want).max() < 1e-6
    out = np.array([[1.0, -2.0], [0.5, 3.0]], np.float32)
    bias = np.array([0.25, -1.0], np.float32)
    p = orc.from_f32_slice(0, [1, 0, 0, 1], 2, 2, 1.0, 0.0)  # identity weights
    y = orc.qmatmul(p, out, order=0, bias=bias, act=act)
    assert np.allclose(y, orc.act_fn(out + bias, act))


@pytest.mark.parametrize("dt", [0, 1])
@pytest.mark.parametrize("zp", [0.0, 0.375])
def test_i8act_exact_integers_and_affine_meaning(orc, dt, zp):
    rng = np.random.default_rng(200 + dt)
    m, k, n = 3, 61, 10
    w = (rng.standard_normal((n, k)) * 0.05).astype(np.float32)
    p = orc.quantize(dt, w)
    x = rng.standard_normal((m, k)).astype(np.float32)
    payload = orc.quantize_activations(x) if zp == 0.0 else orc.quantize_activations(x, 0.03, zp)
    sa = payload[:4].view(np.float32)[0]
    qa = payload[8:].view(np.int8).reshape(m, k).astype(np.int64)
    out, acc = orc.qmatmul_i8act(p, payload, m, want_acc=True)
    bits = 8 if dt == 0 else 4
    items = 32 // bits
    kp = -(-k // items)
    wq = p.words[: n * kp].reshape(n, kp).astype(np.uint64)
    lanes = np.stack([(wq >> np.uint64(bits * i)) & np.uint64((1 << bits) - 1) for i in range(items)], -1)
    lanes = lanes.reshape(n, -1)[:, :k].astype(np.int64)
    qw = np.where(lanes >= (1 << (bits - 1)), lanes - (1 << bits), lanes)
    if zp == 0.0:
        assert np.array_equal(acc, (qa @ qw.T).astype(np.int32))
        assert sa == np.float32(np.abs(x).max()) / np.float32(127.0)
    deq_w = qw * p.scales[:, None].astype(np.float64) + p.zeros[:, None].astype(np.float64)
    deq_a = qa * float(sa) + zp
    want = deq_a @ deq_w.T
    assert np.abs(out - want).max() <= 2e-5 * np.abs(want).max() + 1e-6


def test_quantize_activations_formula(orc):
    x = np.array([0.0, 1.0, -2.0, 0.49, 0.51, 127.0, -127.0, 63.5], np.float32)
    pl = orc.quantize_activations(x)
    s = pl[:4].view(np.float32)[0]
    assert s == np.float32(1.0) and pl[4:8].view(np.float32)[0] == 0.0
    assert list(pl[8:].view(np.int8)) == [0, 1, -2, 0, 1, 127, -127, 64]
    assert orc.quantize_activations(np.zeros(4, np.float32))[:4].view(np.float32)[0] == 1.0


@pytest.mark.parametrize("dt", [0, 1])
@pytest.mark.parametrize("m,threads", [(1, 1), (1, 4), (5, 3)])
def test_tuned_cpu_baseline_agrees_with_the_restatement(orc, dt, m, threads):
    """bench.py's cpu_baseline (AVX2 unpack + FMA dots, weight rows over threads) computes the same MatMul as the
    oracle's restatement; its summation order differs, so the comparison is at 1e-5 of max|out| (f64-accumulated
    reference), with ragged K and N and every epilogue."""
    import fastnn_amd
    rng = np.random.default_rng(50 + dt)
    n, k = 203, 1000 if dt == 0 else 1000 // 8 * 8 + 8
    pw = fastnn_amd.quantize_weights(dt, (rng.standard_normal((n, k)) * 0.05).astype(np.float32))
    po = orc.Packed(pw.dtype, pw.rows, pw.inner, pw.words, pw.scales, pw.zeros, pw.qblock, pw.codebook)
    a = rng.standard_normal((m, k)).astype(np.float32)
    bias = (rng.standard_normal(n) * 0.1).astype(np.float32)
    for act in range(4):
        want = orc.qmatmul(po, a, order=2, bias=bias, act=act)
        got = orc.cpu_qgemm(po, a, bias=bias, act=act, threads=threads)
        assert np.abs(got - want).max() <= 1e-5 * np.abs(want).max(), (dt, act)
    with pytest.raises(ValueError):
        orc.cpu_qgemm(orc.Packed(4, pw.rows, pw.inner, pw.words, pw.scales, pw.zeros), a)
