"""GPU tests of the host-side HipBackend: plans of WriteConst / CallKernel / Fill / MemCopy
instructions dispatched against a device arena, checked with the CPU oracle.  The plans are
laid out the way fastnn's compile step emits them for a quantised model: constants first,
then one CallKernel per layer, kernel names carrying the fused epilogue as a suffix."""
import numpy as np
import pytest

import fastnn_amd
from fastnn_amd import lib as flib
from fastnn_amd.backend import ExecutablePlan, HipBackend, KERNEL_OF, meta_of
from gpu_common import assert_close, to_oracle

pytestmark = pytest.mark.gpu


class Arena:
    """Bump allocator for byte offsets, 64-byte aligned like fastnn's memory planner slots."""

    def __init__(self):
        self.top = 0

    def take(self, nbytes):
        off = self.top
        self.top += (nbytes + 63) // 64 * 64
        return (off, nbytes)


@pytest.fixture(scope="module")
def be():
    b = HipBackend(0)
    yield b
    b.close()


def _w(rng, n, k):
    return (rng.standard_normal((n, k)) * 0.05).astype(np.float32)


def test_name_and_arena_roundtrip(be):
    assert be.name == "hip"
    be.allocate_arena(1000)
    assert not be.read_arena(0, 1000).any()          # a fresh arena is zero-filled
    data = np.arange(250, dtype=np.float32)
    be.write_arena(0, data)
    assert np.array_equal(be.read_arena(0, 1000, np.float32), data)
    be.write_arena(996, np.float32([7.0]))
    assert be.read_arena(996, 4, np.float32)[0] == 7.0
    with pytest.raises(flib.FnnError) as e:
        be.write_arena(998, np.float32([1.0]))
    assert e.value.kind == "Memory"
    with pytest.raises(flib.FnnError):
        be.read_arena(1, 1000)


@pytest.mark.parametrize("m", [1, 8, 64])
def test_mlp_block_plan_fp8_up_fp4_down(be, orc, m):
    """x -> FP8 up-projection + bias + GELU (fused suffix) -> FP4 down-projection -> residual add."""
    rng = np.random.default_rng(90 + m)
    d, f = 256, 1024
    x = rng.standard_normal((m, d)).astype(np.float32)
    up = fastnn_amd.quantize_weights(flib.DT_F8, _w(rng, f, d))
    down = fastnn_amd.quantize_weights(flib.DT_F4, _w(rng, d, f))
    b_up = (rng.standard_normal(f) * 0.1).astype(np.float32)
    a = Arena()
    s_x, s_up, s_bup, s_down = a.take(x.nbytes), a.take(up.words.nbytes), a.take(b_up.nbytes), a.take(down.words.nbytes)
    s_h, s_y, s_out = a.take(m * f * 4), a.take(m * d * 4), a.take(m * d * 4)
    plan = ExecutablePlan(a.top)
    plan.write_const(s_up[0], up.words).write_const(s_bup[0], b_up).write_const(s_down[0], down.words)
    plan.call_kernel("matmul_f8_gelu", [s_x, s_up, s_bup], s_h, [m, d, f], meta_of(up))
    plan.call_kernel("matmul_f4", [s_h, s_down], s_y, [m, f, d], meta_of(down))
    plan.call_kernel("add_f32", [s_y, s_x], s_out, [m * d])
    be.allocate_arena(a.top)
    be.write_arena(s_x[0], x)
    be.dispatch(plan)
    h_ref = orc.qmatmul(to_oracle(orc, up), x, bias=b_up, act=flib.ACT_GELU)
    y_ref = orc.qmatmul(to_oracle(orc, down), h_ref) + x
    got_h = be.read_arena(*s_h, np.float32).reshape(m, f)
    got = be.read_arena(*s_out, np.float32).reshape(m, d)
    assert_close(got_h, h_ref, 2e-5, "hidden")
    assert_close(got, y_ref, 1e-4, "block output")       # the second layer sees got_h, not h_ref
    # second dispatch with a new input: constants stay resident, result follows the input
    x2 = rng.standard_normal((m, d)).astype(np.float32)
    be.write_arena(s_x[0], x2)
    be.dispatch(plan)
    h2 = orc.qmatmul(to_oracle(orc, up), x2, bias=b_up, act=flib.ACT_GELU)
    y2 = orc.qmatmul(to_oracle(orc, down), h2) + x2
    assert_close(be.read_arena(*s_out, np.float32).reshape(m, d), y2, 1e-4, "second dispatch")
    times = be.dispatch_profile(plan)
    assert len(times) == len(plan) and all(t > 0 for t in times[3:])


@pytest.mark.parametrize("dt", list(range(8)))
@pytest.mark.parametrize("act", ["", "_relu", "_silu"])
def test_every_matmul_kernel_name(be, orc, dt, act):
    rng = np.random.default_rng(300 + dt)
    m, k, n = 3, 160, 72
    x = rng.standard_normal((m, k)).astype(np.float32)
    pw = fastnn_amd.quantize_weights(dt, _w(rng, n, k))
    a = Arena()
    s_x, s_w, s_o = a.take(x.nbytes), a.take(pw.words.nbytes), a.take(m * n * 4)
    plan = ExecutablePlan(a.top).write_const(s_x[0], x).write_const(s_w[0], pw.words)
    plan.call_kernel(KERNEL_OF[dt] + act, [s_x, s_w], s_o, [m, k, n], meta_of(pw))
    be.allocate_arena(a.top)
    be.dispatch(plan)
    code = {"": 0, "_relu": 1, "_silu": 3}[act]
    want = orc.qmatmul(to_oracle(orc, pw), x, act=code)
    assert_close(be.read_arena(*s_o, np.float32).reshape(m, n), want, 2e-5, KERNEL_OF[dt] + act)


@pytest.mark.parametrize("dt,name", [(flib.DT_I8, "matmul_i8_i8"), (flib.DT_I4, "matmul_i4_i8")])
@pytest.mark.parametrize("calibrated", [False, True])
def test_i8_activation_chain(be, orc, dt, name, calibrated):
    """quantize_activations -> matmul_*_i8: payload bytes bit-exact, output equal to the oracle's."""
    rng = np.random.default_rng(17)
    m, k, n = 6, 200, 40
    x = rng.standard_normal((m, k)).astype(np.float32)
    pw = fastnn_amd.quantize_weights(dt, _w(rng, n, k))
    a = Arena()
    s_x, s_w, s_q, s_o = a.take(x.nbytes), a.take(pw.words.nbytes), a.take(8 + m * k), a.take(m * n * 4)
    params = [m * k, 0, 0]
    scale, zp = np.float32(0.03), np.float32(0.25)
    if calibrated:
        params += [int(scale.view(np.uint32)), int(zp.view(np.uint32))]
    plan = ExecutablePlan(a.top).write_const(s_w[0], pw.words)
    plan.call_kernel("quantize_activations", [s_x], s_q, params)
    plan.call_kernel(name, [s_q, s_w], s_o, [m, k, n], meta_of(pw))
    be.allocate_arena(a.top)
    be.write_arena(s_x[0], x)
    be.dispatch(plan)
    payload = orc.quantize_activations(x, float(scale), float(zp)) if calibrated else orc.quantize_activations(x)
    assert np.array_equal(be.read_arena(*s_q), payload)
    want = orc.qmatmul_i8act(to_oracle(orc, pw), payload, m)
    assert_close(be.read_arena(*s_o, np.float32).reshape(m, n), want, 1e-6, name)


@pytest.mark.parametrize("calibrated", [False, True])
def test_quantize_then_dequantize_activations(be, orc, calibrated):
    """quantize_activations -> dequantize_activations (per-tensor): payload and the f32 values
    q*scale + zero are bit-identical to the oracle's; an output slice shorter than numel is filled
    as far as it goes."""
    rng = np.random.default_rng(19)
    x = rng.standard_normal(1000).astype(np.float32)
    a = Arena()
    s_x, s_q, s_y, s_short = a.take(x.nbytes), a.take(8 + x.size), a.take(x.nbytes), a.take(400)
    params = [x.size, 0, 0]
    scale, zp = np.float32(0.021), np.float32(-0.3)
    if calibrated:
        params += [int(scale.view(np.uint32)), int(zp.view(np.uint32))]
    plan = ExecutablePlan(a.top)
    plan.call_kernel("quantize_activations", [s_x], s_q, params)
    plan.call_kernel("dequantize_activations", [s_q], s_y, [x.size, 0, 0])
    plan.call_kernel("dequantize_activations", [s_q], s_short, [x.size, 0, 0])
    be.allocate_arena(a.top)
    be.write_arena(s_x[0], x)
    be.dispatch(plan)
    payload = orc.quantize_activations(x, float(scale), float(zp)) if calibrated else orc.quantize_activations(x)
    assert np.array_equal(be.read_arena(*s_q), payload)
    want = orc.dequantize_activations(payload, x.size)
    assert np.array_equal(be.read_arena(*s_y, np.float32), want)
    assert np.array_equal(be.read_arena(*s_short, np.float32), want[:100])


@pytest.mark.parametrize("nc,numel", [(4, 1000), (200, 200 * 11 + 3)])
def test_per_channel_quantize_then_dequantize_activations_plan(be, orc, nc, numel):
    """The per-channel instructions as the reference's compile emits them (src/backend/cpu/mod.rs:2319-2425: params
    [numel, 1, nc, scale bits.., zero-point bits..] for both): payload and values bit-identical to the reference's
    loops (src/backend/cpu/mod.rs:6941-6975, 7026-7061), eager and as a replayed graph; an instruction with too few
    params and a payload slice without room for its header are dispatch errors (the reference panics on both)."""
    rng = np.random.default_rng(23 + nc)
    x = (rng.standard_normal(numel) * 2).astype(np.float32)
    sc = rng.uniform(0.01, 0.1, nc).astype(np.float32)
    zp = rng.uniform(-1, 1, nc).astype(np.float32)
    chunk = numel // nc
    a = Arena()
    s_x, s_q, s_y, s_short = a.take(x.nbytes), a.take(8 + 8 * nc + chunk), a.take(x.nbytes), a.take(4 * (chunk + 3))
    params = [numel, 1, nc] + [int(v) for v in sc.view(np.uint32)] + [int(v) for v in zp.view(np.uint32)]
    plan = ExecutablePlan(a.top)
    plan.call_kernel("quantize_activations", [s_x], s_q, params)
    plan.call_kernel("dequantize_activations", [s_q], s_y, params)
    plan.call_kernel("dequantize_activations", [s_q], s_short, params)
    be.allocate_arena(a.top)
    before_q = np.arange(s_q[1], dtype=np.uint32).astype(np.uint8)
    before_y = np.full(numel, 5.0, np.float32)
    want_q = orc.quantize_activations_per_channel(x, numel, sc, zp, before_q)
    want_y = orc.dequantize_activations_per_channel(want_q, before_y)
    for rep in range(3):
        be.write_arena(s_x[0], x)
        be.write_arena(s_q[0], before_q)
        be.write_arena(s_y[0], before_y)
        be.write_arena(s_short[0], before_y[:chunk + 3])
        be.dispatch(plan)
        assert np.array_equal(be.read_arena(*s_q), want_q), rep
        assert np.array_equal(be.read_arena(*s_y, np.float32), want_y), rep
        assert np.array_equal(be.read_arena(*s_short, np.float32), orc.dequantize_activations_per_channel(want_q, before_y[:chunk + 3])), rep
    with pytest.raises(flib.FnnError) as e:
        be.dispatch(ExecutablePlan(a.top).call_kernel("quantize_activations", [s_x], s_q, params[:-1]))
    assert e.value.kind == "Dispatch"
    with pytest.raises(flib.FnnError) as e:
        be.dispatch(ExecutablePlan(a.top).call_kernel("quantize_activations", [s_x], (s_q[0], 8 * nc), params))
    assert e.value.kind == "Dispatch"


@pytest.mark.parametrize("act,code", [("", 0), ("_relu", 1), ("_silu", 3)])
@pytest.mark.parametrize("wdt,kname", [(flib.DT_I8, "conv2d_i8"), (flib.DT_I4, "conv2d_i4")])
def test_conv2d_i8_plan(be, orc, act, code, wdt, kname):
    """conv2d_i8 / conv2d_i4: the integer kernel is picked by the bit width of the weight metadata."""
    rng = np.random.default_rng(41)
    b, c, h, w, oc, kh, kw, stride, pad, dil, groups = 2, 8, 14, 11, 12, 3, 3, 2, 1, 1, 2
    kk = c // groups * kh * kw
    x = rng.uniform(0, 1, (b, c, h, w)).astype(np.float32)
    pw = fastnn_amd.quantize_weights(wdt, (rng.standard_normal((oc, kk)) * 0.1).astype(np.float32))
    bias = (rng.standard_normal(oc) * 0.05).astype(np.float32)
    want = orc.qconv2d_i8(x, to_oracle(orc, pw), kh, kw, stride, pad, dil, groups, bias=bias, act=code)
    a = Arena()
    s_x, s_w, s_b, s_y = a.take(x.nbytes), a.take(pw.words.nbytes), a.take(bias.nbytes), a.take(want.nbytes)
    plan = ExecutablePlan(a.top).write_const(s_w[0], pw.words).write_const(s_b[0], bias)
    plan.call_kernel(kname + act, [s_x, s_w, s_b], s_y, [stride, pad, dil, groups, c, h, w, kh, kw],
                     meta_of(pw, [oc, c // groups, kh, kw]))
    be.allocate_arena(a.top)
    be.write_arena(s_x[0], x)
    be.dispatch(plan)
    assert_close(be.read_arena(*s_y, np.float32).reshape(want.shape), want, 1e-5, kname + act)


@pytest.mark.parametrize("act,code", [("", 0), ("_relu", 1), ("_gelu", 2), ("_silu", 3)])
@pytest.mark.parametrize("wdt,kname", [(flib.DT_I8, "conv2d_i8_i8"), (flib.DT_I4, "conv2d_i4_i8")])
@pytest.mark.parametrize("calibrated", [False, True])
def test_conv2d_on_i8_payload_plan(be, orc, act, code, wdt, kname, calibrated):
    """quantize_activations -> conv2d_{i8,i4}_i8: the conv reads the int8 payload (no second
    quantisation); the weight kernel is picked by the bit width of the weight metadata.
    Calibrated: scale/zero given as f32 bit patterns, zero != 0 (the dequantised-lane form)."""
    rng = np.random.default_rng(43)
    b, c, h, w, oc, kh, kw, stride, pad, dil, groups = 2, 8, 14, 11, 12, 3, 3, 2, 1, 1, 2
    kk = c // groups * kh * kw
    x = rng.uniform(-1, 1, (b, c, h, w)).astype(np.float32)
    pw = fastnn_amd.quantize_weights(wdt, (rng.standard_normal((oc, kk)) * 0.1).astype(np.float32))
    bias = (rng.standard_normal(oc) * 0.05).astype(np.float32)
    scale, zp = np.float32(0.009), np.float32(0.11)
    payload = orc.quantize_activations(x.reshape(-1), float(scale), float(zp)) if calibrated else orc.quantize_activations(x.reshape(-1))
    want = orc.qconv2d_i8payload(payload, x.shape, to_oracle(orc, pw), kh, kw, stride, pad, dil, groups, bias=bias, act=code)
    a = Arena()
    s_x, s_q, s_w, s_b, s_y = a.take(x.nbytes), a.take(8 + x.size), a.take(pw.words.nbytes), a.take(bias.nbytes), a.take(want.nbytes)
    plan = ExecutablePlan(a.top).write_const(s_w[0], pw.words).write_const(s_b[0], bias)
    qparams = [x.size, 0, 0]
    if calibrated:
        qparams += [int(scale.view(np.uint32)), int(zp.view(np.uint32))]
    plan.call_kernel("quantize_activations", [s_x], s_q, qparams)
    plan.call_kernel(kname + act, [s_q, s_w, s_b], s_y, [stride, pad, dil, groups, c, h, w, kh, kw],
                     meta_of(pw, [oc, c // groups, kh, kw]))
    be.allocate_arena(a.top)
    be.write_arena(s_x[0], x)
    be.dispatch(plan)
    assert np.array_equal(be.read_arena(*s_q), payload)
    tol = 1e-5 if not calibrated else 2e-5      # zero != 0: integer-sum form vs the reference's per-lane f32 sums
    assert_close(be.read_arena(*s_y, np.float32).reshape(want.shape), want, tol, kname + act)


def test_fill_memcopy_and_elementwise(be, orc):
    rng = np.random.default_rng(5)
    x = rng.standard_normal(1000).astype(np.float32)
    a = Arena()
    s_x, s_f, s_c, s_r, s_g, s_s, s_a = (a.take(4000) for _ in range(7))
    s_row = a.take(40)
    plan = ExecutablePlan(a.top).write_const(s_x[0], x).write_const(s_row[0], x[:10])
    plan.fill(s_f[0], s_f[1], -2.5).memcopy(s_c, s_x)
    plan.call_kernel("relu_f32", [s_x], s_r, [1000]).call_kernel("gelu_f32", [s_x], s_g, [1000])
    plan.call_kernel("silu_f32", [s_x], s_s, [1000]).call_kernel("add_f32", [s_x, s_row], s_a, [1000])
    be.allocate_arena(a.top)
    be.dispatch(plan)
    rd = lambda s: be.read_arena(*s, np.float32)
    assert np.all(rd(s_f) == np.float32(-2.5))
    assert np.array_equal(rd(s_c), x)
    assert np.array_equal(rd(s_r), np.maximum(x, 0))
    assert_close(rd(s_g), orc.act_fn(x, flib.ACT_GELU), 1e-6)
    assert_close(rd(s_s), orc.act_fn(x, flib.ACT_SILU), 1e-6)
    assert np.array_equal(rd(s_a), x + np.tile(x[:10], 100))      # second operand broadcast modulo its length


def test_unsupported_and_malformed_instructions(be):
    be.allocate_arena(4096)
    p = ExecutablePlan(4096).call_kernel("softmax_f32", [(0, 64)], (64, 64), [16])
    with pytest.raises(flib.FnnError) as e:
        be.dispatch(p)
    assert e.value.kind == "UnsupportedOp" and e.value.message == "softmax_f32"
    p = ExecutablePlan(4096).call_kernel("conv2d_i4_i8", [(0, 64), (64, 64)], (128, 64), [1] * 9)
    with pytest.raises(flib.FnnError) as e:
        be.dispatch(p)
    assert e.value.kind == "Dispatch" and "missing weight_meta" in e.value.message
    p = ExecutablePlan(4096).call_kernel("conv2d_u8_i8", [(0, 64), (64, 64)], (128, 64), [1] * 9)
    with pytest.raises(flib.FnnError) as e:      # no such name in the reference's dispatch either
        be.dispatch(p)
    assert e.value.kind == "UnsupportedOp" and e.value.message == "conv2d_u8_i8"
    p = ExecutablePlan(4096).call_kernel("conv2d_i4", [(0, 64), (64, 64)], (128, 64), [1] * 9)
    with pytest.raises(flib.FnnError) as e:
        be.dispatch(p)
    assert e.value.kind == "Dispatch" and "missing weight_meta" in e.value.message
    p = ExecutablePlan(4096).call_kernel("matmul_i8", [(0, 64), (64, 64)], (128, 64), [4, 4])
    with pytest.raises(flib.FnnError) as e:
        be.dispatch(p)
    assert e.value.kind == "Dispatch" and "expected params [M,K,N]" in e.value.message
    p = ExecutablePlan(4096).call_kernel("conv2d_i8", [(0, 64), (64, 64)], (128, 64), [1, 0, 1, 0, 1, 4, 4, 1, 1],
                                         dict(bit_width=8, scales=[1.0], zero_points=[0.0], shape=[1, 1]))
    with pytest.raises(flib.FnnError) as e:
        be.dispatch(p)
    assert "groups=0" in e.value.message
    p = ExecutablePlan(4096).call_kernel("conv2d_i8", [(0, 64), (64, 64)], (128, 64), [1, 0, 1, 1, 1, 4, 4, 1, 1])
    with pytest.raises(flib.FnnError) as e:
        be.dispatch(p)
    assert "missing weight_meta" in e.value.message
    p = ExecutablePlan(4096).call_kernel("matmul_i8", [(0, 64), (4090, 64)], (128, 64), [1, 16, 4])
    with pytest.raises(flib.FnnError) as e:
        be.dispatch(p)
    assert "outside the arena" in e.value.message
    p = ExecutablePlan(8192)
    with pytest.raises(flib.FnnError) as e:
        be.dispatch(p)
    assert e.value.kind == "Memory"
    # weight slice shorter than rows*kp words: packed_tensor_from_meta's length check
    p = ExecutablePlan(4096).call_kernel("matmul_i8", [(0, 64), (64, 16)], (128, 64), [1, 16, 4],
                                         dict(bit_width=8, scales=[1.0], zero_points=[0.0], shape=[4, 16]))
    with pytest.raises(flib.FnnError) as e:
        be.dispatch(p)
    assert e.value.kind == "Dispatch"


def test_rewritten_weights_are_re_registered(be, orc):
    """write_arena over a weight slice drops the cached device weight (the CPU cache would go stale)."""
    rng = np.random.default_rng(77)
    m, k, n = 2, 64, 16
    x = rng.standard_normal((m, k)).astype(np.float32)
    pw1 = fastnn_amd.quantize_weights(flib.DT_I8, _w(rng, n, k))
    pw2 = fastnn_amd.quantize_weights(flib.DT_I8, _w(rng, n, k))
    a = Arena()
    s_x, s_w, s_o = a.take(x.nbytes), a.take(pw1.words.nbytes), a.take(m * n * 4)
    be.allocate_arena(a.top)
    be.write_arena(s_x[0], x)
    for pw in (pw1, pw2):
        be.write_arena(s_w[0], pw.words)
        plan = ExecutablePlan(a.top).call_kernel("matmul_i8", [s_x, s_w], s_o, [m, k, n], meta_of(pw))
        be.dispatch(plan)
        assert_close(be.read_arena(*s_o, np.float32).reshape(m, n), orc.qmatmul(to_oracle(orc, pw), x), 2e-5)


def test_resident_plan_replays_as_graph(be, orc):
    """From the second dispatch on a plan whose constants are in place runs as one HIP-graph replay.
    Every replay is checked against the instruction-by-instruction path (dispatch_profile never replays)
    and the oracle, with host writes, reads and eager dispatches between the replays."""
    rng = np.random.default_rng(4242)
    m, d, f = 24, 256, 768
    up = fastnn_amd.quantize_weights(flib.DT_I4, _w(rng, f, d))
    down = fastnn_amd.quantize_weights(flib.DT_F8, _w(rng, d, f))
    b_up = (rng.standard_normal(f) * 0.1).astype(np.float32)
    a = Arena()
    s_x, s_up, s_bup, s_down = a.take(m * d * 4), a.take(up.words.nbytes), a.take(b_up.nbytes), a.take(down.words.nbytes)
    s_h, s_y, s_out, s_cp = a.take(m * f * 4), a.take(m * d * 4), a.take(m * d * 4), a.take(m * d * 4)
    plan = ExecutablePlan(a.top)
    plan.write_const(s_up[0], up.words).write_const(s_bup[0], b_up).write_const(s_down[0], down.words)
    plan.fill(s_y[0], s_y[1], 0.0)
    plan.call_kernel("matmul_i4_silu", [s_x, s_up, s_bup], s_h, [m, d, f], meta_of(up))
    plan.call_kernel("matmul_f8", [s_h, s_down], s_y, [m, f, d], meta_of(down))
    plan.call_kernel("add_f32", [s_y, s_x], s_out, [m * d])
    plan.memcopy(s_cp, s_out)
    be.allocate_arena(a.top)
    replays = 0
    for it in range(6):
        x = rng.standard_normal((m, d)).astype(np.float32)
        be.write_arena(s_x[0], x)                      # touches no constant: the plan stays resident
        be.dispatch(plan)
        replays += plan.replayed
        assert plan.replayed == (it >= 1), f"dispatch {it}"
        got = be.read_arena(*s_cp, np.float32).copy()
        h_ref = orc.qmatmul(to_oracle(orc, up), x, bias=b_up, act=flib.ACT_SILU)
        want = orc.qmatmul(to_oracle(orc, down), h_ref) + x
        assert_close(got.reshape(m, d), want, 1e-4, f"dispatch {it}")
        be.write_arena(s_cp[0], np.zeros(m * d, np.float32))
        be.dispatch_profile(plan)                      # same instructions, one by one
        assert not plan.replayed
        assert np.array_equal(be.read_arena(*s_cp, np.float32), got), f"replay {it} differs from the eager path"
    assert replays == 5
    # rewriting a constant from the host ends residency: the next dispatch uploads and runs eagerly,
    # and its result follows the plan's own payload again
    be.write_arena(s_bup[0], np.zeros_like(b_up))
    be.dispatch(plan)
    assert not plan.replayed
    assert_close(be.read_arena(*s_cp, np.float32).reshape(m, d), want, 1e-4, "after a constant was overwritten")
    be.dispatch(plan)
    assert plan.replayed
    assert_close(be.read_arena(*s_cp, np.float32).reshape(m, d), want, 1e-4, "replay after re-upload")


def test_plan_that_rewrites_its_constants_never_replays(be, orc):
    """A WriteConst target that another instruction overwrites is uploaded on every dispatch (eager path)."""
    rng = np.random.default_rng(5)
    m, k, n = 4, 64, 32
    x = rng.standard_normal((m, k)).astype(np.float32)
    pw = fastnn_amd.quantize_weights(flib.DT_I8, _w(rng, n, k))
    a = Arena()
    s_x, s_w, s_o = a.take(x.nbytes), a.take(pw.words.nbytes), a.take(m * n * 4)
    plan = ExecutablePlan(a.top).write_const(s_x[0], x).write_const(s_w[0], pw.words)
    plan.call_kernel("matmul_i8", [s_x, s_w], s_o, [m, k, n], meta_of(pw))
    plan.call_kernel("relu_f32", [s_x], s_x, [m * k])      # clobbers the constant input
    be.allocate_arena(a.top)
    want = orc.qmatmul(to_oracle(orc, pw), x)
    for _ in range(3):
        be.dispatch(plan)
        assert not plan.replayed
        assert_close(be.read_arena(*s_o, np.float32).reshape(m, n), want, 2e-5, "clobbered constant")


@pytest.mark.parametrize("wdt,kname", [(flib.DT_U8, "conv2d_u8"), (flib.DT_U4, "conv2d_u4"), (flib.DT_F8, "conv2d_f8"),
                                       (flib.DT_F8R, "conv2d_f8r"), (flib.DT_F4, "conv2d_f4"), (flib.DT_I4CB, "conv2d_i4")])
def test_conv2d_float_weight_plans(be, orc, wdt, kname):
    """conv2d_{u8,u4,f8,f8r,f4} and conv2d_i4 with a codebook: f32 convolution with dequantised weights."""
    rng = np.random.default_rng(43 + wdt)
    b, c, h, w, oc, kh, kw, stride, pad, dil, groups = 2, 32, 10, 9, 24, 1, 1, 1, 0, 1, 1
    kk = c // groups * kh * kw
    x = rng.standard_normal((b, c, h, w)).astype(np.float32)
    pw = fastnn_amd.quantize_weights(wdt, (rng.standard_normal((oc, kk)) * 0.2).astype(np.float32))
    bias = (rng.standard_normal(oc) * 0.05).astype(np.float32)
    want = orc.qconv2d_float(x, to_oracle(orc, pw), kh, kw, stride, pad, dil, groups, bias=bias, act=flib.ACT_SILU)
    a = Arena()
    s_x, s_w, s_b, s_y = a.take(x.nbytes), a.take(pw.words.nbytes), a.take(bias.nbytes), a.take(want.nbytes)
    plan = ExecutablePlan(a.top).write_const(s_w[0], pw.words).write_const(s_b[0], bias)
    plan.call_kernel(kname + "_silu", [s_x, s_w, s_b], s_y, [stride, pad, dil, groups, c, h, w, kh, kw],
                     meta_of(pw, [oc, c // groups, kh, kw]))
    be.allocate_arena(a.top)
    be.write_arena(s_x[0], x)
    be.dispatch(plan)
    assert_close(be.read_arena(*s_y, np.float32).reshape(want.shape), want, 2e-5, kname)
    be.write_arena(s_x[0], x * 0.5)                     # resident plan: graph replay of the three launches
    be.dispatch(plan)
    assert plan.replayed
    want2 = orc.qconv2d_float(x * 0.5, to_oracle(orc, pw), kh, kw, stride, pad, dil, groups, bias=bias, act=flib.ACT_SILU)
    assert_close(be.read_arena(*s_y, np.float32).reshape(want.shape), want2, 2e-5, kname + " replay")


def test_data_movement_kernels(be, orc):
    """concat / slice_f32 / pool_f32 (max) / upsample_nearest2d: bit-identical to the oracle (pure data movement)."""
    rng = np.random.default_rng(8)
    n, c, h, w = 2, 6, 8, 10
    x = rng.standard_normal((n, c, h, w)).astype(np.float32)
    x2 = rng.standard_normal((n, 3, h, w)).astype(np.float32)
    a = Arena()
    s_x, s_x2 = a.take(x.nbytes), a.take(x2.nbytes)
    s_cat = a.take((x.size + x2.size) * 4)
    s_lo, s_hi = a.take(n * 2 * h * w * 4), a.take(n * 4 * h * w * 4)
    s_pool = a.take(x.nbytes)
    s_pool2 = a.take(n * c * (h // 2) * (w // 2) * 4)
    s_up = a.take(x.size * 4 * 4)
    s_flat = a.take((x.size + x2.size) * 4)
    plan = ExecutablePlan(a.top).write_const(s_x[0], x).write_const(s_x2[0], x2)
    plan.call_kernel("concat", [s_x, s_x2], s_cat, [1, h * w, n])                 # channel axis: outer = N
    plan.call_kernel("slice_f32", [s_x], s_lo, [1, 0, 2, h * w])                  # channels [0,2)
    plan.call_kernel("slice_f32", [s_x], s_hi, [1, 2, 6, h * w])                  # channels [2,6)
    plan.call_kernel("pool_f32", [s_x], s_pool, [5, 1, 2, 1, n, c, h, w])         # the SPPF pooling
    plan.call_kernel("pool_f32", [s_x], s_pool2, [2, 2, 0, 1, n, c, h, w])
    plan.call_kernel("upsample_nearest2d", [s_x], s_up, [2, 2, h, w])
    plan.call_kernel("concat", [s_x, s_x2], s_flat, [])                           # legacy form: one after the other
    be.allocate_arena(a.top)
    for it in range(2):                                                           # second pass: graph replay
        be.dispatch(plan)
        assert plan.replayed == (it == 1)
        rd = lambda s: be.read_arena(*s, np.float32)
        assert np.array_equal(rd(s_cat), np.concatenate([x, x2], axis=1).reshape(-1))
        assert np.array_equal(rd(s_cat), orc.concat([x, x2], n, x.size + x2.size))
        assert np.array_equal(rd(s_lo), x[:, 0:2].reshape(-1))
        assert np.array_equal(rd(s_hi), orc.slice_f32(x, 2, 6, h * w, n * 4 * h * w))
        assert np.array_equal(rd(s_pool), orc.maxpool2d(x, 5, 1, 2).reshape(-1))
        assert np.array_equal(rd(s_pool2), orc.maxpool2d(x, 2, 2, 0).reshape(-1))
        assert np.array_equal(rd(s_up), orc.upsample_nearest2d(x, 2, 2).reshape(-1))
        assert np.array_equal(rd(s_flat), np.concatenate([x.reshape(-1), x2.reshape(-1)]))
    # in-place pooling (input slot reused as output): the input is staged first, as the CPU arm does
    p2 = ExecutablePlan(a.top).write_const(s_x[0], x).call_kernel("pool_f32", [s_x], s_x, [3, 1, 1, 1, n, c, h, w])
    be.dispatch(p2)
    assert np.array_equal(be.read_arena(*s_x, np.float32), orc.maxpool2d(x, 3, 1, 1).reshape(-1))
    # average pooling (is_max = 0): same summation order as the CPU kernel, so bit-identical too
    be.write_arena(s_x[0], x)
    for (k, s, p) in [(5, 1, 2), (2, 2, 0), (3, 2, 1)]:
        want = orc.avgpool2d(x, k, s, p)
        be.dispatch(ExecutablePlan(a.top).call_kernel("pool_f32", [s_x], (s_pool[0], want.nbytes), [k, s, p, 0, n, c, h, w]))
        assert np.array_equal(be.read_arena(s_pool[0], want.nbytes, np.float32), want.reshape(-1)), (k, s, p)
    with pytest.raises(flib.FnnError) as e:
        be.dispatch(ExecutablePlan(a.top).call_kernel("slice_f32", [s_x], s_lo, [1, 0, 2]))
    assert "expected params [dim, start, end, stride]" in e.value.message


def test_c2f_sppf_neck_fragment_as_one_plan(be, orc):
    """A YOLO-style fragment through the plan dispatcher: C2f (1x1 conv, channel split, two 3x3 convs with a
    residual add, concat, 1x1 conv), an SPPF pooling pyramid and an upsample + concat, I8 convolutions with
    bias + SiLU; compared with the same chain of oracle calls."""
    rng = np.random.default_rng(21)
    n, c, h, w = 1, 16, 12, 12
    hw = h * w
    x = rng.uniform(0, 1, (n, c, h, w)).astype(np.float32)
    def conv_w(oc, ic, k):
        kk = ic * k * k
        pw = fastnn_amd.quantize_weights(flib.DT_I8, (rng.standard_normal((oc, kk)) * np.sqrt(2.0 / kk)).astype(np.float32))
        return pw, (rng.standard_normal(oc) * 0.05).astype(np.float32)
    cv1, m1, m2, cv2 = conv_w(16, 16, 1), conv_w(8, 8, 3), conv_w(8, 8, 3), conv_w(16, 24, 1)
    a = Arena()
    f4 = lambda ch, hh=h, ww=w: a.take(n * ch * hh * ww * 4)
    s_x, s_y, s_a, s_b, s_t, s_u, s_r, s_cat, s_out = f4(16), f4(16), f4(8), f4(8), f4(8), f4(8), f4(8), f4(24), f4(16)
    s_p1, s_p2, s_p3, s_sp = f4(16), f4(16), f4(16), f4(64)
    s_up, s_neck = f4(64, 2 * h, 2 * w), f4(64 + 16, 2 * h, 2 * w)
    skip = rng.uniform(0, 1, (n, 16, 2 * h, 2 * w)).astype(np.float32)
    s_skip = f4(16, 2 * h, 2 * w)
    plan = ExecutablePlan(0)
    slots = {}
    for name, (pw, bias) in dict(cv1=cv1, m1=m1, m2=m2, cv2=cv2).items():
        slots[name] = (a.take(pw.words.nbytes), a.take(bias.nbytes))
    plan = ExecutablePlan(a.top).write_const(s_skip[0], skip)
    for name, (pw, bias) in dict(cv1=cv1, m1=m1, m2=m2, cv2=cv2).items():
        plan.write_const(slots[name][0][0], pw.words).write_const(slots[name][1][0], bias)
    def conv(name, pw, src, dst, ic, k):
        plan.call_kernel("conv2d_i8_silu", [src, slots[name][0], slots[name][1]], dst, [1, k // 2, 1, 1, ic, h, w, k, k],
                         meta_of(pw, [pw.rows, ic, k, k]))
    conv("cv1", cv1[0], s_x, s_y, 16, 1)
    plan.call_kernel("slice_f32", [s_y], s_a, [1, 0, 8, hw]).call_kernel("slice_f32", [s_y], s_b, [1, 8, 16, hw])
    conv("m1", m1[0], s_b, s_t, 8, 3)
    conv("m2", m2[0], s_t, s_u, 8, 3)
    plan.call_kernel("add_f32", [s_b, s_u], s_r, [n * 8 * hw])
    plan.call_kernel("concat", [s_a, s_b, s_r], s_cat, [1, hw, n])
    conv("cv2", cv2[0], s_cat, s_out, 24, 1)
    plan.call_kernel("pool_f32", [s_out], s_p1, [5, 1, 2, 1, n, 16, h, w])
    plan.call_kernel("pool_f32", [s_p1], s_p2, [5, 1, 2, 1, n, 16, h, w])
    plan.call_kernel("pool_f32", [s_p2], s_p3, [5, 1, 2, 1, n, 16, h, w])
    plan.call_kernel("concat", [s_out, s_p1, s_p2, s_p3], s_sp, [1, hw, n])
    plan.call_kernel("upsample_nearest2d", [s_sp], s_up, [2, 2, h, w])
    plan.call_kernel("concat", [s_up, s_skip], s_neck, [1, 4 * hw, n])
    be.allocate_arena(a.top)

    def reference(xin):
        q = lambda pwb, t, k: orc.qconv2d_i8(t, to_oracle(orc, pwb[0]), k, k, 1, k // 2, 1, 1, bias=pwb[1], act=flib.ACT_SILU)
        y = q(cv1, xin, 1)
        ya, yb = y[:, :8], y[:, 8:]
        r = yb + q(m2, q(m1, yb, 3), 3)
        out = q(cv2, np.concatenate([ya, yb, r], axis=1), 1)
        p1 = orc.maxpool2d(out, 5, 1, 2); p2 = orc.maxpool2d(p1, 5, 1, 2); p3 = orc.maxpool2d(p2, 5, 1, 2)
        sp = np.concatenate([out, p1, p2, p3], axis=1)
        return np.concatenate([orc.upsample_nearest2d(sp, 2, 2), skip], axis=1)

    for it in range(3):
        xin = x if it == 0 else rng.uniform(0, 1, x.shape).astype(np.float32)
        be.write_arena(s_x[0], xin)
        be.dispatch(plan)
        assert plan.replayed == (it >= 1)
        got = be.read_arena(*s_neck, np.float32).reshape(n, 80, 2 * h, 2 * w)
        # each conv re-quantises its input from the previous result: differences of one rounding step can
        # propagate, so the chain is compared at 2e-3 of the output range (single convs: 1e-5)
        assert_close(got, reference(xin), 2e-3, f"fragment, dispatch {it}")


def test_backend_kernel_flags_single_f16_activations(be, orc):
    """FNN_FLAG_ACT_F16_SINGLE per backend: the MLP block at 64 tokens agrees to 1e-3 (default: 2e-5), a plan
    captured under the old flags is captured again, and unknown bits are refused."""
    rng = np.random.default_rng(64)
    m, d, f = 64, 256, 1024
    x = rng.standard_normal((m, d)).astype(np.float32)
    up = fastnn_amd.quantize_weights(flib.DT_I4, _w(rng, f, d))
    down = fastnn_amd.quantize_weights(flib.DT_I8, _w(rng, d, f))
    a = Arena()
    s_x, s_up, s_down, s_h, s_y = a.take(x.nbytes), a.take(up.words.nbytes), a.take(down.words.nbytes), a.take(m * f * 4), a.take(m * d * 4)
    plan = ExecutablePlan(a.top).write_const(s_up[0], up.words).write_const(s_down[0], down.words)
    plan.call_kernel("matmul_i4_relu", [s_x, s_up], s_h, [m, d, f], meta_of(up))
    plan.call_kernel("matmul_i8", [s_h, s_down], s_y, [m, f, d], meta_of(down))
    be.allocate_arena(a.top)
    be.write_arena(s_x[0], x)
    h_ref = orc.qmatmul(to_oracle(orc, up), x, act=flib.ACT_RELU)
    want = orc.qmatmul(to_oracle(orc, down), h_ref)
    try:
        be.dispatch(plan); be.dispatch(plan)
        assert plan.replayed
        precise = be.read_arena(*s_y, np.float32).reshape(m, d).copy()
        assert_close(precise, want, 1e-4, "default flags")
        be.set_kernel_flags(flib.FLAG_ACT_F16_SINGLE)
        be.dispatch(plan)                             # the old capture is stale: captured again (or run eagerly)
        fast = be.read_arena(*s_y, np.float32).reshape(m, d).copy()
        assert_close(fast, want, 1e-3, "single f16 activations")
        assert not np.array_equal(fast, precise)      # it really is the other kernel variant
        be.dispatch(plan)
        assert plan.replayed
        assert np.array_equal(be.read_arena(*s_y, np.float32).reshape(m, d), fast)
        with pytest.raises(flib.FnnError):
            be.set_kernel_flags(flib.FLAG_DEVICE_PTRS)
    finally:
        be.set_kernel_flags(0)


def test_two_plans_sharing_an_arena_do_not_trust_stale_constants(be, orc):
    """Plan A and plan B lay their constants over the same bytes of one backend's arena.  Each dispatch of one
    overwrites the other's constants (uploads, kernel outputs): the other plan must notice, upload again and
    run eagerly, and both must keep agreeing with the oracle however they alternate.  Two plans whose byte
    ranges are disjoint keep their residency (and their graph replays) across each other's dispatches."""
    rng = np.random.default_rng(77)
    m, k, n = 4, 256, 128
    xa, xb = rng.standard_normal((m, k)).astype(np.float32), rng.standard_normal((m, k)).astype(np.float32)
    wa = fastnn_amd.quantize_weights(flib.DT_I8, _w(rng, n, k))
    wb = fastnn_amd.quantize_weights(flib.DT_I4, _w(rng, n, k))
    ba = (rng.standard_normal(n) * 0.1).astype(np.float32)
    a = Arena()
    s_x, s_w, s_b, s_o = a.take(xa.nbytes), a.take(wa.words.nbytes), a.take(ba.nbytes), a.take(m * n * 4)
    # A: weight at s_w, bias at s_b, output at s_o.  B: its (shorter) weight at the same offset, and its output lands
    # on A's bias.
    pa = ExecutablePlan(a.top).write_const(s_x[0], xa).write_const(s_w[0], wa.words).write_const(s_b[0], ba)
    pa.call_kernel("matmul_i8_relu", [s_x, s_w, s_b], s_o, [m, k, n], meta_of(wa))
    s_wb = (s_w[0], wb.words.nbytes)
    pb = ExecutablePlan(a.top).write_const(s_x[0], xb).write_const(s_wb[0], wb.words)
    pb.call_kernel("matmul_i4", [s_x, s_wb], (s_b[0], m * n * 4), [m, k, n], meta_of(wb))
    want_a = orc.qmatmul(to_oracle(orc, wa), xa, bias=ba, act=flib.ACT_RELU)
    want_b = orc.qmatmul(to_oracle(orc, wb), xb)
    be.allocate_arena(a.top + m * n * 4)
    for which in "aabbabbaab":
        if which == "a":
            be.dispatch(pa)
            assert_close(be.read_arena(*s_o, np.float32).reshape(m, n), want_a, 2e-5, "plan A after " + which)
        else:
            be.dispatch(pb)
            assert_close(be.read_arena(s_b[0], m * n * 4, np.float32).reshape(m, n), want_b, 2e-5, "plan B")
    # a replay only ever follows a dispatch of the same plan
    be.dispatch(pa); be.dispatch(pa)
    assert pa.replayed
    be.dispatch(pb)
    assert not pb.replayed
    be.dispatch(pa)
    assert not pa.replayed
    assert_close(be.read_arena(*s_o, np.float32).reshape(m, n), want_a, 2e-5, "plan A at the end")
    # disjoint plans: residency and replays survive the other plan's dispatches
    a2 = Arena()
    t_x, t_w, t_o = a2.take(xa.nbytes), a2.take(wa.words.nbytes), a2.take(m * n * 4)
    u_x, u_w, u_o = a2.take(xb.nbytes), a2.take(wb.words.nbytes), a2.take(m * n * 4)
    pc = ExecutablePlan(a2.top).write_const(t_x[0], xa).write_const(t_w[0], wa.words)
    pc.call_kernel("matmul_i8", [t_x, t_w], t_o, [m, k, n], meta_of(wa))
    pd = ExecutablePlan(a2.top).write_const(u_x[0], xb).write_const(u_w[0], wb.words)
    pd.call_kernel("matmul_i4", [u_x, u_w], u_o, [m, k, n], meta_of(wb))
    be.allocate_arena(a2.top)
    want_c = orc.qmatmul(to_oracle(orc, wa), xa)
    for it in range(4):
        be.dispatch(pc); be.dispatch(pd)
        assert pc.replayed == (it >= 1) and pd.replayed == (it >= 1), it
        assert_close(be.read_arena(*t_o, np.float32).reshape(m, n), want_c, 2e-5, "disjoint plan C")
        assert_close(be.read_arena(*u_o, np.float32).reshape(m, n), want_b, 2e-5, "disjoint plan D")


def test_many_forwards_keep_the_plan_resident(be, orc):
    """The write log holds one entry per distinct byte range: a thousand write-input / dispatch cycles neither
    overflow it nor end the plan's residency (every dispatch after the first is a graph replay)."""
    rng = np.random.default_rng(78)
    m, k, n = 2, 128, 64
    pw = fastnn_amd.quantize_weights(flib.DT_I8, _w(rng, n, k))
    a = Arena()
    s_x, s_w, s_o = a.take(m * k * 4), a.take(pw.words.nbytes), a.take(m * n * 4)
    plan = ExecutablePlan(a.top).write_const(s_w[0], pw.words).call_kernel("matmul_i8", [s_x, s_w], s_o, [m, k, n], meta_of(pw))
    be.allocate_arena(a.top)
    x = rng.standard_normal((m, k)).astype(np.float32)
    replays = 0
    for it in range(1000):
        be.write_arena(s_x[0], x)
        be.dispatch(plan)
        replays += plan.replayed
    assert replays == 999
    assert_close(be.read_arena(*s_o, np.float32).reshape(m, n), orc.qmatmul(to_oracle(orc, pw), x), 2e-5, "after 1000 forwards")


def test_maxpool_secondary_output_holds_the_window_positions(be, orc):
    """CallKernel.secondary_output_slice of "pool_f32" (is_max = 1): i64 kh*kernel + kw of each maximum, bit-identical to
    the oracle, eager and replayed; an index slice shorter than the output takes the leading entries only."""
    rng = np.random.default_rng(79)
    n, c, h, w = 2, 5, 9, 7
    x = rng.permutation(n * c * h * w).astype(np.float32).reshape(n, c, h, w)
    x[0, 0, :3, :3] = 1000.0                                   # ties: the first tap in (kh, kw) order stays
    for (k, s, p) in [(5, 1, 2), (2, 2, 0), (3, 2, 1)]:
        want_v, want_i = orc.maxpool2d(x, k, s, p, return_indices=True)
        a = Arena()
        s_x, s_v, s_i = a.take(x.nbytes), a.take(want_v.nbytes), a.take(want_i.nbytes)
        s_short = a.take(8 * 10)
        plan = ExecutablePlan(a.top).write_const(s_x[0], x)
        plan.call_kernel("pool_f32", [s_x], s_v, [k, s, p, 1, n, c, h, w], secondary_output=s_i)
        plan.call_kernel("pool_f32", [s_x], s_v, [k, s, p, 1, n, c, h, w], secondary_output=s_short)
        be.allocate_arena(a.top)
        for it in range(2):
            be.dispatch(plan)
            assert plan.replayed == (it == 1)
            assert np.array_equal(be.read_arena(*s_v, np.float32), want_v.reshape(-1)), (k, s, p)
            assert np.array_equal(be.read_arena(*s_i, np.int64), want_i.reshape(-1)), (k, s, p)
            assert np.array_equal(be.read_arena(*s_short, np.int64), want_i.reshape(-1)[:10]), (k, s, p)
    with pytest.raises(flib.FnnError):
        be.dispatch(ExecutablePlan(a.top).call_kernel("pool_f32", [s_x], s_v, [k, s, p, 1, n, c, h, w], secondary_output=(s_i[0] + 4, 64)))


def test_meta_with_several_codebooks_reads_the_first(be, orc):
    """QuantizedWeightMeta.codebooks is a vector; every decode of the reference reads entry 0."""
    rng = np.random.default_rng(80)
    m, k, n = 3, 128, 48
    x = rng.standard_normal((m, k)).astype(np.float32)
    pw = fastnn_amd.quantize_weights(flib.DT_I4CB, _w(rng, n, k))
    meta = meta_of(pw)
    meta["codebooks"] = np.concatenate([meta["codebooks"], rng.standard_normal((3, 16)).astype(np.float32)])
    a = Arena()
    s_x, s_w, s_o = a.take(x.nbytes), a.take(pw.words.nbytes), a.take(m * n * 4)
    plan = ExecutablePlan(a.top).write_const(s_x[0], x).write_const(s_w[0], pw.words)
    plan.call_kernel("matmul_i4", [s_x, s_w], s_o, [m, k, n], meta)
    be.allocate_arena(a.top)
    be.dispatch(plan)
    assert_close(be.read_arena(*s_o, np.float32).reshape(m, n), orc.qmatmul(to_oracle(orc, pw), x), 2e-5, "codebooks[0]")


def test_graph_replay_switch_and_context_options(be, orc):
    """fnn_backend_set_graph_replay(0) keeps every dispatch instruction by instruction; per-context options select
    kernel variants without changing results beyond the stated tolerance, and refuse values out of range."""
    rng = np.random.default_rng(81)
    m, k, n = 64, 512, 256
    x = rng.standard_normal((m, k)).astype(np.float32)
    pw = fastnn_amd.quantize_weights(flib.DT_I4, _w(rng, n, k))
    a = Arena()
    s_x, s_w, s_o = a.take(x.nbytes), a.take(pw.words.nbytes), a.take(m * n * 4)
    plan = ExecutablePlan(a.top).write_const(s_x[0], x).write_const(s_w[0], pw.words)
    plan.call_kernel("matmul_i4", [s_x, s_w], s_o, [m, k, n], meta_of(pw))
    want = orc.qmatmul(to_oracle(orc, pw), x)
    be.allocate_arena(a.top)
    try:
        be.set_graph_replay(False)
        for _ in range(3):
            be.dispatch(plan)
            assert not plan.replayed
        be.set_graph_replay(True)
        be.dispatch(plan)
        assert plan.replayed
        for opt, val in [(flib.OPT_TILE_SHAPE, 0), (flib.OPT_TILE_SHAPE, 2), (flib.OPT_TILE_SPLIT, 2), (flib.OPT_TILE_SPLIT, 0)]:
            be.set_option(opt, val)
            be.dispatch(plan)                              # the graph is captured again with the new choice
            assert_close(be.read_arena(*s_o, np.float32).reshape(m, n), want, 2e-5, f"option {opt}={val}")
        with pytest.raises(flib.FnnError):
            be.set_option(flib.OPT_TILE_SHAPE, 7)
        with pytest.raises(flib.FnnError):
            be.set_option(99, 0)
    finally:
        be.set_graph_replay(True)
        be.set_option(flib.OPT_TILE_SHAPE, -1)
        be.set_option(flib.OPT_TILE_SPLIT, 0)


def test_loaded_plan_dispatches_with_a_shape_environment(be, orc):
    """The hand-assembled saved plan (tests/golden/executable_plan.bin) runs on the device: constants from its
    WriteConst payloads, [M, K, N] of both MatMuls resolved from param_dims under ShapeEnv {B: 2} (a Symbol and a
    Bounded dim), results against the oracle on the fixture's own words and metadata."""
    import os
    import struct
    from fastnn_amd.backend import ExecutablePlan as EP
    here = os.path.dirname(os.path.abspath(__file__))
    plan = EP.load(os.path.join(here, "golden", "executable_plan.bin"))
    rows = [[1, -1, 2, -2, 3, -3, 4, -4], [5, 6, 7, 8, -5, -6, -7, -8], [127, -128, 0, 1, -1, 64, -64, 10], [0, 0, 0, 9, 0, 0, -9, 0]]
    words = np.frombuffer(b"".join(struct.pack("<8b", *r) for r in rows), np.uint32)
    w8 = orc.Packed(flib.DT_I8, 4, 8, np.concatenate([words, np.zeros(16, np.uint32)]), np.float32([0.5, 0.25, 1.0, 2.0]),
                    np.float32([0.0, 0.5, -1.0, 0.0]))
    idx = [[(3 * k + r) % 16 for k in range(32)] for r in range(2)]
    cbw = np.array([sum(n << (4 * i) for i, n in enumerate(row[w * 8:(w + 1) * 8])) for row in idx for w in range(4)], np.uint32)
    wcb = orc.Packed(flib.DT_I4CB, 2, 32, np.concatenate([cbw, np.zeros(16, np.uint32)]), np.float32([0.75, 1.5]), np.zeros(0, np.float32), 32,
                     np.float32([-1.0 + 2.0 * i / 15.0 for i in range(16)]))
    rng = np.random.default_rng(91)
    x1 = rng.standard_normal((2, 8)).astype(np.float32)
    x2 = rng.standard_normal((2, 32)).astype(np.float32)
    be.allocate_arena(plan.arena_size)
    for it in range(3):
        be.write_arena(0, x1)
        be.write_arena(576, x2)
        be.dispatch(plan, {"B": 2})
        assert plan.replayed == (it >= 1)
        y1 = orc.qmatmul(w8, x1, bias=np.float32([0.5, -0.25, 1.0, 0.0]), act=flib.ACT_RELU)
        assert_close(be.read_arena(256, 32, np.float32).reshape(2, 4), y1, 2e-5, "matmul_i8_relu of the loaded plan")
        assert np.array_equal(be.read_arena(320, 32, np.float32), be.read_arena(256, 32, np.float32))          # MemCopy
        pv, pi = orc.maxpool2d(be.read_arena(320, 32, np.float32).reshape(1, 2, 2, 2), 2, 2, 0, return_indices=True)
        assert np.array_equal(be.read_arena(384, 8, np.float32), pv.reshape(-1))
        assert np.array_equal(be.read_arena(392, 16, np.int64), pi.reshape(-1))
        assert_close(be.read_arena(1152, 16, np.float32).reshape(2, 2), orc.qmatmul(wcb, x2), 2e-5, "codebook matmul of the loaded plan")
    # another binding of the same plan: one row; the graph recorded under B = 2 is not replayed
    be.dispatch(plan, {"B": 1})
    assert_close(be.read_arena(1152, 8, np.float32).reshape(1, 2), orc.qmatmul(wcb, x2[:1]), 2e-5, "B = 1")
    with pytest.raises(flib.FnnError) as e:
        be.dispatch(plan)                              # empty environment
    assert e.value.kind == "Dispatch" and "DimExpr::Symbol 'B' is not bound in the ShapeEnv" in e.value.message
    plan.close()


def test_bounded_dims_fall_back_to_their_maximum_and_refuse_larger_bindings(be, orc):
    rng = np.random.default_rng(92)
    k, n = 64, 24
    pw = fastnn_amd.quantize_weights(flib.DT_F8, _w(rng, n, k))
    x = rng.standard_normal((4, k)).astype(np.float32)
    a = Arena()
    s_x, s_w, s_o = a.take(x.nbytes), a.take(pw.words.nbytes), a.take(4 * n * 4)
    plan = ExecutablePlan(a.top).write_const(s_x[0], x).write_const(s_w[0], pw.words)
    plan.call_kernel("matmul_f8", [s_x, s_w], s_o, [1, k, n], meta_of(pw))       # stored params say M = 1
    plan.set_param_dims(2, [("T", 4), k, n])
    be.allocate_arena(a.top)
    want = orc.qmatmul(to_oracle(orc, pw), x)
    be.dispatch(plan)                                  # unbound Bounded dim: its max, 4 rows
    assert_close(be.read_arena(*s_o, np.float32).reshape(4, n), want, 2e-5, "Bounded -> max")
    be.write_arena(s_o[0], np.zeros(4 * n, np.float32))
    be.dispatch(plan, {"T": 3})
    got = be.read_arena(*s_o, np.float32).reshape(4, n)
    assert_close(got[:3], want[:3], 2e-5, "T = 3")
    assert not got[3].any()
    with pytest.raises(flib.FnnError) as e:
        be.dispatch(plan, {"T": 5})
    assert "DimExpr::Bounded: symbol 'T' resolved to 5, exceeds bound 4" in e.value.message
    plan.set_param_dims(2, [1, k])
    with pytest.raises(flib.FnnError) as e:
        be.dispatch(plan)
    assert "param_dims has 2 elements but expected 3" in e.value.message


def test_segmented_dispatch_hands_unsupported_kernels_to_the_caller(be, orc):
    """A plan with a kernel this library does not implement ("sigmoid_f32") between two quantised MatMuls: the dispatch
    stops at it with the kernel's index, the caller computes it on the host through read_arena / write_arena and
    resumes behind it, as a Rust HipBackend does with CpuBackend.  The constants stay resident between passes."""
    rng = np.random.default_rng(93)
    m, d, f = 4, 64, 96
    w1 = fastnn_amd.quantize_weights(flib.DT_I8, _w(rng, f, d))
    w2 = fastnn_amd.quantize_weights(flib.DT_I4, _w(rng, d, f))
    a = Arena()
    s_x, s_w1, s_w2, s_h, s_g, s_y = a.take(m * d * 4), a.take(w1.words.nbytes), a.take(w2.words.nbytes), a.take(m * f * 4), a.take(m * f * 4), a.take(m * d * 4)
    plan = ExecutablePlan(a.top).write_const(s_w1[0], w1.words).write_const(s_w2[0], w2.words)
    plan.call_kernel("matmul_i8", [s_x, s_w1], s_h, [m, d, f], meta_of(w1))
    plan.call_kernel("sigmoid_f32", [s_h], s_g, [m * f])
    plan.call_kernel("matmul_i4", [s_g, s_w2], s_y, [m, f, d], meta_of(w2))
    be.allocate_arena(a.top)
    with pytest.raises(flib.FnnError) as e:
        be.dispatch(plan)
    assert e.value.kind == "UnsupportedOp" and e.value.message == "sigmoid_f32"
    for it in range(3):
        x = rng.standard_normal((m, d)).astype(np.float32)
        be.write_arena(s_x[0], x)
        first, stops = 0, []
        while True:
            stop = be.dispatch_from(plan, first)
            if stop is None:
                break
            stops.append(stop)
            assert plan.describe(stop)["kernel"] == "sigmoid_f32"
            h = be.read_arena(*s_h, np.float32)
            be.write_arena(s_g[0], (1.0 / (1.0 + np.exp(-h.astype(np.float64)))).astype(np.float32))
            first = stop + 1
        assert stops == [3] and not plan.replayed
        h_ref = orc.qmatmul(to_oracle(orc, w1), x)
        g_ref = (1.0 / (1.0 + np.exp(-h_ref.astype(np.float64)))).astype(np.float32)
        assert_close(be.read_arena(*s_y, np.float32).reshape(m, d), orc.qmatmul(to_oracle(orc, w2), g_ref), 1e-4, f"pass {it}")


@pytest.mark.parametrize("batch", [1, 3])
def test_memcopy_and_fill_feeding_a_convolution(be, orc, batch):
    """A MemCopy whose destination a quantised Conv2d reads runs as a copy kernel that leaves the activation ranges
    (the convolution then does not scan); a Fill into the same slice afterwards must drop them again.  Both against
    the oracle, and the plan's statistics say which path ran."""
    rng = np.random.default_rng(61)
    c, h, w, oc, k = 6, 17, 16, 10, 3
    x = rng.uniform(-1, 1, (batch, c, h, w)).astype(np.float32)
    pw = fastnn_amd.quantize_weights(flib.DT_I8, (rng.standard_normal((oc, c * k * k)) * 0.1).astype(np.float32))
    bias = (rng.standard_normal(oc) * 0.05).astype(np.float32)
    a = Arena()
    s_in, s_x, s_w, s_b = a.take(x.nbytes), a.take(x.nbytes), a.take(pw.words.nbytes), a.take(bias.nbytes)
    s_y = a.take(batch * oc * h * w * 4)
    params, meta = [1, 1, 1, 1, c, h, w, k, k], meta_of(pw, [oc, c, k, k])
    be.allocate_arena(a.top)
    # copy, then convolution
    plan = ExecutablePlan(a.top).write_const(s_w[0], pw.words).write_const(s_b[0], bias)
    plan.memcopy(s_x, s_in).call_kernel("conv2d_i8_silu", [s_x, s_w, s_b], s_y, params, meta)
    be.write_arena(s_in[0], x)
    be.dispatch(plan)
    want = orc.qconv2d_i8(x, to_oracle(orc, pw), k, k, 1, 1, 1, 1, bias=bias, act=flib.ACT_SILU)
    assert_close(be.read_arena(*s_y, np.float32).reshape(want.shape), want, 1e-5, "copy -> conv")
    assert plan.ranges_used == 1
    be.dispatch(plan)   # (graph replay)
    assert_close(be.read_arena(*s_y, np.float32).reshape(want.shape), want, 1e-5, "copy -> conv, replayed")
    # copy, fill of the same slice, convolution: the copy's ranges no longer describe the slice
    plan2 = ExecutablePlan(a.top).write_const(s_w[0], pw.words).write_const(s_b[0], bias)
    plan2.memcopy(s_x, s_in).fill(s_x[0], s_x[1], 0.25).call_kernel("conv2d_i8_silu", [s_x, s_w, s_b], s_y, params, meta)
    be.dispatch(plan2)
    want2 = orc.qconv2d_i8(np.full_like(x, 0.25), to_oracle(orc, pw), k, k, 1, 1, 1, 1, bias=bias, act=flib.ACT_SILU)
    assert_close(be.read_arena(*s_y, np.float32).reshape(want2.shape), want2, 1e-5, "copy -> fill -> conv")
    assert plan2.ranges_used == 0


@pytest.mark.parametrize("wdt,kname", [(flib.DT_F8, "matmul_f8"), (flib.DT_I4, "matmul_i4_relu"), (flib.DT_I4CB, "matmul_i4")])
def test_matmul_followed_by_residual_add_runs_as_one_call(be, orc, wdt, kname):
    """A MatMul whose output the next instruction adds to another tensor stores the sum from its own last kernel
    (FNN_OPT_FUSE_RESIDUAL, the Add is skipped): every arrangement of the Add's operands gives, bit for bit, what
    the two instructions give on their own, the MatMul's own output is still written, and the arrangements that
    cannot ride along (the sum overwriting the MatMul's output, a convolution reading the sum) still run the Add."""
    rng = np.random.default_rng(97 + wdt)
    m, k, n = 64, 1024, 384
    x = rng.standard_normal((m, k)).astype(np.float32)
    r = rng.standard_normal((m, n)).astype(np.float32)
    pw = fastnn_amd.quantize_weights(wdt, _w(rng, n, k))
    cw = fastnn_amd.quantize_weights(flib.DT_I8, _w(rng, 8, 6))
    act = flib.ACT_RELU if kname.endswith("relu") else 0
    want_y = orc.qmatmul(to_oracle(orc, pw), x, act=act)
    a = Arena()
    s_x, s_r, s_w, s_cw = a.take(x.nbytes), a.take(r.nbytes), a.take(pw.words.nbytes), a.take(cw.words.nbytes)
    s_y = [a.take(m * n * 4) for _ in range(5)]
    s_sum = [a.take(m * n * 4) for _ in range(5)]
    s_r2, s_conv = a.take(r.nbytes), a.take(m * 8 * 8 * 8 * 4)
    plan = ExecutablePlan(a.top).write_const(s_w[0], pw.words).write_const(s_cw[0], cw.words)
    mm = lambda dst: plan.call_kernel(kname, [s_x, s_w], dst, [m, k, n], meta_of(pw))
    mm(s_y[0]); plan.call_kernel("add_f32", [s_y[0], s_r], s_sum[0], [m * n])        # MatMul output first
    mm(s_y[1]); plan.call_kernel("add_f32", [s_r, s_y[1]], s_sum[1], [m * n])        # ... second
    plan.memcopy(s_r2, s_r)
    mm(s_y[2]); plan.call_kernel("add_f32", [s_y[2], s_r2], s_r2, [m * n])           # the sum replaces the other operand
    mm(s_y[3]); plan.call_kernel("add_f32", [s_y[3], s_r], s_y[3], [m * n])          # ... replaces the MatMul output: not fused
    mm(s_y[4]); plan.call_kernel("add_f32", [s_y[4], s_r], s_sum[4], [m * n])        # a convolution reads the sum: not fused
    plan.call_kernel("conv2d_i8", [s_sum[4], s_cw], s_conv, [1, 0, 1, 1, 6, 8, 8, 1, 1], meta_of(cw, shape=[8, 6, 1, 1]))
    be.allocate_arena(a.top)
    be.write_arena(s_x[0], x)
    be.write_arena(s_r[0], r)
    got = {}
    try:
        for fuse in (1, 0):
            be.set_option(flib.OPT_FUSE_RESIDUAL, fuse)
            be.dispatch(plan)
            first = be.read_arena(0, a.top).copy()
            be.dispatch(plan)
            assert plan.replayed
            got[fuse] = be.read_arena(0, a.top).copy()
            assert np.array_equal(first, got[fuse]), "replay differs from the first dispatch"
            assert plan.residuals_fused == (3 if fuse else 0)
    finally:
        be.set_option(flib.OPT_FUSE_RESIDUAL, 1)
    assert np.array_equal(got[1], got[0])
    view = lambda s: got[1][s[0]:s[0] + s[1]].view(np.float32).reshape(m, n)
    for i in (0, 1, 2, 4):
        assert_close(view(s_y[i]), want_y, 2e-5, f"MatMul output {i}")
    for s in (s_sum[0], s_sum[1], s_r2, s_y[3], s_sum[4]):
        assert np.array_equal(view(s), view(s_y[0]) + r)


@pytest.mark.parametrize("case", ["parts", "memcopy part", "part without pairs", "part rewritten", "overwritten after", "gap"])
def test_conv_ranges_collected_part_by_part(be, orc, case):
    """A one-image tensor that several instructions write part by part (the slot of a Concat result filled in place):
    each producer leaves its pairs behind those of the parts before it, and the convolution that reads the whole
    tensor takes them once disjoint parts cover it -- not when a part comes from an instruction that leaves no
    pairs, is overwritten afterwards, or is missing; a part that is written again before anything reads it counts with
    its last writer (the first one's values are never read, so it is asked for nothing).  A convolution that reads just
    one part takes that part's pairs.  Either way the arena equals, bit for bit, the one with every convolution scanning."""
    rng = np.random.default_rng(31)
    c, h, w = 16, 32, 32
    half = (c // 2) * h * w
    a0 = rng.standard_normal(half).astype(np.float32)
    a1 = (rng.standard_normal(half) * 3).astype(np.float32)
    pw = fastnn_amd.quantize_weights(flib.DT_I8, (rng.standard_normal((8, c)) * 0.3).astype(np.float32))
    ph = fastnn_amd.quantize_weights(flib.DT_I8, (rng.standard_normal((8, c // 2)) * 0.3).astype(np.float32))
    a = Arena()
    s_a0, s_a1, s_w, s_wh = a.take(half * 4), a.take(half * 4), a.take(pw.words.nbytes), a.take(ph.words.nbytes)
    s_t = a.take(2 * half * 4)
    s_p0, s_p1 = (s_t[0], half * 4), (s_t[0] + half * 4, half * 4)
    s_y, s_yh = a.take(8 * h * w * 4), a.take(8 * h * w * 4)
    plan = ExecutablePlan(a.top).write_const(s_w[0], pw.words).write_const(s_wh[0], ph.words)
    plan.call_kernel("relu_f32", [s_a0], s_p0, [half])
    if case == "memcopy part":
        plan.memcopy(s_p1, s_a1)
    elif case == "part without pairs":
        plan.fill(s_p1[0], s_p1[1], 0.25)
    elif case != "gap":
        plan.call_kernel("silu_f32", [s_a1], s_p1, [half])
    if case == "part rewritten":
        plan.call_kernel("gelu_f32", [s_a1], s_p0, [half])
    if case == "overwritten after":
        plan.fill(s_p0[0] + 64, 64, 9.0)
    plan.call_kernel("conv2d_i8", [s_p0, s_wh], s_yh, [1, 0, 1, 1, c // 2, h, w, 1, 1], meta_of(ph, [8, c // 2, 1, 1]))   # reads one part
    plan.call_kernel("conv2d_i8", [s_t, s_w], s_y, [1, 0, 1, 1, c, h, w, 1, 1], meta_of(pw, [8, c, 1, 1]))               # reads the whole
    be.allocate_arena(a.top)
    got, used = {}, {}
    try:
        for on in (1, 0):
            be.set_option(flib.OPT_CONV_RANGES, on)
            be.write_arena(0, np.zeros(a.top, np.uint8))
            be.write_arena(s_a0[0], a0)
            be.write_arena(s_a1[0], a1)
            be.dispatch(plan)
            first = be.read_arena(0, a.top).copy()
            be.dispatch(plan)
            assert plan.replayed
            got[on], used[on] = be.read_arena(0, a.top).copy(), plan.ranges_used
            assert np.array_equal(first, got[on]), "replay differs from the first dispatch"
    finally:
        be.set_option(flib.OPT_CONV_RANGES, 1)
    assert np.array_equal(got[1], got[0])
    # the reader of the part: its pairs hold unless the Fill wrote into the part; the reader of the whole: only with
    # both parts from producers that leave pairs and nothing written after them
    want = {"parts": 2, "memcopy part": 2, "part without pairs": 1, "part rewritten": 2, "overwritten after": 0, "gap": 1}[case]
    assert used[0] == 0 and used[1] == want, (case, used)
    t = got[1][s_t[0]:s_t[0] + s_t[1]].view(np.float32).reshape(1, c, h, w)
    y = got[1][s_y[0]:s_y[0] + s_y[1]].view(np.float32).reshape(1, 8, h, w)
    assert_close(y, orc.qconv2d_i8(t, to_oracle(orc, pw), 1, 1, 1, 0, 1, 1), 1e-5, case)


@pytest.mark.parametrize("implicit", [0, 1, 2, 3])
@pytest.mark.parametrize("oc,side", [(64, 40), (128, 20), (256, 20), (32, 48)])
def test_conv_ranges_of_a_channel_half(be, orc, implicit, oc, side):
    """The two halves of a one-image convolution output read in place by two convolutions (a Split that is a view):
    the producer groups its range pairs by channel block, so a reader of whole blocks takes just their pairs instead of
    scanning -- where a half is whole blocks of the kernel form that ran; either way the arena equals the one with
    every convolution scanning."""
    rng = np.random.default_rng(41 + oc)
    c, h, w = 16, side, side
    x = rng.uniform(-1, 1, (1, c, h, w)).astype(np.float32)
    pw = fastnn_amd.quantize_weights(flib.DT_I8, (rng.standard_normal((oc, c)) * 0.3).astype(np.float32))
    bias = (rng.standard_normal(oc) * 0.1).astype(np.float32)
    ph = [fastnn_amd.quantize_weights(flib.DT_I8, (rng.standard_normal((8, oc // 2)) * 0.2).astype(np.float32)) for _ in range(2)]
    a = Arena()
    s_x, s_w, s_b = a.take(x.nbytes), a.take(pw.words.nbytes), a.take(bias.nbytes)
    s_wh = [a.take(p.words.nbytes) for p in ph]
    s_y = a.take(oc * h * w * 4)
    half = (oc // 2) * h * w * 4
    s_h = [(s_y[0], half), (s_y[0] + half, half)]
    s_o = [a.take(8 * h * w * 4) for _ in range(2)]
    plan = ExecutablePlan(a.top).write_const(s_w[0], pw.words).write_const(s_b[0], bias)
    for k in range(2):
        plan.write_const(s_wh[k][0], ph[k].words)
    plan.call_kernel("conv2d_i8_silu", [s_x, s_w, s_b], s_y, [1, 0, 1, 1, c, h, w, 1, 1], meta_of(pw, [oc, c, 1, 1]))
    for k in range(2):
        plan.call_kernel("conv2d_i8", [s_h[k], s_wh[k]], s_o[k], [1, 0, 1, 1, oc // 2, h, w, 1, 1], meta_of(ph[k], [8, oc // 2, 1, 1]))
    be.allocate_arena(a.top)
    be.write_arena(s_x[0], x)
    got, used = {}, {}
    try:
        be.set_option(flib.OPT_CONV_IMPLICIT, implicit)
        for on in (1, 0):
            be.set_option(flib.OPT_CONV_RANGES, on)
            be.dispatch(plan)
            first = be.read_arena(0, a.top).copy()
            be.dispatch(plan)
            assert plan.replayed
            got[on], used[on] = be.read_arena(0, a.top).copy(), plan.ranges_used
            assert np.array_equal(first, got[on]), "replay differs from the first dispatch"
    finally:
        be.set_option(flib.OPT_CONV_RANGES, 1)
        be.set_option(flib.OPT_CONV_IMPLICIT, 0)
    assert np.array_equal(got[1], got[0])
    assert used[0] == 0 and used[1] in (0, 2), used
    # the fused kernel has blocks of 32 channels (64 from 129 channels on), the tiles of the GEMM pair 64 or 128
    if (implicit == 3 and oc >= 64) or (implicit == 2 and oc >= 128):
        assert used[1] == 2, used
    y = got[1][s_y[0]:s_y[0] + s_y[1]].view(np.float32).reshape(1, oc, h, w)
    for k in range(2):
        o = got[1][s_o[k][0]:s_o[k][0] + s_o[k][1]].view(np.float32).reshape(1, 8, h, w)
        part = np.ascontiguousarray(y[:, k * (oc // 2):(k + 1) * (oc // 2)])
        assert_close(o, orc.qconv2d_i8(part, to_oracle(orc, ph[k]), 1, 1, 1, 0, 1, 1), 1e-5, f"half {k}")


def test_residual_add_onto_the_matmul_input_stays_an_instruction(be, orc):
    """x = x + MatMul(x) with the sum written over x: workgroups of the MatMul still read x while others would store
    sums, so the Add is not folded into the MatMul's last kernel."""
    rng = np.random.default_rng(5)
    m, d = 48, 512
    x = rng.standard_normal((m, d)).astype(np.float32)
    pw = fastnn_amd.quantize_weights(flib.DT_I8, _w(rng, d, d))
    a = Arena()
    s_x, s_w, s_y = a.take(x.nbytes), a.take(pw.words.nbytes), a.take(x.nbytes)
    plan = ExecutablePlan(a.top).write_const(s_w[0], pw.words)
    plan.call_kernel("matmul_i8", [s_x, s_w], s_y, [m, d, d], meta_of(pw)).call_kernel("add_f32", [s_y, s_x], s_x, [m * d])
    be.allocate_arena(a.top)
    for it in range(2):
        be.write_arena(s_x[0], x)
        be.dispatch(plan)
        assert plan.residuals_fused == 0
        y = be.read_arena(*s_y, np.float32).reshape(m, d)
        assert_close(y, orc.qmatmul(to_oracle(orc, pw), x), 2e-5, "MatMul output")
        assert np.array_equal(be.read_arena(*s_x, np.float32).reshape(m, d), y + x)


@pytest.mark.parametrize("implicit", [0, 1, 2, 3])
@pytest.mark.parametrize("wdt,kname,geom", [
    (flib.DT_I8, "conv2d_i8_silu", (3, 16, 20, 20, 24, 3)),    # (images, C, H, W, OC, kernel side)
    (flib.DT_I4, "conv2d_i4", (2, 8, 9, 9, 40, 3)),            # 81 pixels per image: outputs stored one by one
    (flib.DT_I8, "conv2d_i8_relu", (2, 32, 12, 12, 136, 1)),   # more than 128 channels
    (flib.DT_I8, "conv2d_i8", (1, 144, 16, 16, 16, 3)),        # K = 1296: beyond the kernel that holds its operands in LDS
])
def test_conv_followed_by_residual_add_runs_as_one_call(be, orc, implicit, wdt, kname, geom):
    """A quantised Conv2d whose output the next instruction adds to another tensor stores the sum from its epilogue
    (FNN_OPT_FUSE_RESIDUAL, the Add is skipped), in each of its kernel forms: the whole arena is, bit for bit, what
    the instructions give on their own, including the convolution that reads a sum (whose activation ranges then
    come from the fused epilogue, not from the Add).  The sum overwriting the convolution's output or its input
    still runs the Add."""
    rng = np.random.default_rng(211 + wdt + geom[1])
    n, c, h, w, oc, k = geom
    hw, kk = h * w, c * k * k
    x = rng.uniform(-1, 1, (n, c, h, w)).astype(np.float32)
    r = rng.standard_normal((n, oc, h, w)).astype(np.float32)
    pw = fastnn_amd.quantize_weights(wdt, (rng.standard_normal((oc, kk)) * np.sqrt(2.0 / kk)).astype(np.float32))
    bias = (rng.standard_normal(oc) * 0.05).astype(np.float32)
    pw2 = fastnn_amd.quantize_weights(flib.DT_I8, (rng.standard_normal((8, oc)) * np.sqrt(2.0 / oc)).astype(np.float32))
    pwx = fastnn_amd.quantize_weights(flib.DT_I8, (rng.standard_normal((c, c)) * np.sqrt(2.0 / c)).astype(np.float32))
    a = Arena()
    ybytes = n * oc * hw * 4
    s_x, s_r, s_w, s_b, s_w2, s_wx = a.take(x.nbytes), a.take(r.nbytes), a.take(pw.words.nbytes), a.take(bias.nbytes), a.take(pw2.words.nbytes), a.take(pwx.words.nbytes)
    s_y = [a.take(ybytes) for _ in range(5)]
    s_sum = [a.take(ybytes) for _ in range(5)]
    s_r2, s_next, s_x2, s_y5 = a.take(r.nbytes), [a.take(n * 8 * hw * 4) for _ in range(2)], a.take(x.nbytes), a.take(x.nbytes)
    plan = ExecutablePlan(a.top).write_const(s_w[0], pw.words).write_const(s_b[0], bias).write_const(s_w2[0], pw2.words).write_const(s_wx[0], pwx.words)
    cv = lambda dst, src=s_x: plan.call_kernel(kname, [src, s_w, s_b], dst, [1, k // 2, 1, 1, c, h, w, k, k], meta_of(pw, [oc, c, k, k]))
    reader = lambda src, dst: plan.call_kernel("conv2d_i8", [src, s_w2], dst, [1, 0, 1, 1, oc, h, w, 1, 1], meta_of(pw2, [8, oc, 1, 1]))
    cv(s_y[0]); plan.call_kernel("add_f32", [s_y[0], s_r], s_sum[0], [n * oc * hw])       # convolution output first
    reader(s_sum[0], s_next[0])                                                            # ... and a convolution reads the sum
    cv(s_y[1]); plan.call_kernel("add_f32", [s_r, s_y[1]], s_sum[1], [n * oc * hw])       # ... second
    plan.memcopy(s_r2, s_r)
    cv(s_y[2]); plan.call_kernel("add_f32", [s_y[2], s_r2], s_r2, [n * oc * hw])          # the sum replaces the other operand
    reader(s_r2, s_next[1])
    cv(s_y[3]); plan.call_kernel("add_f32", [s_y[3], s_r], s_y[3], [n * oc * hw])         # ... replaces the convolution's output: not fused
    # x2 = x2 + conv(x2) with C -> C channels: the sum would land where workgroups still read their taps: not fused
    plan.memcopy(s_x2, s_x)
    plan.call_kernel("conv2d_i8", [s_x2, s_wx], s_y5, [1, 0, 1, 1, c, h, w, 1, 1], meta_of(pwx, [c, c, 1, 1]))
    plan.call_kernel("add_f32", [s_y5, s_x2], s_x2, [n * c * hw])
    be.allocate_arena(a.top)
    be.write_arena(s_x[0], x)
    be.write_arena(s_r[0], r)
    got, used = {}, {}
    try:
        be.set_option(flib.OPT_CONV_IMPLICIT, implicit)
        for fuse in (1, 0):
            be.set_option(flib.OPT_FUSE_RESIDUAL, fuse)
            be.dispatch(plan)
            first = be.read_arena(0, a.top).copy()
            be.dispatch(plan)
            assert plan.replayed
            got[fuse] = be.read_arena(0, a.top).copy()
            used[fuse] = plan.ranges_used
            assert np.array_equal(first, got[fuse]), "replay differs from the first dispatch"
            assert plan.residuals_fused == (3 if fuse else 0)
    finally:
        be.set_option(flib.OPT_FUSE_RESIDUAL, 1)
        be.set_option(flib.OPT_CONV_IMPLICIT, 0)
    assert np.array_equal(got[1], got[0])
    # both readers take the ranges of the sums from the Add, or from the fused epilogue when an image holds at least a
    # workgroup's pixels (the third taker is the convolution behind the copy of x)
    assert used[0] == 3 and used[1] <= 3 and (hw < 256 or used[1] == 3), used
    view = lambda s, ch=oc: got[1][s[0]:s[0] + s[1]].view(np.float32).reshape(n, ch, h, w)
    act = {"silu": flib.ACT_SILU, "relu": flib.ACT_RELU}.get(kname.split("_")[-1], 0)
    want_y = orc.qconv2d_i8(x, to_oracle(orc, pw), k, k, 1, k // 2, 1, 1, bias=bias, act=act)
    for i in range(3):
        assert_close(view(s_y[i]), want_y, 1e-5, f"convolution output {i}")
    for s in (s_sum[0], s_sum[1], s_r2, s_y[3]):
        assert np.array_equal(view(s), view(s_y[0]) + r)
    assert np.array_equal(view(s_x2, c), view(s_y5, c) + x)


@pytest.mark.parametrize("m", [64, 40])
@pytest.mark.parametrize("single", [0, 1])
def test_matmul_chain_hands_the_prepared_operand_on(be, orc, m, single):
    """A MatMul whose result the next instruction multiplies leaves that MatMul's prepared activation operand behind
    (FNN_OPT_FUSE_PREP): directly, and through the residual Add that rides in its reduction.  Same conversion code, so
    every tensor of the chain equals, bit for bit, what the plan gives with every MatMul preparing its own operand;
    an integer-weight MatMul (digit planes, another operand format) and a codebook one are not handed anything."""
    rng = np.random.default_rng(131 + m + single)
    d, f = 512, 2048
    x = rng.standard_normal((m, d)).astype(np.float32)
    w1 = fastnn_amd.quantize_weights(flib.DT_F8, _w(rng, f, d))
    w2 = fastnn_amd.quantize_weights(flib.DT_F4, _w(rng, d, f))
    w3 = fastnn_amd.quantize_weights(flib.DT_U8, _w(rng, f, d))
    w4 = fastnn_amd.quantize_weights(flib.DT_I4, _w(rng, d, f))
    b1 = (rng.standard_normal(f) * 0.1).astype(np.float32)
    a = Arena()
    s_x = a.take(x.nbytes)
    s_w = [a.take(w.words.nbytes) for w in (w1, w2, w3, w4)]
    s_b1 = a.take(b1.nbytes)
    s_h, s_y, s_s, s_h2, s_y2 = a.take(m * f * 4), a.take(m * d * 4), a.take(m * d * 4), a.take(m * f * 4), a.take(m * d * 4)
    plan = ExecutablePlan(a.top)
    for s, w in zip(s_w, (w1, w2, w3, w4)):
        plan.write_const(s[0], w.words)
    plan.write_const(s_b1[0], b1)
    plan.call_kernel("matmul_f8_gelu", [s_x, s_w[0], s_b1], s_h, [m, d, f], meta_of(w1))     # -> operand of the next
    plan.call_kernel("matmul_f4", [s_h, s_w[1]], s_y, [m, f, d], meta_of(w2))                # handed; + Add -> operand of the next
    plan.call_kernel("add_f32", [s_y, s_x], s_s, [m * d])
    plan.call_kernel("matmul_u8_relu", [s_s, s_w[2]], s_h2, [m, d, f], meta_of(w3))          # handed; next has integer weights
    plan.call_kernel("matmul_i4", [s_h2, s_w[3]], s_y2, [m, f, d], meta_of(w4))
    be.allocate_arena(a.top)
    be.write_arena(s_x[0], x)
    got = {}
    try:
        be.set_kernel_flags(flib.FLAG_ACT_F16_SINGLE if single else 0)
        for on in (1, 0):
            be.set_option(flib.OPT_FUSE_PREP, on)
            be.dispatch(plan)
            first = be.read_arena(0, a.top).copy()
            be.dispatch(plan)
            assert plan.replayed
            got[on] = be.read_arena(0, a.top).copy()
            assert np.array_equal(first, got[on]), "replay differs from the first dispatch"
            assert plan.operands_handed == (2 if on else 0)
    finally:
        be.set_option(flib.OPT_FUSE_PREP, 1)
        be.set_kernel_flags(0)
    assert np.array_equal(got[1], got[0])
    view = lambda s, cols: got[1][s[0]:s[0] + s[1]].view(np.float32).reshape(m, cols)
    tol = 1e-3 if single else 2e-5
    h_ref = orc.qmatmul(to_oracle(orc, w1), x, bias=b1, act=flib.ACT_GELU)
    assert_close(view(s_h, f), h_ref, tol, "first layer")
    y_ref = orc.qmatmul(to_oracle(orc, w2), view(s_h, f))
    assert_close(view(s_y, d), y_ref, tol, "second layer on the first layer's output")
    assert np.array_equal(view(s_s, d), view(s_y, d) + x)
    h2_ref = orc.qmatmul(to_oracle(orc, w3), view(s_s, d), act=flib.ACT_RELU)
    assert_close(view(s_h2, f), h2_ref, tol, "third layer on the sum")
    y2_ref = orc.qmatmul(to_oracle(orc, w4), view(s_h2, f))
    assert_close(view(s_y2, d), y2_ref, tol, "fourth layer")


@pytest.mark.parametrize("k,s,p", [(5, 1, 2), (3, 2, 2), (2, 1, 1), (5, 2, 4), (3, 1, 0), (4, 2, 1)])
def test_maxpool_windows_with_special_values(be, orc, k, s, p):
    """Max pooling with every tap requested at once from clamped coordinates (2 x 2, 3 x 3, 5 x 5 windows) and the
    tap-by-tap kernel (4 x 4): the same bits as the CPU arm, also for signed zeros, infinities and NaN (never
    selected: a window of NaN gives -inf), on odd map sizes and with the largest padding a window allows."""
    rng = np.random.default_rng(1000 + 10 * k + p)
    n, c, h, w = 2, 3, 7, 9
    x = rng.standard_normal((n, c, h, w)).astype(np.float32)
    x[rng.random(x.shape) < 0.15] = 0.0
    x[rng.random(x.shape) < 0.10] = -0.0
    x[rng.random(x.shape) < 0.05] = np.nan
    x[rng.random(x.shape) < 0.03] = -np.inf
    x[rng.random(x.shape) < 0.03] = np.inf
    x[0, 0, :4, :5] = np.nan                      # whole windows of NaN
    want = orc.maxpool2d(x, k, s, p)
    a = Arena()
    s_x, s_y = a.take(x.nbytes), a.take(want.nbytes)
    plan = ExecutablePlan(a.top).write_const(s_x[0], x).call_kernel("pool_f32", [s_x], s_y, [k, s, p, 1, n, c, h, w])
    be.allocate_arena(a.top)
    be.dispatch(plan)
    got = be.read_arena(*s_y, np.uint32)
    assert np.array_equal(got, want.reshape(-1).view(np.uint32))


@pytest.mark.parametrize("seed", [3, 4])
def test_random_matmul_chains_equal_with_and_without_plan_fusions(be, seed):
    """Random chains of two to five MatMuls (mixed weight types, 17 <= M <= 200, optional bias and activation) with
    residual Adds wherever an earlier tensor has the same width: the whole arena with FNN_OPT_FUSE_RESIDUAL and
    FNN_OPT_FUSE_PREP on equals, byte for byte, the arena with both off, on the first dispatch and on the replay."""
    rng = np.random.default_rng(seed)
    engaged = 0
    for case in range(8):
        m = int(rng.choice([17, 24, 40, 64, 100, 128, 200]))
        nl = int(rng.integers(2, 6))
        dims = [int(rng.choice([64, 128, 192, 512, 1024, 2048, 4096, 512, 1024])) for _ in range(nl + 1)]
        dts = [int(rng.choice([flib.DT_F8, flib.DT_F4, flib.DT_U8, flib.DT_F8R, flib.DT_F8, flib.DT_I4, flib.DT_I8])) for _ in range(nl)]
        a = Arena()
        x = rng.standard_normal((m, dims[0])).astype(np.float32)
        s_x = a.take(x.nbytes)
        ws = [fastnn_amd.quantize_weights(dts[i], (rng.standard_normal((dims[i + 1], dims[i])) / np.sqrt(dims[i])).astype(np.float32)) for i in range(nl)]
        s_w = [a.take(w.words.nbytes) for w in ws]
        plan_calls, consts = [], []
        cur, same_width = s_x, {dims[0]: s_x}
        for i in range(nl):
            k, n = dims[i], dims[i + 1]
            out = a.take(m * n * 4)
            name = KERNEL_OF[dts[i]] + ["", "_relu", "_gelu", "_silu"][int(rng.integers(0, 4))]
            inputs = [cur, s_w[i]]
            if rng.random() < 0.5:
                bias = (rng.standard_normal(n) * 0.1).astype(np.float32)
                s_b = a.take(bias.nbytes)
                consts.append((s_b, bias))
                inputs.append(s_b)
            plan_calls.append((name, inputs, out, [m, k, n], meta_of(ws[i])))
            cur = out
            if n in same_width and rng.random() < 0.7:
                s_sum = a.take(m * n * 4)
                pair = [cur, same_width[n]] if rng.random() < 0.5 else [same_width[n], cur]
                plan_calls.append(("add_f32", pair, s_sum, [m * n], None))
                cur = s_sum
            same_width[n] = cur
        plan = ExecutablePlan(a.top)
        for s, w in zip(s_w, ws):
            plan.write_const(s[0], w.words)
        for s, v in consts:
            plan.write_const(s[0], v)
        for name, inputs, out, par, meta in plan_calls:
            plan.call_kernel(name, inputs, out, par, meta)
        be.allocate_arena(a.top)
        be.write_arena(s_x[0], x)
        got = {}
        try:
            for on in (1, 0):
                be.set_option(flib.OPT_FUSE_PREP, on)
                be.set_option(flib.OPT_FUSE_RESIDUAL, on)
                be.dispatch(plan)
                first = be.read_arena(0, a.top).copy()
                be.dispatch(plan)
                got[on] = be.read_arena(0, a.top).copy()
                assert np.array_equal(first, got[on]), (case, on, "replay differs from the first dispatch")
                if on:
                    engaged += plan.residuals_fused + plan.operands_handed
                else:
                    assert plan.residuals_fused == 0 and plan.operands_handed == 0
        finally:
            be.set_option(flib.OPT_FUSE_PREP, 1)
            be.set_option(flib.OPT_FUSE_RESIDUAL, 1)
        assert np.array_equal(got[1], got[0]), (case, m, dims, dts)
        plan.close()
    assert engaged > 0


@pytest.mark.parametrize("dt", [flib.DT_I8, flib.DT_F4])
def test_three_input_matmul_without_a_suffix_adds_the_bias_and_nothing_else(be, orc, dt):
    """`matmul_<type>` with a third input slice: the slice is the bias, no activation is applied (the epilogue is
    named by the suffix alone, as for conv2d_*); the same three slices under `_relu` apply max(x, 0) on top."""
    rng = np.random.default_rng(410 + dt)
    m, k, n = 5, 192, 80
    x = rng.standard_normal((m, k)).astype(np.float32)
    pw = fastnn_amd.quantize_weights(dt, _w(rng, n, k))
    bias = rng.standard_normal(n).astype(np.float32)
    a = Arena()
    s_x, s_w, s_b, s_o, s_r = a.take(x.nbytes), a.take(pw.words.nbytes), a.take(bias.nbytes), a.take(m * n * 4), a.take(m * n * 4)
    plan = ExecutablePlan(a.top).write_const(s_x[0], x).write_const(s_w[0], pw.words).write_const(s_b[0], bias)
    plan.call_kernel(KERNEL_OF[dt], [s_x, s_w, s_b], s_o, [m, k, n], meta_of(pw))
    plan.call_kernel(KERNEL_OF[dt] + "_relu", [s_x, s_w, s_b], s_r, [m, k, n], meta_of(pw))
    be.allocate_arena(a.top)
    be.dispatch(plan)
    want = orc.qmatmul(to_oracle(orc, pw), x, bias=bias)
    assert (want < 0).any()
    got = be.read_arena(*s_o, np.float32).reshape(m, n)
    assert_close(got, want, 2e-5, "bias, no activation")
    assert np.array_equal(be.read_arena(*s_r, np.float32).reshape(m, n), np.maximum(got, 0.0))


@pytest.mark.parametrize("act,code", [("Relu", flib.ACT_RELU), ("Silu", flib.ACT_SILU)])
def test_matmul_add_activation_nodes_reach_the_library_as_one_tagged_instruction(orc, act, code):
    """MatMul -> Add(bias) -> Relu|Silu through AotExecutor(quantize=8): the native plan (what fnn_plan_add_call_kernel
    received) holds one `matmul_i8_<act>` CallKernel with three input slices, and its result is act(xW + b)."""
    from fastnn_amd.aot import AotExecutor
    rng = np.random.default_rng(77)
    d, f, m = 96, 160, 6
    nodes = [{"name": "fc", "op_type": "MatMul", "inputs": "[x, w]", "outputs": "[h0]"},
             {"name": "b", "op_type": "Add", "inputs": "[h0, bias]", "outputs": "[h1]"},
             {"name": "a", "op_type": act, "inputs": "[h1]", "outputs": "[y]"}]
    params = {"w": (rng.standard_normal((d, f)) * 0.1).astype(np.float32), "bias": rng.standard_normal(f).astype(np.float32)}
    x = rng.standard_normal((m, d)).astype(np.float32)
    ex = AotExecutor(nodes, params, ["x"], ["y"], {"x": [m, d]}, quantize=8)
    try:
        y = ex.forward({"x": x})["y"]
        calls = [ex._plan.describe(i) for i in range(len(ex._plan))]
        calls = [c for c in calls if c["op"] == "CallKernel"]
        assert len(calls) == 1
        assert calls[0]["kernel"] == "matmul_i8_" + act.lower()
        assert len(calls[0]["inputs"]) == 3 and calls[0]["params"] == [m, d, f]
    finally:
        ex.close()
    pw = fastnn_amd.quantize_weights(flib.DT_I8, np.ascontiguousarray(params["w"].T))
    want = orc.qmatmul(to_oracle(orc, pw), x, bias=params["bias"], act=code)
    assert_close(y, want, 2e-5, "act(xW + b)")


def test_plan_fusions_engage_when_param_dims_are_all_known(be, orc):
    """CpuBackend::compile gives every MatMul `param_dims: Some([m, k, n])`, all `Known` for a static graph
    (src/backend/cpu/mod.rs:601-613): such a plan must fuse the residual Add and hand prepared operands on exactly
    like the same plan without param_dims, with a byte-identical arena."""
    rng = np.random.default_rng(141)
    m, d, f = 64, 512, 2048
    x = rng.standard_normal((m, d)).astype(np.float32)
    w1 = fastnn_amd.quantize_weights(flib.DT_F8, _w(rng, f, d))
    w2 = fastnn_amd.quantize_weights(flib.DT_F4, _w(rng, d, f))
    w3 = fastnn_amd.quantize_weights(flib.DT_F8, _w(rng, f, d))
    arenas = {}
    for dims in (False, True):
        a = Arena()
        s_x = a.take(x.nbytes)
        s_w = [a.take(w.words.nbytes) for w in (w1, w2, w3)]
        s_h, s_y, s_s, s_h2 = a.take(m * f * 4), a.take(m * d * 4), a.take(m * d * 4), a.take(m * f * 4)
        plan = ExecutablePlan(a.top)
        for s, w in zip(s_w, (w1, w2, w3)):
            plan.write_const(s[0], w.words)
        plan.call_kernel("matmul_f8_gelu", [s_x, s_w[0]], s_h, [m, d, f], meta_of(w1))
        plan.call_kernel("matmul_f4", [s_h, s_w[1]], s_y, [m, f, d], meta_of(w2))
        plan.call_kernel("add_f32", [s_y, s_x], s_s, [m * d])
        plan.call_kernel("matmul_f8", [s_s, s_w[2]], s_h2, [m, d, f], meta_of(w3))
        if dims:
            plan.set_param_dims(3, [m, d, f]).set_param_dims(4, [m, f, d]).set_param_dims(6, [m, d, f])
        be.allocate_arena(a.top)
        be.write_arena(s_x[0], x)
        be.dispatch(plan)
        be.dispatch(plan)
        assert plan.residuals_fused == 1, dims
        assert plan.operands_handed == 2, dims
        arenas[dims] = be.read_arena(0, a.top).copy()
    assert np.array_equal(arenas[False], arenas[True])
    h = arenas[True][s_h[0]:s_h[0] + s_h[1]].view(np.float32).reshape(m, f)
    assert_close(h, orc.qmatmul(to_oracle(orc, w1), x, act=flib.ACT_GELU), 2e-5, "first layer")
    # a symbolic M keeps every instruction on its own
    plan.set_param_dims(4, [("T", m), f, d])
    be.dispatch(plan)
    assert plan.residuals_fused == 0
    assert np.array_equal(be.read_arena(0, a.top), arenas[True])


def test_dispatch_profile_runs_under_the_shape_environment_it_is_given(be, orc):
    """Backend::dispatch_profile resolves symbolic dims with the ShapeEnv of the call (src/backend/mod.rs:178-211), not
    with whatever an earlier dispatch left behind; without bindings a Bounded dim takes its maximum."""
    rng = np.random.default_rng(93)
    k, n = 64, 24
    pw = fastnn_amd.quantize_weights(flib.DT_F8, _w(rng, n, k))
    x = rng.standard_normal((4, k)).astype(np.float32)
    a = Arena()
    s_x, s_w, s_o = a.take(x.nbytes), a.take(pw.words.nbytes), a.take(4 * n * 4)
    plan = ExecutablePlan(a.top).write_const(s_x[0], x).write_const(s_w[0], pw.words)
    plan.call_kernel("matmul_f8", [s_x, s_w], s_o, [1, k, n], meta_of(pw))
    plan.set_param_dims(2, [("T", 4), k, n])
    be.allocate_arena(a.top)
    want = orc.qmatmul(to_oracle(orc, pw), x)
    be.dispatch(plan, {"T": 2})
    for rows in (3, 1):
        be.write_arena(s_o[0], np.zeros(4 * n, np.float32))
        times = be.dispatch_profile(plan, {"T": rows})
        assert len(times) == 3 and times[2] > 0
        got = be.read_arena(*s_o, np.float32).reshape(4, n)
        assert_close(got[:rows], want[:rows], 2e-5, f"T = {rows}")
        assert not got[rows:].any()
    be.write_arena(s_o[0], np.zeros(4 * n, np.float32))
    be.dispatch_profile(plan)                          # no environment: the bound, not the previous call's T = 1
    assert_close(be.read_arena(*s_o, np.float32).reshape(4, n), want, 2e-5, "Bounded -> max")
    sym = ExecutablePlan(a.top).write_const(s_x[0], x).write_const(s_w[0], pw.words)
    sym.call_kernel("matmul_f8", [s_x, s_w], s_o, [1, k, n], meta_of(pw))
    sym.set_param_dims(2, ["T", k, n])
    be.dispatch(sym, {"T": 2})
    with pytest.raises(flib.FnnError) as e:
        be.dispatch_profile(sym)
    assert "DimExpr::Symbol 'T' is not bound" in e.value.message
