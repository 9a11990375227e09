"""GPU parity at the full sizes of the benchmark configurations that the row-sampled MatMul test does not
reach: the FP8 / FP4 MLP stack (four blocks of Linear 2048->8192 + GELU, Linear 8192->2048 + residual, 64
tokens) through the plan dispatcher against the chained oracle, and the YOLOv8n-shaped I8 convolutions at
640x640 against the oracle's restatement of conv2d_packed_i8x4, layer by layer and as one graph."""
import os
import sys

import numpy as np
import pytest

import fastnn_amd
from fastnn_amd import lib as flib
from fastnn_amd.aot import AotExecutor, _names
from fastnn_amd.backend import ExecutablePlan, HipBackend, KERNEL_OF, meta_of
from gpu_common import assert_close, rel_err, to_oracle

sys.path.insert(0, os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
import bench  # noqa: E402  (the conv list and the graph of the benchmark itself)

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ctx():
    c = fastnn_amd.HipContext(0)
    yield c
    c.close()


# --------------------------------------------------------------------------- C4: MLP stack
@pytest.mark.parametrize("dt", [flib.DT_F8, flib.DT_F4])
def test_mlp_stack_full_size_against_chained_oracle(orc, dt):
    """Every hidden and block output of the 4-block stack at full width.  Each layer is checked twice: against the
    oracle applied to the device's own input of that layer (what the kernel computes, 2e-5) and against the
    oracle chained from the start (what the stack computes; the differences of earlier layers pass through)."""
    rng = np.random.default_rng(40 + dt)
    m, d, f, layers = 64, 2048, 8192, 4
    top = [0]

    def take(nb):
        o = top[0]
        top[0] += (nb + 63) // 64 * 64
        return (o, nb)

    s_x = [take(m * d * 4) for _ in range(layers + 1)]
    s_h = [take(m * f * 4) for _ in range(layers)]
    s_y = [take(m * d * 4) for _ in range(layers)]
    consts = []
    for _ in range(layers):
        w1 = fastnn_amd.quantize_weights(dt, (rng.standard_normal((f, d)) / np.sqrt(d)).astype(np.float32))
        w2 = fastnn_amd.quantize_weights(dt, (rng.standard_normal((d, f)) / np.sqrt(f)).astype(np.float32))
        consts.append((w1, take(w1.words.nbytes), w2, take(w2.words.nbytes)))
    plan = ExecutablePlan(top[0])
    for w1, s1, w2, s2 in consts:
        plan.write_const(s1[0], w1.words).write_const(s2[0], w2.words)
    for i, (w1, s1, w2, s2) in enumerate(consts):
        plan.call_kernel(KERNEL_OF[dt] + "_gelu", [s_x[i], s1], s_h[i], [m, d, f], meta_of(w1))
        plan.call_kernel(KERNEL_OF[dt], [s_h[i], s2], s_y[i], [m, f, d], meta_of(w2))
        plan.call_kernel("add_f32", [s_y[i], s_x[i]], s_x[i + 1], [m * d])
    x = rng.standard_normal((m, d)).astype(np.float32)
    be = HipBackend(0)
    try:
        be.allocate_arena(top[0])
        be.write_arena(s_x[0][0], x)
        be.dispatch(plan)
        be.dispatch(plan)          # the second dispatch replays the captured graph
        chained = x
        for i, (w1, _, w2, _) in enumerate(consts):
            p1, p2 = to_oracle(orc, w1), to_oracle(orc, w2)
            x_dev = be.read_arena(*s_x[i], np.float32).reshape(m, d)
            h_dev = be.read_arena(*s_h[i], np.float32).reshape(m, f)
            y_dev = be.read_arena(*s_y[i], np.float32).reshape(m, d)
            o_dev = be.read_arena(*s_x[i + 1], np.float32).reshape(m, d)
            assert_close(h_dev, orc.qmatmul(p1, x_dev, act=flib.ACT_GELU), 2e-5, f"block {i} up-projection")
            assert_close(y_dev, orc.qmatmul(p2, h_dev), 2e-5, f"block {i} down-projection")
            assert np.array_equal(o_dev, y_dev + x_dev), f"block {i} residual add"
            h = orc.qmatmul(p1, chained, act=flib.ACT_GELU)
            chained = orc.qmatmul(p2, h) + chained
            assert_close(o_dev, chained, 1e-4, f"block {i} output, chained")
    finally:
        plan.close()
        be.close()


# --------------------------------------------------------------------------- C5: real layer shapes
def _conv_case(ctx, orc, rng, b, c, h, oc, k, s, act=flib.ACT_SILU):
    kk = c * k * k
    wt = (rng.standard_normal((oc, kk)) * np.sqrt(2.0 / kk)).astype(np.float32)
    bias = (rng.standard_normal(oc) * 0.05).astype(np.float32)
    x = rng.uniform(0, 1, (b, c, h, h)).astype(np.float32)
    pw = fastnn_amd.quantize_weights(flib.DT_I8, wt)
    hd = ctx.register(pw)
    args = (k, k, s, k // 2, 1, 1)
    want, want_acc, _, _ = orc.qconv2d_i8(x, to_oracle(orc, pw), *args, bias=bias, act=act, want_acc=True)
    got, acc = ctx.qconv2d(hd, x, oc, *args, bias=bias, act=act, want_acc=True)
    ctx.release(hd)
    assert np.array_equal(acc, want_acc), f"accumulators of conv {(c, h, oc, k, s)} B={b}"
    assert_close(got, want, 1e-5, f"conv {(c, h, oc, k, s)} B={b}")


def test_every_yolo_layer_shape_at_batch_1(ctx, orc):
    """All 45 convolutions of the 640x640 network, each on its own U(0,1) input: i32 accumulators (bias_q
    included) bit-exact, outputs within 1e-5 (same f32 formula, expf differs in the last place)."""
    rng = np.random.default_rng(50)
    seen = set()
    for (c, h, oc, k, s) in bench.yolo_convs():
        if (c, h, oc, k, s) in seen:
            continue
        seen.add((c, h, oc, k, s))
        _conv_case(ctx, orc, rng, 1, c, h, oc, k, s)


def _distinct_yolo_shapes():
    seen, out = set(), []
    for shp in bench.yolo_convs():
        if shp not in seen:
            seen.add(shp)
            out.append(shp)
    return out


@pytest.mark.parametrize("c,h,oc,k,s", _distinct_yolo_shapes())
def test_every_yolo_layer_shape_at_batch_16(ctx, orc, c, h, oc, k, s):
    """Every distinct convolution shape of the 640x640 network at batch 16 (every image has its own activation
    range; pixel tiles straddle images from the 40x40 maps down): i32 accumulators bit-exact for all 16 images,
    outputs within 1e-5."""
    _conv_case(ctx, orc, np.random.default_rng(51 + c + h + oc + k + s), 16, c, h, oc, k, s)


def _check_graph_against_oracle(orc, nodes, params, ex, x, tag, images=None):
    """Every node of the graph against the oracle, each on the device's own value of its inputs (one arena slot
    per value, so every intermediate value can be read after the forward).  Convolutions: 1e-5; data movement
    and the residual add: bit for bit.  images: the images of the batch the convolutions are checked on (every
    node treats the images of a batch independently; None = all), the other nodes are always checked whole."""
    vals = {"x": x}
    sel = slice(None) if images is None else list(images)

    def dev(name):
        if name not in vals:
            vals[name] = ex.read_output(name)
        return vals[name]

    skip = set()
    n_conv = 0
    for i, nd in enumerate(nodes):
        if i in skip:
            continue
        ins, o = _names(nd["inputs"]), _names(nd["outputs"])
        op = nd["op_type"]
        if op == "Conv":
            w = params[ins[1]]
            oc, ic, kh, kw = w.shape
            nxt = nodes[i + 1]
            assert nxt["op_type"] == "Silu" and _names(nxt["inputs"]) == o
            skip.add(i + 1)
            pw = to_oracle(orc, fastnn_amd.quantize_weights(flib.DT_I8, w.reshape(oc, ic * kh * kw)))
            want = orc.qconv2d_i8(np.ascontiguousarray(dev(ins[0])[sel]), pw, kh, kw, int(nd["strides"]), int(nd["pads"]), 1, 1,
                                  bias=params[ins[2]], act=flib.ACT_SILU)
            assert_close(dev(_names(nxt["outputs"])[0])[sel], want, 1e-5, f"{tag}: conv node {nd['name']} {w.shape}")
            n_conv += 1
        elif op == "Split":
            a = dev(ins[0])
            half = a.shape[1] // 2
            for name, want in ((o[0], a[:, :half]), (o[1], a[:, half:])):
                if ex.kept(name):
                    assert np.array_equal(dev(name), want), nd["name"]
                else:   # a part that only a Concat wanted: that Concat reads the Split's input, the copy is not made
                    vals[name] = np.ascontiguousarray(want)
        elif op == "Add":
            assert np.array_equal(dev(o[0]), dev(ins[0]) + dev(ins[1])), nd["name"]
        elif op == "Concat":
            want = orc.concat([dev(n) for n in ins], dev(ins[0]).shape[0], int(np.prod(dev(o[0]).shape)))
            assert np.array_equal(dev(o[0]).reshape(-1), want.reshape(-1)), nd["name"]
        elif op == "MaxPool":
            assert np.array_equal(dev(o[0]), orc.maxpool2d(dev(ins[0]), 5, 1, 2)), nd["name"]
        elif op == "Resize":
            assert np.array_equal(dev(o[0]), orc.upsample_nearest2d(dev(ins[0]), 2, 2)), nd["name"]
        else:
            raise AssertionError(op)
    return n_conv


def _activation_codes(v, padded):
    """int8 codes the quantised convolution gives its input, image by image: the range of the im2col matrix (the
    tensor, plus 0 where a tap can fall into the padding), sa = range / 255 (1 when empty), za = min + 128 sa,
    q = clamp(round((x - za) * (1 / sa)), -128, 127) with ties away from zero, all in f32
    (src/backend/cpu/packed_conv.rs:149-156, 199-201; src/backend/cpu/im2col.rs:496-507)."""
    v = np.asarray(v, np.float32)
    out = np.empty(v.shape, np.int16)
    for i in range(v.shape[0]):
        mn, mx = np.float32(v[i].min()), np.float32(v[i].max())
        if padded:
            mn, mx = min(mn, np.float32(0)), max(mx, np.float32(0))
        rng_ = np.float32(mx - mn)
        sa = np.float32(rng_ / np.float32(255)) if rng_ > 0 else np.float32(1)
        za = np.float32(mn + np.float32(128) * sa) if rng_ > 0 else np.float32(0)
        t = ((v[i] - za) * np.float32(np.float32(1) / sa)).astype(np.float32)
        q = np.sign(t) * np.floor(np.abs(t) + np.float32(0.5))
        out[i] = np.clip(q, -128, 127).astype(np.int16)
    return out


@pytest.mark.parametrize("batch,size", [(1, 640), (2, 96), (16, 640)])
def test_yolo_graph_node_by_node_against_oracle(orc, batch, size):
    """The backbone + neck as one resident plan (HIP-graph replay on the second forward) at the benchmark's
    640x640 with batch 1 and batch 16, and a small two-image case.  The batch-16 plan is another instruction stream
    (Slice copies for Split, 44 convolutions taking their ranges from the producer, tiles holding pixels of two
    images); there the convolutions are checked on images 0, 7 and 15 and every other node on the whole batch.

    Parity statement: every node against the oracle on the very input the device saw (convolutions 1e-5, data
    movement and Add bit for bit).

    Chained statement: the oracle is also run from the input on its own, and for every convolution the int8 codes
    that the activation quantiser gives the device's input tensor are compared with the codes it gives the
    chained oracle's.  A network of 8-bit activation quantisers is not continuous: an activation within 1e-5 of
    a rounding boundary may land on the other side, which moves that code by one step.  While such flips are the
    only difference, codes differ by exactly one step in a few positions per hundred thousand: that is required of
    the first six convolutions (every difference +-1, at most 0.2 % of a layer's codes).  Further down the flips
    compound: a moved code moves the next layer's sums, a moved minimum or maximum moves that image's scale and
    zero point and with them half of its codes by a step, and this random-weight network amplifies a perturbation
    from layer to layer (measured at 640x640: 3e-5 of the codes after three layers, 2 % after ten, about half from
    the fifteenth on, largest difference 5 steps of 255).  No implementation-independent bound tighter than a few
    steps exists there, so the deep layers carry a guard against gross divergence only (at most 12 steps, outputs
    within 1e-1 of max|ref| and 1e-2 on average); what pins them is the node-by-node statement above."""
    rng = np.random.default_rng(5)
    nodes, params, shape, outs = bench.yolo_graph(batch, rng, size=size)
    x = rng.uniform(0, 1, shape).astype(np.float32)
    images = None if batch <= 2 else [0, 7, 15]
    sel = slice(None) if images is None else images
    ex = AotExecutor(nodes, params, ["x"], outs, {"x": shape}, quantize=8)
    try:
        first = ex.forward({"x": x})
        got = ex.forward({"x": x})
        assert ex.replayed
        for name in outs:
            assert np.array_equal(first[name], got[name]), name + ": replay differs from the first dispatch"
        assert _check_graph_against_oracle(orc, nodes, params, ex, x, f"B={batch} {size}px", images) == 45
        # chained oracle from the input (on the sampled images: every node treats images independently)
        vals = {"x": np.ascontiguousarray(x[sel])}
        skip = set()
        worst_step, report = 0, []
        for i, nd in enumerate(nodes):
            if i in skip:
                continue
            ins, o = _names(nd["inputs"]), _names(nd["outputs"])
            op = nd["op_type"]
            if op == "Conv":
                w = params[ins[1]]
                oc, ic, kh, kw = w.shape
                skip.add(i + 1)
                dev_in = x if ins[0] == "x" else ex.read_output(ins[0])
                qd = _activation_codes(dev_in[sel], int(nd["pads"]) > 0)
                qo = _activation_codes(vals[ins[0]], int(nd["pads"]) > 0)
                diff = np.abs(qd - qo)
                share, step = float((diff != 0).mean()), int(diff.max())
                report.append((nd["name"], round(share, 5), step))
                worst_step = max(worst_step, step)
                pw = to_oracle(orc, fastnn_amd.quantize_weights(flib.DT_I8, w.reshape(oc, ic * kh * kw)))
                vals[_names(nodes[i + 1]["outputs"])[0]] = orc.qconv2d_i8(vals[ins[0]], pw, kh, kw, int(nd["strides"]),
                                                                           int(nd["pads"]), 1, 1, bias=params[ins[2]],
                                                                           act=flib.ACT_SILU)
            elif op == "Split":
                a = vals[ins[0]]
                half = a.shape[1] // 2
                vals[o[0]], vals[o[1]] = a[:, :half].copy(), a[:, half:].copy()
            elif op == "Add":
                vals[o[0]] = vals[ins[0]] + vals[ins[1]]
            elif op == "Concat":
                vals[o[0]] = np.concatenate([vals[n] for n in ins], axis=1)
            elif op == "MaxPool":
                vals[o[0]] = orc.maxpool2d(vals[ins[0]], 5, 1, 2)
            elif op == "Resize":
                vals[o[0]] = orc.upsample_nearest2d(vals[ins[0]], 2, 2)
        print("chained oracle, per convolution (name, share of differing input codes, largest difference):", report, flush=True)
        assert all(step <= 1 and share <= 2e-3 for _, share, step in report[:6]), report
        assert worst_step <= 12, report
        stats = {}
        for name in outs:
            assert got[name][sel].shape == vals[name].shape
            d = np.abs(got[name][sel].astype(np.float64) - vals[name])
            mx = np.abs(vals[name]).max()
            stats[name] = (d.max() / mx, d.mean() / mx)
        print("chained oracle, (max, mean) of |diff| / max|ref| of the outputs:", stats, flush=True)
        assert all(a <= 1e-1 and b <= 1e-2 for a, b in stats.values()), stats
    finally:
        ex.close()


@pytest.mark.parametrize("implicit", [0, 1, 2, 3])
@pytest.mark.parametrize("batch,size", [(3, 160), (1, 224)])
def test_conv_activation_ranges_from_the_producing_instruction(orc, batch, size, implicit):
    """A quantised Conv2d in a plan takes min / max of its input from partial pairs the instruction before it left
    (conv epilogue, Split / Concat copies, residual Add, MaxPool, Resize) instead of scanning the tensor.  min and
    max do not depend on how the values are grouped, so every output must equal, bit for bit, what the plan gives
    with every convolution scanning its own input; the sizes make output tiles straddle images (20 x 20 = 400 rows
    per image against 64-row tiles) and fall below one tile (5 x 5), where the producer leaves nothing and the
    consumer scans.  implicit: which convolution kernel leaves and takes the pairs (0 = chosen by shape, 1 = the
    implicit-GEMM kernel wherever it runs, 2 = the operand kernel + GEMM pair everywhere, 3 = the fused kernel wherever it
    runs)."""
    rng = np.random.default_rng(11)
    nodes, params, shape, outs = bench.yolo_graph(batch, rng, size=size)
    x = rng.uniform(0, 1, shape).astype(np.float32)
    results = {}
    used = {}
    # (2: with the parts of every Concat copied, as the plan of a batch has them anyway; 1 and 0: parts of a
    # one-image Concat stored in place by their producers, whose pairs then arrive part by part)
    for on in (1, 0, 2):
        ex = AotExecutor(nodes, params, ["x"], outs, {"x": shape}, quantize=8, concat_in_place=on != 2)
        try:
            ex.set_option(flib.OPT_CONV_RANGES, 1 if on else 0)
            ex.set_option(flib.OPT_CONV_IMPLICIT, implicit)
            first = ex.forward({"x": x})
            again = ex.forward({"x": x})
            assert ex.replayed
            used[on] = ex.ranges_used
            for name in outs:
                assert np.array_equal(first[name], again[name]), name + ": replay differs from the first dispatch"
            results[on] = again
            if on:
                assert _check_graph_against_oracle(orc, nodes, params, ex, x, f"ranges B={batch} {size}px") == 45
        finally:
            ex.close()
    assert used[0] == 0
    # every conv but the first has a producer in the plan; the smallest maps fall back, and a part without pairs
    # leaves the reader of the whole in-place Concat to its own scan
    assert used[2] >= 30 and used[1] >= 28, used
    for name in outs:
        assert np.array_equal(results[1][name], results[0][name]), name
        assert np.array_equal(results[1][name], results[2][name]), name


def test_conv_activation_ranges_odd_shapes_and_every_producer(orc):
    """Ranges handed over by every kind of producer (conv epilogue with unaligned image sizes, MaxPool, Resize, Add,
    ReLU, Slice copies of a Split, Concat parts) and the cases that must fall back to a scan (a producer whose output
    map is smaller than one tile; a strided 1x1 convolution that does not touch every input row): 13 x 11 maps (143
    pixels per image: tiles straddle the three images, four pixels of a store group straddle them too), outputs equal
    bit for bit with and without the hand-over."""
    rng = np.random.default_rng(23)
    nodes, params = [], {}
    cnt = [0]

    def uid(p):
        cnt[0] += 1
        return f"{p}{cnt[0]}"

    def conv(x, c, oc, k, s, pad):
        w, b, y0, y = uid("w"), uid("b"), uid("c"), uid("s")
        kk = c * k * k
        params[w] = (rng.standard_normal((oc, c, k, k)) * np.sqrt(2.0 / kk)).astype(np.float32)
        params[b] = (rng.standard_normal(oc) * 0.05).astype(np.float32)
        nodes.append({"name": y0, "op_type": "Conv", "inputs": f"[{x}, {w}, {b}]", "outputs": f"[{y0}]", "strides": str(s),
                      "pads": str(pad), "group": "1"})
        nodes.append({"name": y, "op_type": "Silu", "inputs": f"[{y0}]", "outputs": f"[{y}]"})
        return y

    c1 = conv("x", 5, 24, 3, 1, 1)                      # [3, 24, 13, 11]
    c2 = conv(c1, 24, 40, 3, 2, 1)                      # [3, 40, 7, 6]: ranges from c1's epilogue; leaves none (42 pixels)
    c3 = conv(c2, 40, 16, 1, 2, 0)                      # odd input rows / columns are never read: scans
    nodes.append({"name": "m", "op_type": "MaxPool", "inputs": f"[{c1}]", "outputs": "[m]", "kernel_size": "3", "stride": "1",
                  "padding": "1"})
    c4 = conv("m", 24, 8, 3, 1, 1)
    nodes.append({"name": "u", "op_type": "Resize", "inputs": f"[{c2}]", "outputs": "[u]", "mode": "nearest", "scale_h": "2",
                  "scale_w": "2"})
    c5 = conv("u", 40, 8, 3, 1, 1)
    nodes.append({"name": "a", "op_type": "Add", "inputs": f"[{c1}, m]", "outputs": "[a]"})
    c6 = conv("a", 24, 8, 1, 1, 0)
    nodes.append({"name": "sp", "op_type": "Split", "inputs": f"[{c1}]", "outputs": "[h1, h2]", "axis": "1"})
    c7 = conv("h2", 12, 8, 3, 1, 1)
    nodes.append({"name": "k", "op_type": "Concat", "inputs": f"[{c4}, {c6}]", "outputs": "[k]", "axis": "1"})
    c8 = conv("k", 16, 8, 1, 1, 0)
    nodes.append({"name": "r", "op_type": "Relu", "inputs": "[m]", "outputs": "[r]"})
    c9 = conv("r", 24, 8, 3, 1, 1)
    outs = [c3, c5, c7, c8, c9]
    shape = (3, 5, 13, 11)
    x = rng.uniform(-1, 1, shape).astype(np.float32)
    results, used = {}, {}
    for on in (1, 0):
        ex = AotExecutor(nodes, params, ["x"], outs, {"x": shape}, quantize=8)
        try:
            ex.set_option(flib.OPT_CONV_RANGES, on)
            first = ex.forward({"x": x})
            again = ex.forward({"x": x})
            assert ex.replayed
            for name in outs:
                assert np.array_equal(first[name], again[name]), name
            results[on], used[on] = again, ex.ranges_used
            if on:   # the first convolution against the oracle: the scalar NCHW stores with ranges next to them
                w = params["w1"]
                pw = to_oracle(orc, fastnn_amd.quantize_weights(flib.DT_I8, w.reshape(24, 45)))
                want = orc.qconv2d_i8(x, pw, 3, 3, 1, 1, 1, 1, bias=params["b2"], act=flib.ACT_SILU)
                assert_close(ex.read_output(c1), want, 1e-5, "first convolution")
        finally:
            ex.close()
    assert used[0] == 0
    assert used[1] == 7, used   # c2, c4, c5, c6, c7, c8, c9; c3 and the first convolution scan
    for name in outs:
        assert np.array_equal(results[1][name], results[0][name]), name


@pytest.mark.parametrize("seed", [21, 22, 23])
def test_random_conv_graphs_equal_under_every_range_and_kernel_choice(seed):
    """Random graphs of 3 x 3 / 1 x 1 / strided convolutions with MaxPool, Resize, residual Add, ReLU and Concat
    between them (batch 1-3, maps of 9-40 pixels a side, 8-96 channels): the output of the plan is the same, bit for
    bit, with the activation ranges handed over or scanned, with the implicit-GEMM kernel chosen by shape, forced on or
    forced off, and with the residual Adds inside the convolution before them or as launches of their own, on the first
    dispatch and on the replay."""
    rng = np.random.default_rng(seed)
    for case in range(5):
        b, c0 = int(rng.integers(1, 4)), int(rng.choice([3, 5, 8, 16]))
        h, w = int(rng.integers(9, 41)), int(rng.integers(9, 41))
        nodes, params, cnt = [], {}, [0]

        def uid(p):
            cnt[0] += 1
            return f"{p}{cnt[0]}"

        def conv(x, c, oc, k, s, pad):
            wn, bn, y0, y = uid("w"), uid("b"), uid("c"), uid("s")
            params[wn] = (rng.standard_normal((oc, c, k, k)) * np.sqrt(2.0 / (c * k * k))).astype(np.float32)
            params[bn] = (rng.standard_normal(oc) * 0.05).astype(np.float32)
            nodes.append({"name": y0, "op_type": "Conv", "inputs": f"[{x}, {wn}, {bn}]", "outputs": f"[{y0}]", "strides": str(s),
                          "pads": str(pad), "group": "1"})
            nodes.append({"name": y, "op_type": "Silu", "inputs": f"[{y0}]", "outputs": f"[{y}]"})
            return y

        cur, cc, ch, cw = "x", c0, h, w
        for _ in range(int(rng.integers(3, 8))):
            kind = rng.choice(["conv3", "conv1", "conv3s2", "pool", "up", "res", "relu", "cat", "c2f"], p=[0.25, 0.2, 0.1, 0.08, 0.07, 0.1, 0.05, 0.08, 0.07])
            if kind in ("conv3", "conv1", "conv3s2"):
                oc, k = int(rng.choice([8, 16, 24, 40, 64, 96])), (1 if kind == "conv1" else 3)
                s = 2 if kind == "conv3s2" and min(ch, cw) >= 8 else 1
                cur = conv(cur, cc, oc, k, s, k // 2)
                cc, ch, cw = oc, (ch + 2 * (k // 2) - k) // s + 1, (cw + 2 * (k // 2) - k) // s + 1
            elif kind == "pool":
                y = uid("m")
                nodes.append({"name": y, "op_type": "MaxPool", "inputs": f"[{cur}]", "outputs": f"[{y}]", "kernel_size": "5", "stride": "1", "padding": "2"})
                cur = y
            elif kind == "up" and ch * cw < 900:
                y = uid("u")
                nodes.append({"name": y, "op_type": "Resize", "inputs": f"[{cur}]", "outputs": f"[{y}]", "mode": "nearest", "scale_h": "2", "scale_w": "2"})
                cur, ch, cw = y, ch * 2, cw * 2
            elif kind == "res":
                t, y = conv(cur, cc, cc, 3, 1, 1), uid("a")
                nodes.append({"name": y, "op_type": "Add", "inputs": f"[{cur}, {t}]", "outputs": f"[{y}]"})
                cur = y
            elif kind == "relu":
                y = uid("r")
                nodes.append({"name": y, "op_type": "Relu", "inputs": f"[{cur}]", "outputs": f"[{y}]"})
                cur = y
            elif kind == "cat":
                t, y = conv(cur, cc, 8, 1, 1, 0), uid("k")
                nodes.append({"name": y, "op_type": "Concat", "inputs": f"[{cur}, {t}]", "outputs": f"[{y}]", "axis": "1"})
                cur, cc = y, cc + 8
            elif kind == "c2f":   # conv, channel Split, a residual block on the second half, Concat of the halves and the sum
                oc = int(rng.choice([16, 32, 64, 128]))
                y0, ha, hb, r, y = conv(cur, cc, oc, 1, 1, 0), uid("h"), uid("h"), uid("a"), uid("k")
                nodes.append({"name": uid("sp"), "op_type": "Split", "inputs": f"[{y0}]", "outputs": f"[{ha}, {hb}]", "axis": "1"})
                t = conv(conv(hb, oc // 2, oc // 2, 3, 1, 1), oc // 2, oc // 2, 3, 1, 1)
                nodes.append({"name": r, "op_type": "Add", "inputs": f"[{hb}, {t}]", "outputs": f"[{r}]"})
                nodes.append({"name": y, "op_type": "Concat", "inputs": f"[{ha}, {hb}, {r}]", "outputs": f"[{y}]", "axis": "1"})
                cur, cc = y, oc + oc // 2
        cur = conv(cur, cc, 8, 3, 1, 1)
        shape = (b, c0, h, w)
        x = rng.uniform(-1, 1, shape).astype(np.float32)
        res = {}
        # (the fourth entry: parts of a one-image Concat stored in place by their producers, or copied by the Concat)
        for ranges, implicit, fuse, in_place in [(0, 0, 0, 0), (1, 0, 1, 1), (1, 1, 1, 1), (1, 2, 1, 0), (0, 1, 1, 1), (1, 0, 0, 1), (0, 2, 1, 1),
                                                 (1, 3, 1, 0), (0, 3, 0, 1), (1, 0, 1, 0)]:
            ex = AotExecutor(nodes, params, ["x"], [cur], {"x": shape}, quantize=8, concat_in_place=bool(in_place))
            try:
                ex.set_option(flib.OPT_CONV_RANGES, ranges)
                ex.set_option(flib.OPT_CONV_IMPLICIT, implicit)
                ex.set_option(flib.OPT_FUSE_RESIDUAL, fuse)   # (the Add behind a convolution rides in its epilogue)
                first = ex.forward({"x": x})[cur]
                again = ex.forward({"x": x})[cur]
                assert np.array_equal(first, again), (case, ranges, implicit, fuse, in_place, "replay differs from the first dispatch")
                assert ranges or ex.ranges_used == 0
                assert fuse or ex.residuals_fused == 0
                res[(ranges, implicit, fuse, in_place)] = again
            finally:
                ex.close()
        for key, val in res.items():
            assert np.array_equal(val, res[(0, 0, 0, 0)]), (case, key, shape, len(nodes))
