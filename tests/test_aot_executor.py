"""The host-side mirror of fastnn.AotExecutor(nodes, params, input_names, output_names, input_shapes, quantize):
argument handling and lowering need no GPU; forward() is checked against the oracle on the GPU."""
import numpy as np
import pytest

import fastnn_amd
from fastnn_amd import lib as flib
from fastnn_amd.aot import AotExecutor, weight_dtype_of


def mlp_nodes():
    """x -> MatMul(w1) -> Add(b1) -> Gelu -> MatMul(w2) -> Add(x) (residual), all values strings as the
    reference's Python side passes them (fastnn/io/graph_builder.py)."""
    return [
        {"name": "fc1", "op_type": "MatMul", "inputs": "[x, w1]", "outputs": "[h0]"},
        {"name": "b1", "op_type": "Add", "inputs": "[h0, b1]", "outputs": "[h1]"},
        {"name": "act", "op_type": "Gelu", "inputs": "[h1]", "outputs": "[h2]"},
        {"name": "fc2", "op_type": "MatMul", "inputs": "[h2, w2]", "outputs": "[y0]"},
        {"name": "res", "op_type": "Add", "inputs": "[y0, x]", "outputs": "[y]"},
    ]


def mlp_params(rng, d=64, f=160):
    return {"w1": (rng.standard_normal((d, f)) * 0.1).astype(np.float32), "b1": (rng.standard_normal(f) * 0.1).astype(np.float32),
            "w2": (rng.standard_normal((f, d)) * 0.1).astype(np.float32)}


def test_quantize_argument_mapping_and_errors():
    """src/python/nn.rs:1320-1358."""
    assert weight_dtype_of(None) is None and weight_dtype_of("f32") is None
    assert weight_dtype_of(4) == flib.DT_I4 and weight_dtype_of(8) == flib.DT_I8
    for s, dt in dict(i4=flib.DT_I4, i8=flib.DT_I8, u4=flib.DT_U4, u8=flib.DT_U8, f8=flib.DT_F8, f8r=flib.DT_F8R,
                      f4=flib.DT_F4, i4cb=flib.DT_I4CB).items():
        assert weight_dtype_of(s) == dt
    with pytest.raises(ValueError, match=r"unsupported quantize value for integer: 5 \(expected 4 or 8\)"):
        weight_dtype_of(5)
    with pytest.raises(ValueError, match="unsupported quantize string: 'int8'"):
        weight_dtype_of("int8")
    with pytest.raises(TypeError, match="quantize must be int"):
        weight_dtype_of(4.0)


def test_lowering_needs_no_gpu_and_fuses_bias_and_activation():
    rng = np.random.default_rng(0)
    ex = AotExecutor(mlp_nodes(), mlp_params(rng), ["x"], ["y"], {"x": [3, 64]}, quantize="f8")
    assert [i[0] for i in ex.instructions] == ["matmul_f8_gelu", "matmul_f8", "add_f32"]
    assert ex.instructions[0][3] == [3, 64, 160] and ex.instructions[1][3] == [3, 160, 64]
    assert ex.instructions[0][1] == ["x", "w1", "bias"]          # the Add(b1) went into the epilogue
    assert ex.arena_size % 64 == 0
    # the hidden value is also a graph output: nothing may be folded away behind it
    ex2 = AotExecutor(mlp_nodes(), mlp_params(rng), ["x"], ["y", "h0"], {"x": [3, 64]}, quantize=8)
    assert [i[0] for i in ex2.instructions] == ["matmul_i8", "add_f32", "gelu_f32", "matmul_i8", "add_f32"]


def test_lowering_errors():
    rng = np.random.default_rng(0)
    p = mlp_params(rng)
    with pytest.raises(flib.FnnError) as e:
        AotExecutor(mlp_nodes() + [{"name": "s", "op_type": "Softmax", "inputs": "[y]", "outputs": "[z]"}], p, ["x"], ["z"],
                    {"x": [3, 64]}, quantize=4)
    assert e.value.kind == "UnsupportedOp" and e.value.message == "Softmax"
    with pytest.raises(flib.FnnError) as e:
        AotExecutor(mlp_nodes(), p, ["x"], ["y"], {"x": [3, 64]}, quantize=None)
    assert e.value.kind == "UnsupportedOp"
    with pytest.raises(flib.FnnError):
        AotExecutor(mlp_nodes(), p, ["x"], ["y"], {"x": [-1, 64]}, quantize=4)     # symbolic batch
    with pytest.raises(flib.FnnError):
        AotExecutor(mlp_nodes(), p, ["x"], ["nope"], {"x": [3, 64]}, quantize=4)
    with pytest.raises(flib.FnnError):
        AotExecutor(mlp_nodes(), p, ["x"], ["y"], {"x": [3, 65]}, quantize=4)      # K mismatch


def test_conv_lowering():
    rng = np.random.default_rng(1)
    nodes = [
        {"name": "c1", "op_type": "Conv", "inputs": "[x, w, b]", "outputs": "[c]", "strides": "2", "pads": "1", "group": "1"},
        {"name": "a1", "op_type": "Silu", "inputs": "[c]", "outputs": "[s]"},
        {"name": "p", "op_type": "MaxPool", "inputs": "[s]", "outputs": "[m]", "kernel_shape": "5", "strides": "1", "pads": "2"},
        {"name": "cat", "op_type": "Concat", "inputs": "[s, m]", "outputs": "[k]", "axis": "1"},
        {"name": "up", "op_type": "Resize", "inputs": "[k]", "outputs": "[y]", "mode": "nearest", "scale_h": "2", "scale_w": "2"},
    ]
    params = {"w": rng.standard_normal((8, 3, 3, 3)).astype(np.float32), "b": np.zeros(8, np.float32)}
    ex = AotExecutor(nodes, params, ["x"], ["y"], {"x": [1, 3, 16, 16]}, quantize="i8", concat_in_place=False)
    assert [i[0] for i in ex.instructions] == ["conv2d_i8_silu", "pool_f32", "concat", "upsample_nearest2d"]
    assert ex.instructions[0][3] == [2, 1, 1, 1, 3, 16, 16, 3, 3]
    assert ex.instructions[1][3] == [5, 1, 2, 1, 1, 8, 8, 8]
    assert ex.instructions[2][3] == [1, 64, 1]
    assert ex.instructions[3][3] == [2, 2, 8, 8]
    # by default the parts of a one-image channel Concat live inside its result: the conv and the pool store there
    ex = AotExecutor(nodes, params, ["x"], ["y"], {"x": [1, 3, 16, 16]}, quantize="i8")
    assert [i[0] for i in ex.instructions] == ["conv2d_i8_silu", "pool_f32", "upsample_nearest2d"]
    k, s, m = ex._values["k"].slot, ex._values["s"].slot, ex._values["m"].slot
    assert s == (k[0], 8 * 64 * 4) and m == (k[0] + 8 * 64 * 4, 8 * 64 * 4) and k[1] == 16 * 64 * 4
    # a batch of two: the parts interleave per image, the Concat copies
    ex = AotExecutor(nodes, params, ["x"], ["y"], {"x": [2, 3, 16, 16]}, quantize="i8")
    assert [i[0] for i in ex.instructions] == ["conv2d_i8_silu", "pool_f32", "concat", "upsample_nearest2d"]


def _concat_graph():
    """conv -> Split -> conv on one half -> Concat(a, b, t) -> conv -> Concat(x, u, t, u)."""
    rng = np.random.default_rng(2)
    conv = lambda name, x, y: [{"name": name, "op_type": "Conv", "inputs": f"[{x}, w{name}]", "outputs": f"[{y}]", "strides": "1", "pads": "0"}]
    params = {}
    def w(name, c, oc):
        params["w" + name] = (rng.standard_normal((oc, c, 1, 1)) * 0.3).astype(np.float32)
    nodes = []
    w("c0", 16, 32); nodes += conv("c0", "x", "y")
    nodes += [{"name": "sp", "op_type": "Split", "inputs": "[y]", "outputs": "[a, b]", "axis": "1"}]
    w("c1", 16, 16); nodes += conv("c1", "b", "t")
    nodes += [{"name": "k1", "op_type": "Concat", "inputs": "[a, b, t]", "outputs": "[k]", "axis": "1"}]       # y and t in place
    w("c2", 48, 16); nodes += conv("c2", "k", "u")
    nodes += [{"name": "k2", "op_type": "Concat", "inputs": "[x, u, t, u]", "outputs": "[z]", "axis": "1"}]   # only the first u in place
    return nodes, params


def _nested_concat_graph():
    """Concat results inside Concat results: k1 = (pa, pb), k2 = (k1, pc), z = (k2, pool(k2), pa)."""
    rng = np.random.default_rng(4)
    params = {}
    def conv(name, x, y, c, oc):
        params["w" + name] = (rng.standard_normal((oc, c, 1, 1)) * 0.3).astype(np.float32)
        return {"name": name, "op_type": "Conv", "inputs": f"[{x}, w{name}]", "outputs": f"[{y}]", "strides": "1", "pads": "0"}
    nodes = [conv("a", "x", "pa", 16, 16), conv("b", "x", "pb", 16, 16),
             {"name": "k1", "op_type": "Concat", "inputs": "[pa, pb]", "outputs": "[k1]", "axis": "1"},
             conv("c", "k1", "pc", 32, 16),
             {"name": "k2", "op_type": "Concat", "inputs": "[k1, pc]", "outputs": "[k2]", "axis": "1"},
             {"name": "p", "op_type": "MaxPool", "inputs": "[k2]", "outputs": "[m]", "kernel_shape": "5", "strides": "1", "pads": "2"},
             {"name": "k3", "op_type": "Concat", "inputs": "[k2, m, pa]", "outputs": "[z]", "axis": "1"}]
    return nodes, params


def test_nested_concat_parts_in_place():
    nodes, params = _nested_concat_graph()
    ex = AotExecutor(nodes, params, ["x"], ["z", "k1"], {"x": [1, 16, 8, 8]}, quantize=8)
    assert [(i[0], i[1]) for i in ex.instructions] == [("conv2d_i8", ["x", "wa"]), ("conv2d_i8", ["x", "wb"]), ("conv2d_i8", ["k1", "wc"]),
                                                       ("pool_f32", ["k2"]), ("concat", ["pa"])]
    v = lambda n: ex._values[n].slot
    part = 16 * 64 * 4
    z0 = v("z")[0]
    assert v("k2") == (z0, 3 * part) and v("k1") == (z0, 2 * part) and v("pa") == (z0, part) and v("pb") == (z0 + part, part)
    assert v("pc") == (z0 + 2 * part, part) and v("m") == (z0 + 3 * part, 3 * part) and v("z")[1] == 7 * part
    assert ex._calls[4][2] == (z0 + 6 * part, part)   # the second pa: copied into the last stretch


def test_concat_parts_in_place():
    """Which parts of a one-image Concat get their slot inside its result: values produced by an instruction, the
    value whose Split views are consecutive parts (a C2f block: the views follow it), not the graph input, not a
    value that already lives in another Concat, not a part that comes twice; what is left is copied by a Concat
    over its stretch of the result."""
    nodes, params = _concat_graph()
    ex = AotExecutor(nodes, params, ["x"], ["z"], {"x": [1, 16, 8, 8]}, quantize=8)
    names = [i[0] for i in ex.instructions]
    assert names == ["conv2d_i8", "conv2d_i8", "conv2d_i8", "concat", "concat"], names
    v = lambda n: ex._values[n].slot
    part = 16 * 64 * 4
    assert v("y") == (v("k")[0], 2 * part) and v("a") == (v("k")[0], part) and v("b") == (v("k")[0] + part, part)
    assert v("t") == (v("k")[0] + 2 * part, part)
    assert v("u") == (v("z")[0] + part, part)
    # the two copies: x into the first stretch of z, (t, u) into the last two
    assert ex._calls[3][1] == [v("x")] and ex._calls[3][2] == (v("z")[0], part)
    assert ex._calls[4][1] == [v("t"), v("u")] and ex._calls[4][2] == (v("z")[0] + 2 * part, 2 * part)
    off = AotExecutor(nodes, params, ["x"], ["z"], {"x": [1, 16, 8, 8]}, quantize=8, concat_in_place=False)
    assert [i[0] for i in off.instructions] == ["conv2d_i8", "conv2d_i8", "concat", "conv2d_i8", "concat"]


@pytest.mark.gpu
@pytest.mark.parametrize("quantize", [4, 8, "i4", "i8", "u4", "u8", "f8", "f8r", "f4", "i4cb"])
def test_forward_matches_oracle(orc, quantize):
    from gpu_common import assert_close, to_oracle
    rng = np.random.default_rng(7)
    params = mlp_params(rng)
    ex = AotExecutor(mlp_nodes(), params, ["x"], ["y"], {"x": [5, 64]}, quantize=quantize)
    dt = weight_dtype_of(quantize)
    p1 = to_oracle(orc, fastnn_amd.quantize_weights_kn(dt, params["w1"]))
    p2 = to_oracle(orc, fastnn_amd.quantize_weights_kn(dt, params["w2"]))
    try:
        for it in range(3):
            x = rng.standard_normal((5, 64)).astype(np.float32)
            got = ex.forward({"x": x})["y"]
            h = orc.qmatmul(p1, x, bias=params["b1"], act=flib.ACT_GELU)
            want = orc.qmatmul(p2, h) + x
            assert got.shape == (5, 64)
            assert_close(got, want, 1e-4, f"quantize={quantize} call {it}")
            assert ex.replayed == (it >= 1)
    finally:
        ex.close()


@pytest.mark.gpu
def test_forward_conv_graph(orc):
    from gpu_common import assert_close, to_oracle
    rng = np.random.default_rng(9)
    nodes = [
        {"name": "c1", "op_type": "Conv", "inputs": "[x, w, b]", "outputs": "[c]", "strides": "2", "pads": "1"},
        {"name": "a1", "op_type": "Silu", "inputs": "[c]", "outputs": "[s]"},
        {"name": "p", "op_type": "MaxPool", "inputs": "[s]", "outputs": "[m]", "kernel_shape": "5", "strides": "1", "pads": "2"},
        {"name": "cat", "op_type": "Concat", "inputs": "[s, m]", "outputs": "[k]", "axis": "1"},
        {"name": "up", "op_type": "Resize", "inputs": "[k]", "outputs": "[y]", "mode": "nearest", "scale_h": "2", "scale_w": "2"},
    ]
    w = (rng.standard_normal((8, 3, 3, 3)) * 0.3).astype(np.float32)
    b = (rng.standard_normal(8) * 0.05).astype(np.float32)
    x = rng.uniform(0, 1, (2, 3, 16, 16)).astype(np.float32)
    ex = AotExecutor(nodes, {"w": w, "b": b}, ["x"], ["y"], {"x": list(x.shape)}, quantize=8)
    try:
        got = ex.forward({"x": x})["y"]
        pw = to_oracle(orc, fastnn_amd.quantize_weights(flib.DT_I8, w.reshape(8, 27)))
        s = orc.qconv2d_i8(x, pw, 3, 3, 2, 1, 1, 1, bias=b, act=flib.ACT_SILU)
        want = orc.upsample_nearest2d(np.concatenate([s, orc.maxpool2d(s, 5, 1, 2)], axis=1), 2, 2)
        assert got.shape == want.shape == (2, 16, 16, 16)
        assert_close(got, want, 1e-5, "conv graph")
    finally:
        ex.close()


def test_concat_of_all_split_parts_reads_the_split_source():
    """A batch of two: the parts of a channel Split are copies.  A Concat that joins all of them, in order, reads the
    Split's input instead, and the copy of a part that nothing else reads is not made (reading it says so)."""
    nodes, params = _concat_graph()
    ex = AotExecutor(nodes, params, ["x"], ["z"], {"x": [2, 16, 8, 8]}, quantize=8)
    names = [(i[0], i[1], i[2]) for i in ex.instructions]
    assert names == [("conv2d_i8", ["x", "wc0"], "y"), ("slice_f32", ["y"], "b"), ("conv2d_i8", ["b", "wc1"], "t"),
                     ("concat", ["y", "t"], "k"), ("conv2d_i8", ["k", "wc2"], "u"), ("concat", ["x", "u", "t", "u"], "z")], names
    assert ex.kept("b") and not ex.kept("a")
    with pytest.raises(flib.FnnError):
        ex.read_output("a")
    keep_a = AotExecutor(nodes, params, ["x"], ["z", "a"], {"x": [2, 16, 8, 8]}, quantize=8)
    assert [i[0] for i in keep_a.instructions].count("slice_f32") == 2 and keep_a.kept("a")


@pytest.mark.gpu
def test_forward_with_nested_concat_parts_in_place():
    """Concat results placed inside Concat results: every value equal, bit for bit, to the plan that copies."""
    nodes, params = _nested_concat_graph()
    x = np.random.default_rng(5).uniform(-1, 1, (1, 16, 24, 24)).astype(np.float32)
    outs = ["z", "k2", "k1", "m", "pc", "pb", "pa"]
    got = {}
    for in_place in (True, False):
        ex = AotExecutor(nodes, params, ["x"], outs, {"x": list(x.shape)}, quantize=8, concat_in_place=in_place)
        try:
            ex.forward({"x": x})
            got[in_place] = ex.forward({"x": x})
            assert ex.replayed
        finally:
            ex.close()
    for n in outs:
        assert np.array_equal(got[True][n], got[False][n]), n
    g = got[True]
    assert np.array_equal(g["z"], np.concatenate([g["pa"], g["pb"], g["pc"], g["m"], g["pa"]], axis=1))


@pytest.mark.gpu
@pytest.mark.parametrize("side", [32, 8])
def test_forward_with_concat_parts_in_place(side):
    """The same graph with the parts stored in place and with every Concat copying: every value equal bit for bit.
    The convolution that reads k takes its ranges from the pairs that the producers of k's parts left one after the
    other (no instruction writes k as a whole), on tiles of the 32 x 32 map and on the single tile of the 8 x 8 map."""
    nodes, params = _concat_graph()
    rng = np.random.default_rng(3)
    x = rng.uniform(-1, 1, (1, 16, side, side)).astype(np.float32)
    outs = ["z", "k", "u", "t", "y"]
    got, used = {}, {}
    for in_place in (True, False):
        ex = AotExecutor(nodes, params, ["x"], outs, {"x": list(x.shape)}, quantize=8, concat_in_place=in_place)
        try:
            first = ex.forward({"x": x})
            again = ex.forward({"x": x})
            assert ex.replayed
            for n in outs:
                assert np.array_equal(first[n], again[n]), n
            got[in_place], used[in_place] = again, ex.ranges_used
        finally:
            ex.close()
    for n in outs:
        assert np.array_equal(got[True][n], got[False][n]), n
    assert np.array_equal(got[True]["k"], np.concatenate([got[True]["y"], got[True]["t"]], axis=1))
    assert np.array_equal(got[True]["z"], np.concatenate([x, got[True]["u"], got[True]["t"], got[True]["u"]], axis=1))
    assert used[False] == 1 and used[True] == 1, used
