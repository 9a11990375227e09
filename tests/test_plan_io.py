"""ExecutablePlan::load / save: the bincode reader and writer of the host-side backend, checked on the CPU against a
byte image assembled by hand from the reference's serde layout (tests/golden/executable_plan.bin, listing in
executable_plan.txt, generator make_plan_fixture.py).  No file written by fastnn itself exists here (no Rust toolchain),
so agreement with a real saved plan is unpinned; what is pinned is the layout rules of bincode 1.3 applied to the
struct definitions, field by field."""
import os
import struct

import numpy as np
import pytest

from fastnn_amd import lib as flib
from fastnn_amd.backend import ExecutablePlan

HERE = os.path.dirname(os.path.abspath(__file__))
FIXTURE = os.path.join(HERE, "golden", "executable_plan.bin")


def test_fixture_loads_field_by_field():
    plan = ExecutablePlan.load(FIXTURE)
    assert len(plan) == 8 and plan.arena_size == 1280
    assert plan.describe(0) == {"op": "WriteConst", "dst": [128, 32], "len": 32}
    assert plan.describe(1) == {"op": "WriteConst", "dst": [192, 16], "len": 16}
    assert plan.describe(2) == {"op": "Fill", "dst": [256, 32], "value": 0.5}
    d = plan.describe(3)
    assert d["kernel"] == "matmul_i8_relu" and d["inputs"] == [[0, 64], [128, 32], [192, 16]] and d["output"] == [256, 32]
    assert d["secondary"] is None and d["params"] == [2, 8, 4] and d["node_id"] == 7
    assert d["param_dims"] == ["B", 8, 4]
    assert d["meta"] == {"bit_width": 8, "n_scales": 4, "n_zero_points": 4, "shape": [4, 8], "quant_block_size": 0, "n_codebooks": 0}
    assert plan.describe(4) == {"op": "MemCopy", "dst": [320, 32], "src": [256, 32]}
    d = plan.describe(5)
    assert d["kernel"] == "pool_f32" and d["secondary"] == [392, 16] and d["params"] == [2, 2, 0, 1, 1, 2, 2, 2]
    assert d["node_id"] is None and d["param_dims"] is None and d["meta"] is None
    d = plan.describe(7)
    assert d["kernel"] == "matmul_i4" and d["param_dims"] == [{"sym": "B", "max": 4}, 32, 2]
    assert d["meta"] == {"bit_width": 4, "n_scales": 2, "n_zero_points": 0, "shape": [2, 32], "quant_block_size": 32, "n_codebooks": 1}
    plan.close()


def test_save_reproduces_the_loaded_bytes():
    data = open(FIXTURE, "rb").read()
    plan = ExecutablePlan.load(data)
    assert plan.to_bytes() == data
    plan.close()


def test_a_built_plan_survives_save_and_load():
    p = ExecutablePlan(4096)
    p.write_const(0, np.arange(16, dtype=np.float32)).fill(64, 64, -2.5).memcopy((128, 64), (0, 64))
    p.call_kernel("matmul_f8_gelu", [(0, 64), (256, 64), (512, 16)], (1024, 64), [1, 16, 16],
                  dict(bit_width=8, scales=[1.0, 2.0], zero_points=[0.0, 0.0], shape=[16, 16]))
    p.call_kernel("pool_f32", [(0, 64)], (512, 64), [2, 2, 0, 1, 1, 1, 4, 4], secondary_output=(1024, 128))
    p.set_param_dims(3, ["N", ("T", 16), 16])
    q = ExecutablePlan.load(p.to_bytes())
    assert len(q) == len(p) == 5 and q.arena_size == 4096
    for i in range(5):
        assert q.describe(i) == p.describe(i)
    assert q.to_bytes() == p.to_bytes()
    p.close(); q.close()


def test_malformed_images_are_refused_with_the_offset():
    data = open(FIXTURE, "rb").read()
    for bad, what in ((data[:-1], "truncated"), (data[:200], "truncated"), (data + b"\0", "trailing"),
                      (data[:8] + struct.pack("<I", 9) + data[12:], "unknown Instruction variant"),
                      (struct.pack("<Q", 1 << 60) + data[8:], "truncated"), (b"", "truncated")):
        with pytest.raises(flib.FnnError) as e:
            ExecutablePlan.load(bad)
        assert e.value.kind == "Compilation" and what in e.value.message, e.value.message
    # an Option tag other than 0 / 1
    i = data.index(b"matmul_i8_relu") + 14 + 8 + 3 * 16 + 16
    with pytest.raises(flib.FnnError) as e:
        ExecutablePlan.load(data[:i] + b"\x02" + data[i + 1:])
    assert "Option tag" in e.value.message
