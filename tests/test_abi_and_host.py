"""CPU-only checks of the product: the C-ABI library loads and exports every symbol the
public header declares, and the host-side weight packers are bit-identical to the oracle."""
import ctypes
import os
import re

import numpy as np
import pytest

import fastnn_amd
from fastnn_amd import lib as flib

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_library_exports_every_declared_symbol():
    l = fastnn_amd.load_library()
    header = open(os.path.join(ROOT, "include", "fastnn_hip.h")).read()
    declared = set(re.findall(r"\b(fnn_[a-z0-9_]+)\s*\(", header))
    declared -= {"fnn_status", "fnn_dtype", "fnn_act"}
    assert declared, "no declarations parsed"
    for name in sorted(declared):
        assert hasattr(l, name), f"{name} declared in fastnn_hip.h but not exported"
    assert declared == set(flib.EXPORTED_SYMBOLS)
    assert b"gfx950" in l.fnn_hip_version()


def test_backend_header_symbols_exported():
    path = os.path.join(ROOT, "include", "fastnn_hip_backend.h")
    l = fastnn_amd.load_library()
    declared = set(re.findall(r"\b(fnn_[a-z0-9_]+)\s*\(", open(path).read()))
    assert len(declared) >= 16
    for name in sorted(declared):
        assert hasattr(l, name), f"{name} declared in fastnn_hip_backend.h but not exported"
    assert declared == set(flib.BACKEND_SYMBOLS)


def test_rust_glue_binds_only_declared_functions():
    """integration/ffi.rs (the bindings a fastnn maintainer would add) names no function the headers do not declare,
    and gives each the number of arguments its declaration has."""
    def c_decls(text):
        out = {}
        for name, args in re.findall(r"\b(fnn_[a-z0-9_]+)\s*\(([^;{]*?)\)\s*;", text, re.S):
            args = args.strip()
            out[name] = 0 if args in ("", "void") else args.count(",") + 1
        return out
    headers = {}
    for h in ("fastnn_hip.h", "fastnn_hip_backend.h"):
        headers.update(c_decls(open(os.path.join(ROOT, "include", h)).read()))
    rust = re.sub(r"//[^\n]*", "", open(os.path.join(ROOT, "integration", "ffi.rs")).read())
    bound = re.findall(r"\bfn\s+(fnn_[a-z0-9_]+)\s*\(([^)]*)\)", rust, re.S)
    assert len(bound) >= 20
    for name, args in bound:
        assert name in headers, f"ffi.rs binds {name}, which no header declares"
        n_args = len([a for a in args.split(",") if a.strip()])
        assert n_args == headers[name], f"{name}: {n_args} arguments in ffi.rs, {headers[name]} in the header"


def test_plan_builds_without_a_gpu():
    """Plans are host objects: building one needs no device; malformed instructions are refused."""
    from fastnn_amd.backend import ExecutablePlan
    p = ExecutablePlan(4096)
    p.write_const(0, np.arange(16, dtype=np.float32)).fill(64, 64, 1.5).memcopy((128, 64), (0, 64))
    p.call_kernel("matmul_i8_relu", [(0, 64), (256, 64)], (512, 64), [1, 16, 16],
                  dict(bit_width=8, scales=[1.0], zero_points=[0.0], shape=[16, 16]))
    assert len(p) == 4
    l = fastnn_amd.load_library()
    assert l.fnn_plan_add_call_kernel(p.handle, None, None, 0, flib.Slice(0, 0), None, None, 0, None) != 0
    assert b"NULL argument" in l.fnn_backend_last_error(None)
    # CallKernel.secondary_output_slice and a meta with several codebooks (the kernels read codebooks[0])
    p.call_kernel("pool_f32", [(0, 64)], (512, 64), [2, 2, 0, 1, 1, 1, 4, 4], secondary_output=(1024, 128))
    p.call_kernel("matmul_i4", [(0, 64), (256, 64)], (512, 64), [1, 32, 4],
                  dict(bit_width=4, scales=[1.0] * 4, zero_points=[], shape=[4, 32], quant_block_size=32,
                       codebooks=np.zeros((2, 16), np.float32)))
    assert len(p) == 6
    p.close()


def test_entry_points_refuse_null_handles_with_a_message():
    """No entry point dereferences a NULL handle: each returns a status and leaves a message."""
    l = fastnn_amd.load_library()
    assert l.fnn_hip_set_option(None, flib.OPT_TILE_SPLIT, 2) == 1
    assert b"NULL context" in l.fnn_hip_last_error(None)
    assert l.fnn_hip_sync(None) == 1
    assert l.fnn_backend_set_graph_replay(None, 0) == 1
    assert l.fnn_backend_dispatch(None, None) == 1
    assert l.fnn_hip_stream(None) is None


def test_backend_create_without_gpu_reports_an_error():
    l = fastnn_amd.load_library()
    if l.fnn_hip_device_count() > 0:
        pytest.skip("a GPU is present")
    from fastnn_amd.backend import HipBackend
    with pytest.raises(flib.FnnError):
        HipBackend(0)


def test_missing_library_fails_loudly(tmp_path):
    with pytest.raises(FileNotFoundError):
        flib.load_library(str(tmp_path / "nope.so"))


def test_no_product_file_touches_the_oracle():
    """The shipped package must not import, link or call anything under oracle/."""
    pkg = os.path.join(ROOT, "fastnn_amd")
    for dirpath, _, files in os.walk(pkg):
        if os.path.basename(dirpath) == "build":
            continue
        for f in files:
            if f.endswith((".py", ".cpp", ".hip", ".h")):
                text = open(os.path.join(dirpath, f)).read()
                assert "fnn_oracle" not in text and "import oracle" not in text and "from oracle" not in text, f


DTS = [flib.DT_I8, flib.DT_I4, flib.DT_U8, flib.DT_U4, flib.DT_F8, flib.DT_F8R, flib.DT_F4, flib.DT_I4CB]


@pytest.mark.parametrize("dt", DTS)
@pytest.mark.parametrize("shape", [(16, 64), (7, 37), (3, 5), (64, 512)])
def test_host_packers_bit_identical_to_oracle(orc, dt, shape):
    rng = np.random.default_rng(1000 + dt)
    w = (rng.standard_normal(shape) * 0.02).astype(np.float32)
    mask = rng.random(shape) < 0.01
    w[mask] *= 8
    if shape[0] > 2:
        w[1] = 0.0            # all-zero row
        w[2] = 0.015          # constant row (zero range)
    pw = fastnn_amd.quantize_weights(dt, w)
    po = orc.quantize(dt, w)
    assert np.array_equal(pw.words, po.words)
    assert pw.scales.tobytes() == po.scales.tobytes()
    assert pw.zeros.tobytes() == po.zeros.tobytes()
    if dt == flib.DT_I4CB:
        assert pw.codebook.tobytes() == po.codebook.tobytes()
        assert pw.qblock == 32


def test_host_packers_special_values(orc):
    vals = np.array([[0.0, -0.0, 1e-9, -1e-9, 300.0, -300.0, 0.0146, 0.0147, 0.99999994, 1.0000001,
                      239.9, 240.1, 2.0 ** -9, 2.0 ** -10, 1.5 * 2.0 ** -9, 57344.0, 65536.0, 3e-5, 1.6e-5, 447.0]],
                    np.float32)
    for dt in (flib.DT_F8, flib.DT_F8R, flib.DT_F4, flib.DT_I8, flib.DT_I4):
        pw = fastnn_amd.quantize_weights(dt, vals)
        po = orc.quantize(dt, vals)
        assert np.array_equal(pw.words, po.words), dt
        assert pw.scales.tobytes() == po.scales.tobytes()
    # direct lane encoders through a unit-scale row: scale == 1 when max|row| == MAX_REPRESENTABLE
    row = np.concatenate([vals[0][np.abs(vals[0]) <= 240], [240.0]]).astype(np.float32)[None, :]
    pw = fastnn_amd.quantize_weights(flib.DT_F8, row)
    po = orc.quantize(orc.F8, row)
    assert pw.scales[0] == 1.0 and np.array_equal(pw.words, po.words)


def test_codebook_packer_large_matches_oracle(orc):
    rng = np.random.default_rng(5)
    w = np.where(rng.random((96, 256)) < 0.9, rng.laplace(0, 0.02, (96, 256)), rng.laplace(0, 0.1, (96, 256)))
    w = w.astype(np.float32)
    pw = fastnn_amd.quantize_weights(flib.DT_I4CB, w)
    po = orc.quantize(orc.I4CB, w)
    assert np.array_equal(pw.words, po.words)
    assert pw.codebook.tobytes() == po.codebook.tobytes()
    assert pw.scales.tobytes() == po.scales.tobytes()
    with pytest.raises(fastnn_amd.FnnError):
        bad = w.copy()
        bad[0, 0] = np.nan
        fastnn_amd.quantize_weights(flib.DT_I4CB, bad)


def test_transpose_kn(orc):
    rng = np.random.default_rng(6)
    w = rng.standard_normal((70, 45)).astype(np.float32)
    pw = fastnn_amd.quantize_weights_kn(flib.DT_I8, w)
    po = orc.quantize_kn(orc.I8, w)
    assert pw.rows == 45 and pw.inner == 70
    assert np.array_equal(pw.words, po.words)
