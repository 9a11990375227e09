"""Helpers shared by the GPU parity tests."""
import numpy as np

import fastnn_amd
from fastnn_amd import lib as flib

NAMES = {0: "i8", 1: "i4", 2: "u8", 3: "u4", 4: "f8", 5: "f8r", 6: "f4", 7: "i4cb"}


def to_oracle(orc, pw):
    """The same packed weight as the oracle's container (shares the arrays)."""
    return orc.Packed(pw.dtype, pw.rows, pw.inner, pw.words, pw.scales, pw.zeros, pw.qblock, pw.codebook)


def slice_rows(pw, rows):
    """Packed weight restricted to a set of output rows (rows are independent)."""
    items = 32 // pw.bit_width
    kp = -(-pw.inner // items)
    words = np.concatenate([pw.words[: pw.rows * kp].reshape(pw.rows, kp)[rows].reshape(-1),
                            np.zeros(16, np.uint32)])
    if pw.dtype == flib.DT_I4CB:
        bpr = -(-pw.inner // pw.qblock)
        scales = pw.scales.reshape(pw.rows, bpr)[rows].reshape(-1).copy()
        zeros = pw.zeros
    else:
        scales, zeros = pw.scales[rows].copy(), pw.zeros[rows].copy()
    return fastnn_amd.PackedWeight(pw.dtype, len(rows), pw.inner, words, scales, zeros, pw.qblock, pw.codebook)


def rel_err(got, want):
    """max|got-want| / max|want| over the tensor (the stated float tolerance is on this)."""
    got = np.asarray(got, np.float64)
    want = np.asarray(want, np.float64)
    return float(np.abs(got - want).max() / (np.abs(want).max() + 1e-30))


def assert_close(got, want, tol, what=""):
    """Element-wise |d| <= tol*|ref| + tol*max|ref| and tensor-wise max|d|/max|ref| <= tol."""
    got = np.asarray(got, np.float64)
    want = np.asarray(want, np.float64)
    assert got.shape == want.shape, (got.shape, want.shape)
    assert np.all(np.isfinite(got)), f"{what}: non-finite output"
    mx = np.abs(want).max() + 1e-30
    d = np.abs(got - want)
    assert np.all(d <= tol * np.abs(want) + tol * mx), f"{what}: max rel {d.max() / mx:.3e} > {tol}"
