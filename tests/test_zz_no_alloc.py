"""GPU test of fnn_hip_qmatmul_static, the MatMul entry point that allocates nothing: its workspaces (prepared
activation operands, split-K partial tiles) live in a static array inside the library.  Called through the C ABI
and compared with fnn_hip_qmatmul on the same device inputs (same kernels: bit-identical) and with the oracle
(2e-5 of max|ref|, the MatMul parity bound), on calls in a row that share the array, the later ones smaller."""
import numpy as np
import pytest

import fastnn_amd
from fastnn_amd import lib as flib
from gpu_common import assert_close, to_oracle

pytestmark = pytest.mark.gpu


def _case(ctx, orc, dt, n, k, ms, seed, act, with_bias):
    rng = np.random.default_rng(seed)
    pw = fastnn_amd.quantize_weights(dt, (rng.standard_normal((n, k)) * 0.05).astype(np.float32))
    po = to_oracle(orc, pw)
    h = ctx.register(pw)
    bias = (rng.standard_normal(n) * 0.1).astype(np.float32) if with_bias else None
    dbias = ctx.to_device(bias) if with_bias else None
    try:
        for m in ms:
            a = rng.standard_normal((m, k)).astype(np.float32)
            da = ctx.to_device(a)
            d_ref, d_got = ctx.alloc(m * n * 4), ctx.alloc(m * n * 4)
            # the allocating entry point first: it sizes its own workspaces and builds per-weight side tables
            ctx.qmatmul_dev(h, da.ptr, m, d_ref.ptr, dbias.ptr if dbias else 0, act, 0)
            ctx.sync()
            ref = d_ref.download(np.float32, m * n).reshape(m, n)
            ctx.qmatmul_static(h, da.ptr, m, d_got.ptr, dbias.ptr if dbias else 0, act, 0)
            ctx.sync()
            got = d_got.download(np.float32, m * n).reshape(m, n)
            assert np.array_equal(got, ref), f"dt={dt} M={m}: static entry point differs from fnn_hip_qmatmul"
            want = orc.qmatmul(po, a, bias=bias, act=act)
            assert_close(got, want, 2e-5, f"dt={dt} M={m} vs oracle")
            for d in (da, d_ref, d_got):
                d.free()
    finally:
        ctx.release(h)
        if dbias:
            dbias.free()


def test_static_entry_point_matches_the_allocating_one(orc):
    """Two and more calls in a row on one context share the static array; later calls are smaller than earlier
    ones, so a stale tail of an earlier call's operands or partial tiles would show."""
    with fastnn_amd.HipContext(0) as ctx:
        # I8 with K split four ways: operand region and partial-tile region both in use; then smaller calls
        ctx.set_option(flib.OPT_TILE_SPLIT, 4)
        _case(ctx, orc, flib.DT_I8, 512, 2048, [256, 64, 40, 17], seed=11, act=flib.ACT_NONE, with_bias=False)
        ctx.set_option(flib.OPT_TILE_SPLIT, 0)
        # I4 with bias + SiLU epilogue, ragged M and N
        _case(ctx, orc, flib.DT_I4, 1000, 1024, [200, 33], seed=12, act=flib.ACT_SILU, with_bias=True)
        # FP8, and the one-launch kernels (M <= 16) that use no workspace at all
        _case(ctx, orc, flib.DT_F8, 768, 512, [128, 16, 8, 1], seed=13, act=flib.ACT_GELU, with_bias=True)


def test_static_entry_point_reuses_side_tables_but_never_builds_them(orc):
    """A codebook weight at M >= 5 run through its expanded f16 operand (by option) needs the expansion: built by
    fnn_hip_qmatmul on first use, refused with a message by the static entry point before that, used by it afterwards.
    Decoded inside the kernel (the default at this M: the streaming kernel, on the row-major words as long as their
    tile-major copy does not exist) it needs no side table and works at once, with the bits the other entry point gives."""
    rng = np.random.default_rng(14)
    n, k, m = 256, 512, 48
    pw = fastnn_amd.quantize_weights(flib.DT_I4CB, (rng.laplace(0, 0.02, (n, k))).astype(np.float32))
    a = rng.standard_normal((m, k)).astype(np.float32)
    with fastnn_amd.HipContext(0) as ctx:
        h = ctx.register(pw)
        da, d_ref, d_got = ctx.to_device(a), ctx.alloc(m * n * 4), ctx.alloc(m * n * 4)
        ctx.qmatmul_static(h, da.ptr, m, d_got.ptr)          # decoded in the kernel: nothing to build
        ctx.qmatmul_dev(h, da.ptr, m, d_ref.ptr)
        ctx.sync()
        first = d_got.download(np.float32, m * n).reshape(m, n)
        assert np.array_equal(first, d_ref.download(np.float32, m * n).reshape(m, n))
        assert_close(first, orc.qmatmul(to_oracle(orc, pw), a), 2e-5, "codebook weight decoded in the kernel, static entry point")
        ctx.set_option(flib.OPT_CODEBOOK_EXPANDED, 1)
        with pytest.raises(flib.FnnError) as e:
            ctx.qmatmul_static(h, da.ptr, m, d_got.ptr)
        assert e.value.kind == "Memory" and "fnn_hip_qmatmul_static" in e.value.message
        ctx.qmatmul_dev(h, da.ptr, m, d_ref.ptr)
        ctx.qmatmul_static(h, da.ptr, m, d_got.ptr)
        ctx.sync()
        got = d_got.download(np.float32, m * n).reshape(m, n)
        assert np.array_equal(got, d_ref.download(np.float32, m * n).reshape(m, n))
        assert_close(got, orc.qmatmul(to_oracle(orc, pw), a), 2e-5, "codebook weight through the static entry point")


def test_static_entry_point_refuses_what_does_not_fit(orc):
    """Sizes beyond the static array are refused with a message that names the limit; nothing is launched."""
    rng = np.random.default_rng(15)
    n, k = 128, 4096
    pw = fastnn_amd.quantize_weights(flib.DT_I8, (rng.standard_normal((n, k)) * 0.05).astype(np.float32))
    with fastnn_amd.HipContext(0) as ctx:
        h = ctx.register(pw)
        m = 1024                                   # operands: 2*1024*4096*2 bytes = 16 MiB > 8 MiB
        da, dout = ctx.alloc(m * k * 4), ctx.alloc(m * n * 4)
        with pytest.raises(flib.FnnError) as e:
            ctx.qmatmul_static(h, da.ptr, m, dout.ptr)
        assert e.value.kind == "Memory" and "static buffer holds" in e.value.message
        with pytest.raises(flib.FnnError) as e:
            ctx.qmatmul_static(h, da.ptr, 4097, dout.ptr)
        assert e.value.kind == "Memory" and "4096" in e.value.message
        # the same shape through the allocating entry point works, and so does a fitting static call afterwards
        a = rng.standard_normal((64, k)).astype(np.float32)
        d64, o64 = ctx.to_device(a), ctx.alloc(64 * n * 4)
        ctx.qmatmul_static(h, d64.ptr, 64, o64.ptr)
        ctx.sync()
        assert_close(o64.download(np.float32, 64 * n).reshape(64, n), orc.qmatmul(to_oracle(orc, pw), a), 2e-5, "after refusals")
