"""The allocation-free entry point (w4a16_lin_forward_noalloc) against w4a16_lin_forward on the decode path, through
the C ABI: same bits on two calls in a row, the second on a smaller input, with the split over k across workgroups
(the part that uses the fixed device scratch) active in both; sizes beyond the fixed scratch are refused."""
import numpy as np
import pytest

from llm170_amd import ffi, gen, ops

pytestmark = pytest.mark.gpu


def _forward(dec, fn, name, x, t, n, out_f16=False):
    cc = dec.cc
    xd, yd = cc.to_device(np.ascontiguousarray(x[:t])), cc.alloc(t * n * (2 if out_f16 else 4))
    try:
        cc.memset0(yd, t * n * (2 if out_f16 else 4))
        fn(name, xd, yd, t, out_f16)
        return cc.d2h(yd, (t, n), np.uint16 if out_f16 else np.uint32)
    finally:
        cc.free(xd)
        cc.free(yd)


def test_noalloc_entry_point_equals_lin_forward_two_calls_second_smaller():
    dec = ops.W4a16Dec()
    try:
        cc = dec.cc
        big = (5120, 17408)   # 27B down projection: split into 8 k slices automatically (2.5 MiB of partial tiles)
        small = (208, 2560)   # 13 row blocks, 20 k tiles: split forced below
        qb, sb, xb = gen.make_linear(big[0], big[1], 128, 4, seed=41)
        qs, ss, xs = gen.make_linear(small[0], small[1], 128, 16, seed=42)
        dec.upload_lin_g("big", qb, sb, big[0], big[1], 128, False)
        dec.upload_lin_g("small", qs, ss, small[0], small[1], 128, False)
        ref = lambda name, xd, yd, t, f16: dec.lin_forward(name, xd, yd, t, out_f16=f16, path=ops.PATH_DECODE)
        new = lambda name, xd, yd, t, f16: dec.lin_forward_noalloc(name, xd, yd, t, out_f16=f16)
        want_big = _forward(dec, ref, "big", xb, 4, big[0])
        dec.set_decode_ksplit(5)
        want_small = _forward(dec, ref, "small", xs, 1, small[0])
        want_small16 = _forward(dec, ref, "small", xs, 16, small[0], out_f16=True)
        dec.set_decode_ksplit(0)
        before = cc.allocated_bytes()
        # two calls in a row on the same stream, the second on the smaller input
        xd1, yd1 = cc.to_device(xb[:4]), cc.alloc(4 * big[0] * 4)
        xd2, yd2 = cc.to_device(xs[:1]), cc.alloc(1 * small[0] * 4)
        held = cc.allocated_bytes()
        dec.lin_forward_noalloc("big", xd1, yd1, 4)
        dec.set_decode_ksplit(5)
        dec.lin_forward_noalloc("small", xd2, yd2, 1)
        dec.set_decode_ksplit(0)
        assert cc.allocated_bytes() == held  # the context allocated nothing for them
        got_big, got_small = cc.d2h(yd1, (4, big[0]), np.uint32), cc.d2h(yd2, (1, small[0]), np.uint32)
        for p in (xd1, yd1, xd2, yd2):
            cc.free(p)
        assert cc.allocated_bytes() == before
        assert np.array_equal(got_big, want_big)
        assert np.array_equal(got_small, want_small)
        # again in the other order, and an f16 output with 16 rows
        dec.set_decode_ksplit(5)
        assert np.array_equal(_forward(dec, new, "small", xs, 16, small[0], out_f16=True), want_small16)
        dec.set_decode_ksplit(0)
        assert np.array_equal(_forward(dec, new, "big", xb, 4, big[0]), want_big)
        # an unsplit launch needs no scratch at all
        dec.set_decode_ksplit(-1)
        assert np.array_equal(_forward(dec, new, "small", xs, 3, small[0]), _forward(dec, ref, "small", xs, 3, small[0]))
        dec.set_decode_ksplit(0)
        # limits: prefill-sized t, a split that needs more than the fixed scratch, an unknown name
        xd, yd = cc.to_device(xs), cc.alloc(17 * small[0] * 4)
        with pytest.raises(ops.W4a16Error) as e:
            dec.lin_forward_noalloc("small", xd, yd, 17)
        assert e.value.code == ffi.ERR_SHAPE
        with pytest.raises(ops.W4a16Error) as e:
            dec.lin_forward_noalloc("absent", xd, yd, 1)
        assert e.value.code == ffi.ERR_NOT_FOUND
        cc.free(xd)
        cc.free(yd)
        limit = cc.lib.w4a16_noalloc_workspace_bytes()
        n_wide, k_wide = 34816, 1024  # 2176 row blocks x 8 slices x 1 KiB = 17 MiB of partial tiles
        dec.upload_lin_synth("wide", n_wide, k_wide, 128, 5, 6)
        assert (n_wide // 16) * 1024 * 4 > limit
        xd, yd = cc.to_device(gen.normal_f16(1, (1, k_wide))), cc.alloc(n_wide * 4)
        dec.set_decode_ksplit(4)
        try:
            with pytest.raises(ops.W4a16Error) as e:
                dec.lin_forward_noalloc("wide", xd, yd, 1)
            assert e.value.code == ffi.ERR_SHAPE and str(limit) in str(e.value)
            dec.lin_forward("wide", xd, yd, 1, path=ops.PATH_DECODE)  # the allocating entry point serves it
        finally:
            dec.set_decode_ksplit(0)
        cc.free(xd)
        cc.free(yd)
    finally:
        dec.cc.close()


def test_noalloc_scratch_has_one_owner_per_gpu():
    """The fixed scratch of a GPU serves one context at a time: two contexts sharing its tickets could sum each other's
    partial tiles.  The second context is refused until the first is destroyed."""
    a, b = ops.W4a16Dec(), ops.W4a16Dec()
    try:
        q, s, x = gen.make_linear(208, 2560, 128, 2, seed=43)
        outs = []
        for d in (a, b):
            d.upload_lin_g("lin", q, s, 208, 2560, 128, False)
            d.set_decode_ksplit(4)
        xa, ya = a.cc.to_device(x), a.cc.alloc(2 * 208 * 4)
        xb, yb = b.cc.to_device(x), b.cc.alloc(2 * 208 * 4)
        a.lin_forward_noalloc("lin", xa, ya, 2)
        want = a.cc.d2h(ya, (2, 208), np.uint32)
        with pytest.raises(ops.W4a16Error) as e:
            b.lin_forward_noalloc("lin", xb, yb, 2)
        assert e.value.code == ffi.ERR_ARG and "another context" in str(e.value)
        b.lin_forward("lin", xb, yb, 2, path=ops.PATH_DECODE)  # the allocating entry point is per context and works
        assert np.array_equal(b.cc.d2h(yb, (2, 208), np.uint32), want)
        a.cc.close()
        a = None
        b.lin_forward_noalloc("lin", xb, yb, 2)  # the owner is gone: the array is free again
        assert np.array_equal(b.cc.d2h(yb, (2, 208), np.uint32), want)
    finally:
        if a is not None:
            a.cc.close()
        b.cc.close()
