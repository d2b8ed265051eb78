"""One decode launch over fused linears with one output per part (w4a16_lin_forward_multi), the role of the reference's
multi-linear GEMV (w4a16_dec/kernels/gemv.rs:189-332 over the segment table of w4a16_dec/buffers.rs:229-366).

Checked against the same fused linear's single-output launch at the same launch plan (two row blocks per wave, which
the kernels with one output per part are built for), so that every part must carry the bits of its columns; against the
CPU oracle part by part; and for stray writes (guard words around every output)."""
import numpy as np
import pytest

from llm170_amd import gen, ops, parity

pytestmark = pytest.mark.gpu

GUARD = 64  # elements in front of and behind every output that must keep their fill


def say(*a):
    print("multi", *a, flush=True)


def _upload_parts(dec, parts, k, group, bf):
    ops_ = {}
    for i, (name, n) in enumerate(parts):
        q, s, _ = gen.make_linear(n, k, group, 1, seed=100 + i)
        if bf:
            s = (gen.f16_bits_to_f32(s).view(np.uint32) >> 16).astype(np.uint16)
        dec.upload_lin_g(name, q, s, n, k, group, bf)
        ops_[name] = (q, s)
    return ops_


@pytest.mark.parametrize("group,bf", [(128, False), (32, True)])
@pytest.mark.parametrize("t", [1, 3, 4, 8, 16])
@pytest.mark.parametrize("out_f16", [False, True])
def test_multi_outputs_carry_the_fused_launch_bits(orc, group, bf, t, out_f16):
    say("bits", group, bf, t, out_f16)
    dec = ops.W4a16Dec()
    cc = dec.cc
    try:
        k = 512
        parts = [("q", 320), ("k", 64), ("v", 64), ("g", 160)]
        held = _upload_parts(dec, parts, k, group, bf)
        dec.lin_fuse("qkvg", [p for p, _ in parts])
        n = sum(n_ for _, n_ in parts)
        x = gen.normal_f16(900 + t, (t, k))
        px = cc.to_device(x)
        esz, dt = (2, np.uint16) if out_f16 else (4, np.uint32)
        py = cc.alloc(t * n * esz)
        dec.set_decode_shape(32, 0)  # the single-output launch at the plan of the launch under test
        dec.lin_forward("qkvg", px, py, t, out_f16=out_f16, path=ops.PATH_DECODE)
        whole = cc.d2h(py, (t, n), dt)
        fill = 0x5A5A if out_f16 else 0x5A5A5A5A
        bufs = []
        for _, n_ in parts:
            host = np.full(t * n_ + 2 * GUARD, fill, dt)
            bufs.append(cc.to_device(host))
        dec.lin_forward_multi("qkvg", px, [b + GUARD * esz for b in bufs], t, out_f16=out_f16)
        first = 0
        for (name, n_), b in zip(parts, bufs):
            got = cc.d2h(b, (t * n_ + 2 * GUARD,), dt)
            assert np.all(got[:GUARD] == fill) and np.all(got[-GUARD:] == fill), (name, "guard words were written")
            body = got[GUARD:-GUARD].reshape(t, n_)
            assert np.array_equal(body, whole[:, first:first + n_]), (name, "differs from the fused launch's columns")
            q, s = held[name]
            ref = orc.gemm_lane(x, t, q, s, n_, k, group, scale_bf16=bf, threads=4)
            val = gen.f16_bits_to_f32(body) if out_f16 else body.view(np.float32)
            parity.assert_close(val, ref, "multi part " + name)
            first += n_
        for p in [px, py] + bufs:
            cc.free(p)
    finally:
        cc.close()


def test_multi_split_k_shape(orc):
    """A launch split over k across workgroups: the wave that draws the last ticket writes the parts' outputs."""
    say("split k")
    dec = ops.W4a16Dec()
    cc = dec.cc
    try:
        k, t = 4096, 4
        parts = [("a", 128), ("b", 256)]
        held = _upload_parts(dec, parts, k, 128, False)
        dec.lin_fuse("ab", ["a", "b"])
        dec.set_decode_ksplit(4)  # four k slices across workgroups, for both launches
        dec.set_decode_shape(32, 0)
        x = gen.normal_f16(5, (t, k))
        px = cc.to_device(x)
        py = cc.alloc(t * 384 * 4)
        dec.lin_forward("ab", px, py, t, path=ops.PATH_DECODE)
        whole = cc.d2h(py, (t, 384), np.uint32)
        pa, pb = cc.alloc(t * 128 * 4), cc.alloc(t * 256 * 4)
        for rep in range(2):  # the tickets are left at zero: the second launch must give the same bits
            dec.lin_forward_multi("ab", px, [pa, pb], t)
            assert np.array_equal(cc.d2h(pa, (t, 128), np.uint32), whole[:, :128])
            assert np.array_equal(cc.d2h(pb, (t, 256), np.uint32), whole[:, 128:])
        parity.assert_close(cc.d2h(pb, (t, 256), np.float32),
                            orc.gemm_lane(x, t, held["b"][0], held["b"][1], 256, k, 128, threads=4), "multi split-k b")
        for p in (px, py, pa, pb):
            cc.free(p)
    finally:
        cc.close()


def test_multi_contract():
    say("contract")
    dec = ops.W4a16Dec()
    cc = dec.cc
    try:
        k = 256
        _upload_parts(dec, [("a", 32), ("b", 48), ("c", 40), ("d", 16), ("e", 16), ("f", 16)], k, 128, False)
        dec.lin_fuse("ab", ["a", "b"])
        dec.lin_fuse("ac", ["a", "c"])            # 40 rows: not whole 16-row blocks
        dec.lin_fuse("five", ["a", "b", "d", "e", "f"])
        px = cc.to_device(gen.normal_f16(1, (32, k)))
        outs = [cc.alloc(32 * 64 * 4) for _ in range(5)]
        dec.lin_forward_multi("ab", px, outs[:2], 16)
        with pytest.raises(ops.W4a16Error):
            dec.lin_forward_multi("a", px, outs[:1], 1)        # not a fused linear
        with pytest.raises(ops.W4a16Error):
            dec.lin_forward_multi("ab", px, outs[:3], 1)       # three outputs for two parts
        with pytest.raises(ops.W4a16Error):
            dec.lin_forward_multi("ab", px, [outs[0], 0], 1)   # a null output
        with pytest.raises(ops.W4a16Error):
            dec.lin_forward_multi("ab", px, outs[:2], 0)
        with pytest.raises(ops.W4a16Error) as e:
            dec.lin_forward_multi("ab", px, outs[:2], 17)      # beyond the decode regime
        assert e.value.code == ops.ffi.ERR_UNSUPPORTED
        with pytest.raises(ops.W4a16Error) as e:
            dec.lin_forward_multi("ac", px, outs[:2], 1)
        assert e.value.code == ops.ffi.ERR_SHAPE
        with pytest.raises(ops.W4a16Error) as e:
            dec.lin_forward_multi("five", px, outs, 1)
        assert e.value.code == ops.ffi.ERR_UNSUPPORTED
        for p in [px] + outs:
            cc.free(p)
    finally:
        cc.close()
