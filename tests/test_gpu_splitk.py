"""The k split across workgroups (partial tiles parked in a workspace, a ticket per row-block group, the last
workgroup adds the slices in slice order): bit-for-bit checks at the shapes where it is chosen automatically — the 27B
down projection in the decode kernel and in the 17..64-row streaming kernel — through the C ABI."""
import numpy as np
import pytest

from llm170_amd import gen, ops

pytestmark = pytest.mark.gpu

N, K, G = 5120, 17408, 128  # 27B down projection: 160 workgroups x 136 k tiles, 8 slices of 17 tiles
NKS, KT_SLICE = 8, 17


def say(*a):
    print(*a, flush=True)


def _bits(a):
    return np.ascontiguousarray(a, np.float32).view(np.uint32)


@pytest.fixture(scope="module")
def down():
    d = ops.W4a16Dec()
    q, s, x = gen.make_linear(N, K, G, 64, seed=19)
    d.upload_lin_g("down", q, s, N, K, G, False)
    yield d, q, s, x
    d.cc.close()


def _forward(dec, name, x, t, path):
    cc = dec.cc
    xd, yd = cc.to_device(np.ascontiguousarray(x[:t])), cc.alloc(t * N * 4)
    try:
        dec.lin_forward(name, xd, yd, t, path=path)
        return cc.d2h(yd, (t, N), np.float32)
    finally:
        cc.free(xd)
        cc.free(yd)


@pytest.mark.parametrize("t,path", [(1, ops.PATH_DECODE), (4, ops.PATH_DECODE), (8, ops.PATH_DECODE),
                                    (16, ops.PATH_DECODE), (32, ops.PATH_STREAM), (64, ops.PATH_STREAM)])
def test_split_equals_slice_order_sum_of_slice_launches(down, t, path):
    """The automatically split launch against the sum, taken on the host in slice order in f32, of eight unsplit
    launches that each see one slice of k (the slice's columns of q, s and x as a linear of its own, same waves per
    workgroup): the same partial tiles added in the same order, so every bit agrees."""
    dec, q, s, x = down
    say("split vs slices", t, path)
    got = _forward(dec, "down", x, t, path)
    want = None
    try:
        dec.set_decode_ksplit(-1)
        if path == ops.PATH_DECODE:
            # four waves per workgroup like the split launch; the row blocks per wave (two here, four in the split
            # launch from seven rows on) do not enter a row's arithmetic
            dec.set_decode_shape(32, 4)
        for i in range(NKS):
            lo, hi = i * KT_SLICE, (i + 1) * KT_SLICE
            qi = np.ascontiguousarray(q[:, lo * 16:hi * 16])
            si = np.ascontiguousarray(s[:, lo:hi])
            xi = np.ascontiguousarray(x[:, lo * 128:hi * 128])
            dec.upload_lin_g("slice", qi, si, N, KT_SLICE * 128, G, False)
            xd, yd = dec.cc.to_device(xi[:t]), dec.cc.alloc(t * N * 4)
            dec.lin_forward("slice", xd, yd, t, path=path)
            part = dec.cc.d2h(yd, (t, N), np.float32)
            dec.cc.free(xd)
            dec.cc.free(yd)
            want = part if want is None else (want + part).astype(np.float32)
    finally:
        dec.set_decode_ksplit(0)
        dec.set_decode_shape(0, 0)
    bad = np.argwhere(_bits(got) != _bits(want))
    assert bad.size == 0, "%d outputs differ, first at %s: %r vs %r" % (len(bad), bad[0], got[tuple(bad[0])], want[tuple(bad[0])])
    # and the unsplit launch is a different summation order: the split really happened
    try:
        dec.set_decode_ksplit(-1)
        whole = _forward(dec, "down", x, t, path)
    finally:
        dec.set_decode_ksplit(0)
    assert not np.array_equal(_bits(whole), _bits(got))


@pytest.mark.parametrize("t,path", [(1, ops.PATH_DECODE), (4, ops.PATH_DECODE), (32, ops.PATH_STREAM)])
def test_split_launches_repeat_bit_for_bit_beside_another_stream(down, t, path):
    """A few thousand split launches back to back while a second context keeps the chip streaming another linear on
    its own stream: every result has the bits of the first.  Results are read back in batches of 64 (one output
    buffer per launch of a batch); the check stops at the first mismatch."""
    dec, q, s, x = down
    launches, batch = (3200, 64) if path == ops.PATH_DECODE else (1024, 32)
    other = ops.W4a16Dec()
    try:
        n2, k2 = 34816, 5120
        other.upload_lin_synth("wide", n2, k2, G, 11, 12)
        ox, oy = other.cc.to_device(gen.normal_f16(5, (4, k2))), other.cc.alloc(4 * n2 * 2)
        cc = dec.cc
        xd = cc.to_device(np.ascontiguousarray(x[:t]))
        ys = cc.alloc(batch * t * N * 4)
        first = None
        for b in range(launches // batch):
            for _ in range(batch):  # about as much streaming time as the batch below
                other.lin_forward("wide", ox, oy, 4, out_f16=True, path=ops.PATH_DECODE)
            for i in range(batch):
                dec.lin_forward("down", xd, ys + i * t * N * 4, t, path=path)
            got = cc.d2h(ys, (batch, t * N), np.uint32)
            if first is None:
                first = got[0].copy()
            bad = np.argwhere(got != first[None, :])
            assert bad.size == 0, "launch %d differs from the first at output %d: %#x vs %#x" % (
                b * batch + bad[0][0], bad[0][1], got[tuple(bad[0])], first[bad[0][1]])
            other.cc.sync()
        say("split soak", t, path, launches, "launches identical")
        cc.free(xd)
        cc.free(ys)
    finally:
        other.cc.close()
