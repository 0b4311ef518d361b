"""small_hip_conv2d_u8_noalloc: the uint8 convolution for callers that cannot allocate device memory.  Its filter
pre-pass writes into a static device array instead of an allocated block; results must equal small_hip_conv2d_u8
bit for bit (and the oracle), on two calls in a row that share the array, the second one smaller."""
import ctypes as C

import numpy as np
import pytest

import hip_util as hu
from smallframework_amd import capi, synth
from util import assert_equal_exact

pytestmark = pytest.mark.gpu
CB = 16


@pytest.fixture(scope="module")
def lib():
    return capi.load()


def _oq(q):
    from oracle.binding import quant
    return quant(q.zero, q.multiplier, q.lshift, q.rshift)


def _both(lib, oracle, case, qp, seed):
    batch, kh, kw, s, (pt, pb, pl, pr), Co, Ci, H, W = case
    zi, zf, mul, ls, rs = qp
    x = synth.uniform_u8(seed, batch * Ci * H * W)
    f = synth.uniform_u8(seed + 1, Co * Ci * kh * kw)
    Ho, Wo = oracle.out_hw(kh, kw, s, pt, pb, pl, pr, H, W)
    iq, fq, oq = hu.q(zi), hu.q(zf), hu.q(5, mul, ls, rs)
    dx, df = hu.dev(x), hu.dev(f)
    n = batch * Co * Ho * Wo
    d_new, d_old = hu.dev_empty(n, np.uint8), hu.dev_empty(n, np.uint8)
    args = (batch, kh, kw, s, pt, pb, pl, pr, Co, Ci, H, W)
    print("noalloc case", case, qp, flush=True)
    rc = lib.small_hip_conv2d_u8_noalloc(*args, hu.ptr(dx), hu.qref(iq), hu.ptr(df), hu.qref(fq), hu.ptr(d_new),
                                         hu.qref(oq), hu.stream())
    assert rc == 0, lib.small_hip_last_error()
    got = hu.host(d_new)
    rc = lib.small_hip_conv2d_u8(*args, hu.ptr(dx), hu.qref(iq), hu.ptr(df), hu.qref(fq), hu.ptr(d_old),
                                 hu.qref(oq), hu.stream())
    assert rc == 0, lib.small_hip_last_error()
    assert_equal_exact(got, hu.host(d_old), "noalloc vs small_hip_conv2d_u8 %s" % (case,))
    rco, want = oracle.conv2d_u8(batch, CB, kh, kw, s, pt, pb, pl, pr, Co, Ci, H, W, x, _oq(iq), f, _oq(fq), _oq(oq))
    assert rco == 0
    assert_equal_exact(got, want, "noalloc vs oracle %s" % (case,))
    return got


def test_noalloc_two_calls_in_a_row_second_smaller(lib, oracle):
    qp = (-128, -128, 1518500250, 0, 9)
    big = (2, 3, 3, 1, (1, 1, 1, 1), 64, 64, 16, 16)          # prepared filter: 64*64*9 bytes + table
    small = (3, 3, 3, 2, (0, 1, 0, 1), 32, 16, 12, 12)        # fits inside what the first call left behind
    a = _both(lib, oracle, big, qp, 141)
    b = _both(lib, oracle, small, qp, 151)
    assert len(np.unique(a)) > 50 and len(np.unique(b)) > 50
    # and once more the other way round, with other quantisation parameters and a 1x1 window
    _both(lib, oracle, (1, 1, 1, 2, (0, 0, 0, 0), 32, 16, 8, 8), (100, 156, (1 << 31) - 1, 0, 15), 161)
    _both(lib, oracle, big, (-3, 5, 1234567890, 1, 4), 171)


def test_noalloc_small_channel_stem_and_limits(lib, oracle):
    # 1..3 input channels take the stem kernel: no scratch involved
    _both(lib, oracle, (2, 3, 3, 1, (1, 1, 1, 1), 16, 3, 16, 16), (-128, -128, 1518500250, 0, 9), 181)
    # a filter whose prepared form exceeds the static array is refused before anything runs
    kh = kw = 3
    Co = Ci = 1024
    assert lib.small_hip_conv2d_u8_prepared_filter_bytes(kh, kw, Co, Ci) > (4 << 20)
    fake = hu.dev_empty(1024, np.uint8)
    q = hu.q(0)
    rc = lib.small_hip_conv2d_u8_noalloc(1, kh, kw, 1, 1, 1, 1, 1, Co, Ci, 4, 4, hu.ptr(fake), hu.qref(q), hu.ptr(fake),
                                         hu.qref(q), hu.ptr(hu.dev_empty(1024, np.uint8)), hu.qref(q), hu.stream())
    assert rc == capi.EINVAL
    assert b"static scratch" in lib.small_hip_last_error()


def test_noalloc_under_graph_capture(lib, oracle):
    """The use the entry point exists for: recorded into a HIP graph (capture forbids hipMalloc), replayed several times
    with eager calls on the same array and synchronisations in between, another input every time."""
    import torch
    batch, kh, kw, s, (pt, pb, pl, pr), Co, Ci, H, W = 2, 3, 3, 1, (1, 1, 1, 1), 48, 32, 14, 14
    args = (batch, kh, kw, s, pt, pb, pl, pr, Co, Ci, H, W)
    iq, fq, oq = hu.q(-120), hu.q(-131), hu.q(5, 1518500250, 0, 8)
    f = synth.uniform_u8(7, Co * Ci * kh * kw)
    df = hu.dev(f)
    dx = hu.dev(synth.uniform_u8(8, batch * Ci * H * W))
    n = batch * Co * H * W
    d_graph, d_eager = hu.dev_empty(n, np.uint8), hu.dev_empty(n, np.uint8)

    def call(dst):
        rc = lib.small_hip_conv2d_u8_noalloc(*args, hu.ptr(dx), hu.qref(iq), hu.ptr(df), hu.qref(fq), hu.ptr(dst), hu.qref(oq),
                                             hu.stream())
        assert rc == 0, lib.small_hip_last_error()

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        call(d_graph)                        # module loading and the symbol lookup happen outside the capture
    torch.cuda.synchronize()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g, stream=side):
        call(d_graph)
    for rep in range(3):
        x = synth.uniform_u8(20 + rep, batch * Ci * H * W)
        dx.copy_(torch.from_numpy(x))
        d_graph.zero_()
        torch.cuda.synchronize()
        g.replay()
        torch.cuda.synchronize()
        got = hu.host(d_graph)
        call(d_eager)                        # an eager call re-writes the shared array between the replays
        assert_equal_exact(got, hu.host(d_eager), "graph replay %d vs eager" % rep)
        rco, want = oracle.conv2d_u8(batch, CB, kh, kw, s, pt, pb, pl, pr, Co, Ci, H, W, x, _oq(iq), f, _oq(fq), _oq(oq))
        assert rco == 0
        assert_equal_exact(got, want, "graph replay %d vs oracle" % rep)
        assert len(np.unique(want)) > 20


def test_noalloc_two_streams_share_the_array(lib, oracle):
    """Calls issued in turn on two streams (another filter each time, nothing waited for in between) are ordered by the
    library on the device: every result equals the oracle's."""
    import torch
    s1, s2 = torch.cuda.Stream(), torch.cuda.Stream()
    batch, kh, kw, s, (pt, pb, pl, pr), Co, Ci, H, W = 2, 3, 3, 1, (1, 1, 1, 1), 64, 64, 20, 20
    args = (batch, kh, kw, s, pt, pb, pl, pr, Co, Ci, H, W)
    iq, fq, oq = hu.q(-120), hu.q(-131), hu.q(5, 1518500250, 0, 9)
    x = synth.uniform_u8(31, batch * Ci * H * W)
    dx = hu.dev(x)
    n = batch * Co * H * W
    jobs = []
    torch.cuda.synchronize()
    for i in range(8):
        f = synth.uniform_u8(40 + i, Co * Ci * kh * kw)
        df, dout = hu.dev(f), hu.dev_empty(n, np.uint8)
        jobs.append((f, df, dout))
    torch.cuda.synchronize()
    for i, (f, df, dout) in enumerate(jobs):
        st = (s1, s2)[i & 1]
        rc = lib.small_hip_conv2d_u8_noalloc(*args, hu.ptr(dx), hu.qref(iq), hu.ptr(df), hu.qref(fq), hu.ptr(dout), hu.qref(oq),
                                             C.c_void_p(st.cuda_stream))
        assert rc == 0, lib.small_hip_last_error()
    torch.cuda.synchronize()
    for i, (f, df, dout) in enumerate(jobs):
        rco, want = oracle.conv2d_u8(batch, CB, kh, kw, s, pt, pb, pl, pr, Co, Ci, H, W, x, _oq(iq), f, _oq(fq), _oq(oq))
        assert rco == 0
        assert_equal_exact(hu.host(dout), want, "call %d on stream %d" % (i, i & 1))
