"""GPU parity of the on-device pack_buffer / unpack_buffer (small_hip_pack / small_hip_unpack)
against the CPU oracle's index walk, which the CPU suite pins against the reference build.
Pure data movement: every comparison is bit-exact.  Also the round trip at the benchmark's
full activation sizes (a size-independent property: unpack(pack(x)) == x, and pack is a permutation).
"""
import numpy as np
import pytest

from smallframework_amd import capi, layout, synth
from util import assert_equal_exact
import hip_util as hu

pytestmark = pytest.mark.gpu

INPUT, OUTPUT, FILTER_DW, FILTER_CONV, FILTER_FC = range(5)


@pytest.fixture(scope="module")
def lib():
    import torch
    assert torch.cuda.is_available(), "GPU tests need a GPU"
    return capi.load()


CASES = [
    # (type, d0, d1, d2, d3, cib, cob)
    (INPUT, 1, 3, 32, 32, 16, 16),        # first layer: the channel count is the block
    (INPUT, 1, 1, 49, 10, 16, 16),
    (INPUT, 1, 2, 5, 7, 16, 16),
    (INPUT, 1, 2, 8, 8, 16, 16),          # 2 / 3 channels with whole 16-byte pixel groups: vector kernel
    (INPUT, 2, 3, 16, 20, 16, 16),
    (INPUT, 1, 16, 1, 1, 16, 16),
    (INPUT, 1, 64, 13, 17, 16, 16),       # register transpose, ragged pixel count
    (INPUT, 1, 256, 56, 56, 16, 16),
    (INPUT, 3, 32, 9, 300, 16, 16),       # dim0 > 1: consecutive tensors, more than one pixel block
    (OUTPUT, 1, 128, 7, 7, 16, 16),
    (OUTPUT, 1, 1008, 1, 1, 16, 16),
    (INPUT, 1, 24, 6, 5, 8, 16),          # other blockings take the generic kernel
    (OUTPUT, 1, 24, 6, 5, 16, 12),
    (FILTER_CONV, 32, 3, 3, 3, 16, 16),
    (FILTER_CONV, 64, 32, 3, 3, 16, 16),
    (FILTER_CONV, 128, 64, 1, 1, 16, 16),
    (FILTER_CONV, 64, 1, 10, 4, 16, 16),
    (FILTER_CONV, 24, 16, 2, 5, 8, 12),
    (FILTER_DW, 64, 1, 3, 3, 16, 16),
    (FILTER_FC, 16, 64, 1, 1, 16, 16),
    (FILTER_FC, 1008, 1024, 1, 1, 16, 16),
]


def _data(dtype, n, seed):
    if dtype == np.float32:
        return synth.normal(seed, n)
    return synth.uniform_u8(seed, n)


@pytest.mark.parametrize("dtype", [np.float32, np.uint8], ids=["f32", "u8"])
@pytest.mark.parametrize("case", CASES, ids=str)
def test_pack_unpack_vs_oracle(lib, oracle, case, dtype):
    type_, d0, d1, d2, d3, cib, cob = case
    n = d0 * d1 * d2 * d3
    flat = _data(dtype, n, 5)
    want = oracle.pack(flat, type_, d0, d1, d2, d3, cib, cob)
    esize = flat.itemsize
    dflat = hu.dev(flat)
    dpacked = hu.dev_empty(n, dtype)
    rc = lib.small_hip_pack(type_, 1, d0, d1, d2, d3, cib, cob, hu.ptr(dflat), hu.ptr(dpacked), esize, hu.stream())
    assert rc == 0, lib.small_hip_last_error()
    assert_equal_exact(hu.host(dpacked), want, "pack %s" % (case,))
    dback = hu.dev_empty(n, dtype)
    rc = lib.small_hip_unpack(type_, 1, d0, d1, d2, d3, cib, cob, hu.ptr(dpacked), hu.ptr(dback), esize, hu.stream())
    assert rc == 0, lib.small_hip_last_error()
    assert_equal_exact(hu.host(dback), oracle.unpack(want, type_, d0, d1, d2, d3, cib, cob), "unpack %s" % (case,))
    assert_equal_exact(hu.host(dback), flat, "round trip %s" % (case,))


@pytest.mark.parametrize("case", [(7, 48, 11, 13), (5, 3, 20, 9), (4, 16, 1, 1)], ids=str)
def test_batched_pack_is_per_image(lib, oracle, case):
    batch, Cn, H, W = case
    per = Cn * H * W
    flat = synth.normal(9, batch * per)
    dflat, dp = hu.dev(flat), hu.dev_empty(batch * per, np.float32)
    assert lib.small_hip_pack(INPUT, batch, 1, Cn, H, W, 16, 16, hu.ptr(dflat), hu.ptr(dp), 4, hu.stream()) == 0
    got = hu.host(dp)
    for n in range(batch):
        want = oracle.pack(flat[n * per:(n + 1) * per], INPUT, 1, Cn, H, W, 16, 16)
        assert_equal_exact(got[n * per:(n + 1) * per], want, "image %d of %s" % (n, case))
    # the numpy packer of the package agrees (the models are fed through it)
    assert_equal_exact(got, layout.pack_activations(flat.reshape(batch, Cn, H, W)), "layout.pack_activations")


@pytest.mark.parametrize("shape", [(64, 3, 224, 224), (64, 64, 112, 112), (64, 1008, 1, 1), (256, 3, 32, 32)], ids=str)
@pytest.mark.parametrize("dtype", [np.float32, np.uint8], ids=["f32", "u8"])
def test_round_trip_full_size(lib, shape, dtype):
    """Benchmark-size activations: unpack(pack(x)) == x and pack(x) holds the same multiset of values
    (checked through the exact sum of the uint8 bytes / of the float bit patterns)."""
    import torch
    batch, Cn, H, W = shape
    n = batch * Cn * H * W
    g = torch.Generator(device="cuda").manual_seed(3)
    if dtype == np.float32:
        x = torch.randn(n, device="cuda", generator=g)
    else:
        x = torch.randint(0, 256, (n,), device="cuda", generator=g, dtype=torch.uint8)
    p, back = torch.empty_like(x), torch.empty_like(x)
    es = x.element_size()
    assert lib.small_hip_pack(INPUT, batch, 1, Cn, H, W, 16, 16, hu.ptr(x), hu.ptr(p), es, hu.stream()) == 0
    assert lib.small_hip_unpack(INPUT, batch, 1, Cn, H, W, 16, 16, hu.ptr(p), hu.ptr(back), es, hu.stream()) == 0
    torch.cuda.synchronize()
    assert torch.equal(back, x)
    bits = (lambda t: t.view(torch.int32).to(torch.int64)) if dtype == np.float32 else (lambda t: t.to(torch.int64))
    assert int(bits(p).sum()) == int(bits(x).sum())
    # spot check of the index map itself on image 1, channel block 0: packed [px][c] == flat [c][px]
    cb = Cn if Cn < 16 else 16
    img = x[Cn * H * W:2 * Cn * H * W].view(Cn, H * W)
    pk = p[Cn * H * W:2 * Cn * H * W].view(Cn // cb, H * W, cb)
    assert torch.equal(pk[0], img[:cb].t())


def test_bad_arguments(lib):
    d = hu.dev_empty(4096, np.float32)
    o = hu.dev_empty(4096, np.float32)
    a = (hu.ptr(d), hu.ptr(o), 4, hu.stream())
    assert lib.small_hip_pack(9, 1, 1, 16, 4, 4, 16, 16, *a) == capi.EINVAL          # unknown type
    assert lib.small_hip_pack(INPUT, 1, 1, 20, 4, 4, 16, 16, *a) == capi.EINVAL      # 20 % 16 != 0
    assert lib.small_hip_pack(INPUT, 0, 1, 16, 4, 4, 16, 16, *a) == capi.EINVAL
    assert lib.small_hip_pack(INPUT, 1, 1, 16, 4, 4, 16, 16, hu.ptr(d), hu.ptr(d), 4, hu.stream()) == capi.EINVAL
    assert lib.small_hip_pack(INPUT, 1, 1, 16, 4, 4, 16, 16, hu.ptr(d), hu.ptr(o), 2, hu.stream()) == capi.EINVAL
    assert lib.small_hip_unpack(FILTER_CONV, 1, 20, 16, 1, 1, 16, 16, *a) == capi.EINVAL
