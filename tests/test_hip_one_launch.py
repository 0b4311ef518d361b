"""A whole small model in one launch: one workgroup per image, tensors (and for uint8 every filter) in LDS.
uint8 (small_hip_qmodel_*): bit-exact against the CPU oracle running the same layers one after the other, and
against the layer-by-layer GPU path.  float32 (small_hip_fmodel_*): within the float32 bar of the oracle."""
import ctypes as C

import numpy as np
import pytest

from smallframework_amd import capi, models
from oracle.model_exec import OracleExecutor
from util import assert_close_f32, assert_equal_exact

pytestmark = pytest.mark.gpu


def _run(model, batch, seed=99):
    w = models.make_weights(model)
    x = models.make_input(model, batch, seed=seed)
    ex = models.HipExecutor(model, batch, w, x)
    ex.build_one_launch()
    print("one-launch", model.name, "batch", batch, "LDS bytes", ex.one_launch_lds_bytes(), flush=True)
    ex.forward_one_launch()
    got = ex.output_one_launch().copy()
    ex.forward()
    layered = ex.output().copy()
    want = OracleExecutor(model, batch, w, x).forward()
    ex.close()
    return got, layered, want


@pytest.mark.parametrize("disc", [False, True], ids=["config", "discriminating"])
@pytest.mark.parametrize("batch", [1, 5])
def test_resnet8_u8_one_launch(disc, batch):
    got, layered, want = _run(models.resnet8_u8(discriminating=disc), batch)
    assert_equal_exact(got, want, "one launch vs oracle")
    assert_equal_exact(got, layered, "one launch vs layer by layer")
    if disc:
        assert len(np.unique(want)) > 1          # 0 and 255 both occur: the logits depend on the data


@pytest.mark.parametrize("batch", [1, 3, 64])
def test_dscnn_f32_one_launch(batch):
    """The keyword-spotting DS-CNN (10x4 stride-2 stem with 4 / 5 padded rows, depthwise + pointwise blocks, average
    pool, dense) as one launch: float32 bar against the oracle, unscaled (DS-CNN outputs are of unit scale)."""
    got, layered, want = _run(models.dscnn(), batch)
    assert got.shape == want.shape
    assert_close_f32(got, want, what="DS-CNN one launch vs oracle, batch %d" % batch)
    assert_close_f32(got, layered, what="DS-CNN one launch vs layer by layer, batch %d" % batch)
    assert np.abs(want).max() > 0.1


def test_fmodel_refuses_what_does_not_fit():
    """Tiny-YOLOv2's tensors do not fit LDS: creation is refused with EUNSUPPORTED (use the layer path) and a message that
    names the limit; nothing is launched.  A bad argument is another status."""
    m = models.tiny_yolo_v2()
    ex = models.HipExecutor(m, 1)
    with pytest.raises(capi.SmallHipError) as e:
        ex.build_one_launch()
    assert e.value.status == capi.EUNSUPPORTED and "LDS" in str(e.value)
    ex.close()
    # a genuine argument error (a misaligned filter pointer) is EINVAL, not a quiet fall-back
    m = models.dscnn()
    ex = models.HipExecutor(m, 1)
    layers = ex.fmodel_layers()
    layers[1].filter = layers[1].filter + 4
    h = C.c_void_p()
    assert ex.lib.small_hip_fmodel_create(len(layers), layers, C.byref(h), ex.stream()) == capi.EINVAL
    ex.close()


@pytest.mark.parametrize("name,batch", [("dscnn", 64), ("resnet8_u8", 64)])
def test_one_launch_repeats_bit_for_bit(name, batch):
    """Forty launches on the same input give the same bytes: no workgroup reads a tensor another wave is still writing
    (a fused depthwise + 1x1 layer writes its result to another LDS tensor than the one its 3x3 windows read)."""
    m = getattr(models, name)()
    ex = models.HipExecutor(m, batch, models.make_weights(m), models.make_input(m, batch, seed=7))
    ex.build_one_launch()
    ex.forward_one_launch()
    first = ex.output_one_launch().copy()
    for i in range(40):
        ex.forward_one_launch()
        again = ex.output_one_launch()
        assert np.array_equal(again.view(np.uint8), first.view(np.uint8)), "launch %d differs from the first" % (i + 2)
    ex.close()


@pytest.mark.parametrize("disc", [False, True], ids=["config", "discriminating"])
@pytest.mark.parametrize("batch", [64, 256])
def test_resnet8_u8_one_launch_at_the_benchmark_batches(disc, batch):
    """The launch bench.py reports (batch 64 and 256), on a batch tiled from four distinct images: the four against the
    oracle, every copy against its source, bit for bit."""
    m = models.resnet8_u8(discriminating=disc)
    w = models.make_weights(m)
    distinct = 4
    x = models.make_input(m, distinct, seed=31)
    per = x.size // distinct
    xt = np.ascontiguousarray(np.tile(x.reshape(distinct, per), (batch // distinct, 1))).ravel()
    ex = models.HipExecutor(m, batch, w, xt)
    ex.build_one_launch()
    ex.forward_one_launch()
    got = ex.output_one_launch().reshape(batch, -1).copy()
    ex.close()
    want = OracleExecutor(m, distinct, w, x).forward().reshape(distinct, -1)
    assert_equal_exact(got[:distinct], want, "one launch, batch %d, images 0..3 vs oracle" % batch)
    for i in range(distinct, batch):
        assert_equal_exact(got[i], got[i % distinct], "one launch, batch %d: image %d vs its source" % (batch, i))
    if disc:
        assert len(np.unique(want)) > 1


@pytest.mark.parametrize("name,batch", [("resnet8_u8", 8), ("dscnn", 4)])
def test_one_launch_graph_replays_match_eager(name, batch):
    """small_hip_qmodel_forward / small_hip_fmodel_forward recorded into a HIP graph: every replay, with eager launches
    and synchronisations in between and another input each time, reproduces the eager launch bit for bit."""
    import torch
    m = models.resnet8_u8(discriminating=True) if name == "resnet8_u8" else models.dscnn()
    ex = models.HipExecutor(m, batch, models.make_weights(m), models.make_input(m, batch))
    ex.build_one_launch()
    ex.capture(one_launch=True)
    for rep in range(4):
        xr = models.make_input(m, batch, seed=300 + rep)
        ex.buf["in"].copy_(torch.from_numpy(xr))
        ex.replay()
        got = ex.output_one_launch().copy()
        ex.one_out.zero_()
        ex.forward_one_launch()
        want = ex.output_one_launch().copy()
        assert np.array_equal(got.view(np.uint8), want.view(np.uint8)), "graph replay %d differs from the eager launch" % rep
        assert np.unique(want.view(np.uint8)).size > 1
    ex.close()


def _exposed_u8_net(hw, form):
    """Two or three uint8 convolutions whose bytes stay between 0 and 255 (not saturated), followed by a 1x1 convolution
    with an identity filter and a unit output scale, so that the model's output IS the last tensor, byte for byte:
    form "plain": stem -> b0, 3x3 16->16 -> b1;  "relu": stem + in-place ReLU;  "accum": stem -> b0, 3x3 -> b1, 3x3 -> b2 +
    Accum(b0) + ReLU.
    -> (model, weights)."""
    b = models._Builder("u8_exposed_%s_%d" % (form, hw), "u8", (3, hw, hw), "u8")
    unit = (0, (1 << 31) - 1, 0, 0)
    half = 1 << 30
    b.advance(b.conv(16, 3, 1, "same", dst="b0"))
    q = {"in": (-130, half + 777, 0, 0)}
    if form == "relu":
        b.eltwise("relu")
        q.update(b0=(0, (1 << 31) - 1, 0, 2), b1=unit, b2=unit)
        out = "b2"
    elif form == "plain":
        b.advance(b.conv(16, 3, 1, "same", src="b0", dst="b1"))
        q.update(b0=(0, half + 12345, 0, 7), b1=(0, half + 54321, 0, 10), b2=unit)
        out = "b2"
    else:
        # the Accum source (b0) may not be the convolution's own input: one more convolution in between
        b.advance(b.conv(16, 3, 1, "same", src="b0", dst="b1"))
        b.advance(b.conv(16, 3, 1, "same", src="b1", dst="b2"))
        b.eltwise("accum", src="b0", dst="b2")
        b.eltwise("relu")
        q.update(b0=(0, half + 12345, 0, 7), b1=unit, b2=(0, (1 << 31) - 1, 0, 2))
        out = "b1"
    last = b.conv(16, 1, 1, "valid", src=b.cur, dst=out)
    b.advance(last)
    m = b.done()
    m.quant.update(q)
    for o in m.ops:
        if o.weight:
            m.quant[o.weight] = (-129, half, 0, 0)
    m.quant[last.weight] = (0, half, 0, 0)
    w = models.make_weights(m)
    ident = np.zeros(16 * 16, np.uint8)          # packed 1x1 filter [16 ci][16 co]: 1 where ci == co, filter zero point 0
    ident[np.arange(16) * 16 + np.arange(16)] = 1
    w[last.weight] = ident
    return m, w


@pytest.mark.parametrize("form,hw", [
    ("plain", 24), ("relu", 24), ("accum", 24),     # the short epilogue with its pixel tables in every layer but the last
    ("plain", 60), ("relu", 60),                    # a pixel table of 3600 entries does not fit the table fetch: the general one
])
def test_u8_one_launch_epilogue_forms(form, hw, max_lds=163840):
    """The uint8 one-launch kernel's short epilogue (a table indexed by the product's high word, pixel geometry from a
    table, with and without ReLU / Accum) and the general one it falls back to, on tensors that are NOT saturated and
    that the model hands out unchanged: the oracle's bytes."""
    m, w = _exposed_u8_net(hw, form)
    batch = 3
    x = models.make_input(m, batch, seed=5)
    want = OracleExecutor(m, batch, w, x).forward()
    assert len(np.unique(want)) > 30, "the exposed tensor should hold many different bytes"
    ex = models.HipExecutor(m, batch, w, x)
    ex.build_one_launch()
    lds = ex.one_launch_lds_bytes()
    print("u8 net", form, hw, "LDS bytes", lds, "byte values", len(np.unique(want)), flush=True)
    assert lds <= max_lds
    ex.forward_one_launch()
    got = ex.output_one_launch().copy()
    ex.close()
    assert_equal_exact(got, want, "u8 one launch, %s, %dx%d" % (form, hw, hw))


def test_u8_one_launch_without_room_for_pixel_tables():
    """A model that fits LDS only without the short epilogue's pixel tables is planned without them (and not refused)."""
    m, w = _exposed_u8_net(50, "accum")
    batch = 2
    x = models.make_input(m, batch, seed=6)
    ex = models.HipExecutor(m, batch, w, x)
    ex.build_one_launch()
    print("u8 net 50 LDS bytes", ex.one_launch_lds_bytes(), flush=True)
    ex.forward_one_launch()
    got = ex.output_one_launch().copy()
    ex.close()
    want = OracleExecutor(m, batch, w, x).forward()
    assert_equal_exact(got, want, "u8 one launch without pixel tables")
    assert len(np.unique(want)) > 30
