"""The benchmark configurations at their FULL batch on the GPU, checked through properties that do not need the
scalar CPU oracle to run the whole batch:

  * replication: a batch tiled from a few distinct images must give the same result for every copy (the batched
    kernels treat images independently whatever tile / split-K / fused path the launch shape selects): bit-identical
    for uint8, pooling and activations; within the float32 bar for convolutions, whose last tiles of a launch are
    reduced in another (fixed) order than the rest, so two copies of an image may differ in the last bit;
    the distinct images themselves are compared with the oracle, and a second run must reproduce the first bit for bit;
  * scaling by a power of two commutes with every float32 rounding: conv(2x) == 2 conv(x) bit for bit;
  * uint8: bit-exact against the oracle on the distinct images.

The launch shapes here are the ones bench.py times (MobileNetV1 batch 64, Tiny-YOLOv2 batch 16, ResNet-8 uint8 batch
256, the single-layer sweep at batch 64), which select other kernels than the small-batch parity tests do.
"""
import numpy as np
import pytest

from smallframework_amd import models
from oracle.model_exec import OracleExecutor
from util import assert_close_f32, assert_equal_exact, strict_bar

pytestmark = pytest.mark.gpu


# (fraction of elements, worst excess) allowed outside the unscaled bar: measured figures with head-room
STRICT_LIMITS = {"mobilenet_v1": (0.0, 0.0), "tiny_yolo_v2": (5e-3, 3e-5)}


def _tiled_run(model, batch, distinct, **kw):
    """-> (per-image outputs [batch, n], oracle outputs [distinct, n]) for a batch made of `distinct` images repeated."""
    w = models.make_weights(model)
    x = models.make_input(model, distinct)
    per = x.size // distinct
    xt = np.ascontiguousarray(np.tile(x.reshape(distinct, per), (batch // distinct, 1))).ravel()
    assert xt.size == batch * per
    ex = models.HipExecutor(model, batch, w, xt, **kw)
    ex.forward()
    got = ex.output().reshape(batch, -1).copy()
    ex.forward()
    assert_equal_exact(ex.output(), got, model.name + ": second run")      # deterministic
    want = OracleExecutor(model, distinct, w, x).forward().reshape(distinct, -1)
    if model.dtype == "f32" and len(model.ops) > 1:
        # the stated bar |a-b| <= 1e-4|b| + 1e-5, unscaled, against the float64-accumulating chain
        truth = OracleExecutor(model, distinct, w, x, acc64=1).forward().reshape(distinct, -1)
        strict_bar(got[:distinct], truth, "%s b%d (full batch) images 0..%d" % (model.name, batch, distinct - 1),
                   *STRICT_LIMITS[model.name], reference=want)
    return got, want


def _check_replicas(got, distinct, what, exact=False):
    atol = 1e-5 * max(1.0, float(np.abs(got[:distinct]).max()))
    for i in range(distinct, got.shape[0]):
        msg = "%s: image %d vs its source %d" % (what, i, i % distinct)
        if exact:
            assert_equal_exact(got[i], got[i % distinct], msg)
        else:
            assert_close_f32(got[i], got[i % distinct], atol=atol, what=msg)


def test_mobilenet_v1_batch64():
    got, want = _tiled_run(models.mobilenet_v1(), 64, 2)
    _check_replicas(got, 2, "mobilenet_v1 b64")
    assert np.abs(want).max() > 1e-3
    assert_close_f32(got[:2], want, what="mobilenet_v1 b64 images 0, 1")


def test_tiny_yolo_v2_batch16():
    got, want = _tiled_run(models.tiny_yolo_v2(), 16, 1)
    _check_replicas(got, 1, "tiny_yolo_v2 b16")
    assert_close_f32(got[:1], want, atol=1e-5 * max(1.0, float(np.abs(want).max())), what="tiny_yolo_v2 b16 image 0")


@pytest.mark.parametrize("disc", [True, False], ids=["discriminating", "config"])
@pytest.mark.parametrize("prepared", [True, False], ids=["prepared", "direct"])
def test_resnet8_u8_batch256(prepared, disc):
    """Layer by layer at the configuration's batch: the variant whose logits depend on the data, and the configuration
    as it is written (its requantisation saturates most activations; it is the one the metric names)."""
    m = models.resnet8_u8(discriminating=disc)
    got, want = _tiled_run(m, 256, 4, prepared=prepared)
    _check_replicas(got, 4, "resnet8_u8 b256", exact=True)
    assert_equal_exact(got[:4], want, "resnet8_u8 b256 images 0..3")


@pytest.mark.parametrize("m", models.layer_sweep(), ids=lambda m: m.name)
def test_layer_sweep_batch64(m):
    got, want = _tiled_run(m, 64, 1)
    _check_replicas(got, 1, m.name + " b64", exact=not m.name.startswith("conv"))
    if m.name.startswith(("maxpool", "relu")):
        assert_equal_exact(got[:1], want, m.name)
    else:
        assert_close_f32(got[:1], want, what=m.name + " b64 image 0")
    # power-of-two scaling of the input scales every output exactly
    w = models.make_weights(m)
    x = models.make_input(m, 64)
    ex = models.HipExecutor(m, 64, w, x)
    ex.forward()
    y1 = ex.output().copy()
    import torch
    ex.buf["in"].copy_(torch.from_numpy(x * np.float32(4.0)))
    ex.forward()
    assert_equal_exact(ex.output(), y1 * np.float32(4.0), m.name + " b64: f(4x) == 4 f(x)")
