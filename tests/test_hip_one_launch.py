"""The whole quantised model in one launch (small_hip_qmodel_*): one workgroup per image, every tensor and filter in
LDS.  Bit-exact against the CPU oracle running the same layers one after the other, and against the layer-by-layer
GPU path."""
import ctypes as C

import numpy as np
import pytest

from smallframework_amd import capi, models
from oracle.model_exec import OracleExecutor
from util import assert_equal_exact

pytestmark = pytest.mark.gpu


def _run(model, batch, seed=99):
    w = models.make_weights(model)
    x = models.make_input(model, batch, seed=seed)
    ex = models.HipExecutor(model, batch, w, x)
    ex.build_one_launch()
    print("one-launch", model.name, "batch", batch, "LDS bytes", ex.lib.small_hip_qmodel_lds_bytes(ex.qmodel), flush=True)
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
