"""The reference's 1-D functions (include/small/interface_abstract_1D.hpp) compiled into oracle/_ref (sref_1d_f32)
against their CPU restatement (oracle/layers.py:one_d_f32 = the 2-D function with a 1 x k window on every row).
Scalar build only: bit-identical.  (The reference's ZEN2 build aborts in its 1-D kernels on more than one row, and
its 1-D edge code overflows a stack tile when a side needs two or more padded columns, so those are left out.)
Skipped where oracle/_ref is absent.
"""
import numpy as np
import pytest

from oracle import layers as ol
from smallframework_amd import synth
from util import assert_equal_exact

# (k, stride, l_pad, r_pad, Co, Ci, rows, W)
ONE_D_CASES = [
    (3, 1, 1, 1, 32, 16, 1, 13), (3, 1, 1, 1, 32, 16, 3, 13), (3, 2, 0, 1, 32, 16, 1, 12), (3, 2, 0, 1, 32, 16, 3, 12),
    (1, 1, 0, 0, 16, 32, 1, 9), (1, 1, 0, 0, 16, 32, 4, 9), (3, 1, 1, 1, 16, 3, 1, 13), (2, 2, 0, 0, 16, 16, 2, 10),
    (5, 1, 0, 0, 16, 16, 2, 11),
]
KINDS = ["conv", "partial_conv", "maxpool", "avgpool", "relu", "upsample"]


def one_d_inputs(case, kind, cb, oracle):
    k, s, l, r, Co, Ci, rows, W = case
    x = oracle.pack(synth.normal(1, Ci * rows * W), 0, 1, Ci, rows, W, cb, cb)
    f = oracle.pack(synth.he_normal(2, Co * Ci * k, Ci * k), 3, Co, Ci, 1, k, cb, cb) if kind < 2 else None
    Wo = 1 + (W + l + r - k) // s
    init = synth.normal(3, Co * rows * Wo) if kind == 1 else None
    n_out = {0: Co * rows * Wo, 1: Co * rows * Wo, 2: Ci * rows * Wo, 3: Ci * rows * Wo, 4: Ci * rows * W,
             5: Ci * rows * W * 2}[kind]
    return x, f, init, n_out


@pytest.mark.parametrize("kind", range(6), ids=KINDS)
@pytest.mark.parametrize("case", ONE_D_CASES, ids=str)
def test_one_d_functions(oracle, ref_REF, case, kind):
    ref = ref_REF
    cb = ref.f_cob
    k, s, l, r, Co, Ci, rows, W = case
    if kind >= 2 and Ci % 16:
        pytest.skip("needs whole channel blocks")
    x, f, init, n_out = one_d_inputs(case, kind, cb, oracle)
    bi = ref.fbuf(x.size, x)
    bf = ref.fbuf(f.size, f) if f is not None else ref.fbuf(1)
    bo = ref.fbuf(n_out, init if init is not None else np.full(n_out, 9.0, np.float32))
    kk = 2 if kind == 5 else k
    assert ref.lib.sref_1d_f32(kind, kk, s, l, r, Co, Ci, rows, W, bi.h, bf.h, bo.h) == 0, ref.err()
    want = ol.one_d_f32(oracle, kind, cb, kk, s, l, r, Co, Ci, rows, W, x, f, init)
    assert_equal_exact(want, bo.a, "%s %s" % (KINDS[kind], case))


# (k, stride, l_pad, r_pad, groups, channels per group, rows, W)
GROUP_1D_CASES = [(3, 1, 1, 1, 2, 16, 1, 13), (3, 1, 1, 1, 3, 16, 3, 11), (3, 2, 0, 1, 2, 32, 1, 12), (1, 1, 0, 0, 4, 16, 2, 9)]


@pytest.mark.parametrize("partial", [0, 1])
@pytest.mark.parametrize("case", GROUP_1D_CASES, ids=str)
def test_group_conv1d(oracle, ref_REF, case, partial):
    """GroupConv1D / PartialGroupConv1D (interface_abstract_1D.hpp:1255, 1388) on the scalar build, where the
    tensors are [groups][channels][rows][W] and the filter [groups][channels][channels][k]: every group is a
    Conv1D on its own slab."""
    ref = ref_REF
    k, s, l, r, G, Cg, rows, W = case
    Wo = 1 + (W + l + r - k) // s
    x = synth.normal(1, G * Cg * rows * W)
    f = synth.he_normal(2, G * Cg * Cg * k, Cg * k)
    init = synth.normal(3, G * Cg * rows * Wo) if partial else None
    bi, bf = ref.fbuf(x.size, x), ref.fbuf(f.size, f)
    bo = ref.fbuf(G * Cg * rows * Wo, init if partial else np.full(G * Cg * rows * Wo, 9.0, np.float32))
    assert ref.lib.sref_1d_f32(6 + partial, k, s, l, r, G, Cg, rows, W, bi.h, bf.h, bo.h) == 0, ref.err()
    want = ol.one_d_f32(oracle, 6 + partial, 1, k, s, l, r, G, Cg, rows, W, x, f, init)
    assert_equal_exact(want, bo.a, "group conv1d %s" % (case,))
    # every group differs: a dropped or repeated group cannot pass
    per = want.reshape(G, -1)
    assert all(not np.array_equal(per[a], per[b]) for a in range(G) for b in range(a))
