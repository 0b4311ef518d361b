"""Catalogue of the reference's own regression fixtures (PyTorch-generated, NCHW / OIHW float32).

File naming follows test/test_utils.hpp:get_pathname in the reference:
  <kind>__<layer>_Ci<C>_H<H>_W<W>_k<k>_s<s>_<v|f>[_Co<Co>]_<numel>.bin
A subset small enough to commit lives in tests/golden/ref_regression/.
"""
import glob
import os
import re

from util import GOLDEN, read_ref_bin

DIR = os.path.join(GOLDEN, "ref_regression")
_PAT = re.compile(r"out__(conv2d|dw_conv|pool|averagepool|relu)_Ci(\d+)_H(\d+)_W(\d+)_k(\d+)_s(\d+)_([vf])(?:_Co(\d+))?_(\d+)\.bin$")


def _find(kind, layer, stem):
    hits = glob.glob(os.path.join(DIR, "%s__%s_%s_*.bin" % (kind, layer, stem)))
    return hits[0] if len(hits) == 1 else None


def cases(layer):
    """-> list of dict(Ci,H,W,k,s,pad,Co,in,filter,out) whose files are all present."""
    out = []
    for path in sorted(glob.glob(os.path.join(DIR, "out__%s_*.bin" % layer))):
        m = _PAT.search(os.path.basename(path))
        if not m or m.group(1) != layer:
            continue
        Ci, H, W, k, s = (int(m.group(i)) for i in range(2, 7))
        pad = m.group(7)
        Co = int(m.group(8)) if m.group(8) else Ci
        stem = "Ci%d_H%d_W%d_k%d_s%d_%s" % (Ci, H, W, k, s, pad)
        if m.group(8):
            stem += "_Co%d" % Co
        in_layer = "pool" if layer == "averagepool" else layer
        fin = _find("in", in_layer, stem)
        ffl = _find("filter", layer, stem) if layer in ("conv2d", "dw_conv") else None
        if fin is None or (layer in ("conv2d", "dw_conv") and ffl is None):
            continue
        out.append(dict(Ci=Ci, H=H, W=W, k=k, s=s, pad=pad, Co=Co, fin=fin, ffilter=ffl, fout=path,
                        id="%s_%s" % (layer, stem)))
    return out


def load(case):
    x = read_ref_bin(case["fin"])
    f = read_ref_bin(case["ffilter"]) if case["ffilter"] else None
    y = read_ref_bin(case["fout"])
    return x, f, y
