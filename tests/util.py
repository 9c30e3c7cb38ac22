"""Helpers shared by the tests: identical seeded parameters for every implementation of a
network (CPU checker, compiled reference, HIP library) and the error norms the gates use."""
from __future__ import annotations

import os
import tempfile

import numpy as np

from darknet_amd import synth

REL_TOL = 1e-4   # per conv layer: max|got-want| / max|want|   (the contract's "1e-4 relative")
YOLO_ABS_TOL = 1e-3


def fill_params(setter, layers, seed=1000, bn="random"):
    """Write the same weights / BN vectors into any network object exposing set_conv()."""
    for i, L in enumerate(layers):
        if L["type"] == "convolutional":
            n = L["n"]
            w = synth.conv_weights(seed + i, n, L["c"] // L["groups"], L["size"])
        elif L["type"] == "connected":      # weights [outputs][inputs]: a 1x1 convolution of a 1x1 image
            n = L["outputs"]
            w = synth.conv_weights(seed + i, n, L["inputs"], 1)
        elif L["type"] == "batchnorm":      # c values per vector; the weights file carries no biases for it
            _, s, m, v = synth.bn_random(seed * 2 + i, L["c"]) if bn == "random" else synth.bn_identity(L["c"])
            setter(i, None, np.zeros(L["c"], np.float32), s, m, v)
            continue
        elif L["type"] == "local":          # one [n][c*size*size] matrix per location, one bias per output
            w = synth.conv_weights(seed + i, L["out_h"] * L["out_w"] * L["n"], L["c"], L["size"])
            b = (synth.uniform(seed * 3 + i, L["outputs"], -0.5, 0.5) if bn == "random"
                 else np.zeros(L["outputs"], np.float32))
            setter(i, w, b, None, None, None)
            continue
        else:
            continue
        if L["batch_normalize"]:
            if bn == "random":
                b, s, m, v = synth.bn_random(seed * 2 + i, n)
            else:
                b, s, m, v = synth.bn_identity(n)
            setter(i, w, b, s, m, v)
        else:
            b = synth.uniform(seed * 3 + i, n, -0.5, 0.5) if bn == "random" else np.zeros(n, np.float32)
            setter(i, w, b, None, None, None)


def norm_err(got, want):
    """max|got-want| / max|want| - elementwise relative error is meaningless at cancellation
    zeros (the reference itself misses fp64 truth by >10% there)."""
    want = np.asarray(want, np.float64)
    got = np.asarray(got, np.float64)
    return float(np.abs(got - want).max() / max(np.abs(want).max(), 1e-30))


def write_cfg(text):
    f = tempfile.NamedTemporaryFile("w", suffix=".cfg", delete=False)
    f.write(text)
    f.close()
    return f.name


def have_reference_tree():
    return os.path.isdir("/root/reference/cfg")
