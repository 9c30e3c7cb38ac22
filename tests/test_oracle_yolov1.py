"""Pins for the CPU checker's locally connected layer and yolov1 detection head
(oracle.c: orc_local_forward, orc_detection_forward, orc_detection_detections).

Three independent anchors: the golden vectors the compiled reference wrote for yolov1_net.cfg
(every layer's output, boxes, NMS), the compiled reference itself on other geometries where it
is built, and what the mathematics fixes: with the same weights at every location the layer is
an ordinary convolution; a float64 tensor contraction; hand-made head tensors whose boxes have
closed forms."""
import os

import numpy as np
import pytest

from darknet_amd import synth
from oracle import ref
from oracle.cpu import Oracle
from oracle.net import OracleNet

from util import fill_params, write_cfg

GOLD = os.path.join(os.path.dirname(__file__), "golden")
CFG = open(os.path.join(GOLD, "yolov1_net.cfg")).read()


def test_every_layer_and_the_boxes_match_the_reference_golden_vectors():
    g = np.load(os.path.join(GOLD, "yolov1_case.npz"))
    net = OracleNet(CFG)
    assert [L["type"] for L in net.layers] == ["convolutional", "maxpool", "convolutional", "local", "dropout",
                                               "connected", "detection"]
    fill_params(net.set_conv, net.layers, seed=77, bn="random")
    outs = net.forward(g["input"])
    for i, o in enumerate(outs):
        assert np.array_equal(o, g[f"layer{i}"]), (i, net.layers[i]["type"])
    for name in [k[:-5] for k in g.files if k.endswith("_spec")]:
        w, h, thresh, relative, nms = g[name + "_spec"]
        rows = net.get_boxes(outs, int(w), int(h), float(thresh), int(relative), float(nms))
        if nms > 0:
            rows = rows[rows[:, 4] > 0]
            rows = rows[np.lexsort(rows[:, :5].T[::-1])]
        assert np.array_equal(rows, g[name]), name
        assert len(rows) > 0 and (rows[:, 5:] > 0).any()
    soft = OracleNet(CFG.replace("softmax=0", "softmax=1"))
    fill_params(soft.set_conv, soft.layers, seed=77, bn="random")
    got = soft.forward(g["input"])[-1]
    assert np.array_equal(got, g["softmax_out"])
    L = soft.layers[-1]
    cls = got[0][:L["side"] ** 2 * L["classes"]].reshape(-1, L["classes"])
    assert np.allclose(cls.sum(1), 1, atol=1e-6) and np.array_equal(got[0][cls.size:], outs[-1][0][cls.size:])


LOCAL_GEOMETRIES = [  # c, h, w, n, size, stride, pad, batch, activation
    (3, 7, 9, 5, 3, 1, 1, 2, "leaky"),
    (4, 8, 6, 3, 2, 2, 0, 1, "linear"),
    (2, 9, 9, 4, 3, 2, 1, 3, "logistic"),
    (5, 6, 5, 2, 1, 1, 0, 2, "relu"),
    (3, 11, 7, 4, 5, 1, 2, 1, "leaky"),
]


@pytest.mark.skipif(not ref.available(), reason="compiled reference not built")
@pytest.mark.parametrize("c,h,w,n,size,stride,pad,batch,act", LOCAL_GEOMETRIES)
def test_local_matches_compiled_reference(c, h, w, n, size, stride, pad, batch, act):
    # a convolution ahead of the local layer gives the reference a workspace large enough for the
    # local layer's im2col (the local layer sizes its own request in floats, not bytes)
    text = (f"[net]\nbatch={batch}\nheight={h}\nwidth={w}\nchannels={c}\n"
            f"[convolutional]\nfilters={c}\nsize={size | 1}\nstride=1\npad=1\nactivation=linear\n"
            f"[local]\nfilters={n}\nsize={size}\nstride={stride}\npad={pad}\nactivation={act}\n")
    p = write_cfg(text)
    r = ref.RefNet(p)
    os.unlink(p)
    o = OracleNet(text)
    Lr, Lo = r.layers[1], o.layers[1]
    for k in ("h", "w", "c", "out_h", "out_w", "out_c", "inputs", "outputs", "n", "size", "stride", "pad"):
        assert Lr[k] == Lo[k], k
    fill_params(r.set_conv, r.layers, seed=9, bn="random")
    fill_params(o.set_conv, o.layers, seed=9, bn="random")
    x = synth.uniform(4, batch * c * h * w, -1, 1)
    want = r.forward_layer(1, x)
    got = np.ascontiguousarray(o.forward_layer(1, x.reshape(batch, -1), None)).reshape(batch, -1)
    assert np.array_equal(got, want)


def test_local_with_shared_weights_is_a_convolution(orc):
    """The same [n][K] matrix at every location and zero biases: forward_local_layer must equal
    the convolution of those weights bit for bit (both accumulate over k in the same order)."""
    c, h, w, n, size, stride, pad, b = 3, 8, 7, 4, 3, 1, 1, 2
    x = synth.uniform(1, b * c * h * w, -1, 1).reshape(b, c, h, w)
    wt = synth.conv_weights(2, n, c, size).reshape(n, -1)
    loc = h * w
    local_w = np.tile(wt[None], (loc, 1, 1))
    got = orc.local(x, local_w, np.zeros(loc * n, np.float32), n=n, size=size, stride=stride, pad=pad,
                    activation="leaky")
    want = orc.conv(x, wt, np.zeros(n, np.float32), n=n, size=size, stride=stride, pad=pad, activation="leaky")
    assert np.array_equal(got.reshape(-1), np.asarray(want).reshape(-1))
    # strided, unpadded, and a bias per output element
    bias = synth.uniform(3, 3 * 3 * n, -1, 1)
    xs = np.ascontiguousarray(x[:, :, :7, :7])
    got = orc.local(xs, np.tile(wt[None], (9, 1, 1)), bias, n=n, size=3, stride=2, pad=0,
                    activation="linear")
    want = np.asarray(orc.conv(xs, wt, np.zeros(n, np.float32), n=n, size=3, stride=2, pad=0,
                               activation="linear")).reshape(b, n, 3, 3)
    assert np.abs(got - (want + bias.reshape(1, n, 3, 3))).max() <= 2e-6


def test_local_against_a_float64_contraction(orc):
    c, h, w, n, size, stride, pad, b = 4, 6, 5, 3, 3, 1, 1, 2
    x = synth.uniform(11, b * c * h * w, -1, 1).reshape(b, c, h, w)
    loc = h * w
    wt = synth.uniform(12, loc * n * c * size * size, -1, 1).reshape(loc, n, c, size, size)
    bias = synth.uniform(13, n * loc, -1, 1)
    got = orc.local(x, wt, bias, n=n, size=size, stride=stride, pad=pad, activation="linear")
    xp = np.zeros((b, c, h + 2, w + 2))
    xp[:, :, 1:-1, 1:-1] = x
    want = np.zeros((b, n, h, w))
    for oy in range(h):
        for ox in range(w):
            patch = xp[:, :, oy:oy + 3, ox:ox + 3]
            want[:, :, oy, ox] = np.einsum("bckl,nckl->bn", patch, wt[oy * w + ox].astype(np.float64))
    want += bias.reshape(1, n, h, w)
    assert np.abs(got - want).max() <= 1e-5
    # a transposed weight block, a shifted patch or a per-filter bias would all miss by O(1)
    assert np.abs(want).max() > 1


def test_detection_boxes_closed_form(orc):
    side, n, classes = 2, 2, 3
    cells = side * side
    pred = np.zeros(cells * (classes + 5 * n), np.float32)
    prob = pred[:cells * classes].reshape(cells, classes)
    scale = pred[cells * classes:cells * (classes + n)].reshape(cells, n)
    box = pred[cells * (classes + n):].reshape(cells, n, 4)
    prob[:] = [[.5, .25, 0], [1, 0, 0], [0, 0, 1], [.125, .5, .25]]
    scale[:] = [[1, .5], [.25, 0], [.5, .5], [1, .25]]
    box[..., 0] = .5
    box[..., 1] = .25
    box[..., 2] = .5
    box[..., 3] = [[.25, 1], [.5, .5], [.75, .125], [1, 0]]
    rows = orc.detection_detections(pred, side, n, classes, 1, 64, 32, 0.2)
    assert rows.shape == (cells * n, 5 + classes)
    for cell in range(cells):
        row, col = divmod(cell, side)
        for k in range(n):
            r = rows[cell * n + k]
            assert r[0] == (0.5 + col) / side * 64 and r[1] == (0.25 + row) / side * 32
            assert r[2] == 0.25 * 64 and r[3] == box[cell, k, 3] ** 2 * 32     # sqrt=1: the square
            assert r[4] == scale[cell, k]                                      # whatever the threshold
            want = scale[cell, k] * prob[cell]
            assert np.array_equal(r[5:], np.where(want > 0.2, want, 0))
    plain = orc.detection_detections(pred, side, n, classes, 0, 64, 32, 0.2)
    assert np.array_equal(plain[:, 2], np.full(cells * n, 0.5 * 64, np.float32))
    assert np.array_equal(plain[:, [0, 1, 4]], rows[:, [0, 1, 4]])
