"""Pins the CPU checker's detection decode and NMS (oracle.c: orc_yolo_detections, orc_box_iou,
orc_nms_sort; oracle/net.py: get_boxes) against the compiled reference's golden rows, against
the compiled reference itself where it is built, and against independent mathematics."""
import os

import numpy as np
import pytest

from darknet_amd import cfgs, synth
from oracle import ref
from oracle.cpu import Oracle
from oracle.net import OracleNet

from util import fill_params, write_cfg

GOLD = os.path.join(os.path.dirname(__file__), "golden")


def lexsorted(rows):
    return rows if len(rows) == 0 else rows[np.lexsort(rows[:, :5].T[::-1])]


def test_get_boxes_matches_golden_rows_of_the_reference():
    g = np.load(os.path.join(GOLD, "detections_case.npz"))
    net = OracleNet(cfgs.yolov3_tiny(1, 96))
    outs = [g[f"yolo{i}"] if f"yolo{i}" in g.files else None for i in range(net.net["n"])]
    cases = [k[:-5] for k in g.files if k.endswith("_spec")]
    assert len(cases) == 5
    for name in cases:
        w, h, thresh, relative, nms = g[name + "_spec"]
        rows = net.get_boxes(outs, int(w), int(h), float(thresh), int(relative), float(nms))
        want = g[name]
        if nms > 0:
            rows = lexsorted(rows)
            assert (want[:, 5:] > 0).sum() > 1000 and (want[:, 5:] == 0).sum() > 1000
        assert rows.shape == want.shape, name
        assert np.array_equal(rows, want), name


@pytest.mark.skipif(not ref.available(), reason="oracle/_ref (compiled reference) not built")
@pytest.mark.parametrize("w,h,thresh,relative,nms", [(160, 160, 0.5, 1, 0.0), (640, 360, 0.3, 0, 0.45),
                                                     (333, 500, 0.22, 1, 0.3)])
def test_get_boxes_matches_compiled_reference(w, h, thresh, relative, nms):
    text = cfgs.yolov3_tiny(1, 160)
    p = write_cfg(text)
    r = ref.RefNet(p)
    os.unlink(p)
    fill_params(r.set_conv, r.layers, seed=900, bn="random")
    outs = r.predict(synth.uniform01(5, r.inputs))
    want = r.get_boxes(w, h, thresh, relative, nms)
    got = OracleNet(text).get_boxes(outs, w, h, thresh, relative, nms)
    assert len(want) > 50
    if nms > 0:
        want, got = lexsorted(want), lexsorted(got)
    assert np.array_equal(got, want)


def test_box_iou_closed_forms():
    o = Oracle()
    a = np.array([0.5, 0.5, 0.25, 0.5], np.float32)
    assert o.box_iou(a, a) == 1.0
    assert o.box_iou(a, np.array([2.0, 2.0, 0.25, 0.5], np.float32)) == 0.0          # disjoint
    assert o.box_iou(a, np.array([0.75, 0.5, 0.25, 0.5], np.float32)) == 0.0         # touching edges
    # shifted by half a width: intersection 1/2 of each, union 3/2 -> 1/3
    assert o.box_iou(a, np.array([0.625, 0.5, 0.25, 0.5], np.float32)) == np.float32(1) / np.float32(3)
    # a box inside another: ratio of the areas
    assert o.box_iou(a, np.array([0.5, 0.5, 0.125, 0.25], np.float32)) == 0.25
    # symmetric
    b = np.array([0.55, 0.4, 0.3, 0.2], np.float32)
    assert o.box_iou(a, b) == o.box_iou(b, a)


def test_decode_closed_form_single_cell():
    """One cell above the threshold; with a square image equal to the network's aspect the
    letterbox correction is the identity and the box is (col+tx)/lw, (row+ty)/lh, e^tw*pw/netw."""
    o = Oracle()
    lw, lh, n, classes = 4, 3, 2, 3
    pred = np.zeros((n * (5 + classes), lh, lw), np.float32)
    a, row, col = 1, 2, 3
    base = a * (5 + classes)
    pred[base + 0, row, col] = 0.25
    pred[base + 1, row, col] = 0.75
    pred[base + 2, row, col] = np.log(2.0)
    pred[base + 3, row, col] = 0.0
    pred[base + 4, row, col] = 0.75
    pred[base + 5:base + 8, row, col] = [0.5, 1.0, 0.125]
    biases = np.array([10, 20, 30, 40, 50, 60], np.float32)
    mask = [2, 0]                                  # anchor 1 -> pair 0 = (10, 20)
    rows = o.yolo_detections(pred, n, classes, biases, mask, 128, 96, 256, 192, 1, 0.3)
    assert rows.shape == (1, 8)
    x, y, w, h, obj = rows[0, :5]
    assert (x, y) == (np.float32(3.25) / 4, np.float32(2.75) / 3)
    assert abs(w - 2.0 * 10 / 128) < 1e-7 and h == np.float32(20 / 96)
    assert obj == 0.75
    assert list(rows[0, 5:]) == [0.375, 0.75, 0.0]          # 0.09375 <= thresh -> 0
    # absolute coordinates scale by the image size
    ra = o.yolo_detections(pred, n, classes, biases, mask, 128, 96, 256, 192, 0, 0.3)
    assert np.allclose(ra[0, :4], rows[0, :4] * [256, 192, 256, 192], rtol=1e-7)
    # a 2:1 image in a square network is letterboxed to half the height: y stretches about 0.5
    rl = o.yolo_detections(pred, n, classes, biases, mask, 96, 96, 200, 100, 1, 0.3)
    sq = o.yolo_detections(pred, n, classes, biases, mask, 96, 96, 100, 100, 1, 0.3)
    assert rl[0, 0] == sq[0, 0] and rl[0, 2] == sq[0, 2]
    assert abs(rl[0, 1] - ((sq[0, 1] - 0.25) / 0.5)) < 1e-6 and abs(rl[0, 3] - 2 * sq[0, 3]) < 1e-6
    # order: cells row-major, anchors inside a cell
    pred[4, 0, 1] = 0.9
    pred[base + 4, 0, 1] = 0.8
    pred[4, 2, 3] = 0.6
    r3 = o.yolo_detections(pred, n, classes, biases, mask, 128, 96, 128, 96, 1, 0.3)
    assert [float(v) for v in r3[:, 4]] == [np.float32(0.9), np.float32(0.8), np.float32(0.6), 0.75]


def brute_force_nms(rows, classes, thresh):
    """Greedy per-class NMS written from the definition, corner coordinates in float64."""
    out = rows.astype(np.float64).copy()
    x0, x1 = out[:, 0] - out[:, 2] / 2, out[:, 0] + out[:, 2] / 2
    y0, y1 = out[:, 1] - out[:, 3] / 2, out[:, 1] + out[:, 3] / 2
    area = out[:, 2] * out[:, 3]
    for k in range(classes):
        order = sorted(range(len(out)), key=lambda i: (-out[i, 5 + k], i))
        for a, i in enumerate(order):
            if out[i, 5 + k] == 0:
                continue
            for j in order[a + 1:]:
                iw = min(x1[i], x1[j]) - max(x0[i], x0[j])
                ih = min(y1[i], y1[j]) - max(y0[i], y0[j])
                inter = iw * ih if iw > 0 and ih > 0 else 0.0
                if inter / (area[i] + area[j] - inter) > thresh:
                    out[j, 5 + k] = 0
    return out.astype(np.float32)


def test_nms_matches_brute_force_on_grid_boxes():
    """Boxes on a 1/64 grid keep every float32 operation exact, and the thresholds sit away from
    every attainable IoU, so the float32 restatement must agree with float64 brute force."""
    rng = np.random.default_rng(11)
    total, classes = 120, 4
    rows = np.zeros((total, 5 + classes), np.float32)
    rows[:, 0:2] = rng.integers(16, 48, (total, 2)) / 64.0
    rows[:, 2:4] = rng.integers(6, 14, (total, 2)) * 2 / 64.0
    rows[:, 4] = rng.uniform(0.3, 1.0, total)
    p = rng.uniform(0.05, 1.0, (total, classes)).astype(np.float32)
    p[rng.uniform(size=p.shape) < 0.3] = 0
    rows[:, 5:] = p
    rows[::9, 4] = 0                                  # objectness 0: takes no part
    o = Oracle()
    for thresh in (0.2003, 0.4501, 0.7007):
        got = o.nms_sort(rows, classes, thresh)
        live = rows[:, 4] != 0
        want = rows.copy()
        want[live] = brute_force_nms(rows[live], classes, thresh)
        assert np.array_equal(got, want)
        assert (got[:, 5:] != rows[:, 5:]).sum() > (100 if thresh < 0.3 else 5)


# ---- region head (yolov2) ----------------------------------------------------------------------
REGION_CFG = open(os.path.join(GOLD, "region_net.cfg")).read()


def test_region_forward_and_boxes_match_golden():
    g = np.load(os.path.join(GOLD, "region_case.npz"))
    net = OracleNet(REGION_CFG)
    L = net.layers[-1]
    assert L["type"] == "region" and L["softmax"] == 1 and L["n"] == 6
    out = net.forward_layer(net.net["n"] - 1, g["region_in"], None)
    assert np.array_equal(np.ascontiguousarray(out).reshape(1, -1), g["region_out"])
    outs = [None] * (net.net["n"] - 1) + [g["region_out"]]
    for name in [k[:-5] for k in g.files if k.endswith("_spec")]:
        w, h, thresh, relative, nms = g[name + "_spec"]
        rows = net.get_boxes(outs, int(w), int(h), float(thresh), int(relative), float(nms))
        if nms > 0:
            rows = lexsorted(rows[rows[:, 4] > 0])
        assert np.array_equal(rows, g[name]), name
    assert (g["wide_abs_nms"][:, 5:] > 0).sum() > 300


@pytest.mark.skipif(not ref.available(), reason="oracle/_ref (compiled reference) not built")
def test_region_matches_compiled_reference():
    p = write_cfg(REGION_CFG.replace("softmax=1", "softmax=0").replace("height=96", "height=64"))
    r = ref.RefNet(p)
    text = open(p).read()
    os.unlink(p)
    o = OracleNet(text)
    fill_params(r.set_conv, o.layers, seed=77)
    fill_params(o.set_conv, o.layers, seed=77)
    x = synth.uniform01(8, r.inputs)
    ro, oo = r.predict(x), o.forward(x)
    assert np.array_equal(ro[-1].reshape(-1), oo[-1].reshape(-1))          # logistic class scores
    assert np.array_equal(r.get_boxes(100, 80, 0.3, 1, 0.0), o.get_boxes(ro, 100, 80, 0.3, 1, 0.0))


def test_region_forward_properties():
    o = Oracle()
    n, classes = 3, 5
    x = synth.uniform(2, 2 * n * (5 + classes) * 4 * 6, -3, 3).reshape(2, n * (5 + classes), 4, 6)
    y = o.region(x, n, classes, softmax=1).reshape(2, n, 5 + classes, 4, 6)
    xv = x.reshape(2, n, 5 + classes, 4, 6).astype(np.float64)
    assert np.allclose(y[:, :, 5:].sum(axis=2), 1.0, atol=1e-6)                      # softmax over classes
    e = np.exp(xv[:, :, 5:] - xv[:, :, 5:].max(axis=2, keepdims=True))
    assert np.abs(y[:, :, 5:] - e / e.sum(axis=2, keepdims=True)).max() <= 1e-6
    assert np.abs(y[:, :, [0, 1, 4]] - 1 / (1 + np.exp(-xv[:, :, [0, 1, 4]]))).max() <= 1e-6
    assert np.array_equal(y[:, :, 2:4], x.reshape(2, n, 5 + classes, 4, 6)[:, :, 2:4])   # w, h stay raw
    # without softmax the classes get the logistic; with background the objectness stays raw
    y2 = o.region(x, n, classes, softmax=0).reshape(2, n, 5 + classes, 4, 6)
    assert np.abs(y2[:, :, 5:] - 1 / (1 + np.exp(-xv[:, :, 5:]))).max() <= 1e-6
    y3 = o.region(x, n, classes, background=1, softmax=1).reshape(2, n, 5 + classes, 4, 6)
    assert np.allclose(y3[:, :, 4:].sum(axis=2), 1.0, atol=1e-6)                     # softmax spans objectness too


def test_region_decode_closed_form():
    """Anchors are in cell units and divided by the LAYER size (yolo: pixels / network size)."""
    o = Oracle()
    lw, lh, n, classes = 4, 3, 2, 3
    pred = np.zeros((n * (5 + classes), lh, lw), np.float32)
    a, row, col = 1, 2, 3
    base = a * (5 + classes)
    pred[base + 0:base + 5, row, col] = [0.25, 0.75, np.log(2.0), 0.0, 0.75]
    pred[base + 5:base + 8, row, col] = [0.5, 1.0, 0.125]
    rows = o.region_detections(pred, n, classes, 4, 0, [1, 2, 1.5, 0.75], 128, 96, 256, 192, 1, 0.3)
    assert rows.shape == (lw * lh * n, 8)
    r = rows[a * lw * lh + row * lw + col]                      # anchor-major row index
    assert (r[0], r[1]) == (np.float32(3.25) / 4, np.float32(2.75) / 3)
    assert abs(r[2] - 2.0 * 1.5 / 4) < 1e-7 and r[3] == np.float32(0.75 / 3)
    assert r[4] == 0.75 and list(r[5:]) == [0.375, 0.75, 0.0]
    others = np.delete(rows, a * lw * lh + row * lw + col, axis=0)
    assert not others[:, 4:].any()                              # objectness 0 <= thresh: stored as 0, no classes
    assert np.all(others[:, 2] > 0)                             # but every cell still has its box
