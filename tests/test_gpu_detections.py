"""Detections on the device (yolo_decode_gpu, nms_sort_gpu and the reference-named host calls
above them) against the CPU checker, through the C-ABI.

Bar: the set and order of detections, objectness and class probabilities bit-exact (threshold
tests and float products on identical inputs); box coordinates <= 1e-6 relative (they pass
through exp() in double on both sides, device libm vs glibc); NMS decisions bit-exact."""
import ctypes as C
import os

import numpy as np
import pytest

from darknet_amd import api, cfgs, synth
from oracle.cpu import Oracle
from oracle.net import OracleNet

from util import REL_TOL, fill_params, norm_err

pytestmark = pytest.mark.gpu
GOLD = os.path.join(os.path.dirname(__file__), "golden")
D = api.DeviceArray
BOX_RTOL = 1e-6


def check_rows(got, want):
    assert got.shape == want.shape
    assert np.array_equal(got[:, 4:], want[:, 4:])
    assert np.allclose(got[:, :4], want[:, :4], rtol=BOX_RTOL, atol=1e-7)


def device_count(dn, cnt):
    v = np.zeros(1, np.int32)
    dn.hip_pull_int_array(cnt, v.ctypes.data_as(C.POINTER(C.c_int)), 1)
    return int(v[0])


def test_decode_and_nms_kernels_on_the_reference_golden_tensors(dn):
    g = np.load(os.path.join(GOLD, "detections_case.npz"))
    onet = OracleNet(cfgs.yolov3_tiny(1, 96))
    heads = [(i, L) for i, L in enumerate(onet.layers) if L["type"] == "yolo"]
    for name in [k[:-5] for k in g.files if k.endswith("_spec")]:
        w, h, thresh, relative, nms = g[name + "_spec"]
        cap = sum(L["w"] * L["h"] * L["n"] for _, L in heads)
        rows = D(n=cap * 85)
        cnt = dn.hip_make_int_array(None, 1)
        keep = []
        for i, L in heads:
            pred = D(g[f"yolo{i}"])
            keep.append(pred)
            an = np.array([L["anchors"][2 * m + k] for m in L["mask"] for k in (0, 1)], np.float32)
            dn.yolo_decode_gpu(pred.ptr, L["w"], L["h"], L["n"], L["classes"], an.ctypes.data_as(api._F), 96, 96,
                               int(w), int(h), int(relative), float(thresh), rows.ptr, cap, cnt)
        n = device_count(dn, cnt)
        if nms > 0:
            dn.nms_sort_gpu(rows.ptr, n, 80, float(nms))
        got = rows.numpy((cap, 85))[:n]
        want = g[name]
        if nms > 0:   # the golden rows of the NMS cases are stored in canonical (sorted) order
            got = got[np.lexsort(got[:, :5].T[::-1])]
            # a box coordinate that differs in the last bit could swap neighbours in the sort
            assert np.array_equal(got[:, 4], want[:, 4])
        check_rows(got, want)
        dn.hip_free(cnt)


def test_decode_overflow_is_reported_not_written(dn):
    g = np.load(os.path.join(GOLD, "detections_case.npz"))
    pred = D(g["yolo23"])
    rows = D(np.full(10 * 85 + 85, -7.0, np.float32))
    cnt = dn.hip_make_int_array(None, 1)
    an = np.array([10, 14, 23, 27, 37, 58], np.float32)
    dn.yolo_decode_gpu(pred.ptr, 6, 6, 3, 80, an.ctypes.data_as(api._F), 96, 96, 96, 96, 1, 0.2, rows.ptr, 10, cnt)
    assert device_count(dn, cnt) == 108          # every candidate passes 0.2; only 10 rows fit
    out = rows.numpy((11, 85))
    assert np.all(out[10] == -7.0) and np.all(out[:10, 4] > 0.2)
    dn.hip_free(cnt)


def test_nms_kernel_matches_checker_on_dense_grid_boxes(dn):
    rng = np.random.default_rng(5)
    total, classes = 700, 6           # several sweeps of the 256-thread workgroup per class
    rows = np.zeros((total, 5 + classes), np.float32)
    rows[:, 0:2] = rng.integers(16, 48, (total, 2)) / 64.0
    rows[:, 2:4] = rng.integers(4, 14, (total, 2)) * 2 / 64.0
    rows[:, 4] = rng.uniform(0.3, 1.0, total)
    p = rng.uniform(0.05, 1.0, (total, classes)).astype(np.float32)
    p[rng.uniform(size=p.shape) < 0.4] = 0
    p[10:20, 2] = p[10, 2]            # ties: the lower row wins on both sides
    rows[:, 5:] = p
    want = Oracle().nms_sort(rows, classes, 0.4501)
    dev = D(rows)
    dn.nms_sort_gpu(dev.ptr, total, classes, 0.4501)
    got = dev.numpy(rows.shape)
    assert np.array_equal(got, want)
    assert (got != rows).sum() > 1000
    # the host call over detection structs gives the same suppression
    assert np.array_equal(api.do_nms_sort(rows, classes, 0.4501), want)


def test_network_boxes_against_checker_on_the_librarys_own_outputs(dn):
    text = cfgs.yolov3_tiny(2, 160)
    net = api.Network(cfg_text=text)
    onet = OracleNet(text)
    fill_params(net.set_conv, net.layers, seed=900, bn="random")
    net.predict(synth.uniform01(5, net.inputs * 2))
    outs = [net.layer_output(i) if L["type"] == "yolo" else None for i, L in enumerate(net.layers)]
    # the reference's call: image 0, no suppression
    check_rows(net.get_network_boxes(640, 360, 0.3, relative=0), onet.get_boxes(outs, 640, 360, 0.3, 0, 0.0))
    for image, (w, h, thresh, relative, nms) in [(0, (160, 160, 0.5, 1, 0.0)), (1, (333, 500, 0.22, 1, 0.3)),
                                                  (1, (640, 360, 0.3, 0, 0.45))]:
        got = net.get_boxes(w, h, thresh, relative, nms, image)
        want = onet.get_boxes(outs, w, h, thresh, relative, nms, image)
        assert len(want) > 20
        check_rows(got, want)
    # an impossible threshold: no detections, valid empty result
    assert net.get_boxes(160, 160, 2.0).shape == (0, 85)
    assert net.L.num_detections(net.net, 2.0) == 0
    net.free()


# ---- region head (yolov2) ----------------------------------------------------------------------
def test_region_forward_and_decode_on_the_reference_golden_tensors(dn):
    g = np.load(os.path.join(GOLD, "region_case.npz"))
    text = open(os.path.join(GOLD, "region_net.cfg")).read()
    onet = OracleNet(text)
    L = onet.layers[-1]
    x = D(g["region_in"])
    y = D(n=g["region_in"].size)
    dn.forward_region_gpu(x.ptr, y.ptr, 1, L["w"], L["h"], L["n"], L["classes"], L["coords"], L["background"],
                          L["softmax"])
    got = y.numpy(g["region_out"].shape)
    assert np.abs(got - g["region_out"]).max() <= 1e-6          # logistic / exp: device libm vs glibc
    assert np.array_equal(got.reshape(6, 9, -1)[:, 2:4], g["region_in"].reshape(6, 9, -1)[:, 2:4])
    # decode the REFERENCE's region output, so that every threshold decision is on identical inputs
    pred = D(g["region_out"])
    an = np.array(L["anchors"], np.float32)
    cap = L["w"] * L["h"] * L["n"]
    for name in [k[:-5] for k in g.files if k.endswith("_spec")]:
        w, h, thresh, relative, nms = g[name + "_spec"]
        rows = D(n=cap * 9)
        cnt = dn.hip_make_int_array(None, 1)
        dn.region_decode_gpu(pred.ptr, L["w"], L["h"], L["n"], L["classes"], 4, 0, an.ctypes.data_as(api._F), 64, 96,
                             int(w), int(h), int(relative), float(thresh), rows.ptr, cap, cnt)
        assert device_count(dn, cnt) == cap
        if nms > 0:
            dn.nms_sort_gpu(rows.ptr, cap, L["classes"], float(nms))
        r = rows.numpy((cap, 9))
        if nms > 0:
            r = r[r[:, 4] > 0]
            r = r[np.lexsort(r[:, :5].T[::-1])]
            assert np.array_equal(r[:, 4], g[name][:, 4])
        check_rows(r, g[name])
        dn.hip_free(cnt)


def test_region_network_boxes_against_checker(dn):
    text = open(os.path.join(GOLD, "region_net.cfg")).read().replace("batch=1", "batch=3")
    net = api.Network(cfg_text=text)
    onet = OracleNet(text)
    fill_params(net.set_conv, net.layers, seed=40, bn="random")
    fill_params(onet.set_conv, onet.layers, seed=40, bn="random")
    x = synth.uniform01(3, net.inputs * 3)
    net.predict(x)
    want = onet.forward(x)
    for i in range(net.n):
        assert norm_err(net.layer_output(i), want[i]) <= REL_TOL, i
    outs = [None] * (net.n - 1) + [net.layer_output(net.n - 1)]
    check_rows(net.get_network_boxes(200, 100, 0.25, relative=0), onet.get_boxes(outs, 200, 100, 0.25, 0, 0.0))
    for image in (1, 2):
        got = net.get_boxes(200, 100, 0.2, 0, 0.4, image)
        check_rows(got, onet.get_boxes(outs, 200, 100, 0.2, 0, 0.4, image))
        assert (got[:, 5:] > 0).sum() > 100
    net.free()
