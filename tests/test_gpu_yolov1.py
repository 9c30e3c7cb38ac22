"""The yolov1 tail on the device, through the C-ABI: the locally connected layer
(forward_local_gpu), the detection head (forward_detection_layer_gpu, detection_decode_gpu) and
the weights-file block of a local layer, against the CPU checker and the golden vectors the
compiled reference wrote for yolov1_net.cfg.

Bars: local layer <= 1e-4 max-normalised (fp32 sums in another order); the detection layer is a
copy: bit-exact (with softmax=1 the class scores <= 1e-6, device exp vs glibc); boxes out of
identical head tensors bit-exact, NMS decisions included."""
import ctypes as C
import os

import numpy as np
import pytest

from darknet_amd import api, synth
from oracle.cpu import ACTIVATIONS
from oracle.net import OracleNet

from util import REL_TOL, fill_params, norm_err

pytestmark = pytest.mark.gpu
GOLD = os.path.join(os.path.dirname(__file__), "golden")
CFG_PATH = os.path.join(GOLD, "yolov1_net.cfg")
CFG = open(CFG_PATH).read()
D = api.DeviceArray

LOCAL_CASES = [  # batch, c, h, w, n, size, stride, pad, activation
    (1, 3, 7, 9, 5, 3, 1, 1, "leaky"),
    (3, 20, 6, 5, 16, 3, 1, 1, "leaky"),
    (17, 8, 5, 5, 37, 2, 1, 0, "linear"),       # batch and filters past one workgroup's 16, ragged
    (33, 4, 9, 8, 4, 3, 2, 1, "logistic"),      # three image groups, stride 2
    (2, 64, 4, 4, 18, 3, 1, 1, "relu"),         # K = 576: two staged chunks, the second partial
    (2, 130, 3, 3, 3, 3, 1, 1, "leaky"),        # K = 1170: three chunks
    (5, 7, 6, 4, 6, 1, 1, 0, "tanh"),           # 1x1
    (2, 3, 11, 7, 4, 5, 1, 2, "leaky"),         # 5x5, two pixels of padding
]


@pytest.mark.parametrize("batch,c,h,w,n,size,stride,pad,act", LOCAL_CASES,
                         ids=["%dx%dx%dx%d_n%d_k%d_s%d_p%d" % t[:8] for t in LOCAL_CASES])
def test_local_layer_against_checker(dn, orc, batch, c, h, w, n, size, stride, pad, act):
    oh = (h - (1 if pad else size)) // stride + 1
    ow = (w - (1 if pad else size)) // stride + 1
    x = synth.uniform(21, batch * c * h * w, -1, 1).reshape(batch, c, h, w)
    wt = synth.conv_weights(22, oh * ow * n, c, size)
    bias = synth.uniform(23, oh * ow * n, -0.5, 0.5)
    want = orc.local(x, wt, bias, n=n, size=size, stride=stride, pad=pad, activation=act)
    dx, dw, db = D(x), D(wt), D(bias)
    guard = np.full(want.size + 64, 7.5, np.float32)
    out = D(guard)
    dn.forward_local_gpu(dx.ptr, dw.ptr, db.ptr, out.ptr, batch, c, h, w, n, size, stride, pad,
                         ACTIVATIONS.index(act))
    got = out.numpy((want.size + 64,))
    assert np.array_equal(got[want.size:], guard[want.size:])        # nothing written past the output
    assert norm_err(got[:want.size], want.reshape(-1)) <= REL_TOL
    dn.forward_local_gpu(dx.ptr, dw.ptr, db.ptr, out.ptr, batch, c, h, w, n, size, stride, pad,
                         ACTIVATIONS.index(act))
    assert np.array_equal(out.numpy((want.size + 64,)), got)         # same bits from run to run


def test_local_layer_in_image_slices_changes_no_bit(dn):
    """A patch budget of two images' worth: a batch of five runs as 2 + 2 + 1."""
    batch, c, h, w, n, size = 5, 6, 5, 4, 7, 3
    x = synth.uniform(41, batch * c * h * w, -1, 1)
    wt = synth.conv_weights(42, h * w * n, c, size)
    bias = synth.uniform(43, h * w * n, -0.5, 0.5)
    dx, dw, db = D(x), D(wt), D(bias)
    outs = []
    for budget in (1 << 28, 2 * h * w * c * size * size):
        dn.local_set_patch_budget(budget)
        out = D(n=batch * n * h * w)
        dn.forward_local_gpu(dx.ptr, dw.ptr, db.ptr, out.ptr, batch, c, h, w, n, size, 1, 1, ACTIVATIONS.index("leaky"))
        outs.append(out.numpy())
    dn.local_set_patch_budget(1 << 28)
    assert np.array_equal(outs[0], outs[1]) and np.abs(outs[0]).max() > 0.1


def test_yolov1_network_on_the_reference_weights_file_and_golden_vectors(dn, tmp_path):
    g = np.load(os.path.join(GOLD, "yolov1_case.npz"))
    src = os.path.join(GOLD, "yolov1_net.weights")
    net = api.Network(cfg_path=CFG_PATH, weights=src)
    final = net.predict(g["input"])
    for i, L in enumerate(net.layers):
        got = net.layer_output(i)
        if L["type"] in ("maxpool", "dropout", "detection"):
            prev = net.layer_output(i - 1)
            if L["type"] != "maxpool":
                assert np.array_equal(got, prev), (i, L["type"])     # copies of the layer before
        assert norm_err(got, g[f"layer{i}"]) <= REL_TOL, (i, L["type"])
    assert np.array_equal(final, net.layer_output(net.n - 1))
    out = str(tmp_path / "again.weights")
    net.save_weights(out)
    assert open(out, "rb").read() == open(src, "rb").read()
    net.free()


def test_detection_decode_on_the_reference_golden_head(dn):
    g = np.load(os.path.join(GOLD, "yolov1_case.npz"))
    L = OracleNet(CFG).layers[-1]
    side, n, classes = L["side"], L["n"], L["classes"]
    cap = side * side * n
    pred = D(g["layer6"])
    for name in [k[:-5] for k in g.files if k.endswith("_spec")]:
        w, h, thresh, relative, nms = g[name + "_spec"]
        rows = D(n=cap * (5 + classes))
        cnt = dn.hip_make_int_array(None, 1)
        dn.detection_decode_gpu(pred.ptr, side, n, classes, L["sqrt"], int(w), int(h), float(thresh), rows.ptr, cap,
                                cnt)
        v = np.zeros(1, np.int32)
        dn.hip_pull_int_array(cnt, v.ctypes.data_as(C.POINTER(C.c_int)), 1)
        assert int(v[0]) == cap
        if nms > 0:
            dn.nms_sort_gpu(rows.ptr, cap, classes, float(nms))
        r = rows.numpy((cap, 5 + classes))
        if nms > 0:
            r = r[r[:, 4] > 0]
            r = r[np.lexsort(r[:, :5].T[::-1])]
        assert np.array_equal(r, g[name]), name
        dn.hip_free(cnt)


def test_yolov1_batch_boxes_and_softmax_head_against_checker(dn):
    for softmax in (0, 1):
        text = CFG.replace("batch=1", "batch=5").replace("softmax=0", "softmax=%d" % softmax)
        net = api.Network(cfg_text=text)
        onet = OracleNet(text)
        fill_params(net.set_conv, net.layers, seed=31, bn="random")
        fill_params(onet.set_conv, onet.layers, seed=31, bn="random")
        x = synth.uniform01(8, net.inputs * net.batch)
        net.predict(x)
        want = onet.forward(x)
        for i in range(net.n):
            assert norm_err(net.layer_output(i), want[i]) <= REL_TOL, (softmax, i)
        head_in, head = net.layer_output(net.n - 2), net.layer_output(net.n - 1)
        L = onet.layers[-1]
        ncls = L["side"] ** 2 * L["classes"]
        assert np.array_equal(head[:, ncls:], head_in[:, ncls:])
        if softmax:
            again = onet.forward_layer(net.n - 1, head_in, None)      # the checker's head on the library's input
            assert np.abs(head - again).max() <= 1e-6
            assert np.allclose(head[:, :ncls].reshape(net.batch, -1, L["classes"]).sum(2), 1, atol=1e-5)
        else:
            assert np.array_equal(head, head_in)
        outs = [None] * (net.n - 1) + [head]
        for image in (0, 3, 4):
            got = net.get_boxes(120, 90, 0.05, 0, 0.0, image)
            assert np.array_equal(got, onet.get_boxes(outs, 120, 90, 0.05, 0, 0.0, image)), (softmax, image)
            got = net.get_boxes(120, 90, 0.02, 1, 0.4, image)
            assert np.array_equal(got, onet.get_boxes(outs, 120, 90, 0.02, 1, 0.4, image)), (softmax, image)
        assert np.array_equal(net.get_network_boxes(64, 64, 0.1), onet.get_boxes(outs, 64, 64, 0.1, 1, 0.0))
        net.free()


def test_yolov1_tiny_448(dn):
    from test_gpu_network import check_network
    from darknet_amd import cfgs
    assert check_network(cfgs.yolov1_tiny(2, 448)) <= REL_TOL


def test_yolov1_448_with_its_local_layer(dn):
    """The full network of cfg/yolov1.cfg: 24 convolutions, the 7x7x1024 -> 256 locally connected
    layer (115.6 M weights), dropout, connected, detection."""
    from test_gpu_network import check_network
    from darknet_amd import cfgs
    assert check_network(cfgs.yolov1(1, 448)) <= REL_TOL


STREAM_CASES = [  # batch, inputs, outputs, activation
    (1, 9216, 1000, "relu"),        # K a multiple of both chunk widths, ragged filter tile
    (3, 1000, 37, "linear"),        # ragged K: the last chunk is partial
    (4, 2500, 256, "leaky"),
    (5, 777, 130, "logistic"),      # the 16-image tile, ragged everything
    (16, 4096, 64, "leaky"),
    (17, 1030, 9, "linear"),        # two image groups, the second with one image
]


@pytest.mark.parametrize("batch,inputs,outputs,act", STREAM_CASES, ids=["b%d_%d_%d" % t[:3] for t in STREAM_CASES])
def test_connected_stream_against_checker(dn, orc, batch, inputs, outputs, act):
    x = synth.uniform(51, batch * inputs, -1, 1).reshape(batch, inputs)
    wt = synth.conv_weights(52, outputs, inputs, 1)
    bias = synth.uniform(53, outputs, -0.5, 0.5)
    want = orc.connected(x, wt, bias, outputs=outputs, batch_normalize=0, activation=act)
    guard = np.full(want.size + 64, 7.5, np.float32)
    dx, dw, db, out = D(x), D(wt), D(bias), D(guard)
    dn.forward_connected_stream_gpu(dx.ptr, dw.ptr, db.ptr, out.ptr, batch, inputs, outputs, ACTIVATIONS.index(act))
    got = out.numpy()
    assert np.array_equal(got[want.size:], guard[want.size:])
    assert norm_err(got[:want.size], want.reshape(-1)) <= REL_TOL


def test_connected_layer_takes_the_streaming_kernel_at_small_batches(dn):
    """The layer-level call: batch 2 (streaming kernel) and batch 32 (matrix cores) of the same
    head agree with the checker; with batch-norm the tiled kernel serves every batch."""
    from test_gpu_network import build_pair
    for batch in (2, 32):
        text = (f"[net]\nbatch={batch}\nsubdivisions=1\nwidth=4\nheight=4\nchannels=64\n"
                "[connected]\noutput=300\nactivation=leaky\n"
                "[connected]\noutput=50\nbatch_normalize=1\nactivation=linear\n")
        net, onet = build_pair(text, seed=61)
        x = synth.uniform(6, net.inputs * net.batch, -1, 1)
        net.predict(x)
        want = onet.forward(x)
        for i in range(net.n):
            assert norm_err(net.layer_output(i), want[i]) <= REL_TOL, (batch, i)
        net.free()
