"""Every benchmark configuration at the batch size it is quoted on.

The CPU checker needs seconds per image on these networks, so a whole batch cannot be checked
against it directly.  Instead: (a) single layers at batch 64 are compared with the checker on a
subset of their images; (b) for whole networks, image k of the batch must equal the batch-1
forward of that image, which the checker verifies layer by layer elsewhere
(test_gpu_network.py: yolov3-416 / 608 / tiny, resnext50) - images of a batch are independent in
every layer of the path, and the batch size changes the tile schedule and the K-split, i.e. the
code path, not the mathematics; (c) XNOR layers at batch 64 get the checker's own input injected,
layer by layer (an end-to-end comparison of a binarised network is ill-posed: ties at zero flip
signs between summation orders)."""
import numpy as np
import pytest

from darknet_amd import api, cfgs, synth
from oracle.cpu import ACTIVATIONS
from oracle.net import OracleNet

from util import REL_TOL, YOLO_ABS_TOL, fill_params, norm_err

pytestmark = pytest.mark.gpu
D = api.DeviceArray

# the same image at two batch sizes: only the summation order over K may differ
SAME_IMAGE_TOL = 2e-5


def conv_layer_gpu(dn, x, wt, bias, sc, mu, var, n, size, stride, pad):
    b, c, h, w = x.shape
    oh, ow = (h + 2 * pad - size) // stride + 1, (w + 2 * pad - size) // stride + 1
    dev = [D(a) for a in (x, wt, bias, sc, mu, var)]
    out = D(n=b * n * oh * ow)
    pk = D(n=dn.conv_packed_floats(n, c, 1, size))
    dn.conv_pack_weights_gpu(dev[1].ptr, pk.ptr, n, c, 1, size)
    dn.forward_convolutional_gpu(dev[0].ptr, dev[1].ptr, pk.ptr, dev[2].ptr, dev[3].ptr, dev[4].ptr, dev[5].ptr,
                                 out.ptr, b, c, h, w, n, 1, size, stride, pad, 1, ACTIVATIONS.index("leaky"))
    return out.numpy((b, n, oh, ow))


@pytest.mark.parametrize("name", sorted(cfgs.SWEEP))
@pytest.mark.parametrize("batch", [1, 64])
def test_single_layer_sweep_at_batch_1_and_64(dn, orc, name, batch):
    """The three single-layer shapes (3x3 s1 256->512 @26, 1x1 512->256 @52, 3x3 s2 128->256 @104,
    batch-norm + leaky, activations and weights uniform(-1,1)) against the checker: every image at
    batch 1, images 0 / 37 / 63 at batch 64."""
    c, h, w, n, size, stride = cfgs.SWEEP[name]
    pad = size // 2
    x = synth.uniform(11, batch * c * h * w).reshape(batch, c, h, w)
    wt = synth.uniform(12, n * c * size * size).reshape(n, c, size, size)
    bias, sc, mu, var = synth.bn_random(13, n)
    got = conv_layer_gpu(dn, x, wt, bias, sc, mu, var, n, size, stride, pad)
    for k in ([0] if batch == 1 else [0, 37, 63]):
        want = orc.conv(x[k:k + 1], wt, bias, sc, mu, var, n=n, size=size, stride=stride, pad=pad, groups=1,
                        batch_normalize=1, activation="leaky")
        assert norm_err(got[k:k + 1], want) <= REL_TOL, (name, batch, k)


def batch_equals_batch_1(make_cfg, batch, images, layers=None, bn="identity"):
    """Image k of a batch-`batch` forward against the batch-1 forward of the same image."""
    net_b, net_1 = api.Network(cfg_text=make_cfg(batch)), api.Network(cfg_text=make_cfg(1))
    fill_params(net_b.set_conv, net_b.layers, bn=bn)
    fill_params(net_1.set_conv, net_1.layers, bn=bn)
    x = synth.uniform01(5, net_b.inputs * batch).reshape(batch, -1)
    net_b.predict(x)
    idx = list(range(net_b.n)) if layers is None else layers
    outs = {i: net_b.layer_output(i)[images] for i in idx}   # one pull per layer, the images of interest kept
    worst = 0.0
    for j, k in enumerate(images):
        net_1.predict(x[k])
        for i in idx:
            L = net_b.layers[i]
            a, b1 = outs[i][j], net_1.layer_output(i)[0]
            if L["type"] == "yolo":
                assert np.abs(a - b1).max() <= YOLO_ABS_TOL, (k, i)
            e = norm_err(a, b1)
            worst = max(worst, e)
            assert e <= SAME_IMAGE_TOL, (k, i, L["type"], e)
    net_b.free()
    net_1.free()
    return worst


def test_yolov3_416_batch_8(dn):
    batch_equals_batch_1(lambda b: cfgs.yolov3(b, 416), 8, [0, 5, 7])


def test_yolov3_608_batch_8(dn):
    batch_equals_batch_1(lambda b: cfgs.yolov3(b, 608), 8, [2, 7])


def test_yolov3_416_batch_64(dn):
    """The headline configuration: three images of the batch, per layer at the same-image tolerance,
    on the first layers, two layers of every scale (a 1x1 and a 3x3, with their fused shortcuts),
    the neck and the three heads."""
    batch_equals_batch_1(lambda b: cfgs.yolov3(b, 416), 64, [0, 40, 63],
                         layers=[0, 1, 2, 3, 4, 5, 11, 12, 13, 14, 15, 36, 37, 38, 39, 40, 61, 62, 63, 64, 65, 74,
                                 79, 80, 81, 82, 84, 85, 86, 87, 93, 94, 96, 97, 98, 99, 105, 106])


def test_yolov3_608_batch_64(dn):
    """The largest configuration (30 GB of layer outputs): the three yolo heads, the first
    layers and one layer of every scale, for two images."""
    batch_equals_batch_1(lambda b: cfgs.yolov3(b, 608), 64, [1, 63], layers=[0, 1, 4, 11, 36, 61, 74, 81, 82, 93, 94, 105, 106])


def test_resnext50_224_batch_64(dn):
    batch_equals_batch_1(lambda b: cfgs.resnext50(b, 224), 64, [0, 33, 63], bn="random")


def test_yolov3_tiny_xnor_416_batch_64(dn):
    """binary=1 xnor=1 on every conv but the first and the last, at 416x416 and batch 64.  The
    checker runs four images; the batch of 64 holds them in a scrambled order (image j = checker
    image (5j + 3) mod 4), and every XNOR layer is fed the checker's input for its images and
    compared with the checker's output for them.  Then the whole network runs at batch 64."""
    text4 = cfgs.yolov3_tiny(4, 416, xnor=True)
    orc = OracleNet(text4)
    fill_params(orc.set_conv, orc.layers)
    x4 = synth.uniform01(7, orc.net["inputs"] * 4)
    want = orc.forward(x4)
    perm = np.array([(5 * j + 3) % 4 for j in range(64)])
    lib = api._lib.load()
    checked = 0
    for i, L in enumerate(orc.layers):
        if L["type"] != "convolutional" or not L["xnor"]:
            continue
        wt, bias, sc, mu, var = orc.params[i]
        xin = np.ascontiguousarray(want[i - 1].reshape(4, L["c"], L["h"], L["w"])[perm])
        b, c, h, w = xin.shape
        n, size, stride, pad = L["n"], L["size"], L["stride"], L["pad"]
        oh, ow = (h + 2 * pad - size) // stride + 1, (w + 2 * pad - size) // stride + 1
        dev = [D(a) if a is not None else None for a in (xin, wt, bias, sc, mu, var)]
        ptr = [d.ptr if d else None for d in dev]
        wbits = D(n=lib.xnor_weight_words(n, c, size), dtype=np.int32)
        xbits = D(n=lib.xnor_input_words(b, c, h, w), dtype=np.int32)
        wmean, out = D(n=n), D(n=b * n * oh * ow)
        lib.forward_convolutional_xnor_gpu(ptr[0], ptr[1], wbits.ptr, wmean.ptr, xbits.ptr, ptr[2], ptr[3], ptr[4],
                                           ptr[5], out.ptr, b, c, h, w, n, size, stride, pad,
                                           0 if sc is None else 1, ACTIVATIONS.index(L["activation"]))
        got = out.numpy((64, -1))
        ref = want[i].reshape(4, -1)[perm]
        assert norm_err(got, ref) <= REL_TOL, i
        checked += 1
    assert checked == 11
    # the whole network at batch 64 through parse_network_cfg / network_predict
    net = api.Network(cfg_text=cfgs.yolov3_tiny(64, 416, xnor=True))
    fill_params(net.set_conv, net.layers)
    out = net.predict(np.ascontiguousarray(x4.reshape(4, -1)[perm]))
    assert np.isfinite(out).all()
    # images that hold the same input give the same result wherever they sit in the batch (XNOR sums
    # are integers; the fp32 layers at both ends may sum K in another order for another column)
    first = net.layer_output(net.n - 1)
    for j in (1, 17, 63):
        twin = int(np.flatnonzero(perm == perm[j])[0])
        assert np.abs(first[j] - first[twin]).max() <= 1e-5, j
    # at this size too, the passes that run several layers in one launch (first layer + maxpool + sign bits,
    # xnor convolution + maxpool + sign bits) leave the bits of the layer-by-layer run in both yolo heads, and
    # so does the mode that does not write the maps only a fused maxpool reads
    heads = [i for i, L in enumerate(net.layers) if L["type"] == "yolo"]
    xin = np.ascontiguousarray(x4.reshape(4, -1)[perm])
    try:
        lib.network_set_fusion(0)
        net.predict(xin)
        plain = [net.layer_output(i) for i in heads]
        for level in (1, 2):
            lib.network_set_fusion(level)
            net.predict(xin)
            for i, ref in zip(heads, plain):
                assert np.array_equal(net.layer_output(i), ref), (level, i)
    finally:
        lib.network_set_fusion(1)
    net.free()
