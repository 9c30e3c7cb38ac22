"""The input side on the device (resize_image_gpu, letterbox_image_gpu, the reference-named host
calls and the letterbox straight into the network input) against the CPU checker: bit-exact."""
import os

import numpy as np
import pytest

from darknet_amd import api, cfgs, synth

from util import fill_params

pytestmark = pytest.mark.gpu
GOLD = os.path.join(os.path.dirname(__file__), "golden")
D = api.DeviceArray


def test_kernels_on_the_reference_golden_images(dn):
    g = np.load(os.path.join(GOLD, "image_cases.npz"))
    for n in [k[:-3] for k in g.files if k.endswith("_in")]:
        im, box, rs = g[n + "_in"], g[n + "_box"], g[n + "_resized"]
        c, h, w = im.shape
        src = D(im)
        out = D(n=box.size)
        dn.letterbox_image_gpu(src.ptr, w, h, c, out.ptr, box.shape[2], box.shape[1])
        assert np.array_equal(out.numpy(box.shape), box), n
        out2 = D(n=rs.size)
        dn.resize_image_gpu(src.ptr, w, h, c, out2.ptr, rs.shape[2], rs.shape[1])
        assert np.array_equal(out2.numpy(rs.shape), rs), n


@pytest.mark.parametrize("c,h,w,bw,bh", [(3, 480, 640, 416, 416), (3, 375, 500, 608, 608), (3, 1080, 1920, 416, 416),
                                         (1, 20, 10, 16, 24), (3, 30, 300, 64, 64), (3, 100, 100, 416, 416)])
def test_host_calls_match_checker(dn, orc, c, h, w, bw, bh):
    im = synth.uniform01(6, c * h * w).reshape(c, h, w)
    assert np.array_equal(api.letterbox_image(im, bw, bh), orc.letterbox_image(im, bw, bh))
    assert np.array_equal(api.resize_image(im, bw, bh), orc.resize_image(im, bw, bh))


def test_letterbox_into_the_network_input_and_predict_image(dn, orc):
    net = api.Network(cfg_text=cfgs.yolov3_tiny(3, 160))
    fill_params(net.set_conv, net.layers)
    frames = [synth.uniform01(40 + k, 3 * h * w).reshape(3, h, w) for k, (h, w) in enumerate([(120, 200), (300, 90),
                                                                                            (160, 160)])]
    for b, f in enumerate(frames):
        net.letterbox_input(b, f)
    boxed = np.stack([orc.letterbox_image(f, 160, 160) for f in frames])
    got = np.empty_like(boxed)                          # the network's own input buffer
    dn.hip_pull_array(net.L.network_input_gpu(net.net), api._fp(got), got.size)
    assert np.array_equal(got, boxed)
    # device-resident forward on those inputs == network_predict on the checker's letterboxed frames
    net.forward_device()
    net.synchronize()
    dev = net.layer_output(net.n - 1)
    assert np.array_equal(dev, net.predict(boxed))
    # network_predict_image: batch 1, letterbox on the device, same result as predicting the boxed frame
    # (the K-split of a small layer depends on the batch size, so the summation order does too:
    # equal to rounding, not bit for bit)
    one = net.predict_image(frames[1])
    assert np.abs(one[0] - dev[1]).max() <= 1e-5 * max(np.abs(dev[1]).max(), 1.0)
    net.free()
