"""XNOR layers: bit-exact sign/pack stage, layer output within tolerance, one layer at a time
with the CPU checker's input injected (end-to-end comparison of an XNOR network is ill-posed:
exact ties at zero flip sign between fp32 summation orders and the next layer binarises them)."""
import os

import numpy as np
import pytest

from darknet_amd import api, cfgs, synth
from oracle.cpu import ACTIVATIONS
from oracle.net import OracleNet

from util import REL_TOL, fill_params, norm_err

pytestmark = pytest.mark.gpu
GOLD = os.path.join(os.path.dirname(__file__), "golden")
D = api.DeviceArray


def xnor_layer(dn, x, wt, bias, sc, mu, var, n, size, stride, pad, act="leaky"):
    b, c, h, w = x.shape
    oh = (h + 2 * pad - size) // stride + 1
    ow = (w + 2 * pad - size) // stride + 1
    bn = 0 if sc is None else 1
    keep = [D(x), D(wt), D(bias)] + [D(a) if a is not None else None for a in (sc, mu, var)]
    wbits = D(n=dn.xnor_weight_words(n, c, size), dtype=np.int32)
    xbits = D(n=dn.xnor_input_words(b, c, h, w), dtype=np.int32)
    wmean, out = D(n=n), D(n=b * n * oh * ow)
    dn.forward_convolutional_xnor_gpu(keep[0].ptr, keep[1].ptr, wbits.ptr, wmean.ptr, xbits.ptr, keep[2].ptr,
                                      *[k.ptr if k else None for k in keep[3:]], out.ptr, b, c, h, w, n, size,
                                      stride, pad, bn, ACTIVATIONS.index(act))
    return (out.numpy((b, n, oh, ow)), wbits.numpy().view(np.uint32), xbits.numpy().view(np.uint32),
            wmean.numpy())


def pack_bits(sign_pos, axis_len):
    """bit j of word k <-> channel 32k + j."""
    cw = (axis_len + 31) // 32
    padded = np.zeros(sign_pos.shape[:-1] + (cw * 32,), np.uint8)
    padded[..., :axis_len] = sign_pos
    return np.packbits(padded.reshape(sign_pos.shape[:-1] + (cw, 32)), axis=-1, bitorder="little").view(np.uint32)[..., 0]


@pytest.mark.parametrize("b,c,h,w,n,size,stride", [(2, 32, 9, 9, 24, 3, 1), (1, 48, 13, 13, 40, 3, 1),
                                                   (2, 64, 12, 12, 32, 3, 2), (2, 100, 7, 7, 17, 1, 1)])
def test_xnor_pack_bits_and_layer_output(dn, orc, b, c, h, w, n, size, stride):
    pad = size // 2
    x = synth.uniform(9, b * c * h * w).reshape(b, c, h, w)
    x.reshape(-1)[::17] = 0.0
    wt = synth.conv_weights(1, n, c, size)
    wt[3] = 0.0
    bias, sc, mu, var = synth.bn_random(2, n)
    want, bw, bi = orc.conv(x, wt, bias, sc, mu, var, n=n, size=size, stride=stride, pad=pad, batch_normalize=1,
                            activation="leaky", xnor=1, return_binary=True)
    got, wbits, xbits, wmean = xnor_layer(dn, x, wt, bias, sc, mu, var, n, size, stride, pad)
    # sign/pack stage: bit-exact against the CPU checker's binarised tensors
    want_x = pack_bits((bi.reshape(b, c, h * w) > 0).transpose(0, 2, 1), c)          # [b][hw][cw]
    assert np.array_equal(xbits.reshape(b, -1, h * w).transpose(0, 2, 1), want_x)
    want_w = pack_bits((bw.reshape(n, c, size * size) > 0).transpose(0, 2, 1), c)     # [n][tap][cw]
    # device layout: [tap][slice][n padded to 16], then the per-(filter, tap) popcounts
    cw, npad, ss = (c + 31) // 32, (n + 15) // 16 * 16, size * size
    dev_w = wbits[:ss * cw * npad].reshape(ss, cw, npad)
    assert np.array_equal(dev_w[:, :, :n].transpose(2, 0, 1), want_w) and not dev_w[:, :, n:].any()
    pops = np.array([[sum(bin(int(v)).count("1") for v in want_w[f, t]) for t in range(ss)] for f in range(n)])
    assert np.array_equal(wbits[ss * cw * npad:].view(np.int32).reshape(n, ss), pops)
    assert np.array_equal(wmean, np.abs(bw.reshape(n, -1))[:, 0])                     # mean|w| per filter
    assert norm_err(got, want) <= REL_TOL


def test_xnor_golden_case(dn):
    g = np.load(os.path.join(GOLD, "xnor_case.npz"))
    L = [{"type": "convolutional", "n": 24, "c": 32, "groups": 1, "size": 3, "batch_normalize": 1}]
    params = {}
    fill_params(lambda i, *a: params.update(p=a), L, seed=33, bn="random")
    wt, bias, sc, mu, var = params["p"]
    got, wbits, xbits, wmean = xnor_layer(dn, g["input"].reshape(2, 32, 9, 9), wt, bias, sc, mu, var, 24, 3, 1, 1)
    assert norm_err(got.reshape(2, -1), g["output"]) <= REL_TOL
    assert np.array_equal(xbits.reshape(2, 1, 81)[:, 0], pack_bits((g["binary_input"].reshape(2, 32, 81) > 0).transpose(0, 2, 1), 32)[..., 0])


def test_xnor_network_layer_by_layer_with_injected_inputs(dn):
    """yolov3-tiny with binary=1 xnor=1 on every conv but the first and the last: each XNOR layer
    is fed the CPU checker's input for that layer."""
    text = cfgs.yolov3_tiny(2, 160, xnor=True)
    orc = OracleNet(text)
    fill_params(orc.set_conv, orc.layers)
    x = synth.uniform01(7, orc.net["inputs"] * 2)
    want = orc.forward(x)
    checked = 0
    for i, L in enumerate(orc.layers):
        if L["type"] != "convolutional" or not L["xnor"]:
            continue
        wt, bias, sc, mu, var = orc.params[i]
        xin = want[i - 1].reshape(2, L["c"], L["h"], L["w"])
        got, _, _, _ = xnor_layer(dn, xin, wt, bias, sc, mu, var, L["n"], L["size"], L["stride"], L["pad"],
                                  L["activation"])
        assert norm_err(got.reshape(2, -1), want[i]) <= REL_TOL, i
        checked += 1
    assert checked == 11      # 13 convs minus the first and the last
    # the whole network also runs through parse_network_cfg / network_predict; reported, not gated
    net = api.Network(cfg_text=text)
    fill_params(net.set_conv, net.layers)
    out = net.predict(x)
    print("\n  end-to-end xnor tiny: max|hip-cpu| on the last yolo head =", float(np.abs(out - want[-1]).max()))
    assert np.isfinite(out).all()
    net.free()


class FusedCase:
    """One xnor convolution through forward_convolutional_xnor_fused_gpu and through the separate
    calls it stands for (packed convolution, maxpool, input pack of the next layer)."""

    def __init__(self, dn, seed, b, c, h, w, n, size, act="leaky", negative_scales=True, bn=1):
        self.dn, self.geom = dn, (b, c, h, w, n, size)
        pad = size // 2
        self.pad = pad
        self.x = synth.uniform(seed, b * c * h * w).reshape(b, c, h, w)
        self.x.reshape(-1)[::13] = 0.0
        wt = synth.conv_weights(seed + 1, n, c, size)
        bias, sc, mu, var = synth.bn_random(seed + 2, n)
        if negative_scales:
            sc = sc.copy()
            sc[::3] *= -1.0            # a falling tail: the lean form must take the smallest dot product
        self.act, self.bn = ACTIVATIONS.index(act), bn
        self.dev = [D(a) for a in (self.x, wt, bias, sc, mu, var)]
        self.wbits = D(n=dn.xnor_weight_words(n, c, size), dtype=np.int32)
        self.wmean = D(n=n)
        dn.xnor_pack_weights_gpu(self.dev[1].ptr, self.wbits.ptr, self.wmean.ptr, n, c, size)
        self.xbits = D(n=dn.xnor_input_words(b, c, h, w), dtype=np.int32)

    def tail_args(self):
        b, c, h, w, n, size = self.geom
        return [b, c, h, w, n, size, 1, self.pad, self.bn, self.act]

    def separate(self, pool):
        """-> conv map, pooled map (or None), sign bits of the last of the two."""
        dn = self.dn
        b, c, h, w, n, size = self.geom
        d = self.dev
        out = D(np.full(b * n * h * w, np.nan, np.float32))
        dn.forward_convolutional_xnor_packed_gpu(d[0].ptr, self.wbits.ptr, self.wmean.ptr, self.xbits.ptr, d[2].ptr,
                                                 d[3].ptr, d[4].ptr, d[5].ptr, out.ptr, *self.tail_args())
        last, lh, lw, pooled = out, h, w, None
        if pool:
            pooled = D(np.full(b * n * (h // 2) * (w // 2), np.nan, np.float32))
            dn.forward_maxpool_gpu(out.ptr, pooled.ptr, None, b, n, h, w, 2, 2, 1)
            last, lh, lw = pooled, h // 2, w // 2
        bits = D(n=dn.xnor_input_words(b, n, lh, lw), dtype=np.int32)
        dn.xnor_pack_input_gpu(last.ptr, bits.ptr, b, n, lh, lw)
        return (out.numpy().view(np.uint32), pooled.numpy().view(np.uint32) if pool else None,
                bits.numpy().view(np.uint32))

    def fused(self, pool, write_map=True, ready=False):
        dn = self.dn
        b, c, h, w, n, size = self.geom
        d = self.dev
        out = D(np.full(b * n * h * w, np.nan, np.float32))
        pooled = D(np.full(b * n * (h // 2) * (w // 2), np.nan, np.float32)) if pool else None
        lh, lw = (h // 2, w // 2) if pool else (h, w)
        bits = D(np.full(dn.xnor_input_words(b, n, lh, lw), -1, np.int32))     # poisoned: every word must be written
        dn.forward_convolutional_xnor_fused_gpu(None if ready else d[0].ptr, self.wbits.ptr, self.wmean.ptr,
                                                self.xbits.ptr, 1 if ready else 0, d[2].ptr, d[3].ptr, d[4].ptr,
                                                d[5].ptr, out.ptr if write_map else None,
                                                pooled.ptr if pool else None, bits.ptr, *self.tail_args())
        return (out.numpy().view(np.uint32), pooled.numpy().view(np.uint32) if pool else None,
                bits.numpy().view(np.uint32))


@pytest.mark.parametrize("b,c,h,w,n", [(3, 16, 16, 12, 32), (2, 64, 26, 26, 48), (1, 40, 8, 8, 17), (2, 32, 52, 52, 64)])
@pytest.mark.parametrize("act", ["leaky", "linear", "logistic"])
def test_xnor_convolution_pool_and_next_bits_in_one_pass(dn, b, c, h, w, n, act):
    """The pooled kernel against the three calls it replaces: the convolution's map, the 2x2/2
    maximum and the sign bits of the pooled map, bit for bit; the lean form (map not written)
    gives the same pooled map and bits with scales of both signs; and the bits a fused call left in
    xbits serve a second call that reads no input."""
    cs = FusedCase(dn, 5, b, c, h, w, n, 3, act=act)
    want_map, want_pool, want_bits = cs.separate(pool=True)
    got_map, got_pool, got_bits = cs.fused(pool=True)
    assert np.array_equal(got_map, want_map)
    assert np.array_equal(got_pool, want_pool)
    assert np.array_equal(got_bits, want_bits)
    lean_map, lean_pool, lean_bits = cs.fused(pool=True, write_map=False)
    assert np.array_equal(lean_pool, want_pool) and np.array_equal(lean_bits, want_bits)
    assert np.isnan(lean_map.view(np.float32)).all()            # untouched
    again = cs.fused(pool=True, ready=True)                     # xbits as the previous calls left it
    assert np.array_equal(again[0], want_map) and np.array_equal(again[1], want_pool)


@pytest.mark.parametrize("b,c,h,w,n,size", [(2, 32, 13, 13, 255, 1), (2, 96, 13, 13, 40, 3), (1, 16, 9, 7, 16, 3),
                                            (3, 512, 5, 5, 33, 1)])
def test_xnor_convolution_writes_the_next_layers_bits(dn, b, c, h, w, n, size):
    cs = FusedCase(dn, 8, b, c, h, w, n, size)
    want_map, _, want_bits = cs.separate(pool=False)
    got_map, _, got_bits = cs.fused(pool=False)
    assert np.array_equal(got_map, want_map)
    assert np.array_equal(got_bits, want_bits)


def test_xnor_network_fused_equals_layer_by_layer(dn):
    """yolov3-tiny-xnor through the network loop: with the pairing on (convolution + maxpool in one
    pass, sign bits handed from layer to layer) every layer holds the bits of the layer-by-layer
    run; in lean mode every layer but the maps that are not written does."""
    text = cfgs.yolov3_tiny(3, 160, xnor=True)
    net = api.Network(cfg_text=text)
    fill_params(net.set_conv, net.layers)
    x = synth.uniform01(7, net.inputs * 3)
    try:
        dn.network_set_fusion(0)
        net.predict(x)
        want = [net.layer_output(i) for i in range(net.n)]
        dn.network_set_fusion(1)
        net.predict(x)
        for i in range(net.n):
            assert np.array_equal(net.layer_output(i), want[i]), i
        dn.network_set_fusion(2)
        net.predict(x)
        skipped = [i for i, L in enumerate(net.layers)
                   if L["type"] == "convolutional" and net.layers[i + 1]["type"] == "maxpool"
                   and net.layers[i + 1]["stride"] == 2 and i != 8]         # layer 8 is also read by a route
        assert skipped == [0, 2, 4, 6]                                      # the first layer pairs with its pool too
        for i in range(net.n):
            if i not in skipped:
                assert np.array_equal(net.layer_output(i), want[i]), i
    finally:
        dn.network_set_fusion(1)
    net.free()
