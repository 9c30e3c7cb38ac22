"""The first-layer kernel (3x3, stride 1, pad 1 over 3 channels, or over the 16 channels behind a pooled
first layer) through the C-ABI: against the CPU
checker and the fp64 convolution as every convolution is, and its pooled forms against the separate
calls they stand for - forward_convolutional_gpu, forward_maxpool_gpu, xnor_pack_input_gpu - bit
for bit.  Widths of one to several 128-column tiles with and without a ragged last tile, two-row
images, 1 to 64 filters, batches whose tiles cross images, both signs of the batch-norm scale."""
import numpy as np
import pytest

from darknet_amd import api, cfgs, synth
from oracle.cpu import ACTIVATIONS

from util import REL_TOL, fill_params, norm_err

pytestmark = pytest.mark.gpu
D = api.DeviceArray


class First:
    def __init__(self, dn, seed, b, h, w, n, act="leaky", bn=1, c=3):
        self.dn, self.geom, self.act, self.bn, self.c = dn, (b, h, w, n), act, bn, c
        self.x = synth.uniform(seed, b * c * h * w).reshape(b, c, h, w)
        self.wt = synth.conv_weights(seed + 1, n, c, 3)
        self.bias, self.sc, self.mu, self.var = synth.bn_random(seed + 2, n)
        self.sc = self.sc.copy()
        self.sc[1::3] *= -1.0
        self.dev = [D(a) for a in (self.x, self.wt, self.bias, self.sc, self.mu, self.var)]

    def tail(self):
        b, h, w, n = self.geom
        return [b, self.c, h, w, n, 1, 3, 1, 1, self.bn, ACTIVATIONS.index(self.act)]

    GUARD = 256  # floats behind every output buffer that no kernel may touch

    def guarded(self, count, dtype=np.float32):
        """A device buffer of `count` elements plus GUARD sentinels behind it, all preset to a NaN pattern."""
        host = np.full(count + self.GUARD, 0x7FC0BEEF, np.uint32).view(dtype)
        return D(host, dtype=dtype)

    def unguard(self, dev, count):
        """The buffer's first `count` elements as uint32, after checking that the sentinels are intact."""
        bits = dev.numpy().view(np.uint32)
        assert (bits[count:] == 0x7FC0BEEF).all(), "a kernel wrote past the end of its output"
        return bits[:count].copy()

    def conv(self):
        b, h, w, n = self.geom
        d = self.dev
        count = b * n * h * w
        out = self.guarded(count)
        self.dn.forward_convolutional_gpu(d[0].ptr, d[1].ptr, None, d[2].ptr, d[3].ptr, d[4].ptr, d[5].ptr, out.ptr,
                                          *self.tail())
        return D(self.unguard(out, count).view(np.float32))

    def separate(self):
        b, h, w, n = self.geom
        out = self.conv()
        pooled = D(np.full(b * n * (h // 2) * (w // 2), np.nan, np.float32))
        self.dn.forward_maxpool_gpu(out.ptr, pooled.ptr, None, b, n, h, w, 2, 2, 1)
        bits = D(n=self.dn.xnor_input_words(b, n, h // 2, w // 2), dtype=np.int32)
        self.dn.xnor_pack_input_gpu(pooled.ptr, bits.ptr, b, n, h // 2, w // 2)
        return out.numpy().view(np.uint32), pooled.numpy().view(np.uint32), bits.numpy().view(np.uint32)

    def fused(self, write_map=True):
        b, h, w, n = self.geom
        d = self.dev
        n_map, n_pool, n_bits = b * n * h * w, b * n * (h // 2) * (w // 2), self.dn.xnor_input_words(b, n, h // 2, w // 2)
        out, pooled, bits = self.guarded(n_map), self.guarded(n_pool), self.guarded(n_bits, np.int32)
        self.dn.forward_convolutional_maxpool_gpu(d[0].ptr, d[1].ptr, d[2].ptr, d[3].ptr, d[4].ptr, d[5].ptr,
                                                  out.ptr if write_map else None, pooled.ptr, bits.ptr, *self.tail())
        return self.unguard(out, n_map), self.unguard(pooled, n_pool), self.unguard(bits, n_bits)


GEOMS = [(1, 2, 32, 16), (2, 6, 64, 32), (3, 10, 160, 17), (1, 16, 416, 32), (2, 8, 128, 64), (5, 4, 96, 33),
         (1, 34, 256, 1), (2, 12, 288, 48), (2, 8, 104, 24), (1, 4, 40, 64), (3, 6, 200, 9),
         (2, 416, 416, 16), (1, 416, 416, 32), (1, 448, 448, 64)]   # the first layers of yolov3-tiny, yolov3 and yolov1 at full size
# 16 channels, up to 32 filters: the second convolution of the tiny networks (16 -> 32 at 208 x 208)
GEOMS16 = [(1, 2, 32, 32), (2, 8, 64, 32), (1, 16, 208, 32), (3, 12, 128, 17), (2, 24, 96, 1), (1, 6, 160, 31),
           (2, 8, 56, 32), (1, 4, 104, 20), (2, 208, 208, 32)]   # the last: yolov3-tiny's second convolution at full size


@pytest.mark.parametrize("b,h,w,n", GEOMS)
def test_first_layer_against_the_checker(dn, orc, b, h, w, n):
    assert dn.conv_maxpool_fusable(b, 3, h, w, n, 1, 3, 1, 1, ACTIVATIONS.index("leaky")) == 1
    assert dn.conv_kernel_name_geometry(b, 3, h, w, n, 1, 3, 1, 1).decode().startswith("conv_first")
    cs = First(dn, 3, b, h, w, n)
    got = cs.conv().numpy((b, n, h, w))
    want = orc.conv(cs.x, cs.wt, cs.bias, cs.sc, cs.mu, cs.var, n=n, size=3, stride=1, pad=1, groups=1,
                    batch_normalize=1, activation="leaky")
    assert not np.isnan(got).any()
    assert norm_err(got, want) <= REL_TOL
    # the same layer on the generic kernel (conv_set_algo(3) leaves the first-layer kernels out), which pairs
    # the k of an MFMA differently: the same values to rounding
    dn.conv_set_algo(3)
    try:
        other = cs.conv().numpy((b, n, h, w))
    finally:
        dn.conv_set_algo(0)
    assert norm_err(got, other) <= 2e-6


@pytest.mark.parametrize("b,h,w,n", GEOMS)
@pytest.mark.parametrize("act,bn", [("leaky", 1), ("relu", 0), ("linear", 1)])
def test_first_layer_with_pool_and_bits_in_one_pass(dn, b, h, w, n, act, bn):
    cs = First(dn, 11, b, h, w, n, act=act, bn=bn)
    want_map, want_pool, want_bits = cs.separate()
    got_map, got_pool, got_bits = cs.fused()
    assert np.array_equal(got_map, want_map)
    assert np.array_equal(got_pool, want_pool)
    assert np.array_equal(got_bits, want_bits)
    lean_map, lean_pool, lean_bits = cs.fused(write_map=False)
    assert np.array_equal(lean_pool, want_pool) and np.array_equal(lean_bits, want_bits)
    assert np.isnan(lean_map.view(np.float32)).all()


@pytest.mark.parametrize("c,b,h,w,n", [(3, 2, 8, 128, 32), (3, 1, 16, 192, 17), (3, 3, 8, 64, 64), (3, 1, 24, 416, 33),
                                       (3, 2, 16, 256, 5), (16, 2, 8, 128, 32), (16, 1, 16, 192, 17), (16, 1, 24, 416, 9)])
def test_every_tile_shape_gives_the_same_bits(dn, c, b, h, w, n):
    """The tile is 2 x 128, 4 x 64 or 8 x 32 pixels by what divides the image; forced one after the other
    on images that allow several, the map, the pooled map and the bits are the same."""
    cs = First(dn, 23, b, h, w, n, c=c)
    results, names = [], set()
    try:
        for shape in (4, 2, 1):
            dn.conv_first_set_shape(shape)
            names.add(dn.conv_kernel_name_geometry(b, c, h, w, n, 1, 3, 1, 1).decode())
            results.append((cs.conv().numpy().view(np.uint32),) + cs.fused() + cs.fused(write_map=False)[1:])
    finally:
        dn.conv_first_set_shape(0)
    assert len(names) == 3, names                      # all three heights divide these images
    for other in results[1:]:
        for got, want in zip(other, results[0]):
            assert np.array_equal(got, want)
    assert np.array_equal(results[0][0], results[0][1])


def test_geometries_the_pair_does_not_serve(dn):
    leaky, logistic = ACTIVATIONS.index("leaky"), ACTIVATIONS.index("logistic")
    assert dn.conv_maxpool_fusable(1, 3, 416, 416, 16, 1, 3, 1, 1, logistic) == 0     # activation outside the tail
    assert dn.conv_maxpool_fusable(1, 3, 417, 416, 16, 1, 3, 1, 1, leaky) == 0        # odd height
    assert dn.conv_maxpool_fusable(1, 3, 416, 404, 16, 1, 3, 1, 1, leaky) == 0        # width not a multiple of 8
    assert dn.conv_maxpool_fusable(1, 3, 416, 416, 65, 1, 3, 1, 1, leaky) == 0        # more than 64 filters
    assert dn.conv_maxpool_fusable(1, 4, 416, 416, 16, 1, 3, 1, 1, leaky) == 0        # not 3 channels
    assert dn.conv_maxpool_fusable(1, 3, 416, 416, 16, 1, 3, 2, 1, leaky) == 0        # stride 2


def test_tiny_network_fused_equals_layer_by_layer(dn):
    """yolov3-tiny: first layer + maxpool in one pass (and in the xnor variant the sign bits for layer 2):
    every layer holds the bits of the layer-by-layer run; lean mode leaves only layer 0's map out."""
    for xnor in (False, True):
        net = api.Network(cfg_text=cfgs.yolov3_tiny(2, 160, xnor=xnor))
        fill_params(net.set_conv, net.layers)
        x = synth.uniform01(7, net.inputs * 2)
        try:
            dn.network_set_fusion(0)
            assert not any(dn.network_layer_runs_fused(net.net, i) for i in range(net.n))
            net.predict(x)
            want = [net.layer_output(i) for i in range(net.n)]
            dn.network_set_fusion(1)
            # what runs inside the convolution in front of it: the 2x2/2 maxpools behind the first layer, behind
            # the 16-channel second layer when it is an fp32 convolution and, in the xnor network, behind the
            # xnor convolutions (not the stride-1 pool 11), and the yolo heads
            # behind fp32 convolutions (in the xnor network only the last convolution is one)
            assert [i for i in range(net.n) if dn.network_layer_runs_fused(net.net, i)] == \
                ([1, 3, 5, 7, 9, 23] if xnor else [1, 3, 16, 23])
            assert not any(dn.network_layer_output_skipped(net.net, i) for i in range(net.n))
            net.predict(x)
            for i in range(net.n):
                assert np.array_equal(net.layer_output(i), want[i]), (xnor, i)
            dn.network_set_fusion(2)
            net.predict(x)
            skipped = [0, 2, 4, 6] if xnor else [0, 2]
            assert [i for i in range(net.n) if dn.network_layer_output_skipped(net.net, i)] == skipped
            for i in range(net.n):
                if i not in skipped:
                    assert np.array_equal(net.layer_output(i), want[i]), (xnor, i)
        finally:
            dn.network_set_fusion(1)
        net.free()


@pytest.mark.parametrize("b,h,w,n", GEOMS16)
def test_sixteen_channel_layer_against_the_checker(dn, orc, b, h, w, n):
    leaky = ACTIVATIONS.index("leaky")
    assert dn.conv_maxpool_fusable(b, 16, h, w, n, 1, 3, 1, 1, leaky) == 1
    assert dn.conv_maxpool_fusable(b, 16, h, w, 33, 1, 3, 1, 1, leaky) == 0     # a lane's registers hold 32 filters' weights
    name = dn.conv_kernel_name_geometry(b, 16, h, w, n, 1, 3, 1, 1).decode()
    assert name.startswith("conv_first_kernel") and name.endswith(",16>"), name
    cs = First(dn, 5, b, h, w, n, c=16)
    got = cs.conv().numpy((b, n, h, w))
    want = orc.conv(cs.x, cs.wt, cs.bias, cs.sc, cs.mu, cs.var, n=n, size=3, stride=1, pad=1, groups=1,
                    batch_normalize=1, activation="leaky")
    assert not np.isnan(got).any()
    assert norm_err(got, want) <= REL_TOL
    # exact on small integers: every product and partial sum is representable, so the order of the k pairs
    # (tap by tap over channels ch and ch + 8) cannot show
    xi = np.round(cs.x * 4).astype(np.float32)
    wi = np.round(cs.wt * 8).astype(np.float32)
    ones, zeros = np.ones(n, np.float32), np.zeros(n, np.float32)
    d = [D(a) for a in (xi, wi, zeros)]
    out = D(np.full(b * n * h * w, np.nan, np.float32))
    dn.forward_convolutional_gpu(d[0].ptr, d[1].ptr, None, d[2].ptr, None, None, None, out.ptr, b, 16, h, w, n, 1, 3, 1, 1,
                                 0, ACTIVATIONS.index("linear"))
    exact = orc.conv(xi.reshape(b, 16, h, w), wi, zeros, ones, zeros, ones, n=n, size=3, stride=1, pad=1, groups=1,
                     batch_normalize=0, activation="linear")
    assert np.array_equal(out.numpy((b, n, h, w)), exact)


@pytest.mark.parametrize("b,h,w,n", GEOMS16)
@pytest.mark.parametrize("act,bn", [("leaky", 1), ("linear", 0)])
def test_sixteen_channel_layer_with_pool_and_bits_in_one_pass(dn, b, h, w, n, act, bn):
    cs = First(dn, 13, b, h, w, n, act=act, bn=bn, c=16)
    want_map, want_pool, want_bits = cs.separate()
    got_map, got_pool, got_bits = cs.fused()
    assert np.array_equal(got_map, want_map)
    assert np.array_equal(got_pool, want_pool)
    assert np.array_equal(got_bits, want_bits)
    lean_map, lean_pool, lean_bits = cs.fused(write_map=False)
    assert np.array_equal(lean_pool, want_pool) and np.array_equal(lean_bits, want_bits)
    assert np.isnan(lean_map.view(np.float32)).all()


def test_tiny_network_at_416_batch_64_fused_equals_layer_by_layer(dn):
    """The benchmark size: both pooled first layers (3 -> 16 and 16 -> 32 with their maxpools) and both yolo
    heads of yolov3-tiny hold the bits of the layer-by-layer run at fusion levels 1 and 2."""
    net = api.Network(cfg_text=cfgs.yolov3_tiny(64, 416))
    fill_params(net.set_conv, net.layers)
    x = synth.uniform01(9, net.inputs * 64)
    watch = [1, 3] + [i for i, L in enumerate(net.layers) if L["type"] == "yolo"]
    try:
        dn.network_set_fusion(0)
        net.predict(x)
        want = {i: net.layer_output(i) for i in watch}
        for level in (1, 2):
            dn.network_set_fusion(level)
            net.predict(x)
            for i in watch:
                assert np.array_equal(net.layer_output(i), want[i]), (level, i)
    finally:
        dn.network_set_fusion(1)
    net.free()


def random_first_layers(seed, count):
    rng = np.random.default_rng(seed)
    out = []
    for _ in range(count):
        c = int(rng.choice([3, 3, 16]))
        n = int(rng.integers(1, 65 if c == 3 else 33))
        h = 2 * int(rng.integers(1, 21))
        w = 8 * int(rng.integers(4, 38))
        b = int(rng.integers(1, 5))
        act, bn = [("leaky", 1), ("linear", 0), ("relu", 1)][int(rng.integers(0, 3))]
        out.append((c, b, h, w, n, act, bn))
    return out


@pytest.mark.parametrize("c,b,h,w,n,act,bn", random_first_layers(20250, 32))
def test_random_first_layers(dn, orc, c, b, h, w, n, act, bn):
    """Random heights, widths (any multiple of 8: short last tiles, every tile shape the height allows), filter
    counts and batches: the map against the checker, the one-pass pooled forms against the separate calls."""
    cs = First(dn, 77, b, h, w, n, act=act, bn=bn, c=c)
    want_map, want_pool, want_bits = cs.separate()
    args = (cs.x, cs.wt, cs.bias, cs.sc, cs.mu, cs.var) if bn else (cs.x, cs.wt, cs.bias)
    ref = orc.conv(*args, n=n, size=3, stride=1, pad=1, groups=1, batch_normalize=bn, activation=act)
    assert norm_err(want_map.view(np.float32).reshape(b, n, h, w), ref) <= REL_TOL
    got_map, got_pool, got_bits = cs.fused()
    assert np.array_equal(got_map, want_map) and np.array_equal(got_pool, want_pool) and np.array_equal(got_bits, want_bits)
    lean = cs.fused(write_map=False)
    assert np.array_equal(lean[1], want_pool) and np.array_equal(lean[2], want_bits)

