"""Parity of the convolution kernels against the CPU checker through the C-ABI.

Gate (the contract's "within 1e-4 relative of the fp32 reference"): per layer,
max|hip - cpu| / max|cpu| <= 1e-4, with the fp64 direct convolution as referee for both fp32
summation orders.  Shapes cover every kernel variant and tile edge: tap-blocked 1x1 / 3x3
(stride 1 and 2), the reference-order kernels (3 input channels, 7x7, odd channel counts), ragged
M (255), K not a multiple of 16 (27), N not a multiple of the tile, columns crossing images,
grouped convolutions, all three tile shapes (M <= 32, <= 64, > 64)."""
import os

import numpy as np
import pytest

from darknet_amd import api, cfgs, synth
from oracle.cpu import ACTIVATIONS

from util import REL_TOL, fill_params, norm_err

pytestmark = pytest.mark.gpu
GOLD = os.path.join(os.path.dirname(__file__), "golden")
D = api.DeviceArray


def run_conv(dn, x, wt, bias, sc, mu, var, *, n, size, stride, pad, groups, bn, act, packed=True):
    b, c, h, w = x.shape
    oh = (h + 2 * pad - size) // stride + 1
    ow = (w + 2 * pad - size) // stride + 1
    keep = [D(x), D(wt), D(bias)] + [D(a) if a is not None else None for a in (sc, mu, var)]
    out = D(n=b * n * oh * ow)
    pf = dn.conv_packed_floats(n, c, groups, size)
    pk = None
    if packed and pf:
        pk = D(n=pf)
        dn.conv_pack_weights_gpu(keep[1].ptr, pk.ptr, n, c, groups, size)
    dn.forward_convolutional_gpu(keep[0].ptr, keep[1].ptr, pk.ptr if pk else None, keep[2].ptr,
                                 keep[3].ptr if keep[3] else None, keep[4].ptr if keep[4] else None,
                                 keep[5].ptr if keep[5] else None, out.ptr, b, c, h, w, n, groups, size, stride,
                                 pad, bn, ACTIVATIONS.index(act))
    return out.numpy((b, n, oh, ow))


SHAPES = [  # b, c, h, w, n, size, stride, pad, groups, act
    (2, 256, 26, 26, 512, 3, 1, 1, 1, "leaky"),     # sweep (i)
    (2, 512, 52, 52, 256, 1, 1, 0, 1, "leaky"),     # sweep (ii)
    (2, 128, 104, 104, 256, 3, 2, 1, 1, "leaky"),   # sweep (iii)
    (3, 3, 41, 37, 32, 3, 1, 1, 1, "leaky"),        # K = 27, reference K order, BM = 32
    (2, 32, 30, 30, 64, 3, 2, 1, 1, "leaky"),       # BM = 64
    (1, 64, 19, 19, 32, 1, 1, 0, 1, "leaky"),
    (2, 1024, 13, 13, 255, 1, 1, 0, 1, "linear"),   # detection head: ragged M, no BN
    (5, 16, 7, 9, 130, 3, 1, 1, 1, "logistic"),     # tiny images: tile columns cross images
    (1, 3, 38, 40, 64, 7, 2, 3, 1, "leaky"),        # 7x7 stem
    (2, 20, 11, 11, 48, 3, 1, 1, 1, "leaky"),       # c % 16 != 0 -> reference K order
    (2, 48, 9, 9, 40, 3, 1, 0, 1, "relu"),          # 3x3 without padding -> direct kernel
    (2, 128, 14, 14, 128, 3, 1, 1, 32, "leaky"),    # resnext grouped 3x3, 4 channels per group
    (2, 256, 14, 14, 256, 3, 2, 1, 32, "leaky"),    # grouped, stride 2
    (1, 16, 1, 1, 16, 3, 1, 1, 1, "leaky"),         # 1x1 image
    (2, 512, 7, 7, 512, 3, 1, 1, 32, "leaky"),      # grouped, 16 per group (block-diagonal MFMA tiles)
    (1, 1024, 9, 7, 1024, 3, 2, 1, 32, "leaky"),    # grouped, 32 per group: one group per tile, stride 2
    (3, 64, 10, 10, 64, 1, 1, 0, 16, "linear"),     # grouped 1x1, 4 per group
    (2, 64, 12, 12, 64, 3, 1, 1, 64, "relu"),       # depthwise: 1 per group
    (2, 48, 9, 9, 96, 3, 1, 1, 3, "leaky"),         # 16 channels -> 32 filters per group: direct kernel
    (2, 96, 9, 9, 96, 3, 1, 1, 2, "leaky"),         # 48 per group: direct kernel
    (2, 3, 16, 16, 32, 3, 1, 1, 1, "leaky"),        # first-layer kernel (3 channels, pixels a multiple of 256)
    (1, 3, 32, 24, 16, 3, 1, 1, 1, "leaky"),        # the same with 16 filters (half a filter block)
    (3, 3, 16, 48, 64, 3, 1, 1, 1, "linear"),       # two filter blocks, tiles of 5.3 rows
    (1, 3, 64, 20, 20, 3, 1, 1, 1, "relu"),         # ragged filter count, narrow image (13 rows per tile)
    (2, 3, 8, 512, 8, 3, 1, 1, 1, "leaky"),         # rows longer than a tile
]


@pytest.mark.parametrize("b,c,h,w,n,size,stride,pad,groups,act", SHAPES)
@pytest.mark.parametrize("bn", [1, 0])
def test_conv_layer_parity(dn, orc, b, c, h, w, n, size, stride, pad, groups, act, bn):
    x = synth.uniform(1, b * c * h * w).reshape(b, c, h, w)
    wt = synth.conv_weights(2, n, c // groups, size)
    bias, sc, mu, var = synth.bn_random(3, n)
    if not bn:
        sc = mu = var = None
    want = orc.conv(x, wt, bias, sc, mu, var, n=n, size=size, stride=stride, pad=pad, groups=groups,
                    batch_normalize=bn, activation=act)
    got = run_conv(dn, x, wt, bias, sc, mu, var, n=n, size=size, stride=stride, pad=pad, groups=groups, bn=bn,
                   act=act)
    assert norm_err(got, want) <= REL_TOL
    ref64 = orc.conv_f64(x, wt, bias, sc, mu, var, n=n, size=size, stride=stride, pad=pad, groups=groups,
                         batch_normalize=bn, activation=act)
    assert norm_err(got, ref64) <= 5e-6      # the MFMA order sits as close to fp64 as the CPU order
    # measured error is reported for the record
    print(f"\n  {size}x{size}/{stride} {c}->{n} @{w}x{h} g{groups} bn{bn}: vs cpu {norm_err(got, want):.2e}, "
          f"vs fp64 {norm_err(got, ref64):.2e}, cpu vs fp64 {norm_err(want, ref64):.2e}")


def test_conv_exact_on_small_integers(dn, orc):
    """Integer data: every partial sum is exact in fp32, so any order gives the same bits."""
    rng = np.random.default_rng(0)
    b, c, h, w, n = 2, 32, 12, 12, 64
    x = rng.integers(-4, 5, (b, c, h, w)).astype(np.float32)
    wt = rng.integers(-3, 4, n * c * 9).astype(np.float32)
    bias = rng.integers(-5, 6, n).astype(np.float32)
    want = orc.conv(x, wt, bias, n=n, size=3, stride=1, pad=1, activation="linear")
    got = run_conv(dn, x, wt, bias, None, None, None, n=n, size=3, stride=1, pad=1, groups=1, bn=0, act="linear")
    assert np.array_equal(got, want)


def random_geometries(seed, count):
    """Seeded draw of legal layer geometries over every dispatch branch: 1x1 / 3x3 / 5x5 / 7x7,
    strides 1-3, any padding up to the kernel size, channel counts on and off the 16-multiple that
    selects the tap-blocked order, groups (equal, unequal, depthwise), filters around the tile
    sizes, images smaller than the kernel window allows to skip."""
    rng = np.random.default_rng(seed)
    out = []
    while len(out) < count:
        size = int(rng.choice([1, 3, 3, 3, 5, 7]))
        stride = 1 if size == 1 else int(rng.choice([1, 1, 2, 3]))
        pad = 0 if size == 1 else int(rng.integers(0, size // 2 + 2))
        groups = int(rng.choice([1, 1, 1, 2, 4, 8, 32]))
        cg = int(rng.choice([1, 2, 3, 4, 8, 16, 20, 32, 48]))
        fg = cg if (groups > 1 and rng.random() < 0.6) else int(rng.choice([1, 3, 8, 16, 31, 40, 65, 130, 260]))
        c, n = cg * groups, fg * groups
        if c > 512 or n > 600:
            continue
        h, w = int(rng.integers(1, 30)), int(rng.integers(1, 30))
        if (h + 2 * pad - size) // stride + 1 <= 0 or (w + 2 * pad - size) // stride + 1 <= 0:
            continue
        b = int(rng.integers(1, 4))
        act = str(rng.choice(["leaky", "linear", "relu", "logistic"]))
        out.append((b, c, h, w, n, size, stride, pad, groups, act, int(rng.integers(0, 2))))
    return out


@pytest.mark.parametrize("b,c,h,w,n,size,stride,pad,groups,act,bn", random_geometries(20241, 48))
def test_conv_random_geometries(dn, orc, b, c, h, w, n, size, stride, pad, groups, act, bn):
    x = synth.uniform(31, b * c * h * w).reshape(b, c, h, w)
    wt = synth.conv_weights(32, n, c // groups, size)
    bias, sc, mu, var = synth.bn_random(33, n)
    if not bn:
        sc = mu = var = None
    kw = dict(n=n, size=size, stride=stride, pad=pad, groups=groups)
    want = orc.conv(x, wt, bias, sc, mu, var, batch_normalize=bn, activation=act, **kw)
    got = run_conv(dn, x, wt, bias, sc, mu, var, bn=bn, act=act, **kw)
    assert got.shape == want.shape
    assert norm_err(got, want) <= REL_TOL, dn.conv_kernel_name(n, c, groups, size)


TILE_CASES = [  # b, c, h, w, n, size, stride: enough columns for whole rounds of tiles plus a K-split tail
    (24, 64, 40, 40, 160, 3, 1),     # ragged filter tiles, 3x3 tap-blocked
    (24, 96, 40, 40, 64, 1, 1),      # up to 64 filters, 1x1
    (16, 80, 52, 52, 192, 1, 1),     # 1x1, more than 64 filters
    (12, 20, 36, 36, 48, 3, 2),      # reference K order (c % 16 != 0), stride 2
    (12, 20, 40, 40, 160, 3, 1),     # reference K order on the 128-row tiles
    (8, 24, 48, 48, 136, 1, 1),      # 1x1 in reference K order, ragged filter tiles
]


@pytest.mark.parametrize("b,c,h,w,n,size,stride", TILE_CASES)
def test_every_tile_shape_split_and_band_count_computes_the_same_layer(dn, orc, b, c, h, w, n, size, stride):
    """The tuning hooks pick the tile (0 = the library's rule, 128 = wide, 64 = narrow, 1 = 64x64),
    the K-split factor and the band count of the tile order; none may change a layer beyond the
    summation order over K.  Image 0 and the last image against the checker, every variant against
    the default."""
    pad = size // 2
    x = synth.uniform(41, b * c * h * w).reshape(b, c, h, w)
    wt = synth.conv_weights(42, n, c, size)
    bias, sc, mu, var = synth.bn_random(43, n)
    kw = dict(n=n, size=size, stride=stride, pad=pad, groups=1)
    base = run_conv(dn, x, wt, bias, sc, mu, var, bn=1, act="leaky", **kw)
    for k in (0, b - 1):
        want = orc.conv(x[k:k + 1], wt, bias, sc, mu, var, batch_normalize=1, activation="leaky", **kw)
        assert norm_err(base[k:k + 1], want) <= REL_TOL, k
    names = set()
    try:
        for tile_n in (0, 128, 64, 1):
            for split in (0, 1, 3):
                for bands in (0, 1, 2, 8):
                    dn.conv_set_ksplit(split, tile_n)
                    dn.conv_set_bands(bands)
                    oh = (h + 2 * pad - size) // stride + 1
                    names.add(dn.conv_kernel_name_columns(n, c, 1, size, b * oh * oh))
                    got = run_conv(dn, x, wt, bias, sc, mu, var, bn=1, act="leaky", **kw)
                    assert norm_err(got, base) <= 2e-5, (tile_n, split, bands)
    finally:
        dn.conv_set_ksplit(0, 0)
        dn.conv_set_bands(0)
    assert len(names) >= 2      # the hooks did switch kernels


def test_small_and_chip_filling_launches_run_their_own_variant_and_agree(dn, orc):
    """A 3x3 layer of 128..256 channels runs the 128x64 tile; a launch with fewer tiles than the chip
    has CUs takes the variant whose K-order number carries +100 (another form of the same loop).  The
    same image through both against the checker and against each other."""
    c, h, w, n = 128, 26, 26, 256
    x = synth.uniform(51, 32 * c * h * w).reshape(32, c, h, w)
    wt = synth.conv_weights(52, n, c, 3)
    bias, sc, mu, var = synth.bn_random(53, n)
    kw = dict(n=n, size=3, stride=1, pad=1, groups=1)
    small_name = dn.conv_kernel_name_columns(n, c, 1, 3, 1 * h * w).decode()
    big_name = dn.conv_kernel_name_columns(n, c, 1, 3, 32 * h * w).decode()
    assert small_name == "conv_mfma_kernel<128,64,64,32,113>" and big_name == "conv_mfma_kernel<128,64,64,32,13>"
    big = run_conv(dn, x, wt, bias, sc, mu, var, bn=1, act="leaky", **kw)
    for k in (0, 31):
        small = run_conv(dn, x[k:k + 1], wt, bias, sc, mu, var, bn=1, act="leaky", **kw)
        want = orc.conv(x[k:k + 1], wt, bias, sc, mu, var, batch_normalize=1, activation="leaky", **kw)
        assert norm_err(small, want) <= REL_TOL and norm_err(big[k:k + 1], want) <= REL_TOL, k
        assert norm_err(small, big[k:k + 1]) <= 2e-5, k


def test_mfma_kernel_agrees_with_direct_kernel_and_unpacked_call(dn):
    b, c, h, w, n = 2, 64, 20, 20, 96
    x = synth.uniform(1, b * c * h * w).reshape(b, c, h, w)
    wt = synth.conv_weights(2, n, c, 3)
    bias, sc, mu, var = synth.bn_random(3, n)
    kw = dict(n=n, size=3, stride=1, pad=1, groups=1, bn=1, act="leaky")
    fast = run_conv(dn, x, wt, bias, sc, mu, var, **kw)
    nopack = run_conv(dn, x, wt, bias, sc, mu, var, packed=False, **kw)   # library repacks per call
    assert np.array_equal(fast, nopack)
    dn.conv_set_algo(1)
    try:
        direct = run_conv(dn, x, wt, bias, sc, mu, var, **kw)
    finally:
        dn.conv_set_algo(0)
    assert norm_err(fast, direct) <= 2e-6


def test_grouped_mfma_tiles_agree_with_direct_kernel_and_unpacked_call(dn):
    """Block-diagonal 32-filter tiles (8 channels per group here) against the per-group direct loop."""
    b, c, h, w, n, groups = 3, 128, 15, 17, 128, 16
    x = synth.uniform(4, b * c * h * w).reshape(b, c, h, w)
    wt = synth.conv_weights(5, n, c // groups, 3)
    bias, sc, mu, var = synth.bn_random(6, n)
    kw = dict(n=n, size=3, stride=2, pad=1, groups=groups, bn=1, act="leaky")
    assert dn.conv_kernel_name(n, c, groups, 3).decode() == "conv_mfma_kernel<32,256,32,64,13>"
    # (8 per group at stride 1 would run on the vector-ALU kernel of small groups; at stride 2 the matrix cores keep it)
    assert dn.conv_kernel_name_geometry(b, c, h, w, n, groups, 3, 2, 1).decode() == "conv_mfma_kernel<32,256,32,64,13>"
    fast = run_conv(dn, x, wt, bias, sc, mu, var, **kw)
    assert np.array_equal(fast, run_conv(dn, x, wt, bias, sc, mu, var, packed=False, **kw))
    dn.conv_set_algo(1)
    try:
        assert dn.conv_kernel_name(n, c, groups, 3).decode() == "conv_direct_kernel"
        direct = run_conv(dn, x, wt, bias, sc, mu, var, **kw)
    finally:
        dn.conv_set_algo(0)
    assert norm_err(fast, direct) <= 2e-6


@pytest.mark.parametrize("b,c,h,w,groups,stride,act,bn", [
    (2, 128, 56, 56, 32, 1, "leaky", 1),      # resnext50 stage 1: 4 per group
    (1, 128, 57, 41, 32, 2, "leaky", 1),      # 4 per group, stride 2, odd sizes: ragged tiles on both axes
    (3, 16, 9, 70, 4, 1, "linear", 0),        # 4 per group, three tiles across, no batch-norm
    (2, 64, 33, 8, 8, 1, "relu", 1),          # 8 per group, narrower than a tile
    (2, 16, 12, 66, 4, 2, "relu", 1),         # 4 per group, stride 2, one column into the second tile
    (1, 8, 1, 1, 2, 1, "leaky", 1),           # a single pixel
    (2, 32, 17, 33, 4, 1, "leaky", 1)])       # 8 per group, stride 1, one column into the second tile
def test_small_group_kernel(dn, orc, b, c, h, w, groups, stride, act, bn):
    """Grouped 3x3 layers of 4 or 8 channels per group on the vector-ALU kernel: against the CPU checker and
    the fp64 convolution as every convolution, and against the same layer on the matrix cores; sentinels
    behind the output."""
    n = c
    name = dn.conv_kernel_name_geometry(b, c, h, w, n, groups, 3, stride, 1).decode()
    assert name == f"conv_group_kernel<{c // groups},{stride}>", name
    x = synth.uniform(41, b * c * h * w).reshape(b, c, h, w)
    wt = synth.conv_weights(42, n, c // groups, 3)
    bias, sc, mu, var = synth.bn_random(43, n)
    sc = sc.copy()
    sc[2::5] *= -1.0
    kw = dict(n=n, size=3, stride=stride, pad=1, groups=groups)
    oh, ow = (h - 1) // stride + 1, (w - 1) // stride + 1
    count, guard = b * n * oh * ow, 512
    dev = [D(a) for a in (x, wt, bias, sc, mu, var)]
    out = D(np.full(count + guard, 0x7FC0BEEF, np.uint32).view(np.float32))
    dn.forward_convolutional_gpu(dev[0].ptr, dev[1].ptr, None, dev[2].ptr, *[d.ptr if bn else None for d in dev[3:]],
                                 out.ptr, b, c, h, w, n, groups, 3, stride, 1, bn, ACTIVATIONS.index(act))
    bits = out.numpy().view(np.uint32)
    assert (bits[count:] == 0x7FC0BEEF).all(), "the kernel wrote past the end of its output"
    got = bits[:count].view(np.float32).reshape(b, n, oh, ow)
    assert not np.isnan(got).any()
    args = (x, wt, bias, sc, mu, var) if bn else (x, wt, bias)
    want = orc.conv(*args, batch_normalize=bn, activation=act, **kw)
    assert norm_err(got, want) <= REL_TOL
    assert norm_err(got, orc.conv_f64(*args, batch_normalize=bn, activation=act, **kw)) <= 5e-6
    dn.conv_set_algo(3)
    try:
        mfma = run_conv(dn, x, wt, bias, sc if bn else None, mu if bn else None, var if bn else None, bn=bn, act=act, **kw)
    finally:
        dn.conv_set_algo(0)
    assert norm_err(got, mfma) <= 2e-6


def test_conv_golden_vectors(dn):
    g = np.load(os.path.join(GOLD, "conv_cases.npz"))
    for name in sorted(k[:-5] for k in g.files if k.endswith("_spec")):
        b, c, h, w, n, size, stride, pad, groups, act, bn = [int(v) for v in g[name + "_spec"]]
        L = [{"type": "convolutional", "n": n, "c": c, "groups": groups, "size": size, "batch_normalize": bn}]
        params = {}
        fill_params(lambda i, *a: params.update(p=a), L, seed=77, bn="random")
        wt, bias, sc, mu, var = params["p"]
        got = run_conv(dn, g[name + "_in"].reshape(b, c, h, w), wt, bias, sc, mu, var, n=n, size=size,
                       stride=stride, pad=pad, groups=groups, bn=bn, act=ACTIVATIONS[act])
        assert norm_err(got.reshape(b, -1), g[name + "_out"]) <= REL_TOL, name


def test_conv_linearity_at_full_size(dn):
    """Size-independent property at the benchmark shape (batch 64): conv(x1 + x2) = conv(x1) + conv(x2)
    without bias/BN/activation, and a batch of copies gives copies."""
    c, h, w, n, b = 256, 26, 26, 512, 64
    x1 = synth.uniform(1, b * c * h * w).reshape(b, c, h, w)
    x1[1:] = x1[0]                                       # every image identical
    wt = synth.conv_weights(2, n, c, 3)
    zero = np.zeros(n, np.float32)
    kw = dict(n=n, size=3, stride=1, pad=1, groups=1, bn=0, act="linear")
    y = run_conv(dn, x1, wt, zero, None, None, None, **kw)
    # copies agree to rounding: tiles of the last, partial round are summed in K-slices, so an
    # image that falls there sees a different (fixed) summation order than one that does not
    assert all(norm_err(y[i], y[0]) <= 1e-5 for i in (1, 17, 63))
    y_again = run_conv(dn, x1, wt, zero, None, None, None, **kw)
    assert np.array_equal(y, y_again)                      # run-to-run deterministic
    x2 = synth.uniform(5, b * c * h * w).reshape(b, c, h, w)
    y2 = run_conv(dn, x2, wt, zero, None, None, None, **kw)
    y12 = run_conv(dn, x1 + x2, wt, zero, None, None, None, **kw)
    assert norm_err(y12, y + y2) <= 1e-5


FUSED = [  # b, c, h, w, n, size, stride, pad, groups, act, alpha, beta, shortcut act
    (2, 64, 26, 26, 128, 3, 1, 1, 1, "leaky", 1.0, 1.0, "linear"),     # darknet53 residual block
    (3, 128, 13, 13, 255, 1, 1, 0, 1, "linear", 0.5, -1.25, "leaky"),  # ragged M, scaled, activated
    (1, 256, 13, 13, 512, 3, 1, 1, 1, "leaky", 1.0, 1.0, "linear"),    # batch 1: every tile K-split
    (5, 16, 7, 9, 130, 3, 1, 1, 1, "leaky", 1.0, 2.0, "logistic"),     # tile columns cross images
    (2, 3, 21, 23, 32, 3, 1, 1, 1, "leaky", 1.0, 1.0, "linear"),       # reference-order kernel, BM = 32
    (2, 64, 14, 14, 64, 3, 1, 1, 32, "leaky", 1.0, 1.0, "linear"),     # grouped -> direct kernel + add
]


@pytest.mark.parametrize("b,c,h,w,n,size,stride,pad,groups,act,alpha,beta,sact", FUSED)
def test_conv_shortcut_fused_equals_separate_calls(dn, b, c, h, w, n, size, stride, pad, groups, act, alpha,
                                                    beta, sact):
    """forward_convolutional_shortcut_gpu == forward_convolutional_gpu then forward_shortcut_gpu, bit for
    bit, on both outputs (the shortcut itself is checked against the CPU in test_gpu_kernels)."""
    x = synth.uniform(11, b * c * h * w).reshape(b, c, h, w)
    wt = synth.conv_weights(12, n, c // groups, size)
    bias, sc, mu, var = synth.bn_random(13, n)
    oh = (h + 2 * pad - size) // stride + 1
    ow = (w + 2 * pad - size) // stride + 1
    total = b * n * oh * ow
    res = synth.uniform(14, total)
    dx, dw, db, ds, dm, dv, dres = D(x), D(wt), D(bias), D(sc), D(mu), D(var), D(res)
    pk = None
    pf = dn.conv_packed_floats(n, c, groups, size)
    if pf:
        pk = D(n=pf)
        dn.conv_pack_weights_gpu(dw.ptr, pk.ptr, n, c, groups, size)
    conv_args = (dx.ptr, dw.ptr, pk.ptr if pk else None, db.ptr, ds.ptr, dm.ptr, dv.ptr)
    geom = (b, c, h, w, n, groups, size, stride, pad, 1, ACTIVATIONS.index(act))
    out_a, sum_a = D(n=total), D(n=total)
    dn.forward_convolutional_gpu(*conv_args, out_a.ptr, *geom)
    dn.forward_shortcut_gpu(out_a.ptr, dres.ptr, sum_a.ptr, b, ow, oh, n, ow, oh, n, alpha, beta,
                            ACTIVATIONS.index(sact))
    out_b, sum_b = D(n=total), D(n=total)
    dn.forward_convolutional_shortcut_gpu(*conv_args, out_b.ptr, *geom, dres.ptr, sum_b.ptr, alpha, beta,
                                          ACTIVATIONS.index(sact))
    assert np.array_equal(out_a.numpy((total,)), out_b.numpy((total,)))
    assert np.array_equal(sum_a.numpy((total,)), sum_b.numpy((total,)))
    assert np.abs(sum_b.numpy((total,))).max() > 0


def test_batches_beyond_4_gib_run_in_slices_of_whole_images(dn):
    """The MFMA kernels address their input with 32-bit offsets.  A batch whose input exceeds 4 GiB
    is cut into slices of whole images on the host instead of falling back to the direct kernel:
    every image must equal the result of convolving it alone (summation order aside)."""
    b, c, h, w, n = 63, 16, 1040, 1040, 16          # 63 x 69.2 MB = 4.36 GB in, the same out
    assert b * c * h * w * 4 > (1 << 32)
    rng = np.random.default_rng(5)
    x = rng.random((b, c, h, w), dtype=np.float32) - 0.5
    wt = synth.conv_weights(61, n, c, 3)
    bias, sc, mu, var = synth.bn_random(62, n)
    kw = dict(n=n, size=3, stride=1, pad=1, groups=1, bn=1, act="leaky")
    assert dn.conv_kernel_name(n, c, 1, 3).decode().startswith("conv_mfma_kernel")
    ev = dn.hip_event_create(), dn.hip_event_create()
    dn.conv_profile_next(ev[0], ev[1])         # only an MFMA launch takes the pair of events
    got = run_conv(dn, x, wt, bias, sc, mu, var, **kw)
    assert dn.conv_profile_pending() == 0 and dn.hip_event_elapsed_ms(ev[0], ev[1]) > 0
    assert got.shape == (b, n, h, w)
    per = ((1 << 32) - (2 << 20)) // (c * h * w * 4)      # images per slice
    for i in (0, per - 1, per, b - 1):
        alone = run_conv(dn, x[i:i + 1], wt, bias, sc, mu, var, **kw)
        assert norm_err(got[i:i + 1], alone) <= 1e-5, i


def random_small_groups(seed, count):
    rng = np.random.default_rng(seed)
    out = []
    for _ in range(count):
        cg = int(rng.choice([4, 8]))
        groups = int(rng.choice([2, 3, 8, 32]))
        stride = 1 if cg == 8 else int(rng.choice([1, 2]))
        h, w = int(rng.integers(1, 40)), int(rng.integers(1, 80))
        b = int(rng.integers(1, 4))
        act, bn = [("leaky", 1), ("linear", 0), ("relu", 1)][int(rng.integers(0, 3))]
        out.append((b, cg * groups, h, w, groups, stride, act, bn))
    return out


@pytest.mark.parametrize("b,c,h,w,groups,stride,act,bn", random_small_groups(20251, 16))
def test_small_group_kernel_random_geometries(dn, orc, b, c, h, w, groups, stride, act, bn):
    test_small_group_kernel(dn, orc, b, c, h, w, groups, stride, act, bn)

