"""The two opt-in modes of the tap-blocked MFMA convolution kernels that run on the bf16 matrix cores.

bf16-operand mode (conv_set_precision(1)).  What it computes is pinned exactly: the CPU checker run
on operands rounded to bf16 (round to nearest even, done here in integer arithmetic) must agree with
the kernel to the fp32 bar (<= 1e-4 max-normalised; the products of two bf16 numbers are exact in
fp32, so only the summation order differs).  Against the unrounded fp32 checker the mode's error is
measured and bounded loosely (it is a precision trade, not a parity claim), and the default fp32
mode must be untouched by a round trip through the switch.

Three-piece mode (conv_set_precision(2)): fp32 emulated with three bf16 pieces per operand.  It is
held to the fp32 parity bar itself, with the fp64 convolution as referee."""
import numpy as np
import pytest

from darknet_amd import api, cfgs, synth
from oracle.net import OracleNet

from test_gpu_conv import run_conv
from util import REL_TOL, fill_params, norm_err

pytestmark = pytest.mark.gpu


def round_bf16(x):
    """fp32 -> nearest bf16 (ties to even) -> fp32, on the bit patterns."""
    u = np.ascontiguousarray(x, dtype=np.float32).view(np.uint32).astype(np.uint64)
    u = (u + 0x7FFF + ((u >> 16) & 1)) & 0xFFFF0000
    return u.astype(np.uint32).view(np.float32).reshape(np.shape(x))


def test_round_bf16_helper():
    x = np.array([1.0, 1.0 + 2.0 ** -8, 1.0 + 3 * 2.0 ** -8, 1.0 + 2.0 ** -8 + 2.0 ** -20, -0.1, 0.0], np.float32)
    r = round_bf16(x)
    # ties go to the even mantissa: 1+2^-8 -> 1, 1+3*2^-8 -> 1+2^-6; above a tie rounds up
    assert r[0] == 1.0 and r[1] == 1.0 and r[2] == np.float32(1.0 + 2.0 ** -6) and r[3] == np.float32(1 + 2.0 ** -7)
    assert abs(r[4] + 0.1) < 0.1 * 2.0 ** -8 and r[5] == 0.0
    assert np.all((r.view(np.uint32) & 0xFFFF) == 0)


@pytest.fixture
def bf16(dn):
    dn.conv_set_precision(1)
    yield dn
    dn.conv_set_precision(0)


BF16_SHAPES = [  # b, c, h, w, n, size, stride, pad, groups, act
    (2, 256, 26, 26, 512, 3, 1, 1, 1, "leaky"),
    (2, 512, 52, 52, 256, 1, 1, 0, 1, "leaky"),
    (2, 128, 104, 104, 256, 3, 2, 1, 1, "leaky"),
    (2, 32, 30, 30, 64, 3, 2, 1, 1, "leaky"),       # 64-row tile
    (1, 64, 19, 19, 32, 1, 1, 0, 1, "linear"),      # 32-row tile
    (2, 1024, 13, 13, 255, 1, 1, 0, 1, "linear"),   # ragged M, K-split at this size
    (2, 128, 14, 14, 128, 3, 1, 1, 32, "leaky"),    # grouped 32-filter tiles
    (5, 16, 7, 9, 130, 3, 1, 1, 1, "logistic"),     # one chunk per tap, tiny images, ragged M on the 128-row tile
    (3, 64, 10, 10, 300, 3, 1, 1, 1, "leaky"),      # 256-row tiles, the second one ragged; N below one tile
    (1, 32, 20, 21, 32, 3, 2, 1, 1, "relu"),        # 32-row tile on the staged-input variant, stride 2, odd width
    (2, 48, 13, 13, 200, 1, 1, 0, 1, "leaky"),      # 1x1, 3 chunks (shorter than the pipeline), 169 pixels per image
    (2, 16, 6, 6, 256, 1, 1, 0, 1, "linear"),       # a single chunk
]


@pytest.mark.parametrize("b,c,h,w,n,size,stride,pad,groups,act", BF16_SHAPES)
def test_bf16_mode_is_fp32_conv_of_rounded_operands(bf16, orc, b, c, h, w, n, size, stride, pad, groups, act):
    x = synth.uniform(11, b * c * h * w).reshape(b, c, h, w)
    wt = synth.conv_weights(12, n, c // groups, size)
    bias, sc, mu, var = synth.bn_random(13, n)
    kw = dict(n=n, size=size, stride=stride, pad=pad, groups=groups)
    name = bf16.conv_kernel_name(n, c, groups, size).decode()
    assert name.count(",") == 5 and name.endswith(",2>" if size == 3 else ",1>")     # <BM,BN,WM,WN,mode,variant>
    got = run_conv(bf16, x, wt, bias, sc, mu, var, bn=1, act=act, **kw)
    want = orc.conv(round_bf16(x), round_bf16(wt), bias, sc, mu, var, batch_normalize=1, activation=act, **kw)
    assert norm_err(got, want) <= REL_TOL
    full = orc.conv(x, wt, bias, sc, mu, var, batch_normalize=1, activation=act, **kw)
    err = norm_err(got, full)
    print(f"bf16-operand error vs fp32, {size}x{size}/{stride} {c}->{n} g{groups}: {err:.2e}")
    assert 1e-5 < err < 2e-2          # really reduced precision, and no worse than bf16 rounding explains


@pytest.mark.parametrize("b,c,h,w,n,size,stride,pad,groups,act,bn", __import__("test_gpu_conv").random_geometries(777, 32))
def test_bf16_mode_random_geometries(bf16, orc, b, c, h, w, n, size, stride, pad, groups, act, bn):
    """Whatever kernel a geometry lands on with the switch on - bf16 variants or untouched fp32
    ones - the result is the fp32 convolution of operands rounded (or not) accordingly."""
    x = synth.uniform(41, b * c * h * w).reshape(b, c, h, w)
    wt = synth.conv_weights(42, n, c // groups, size)
    bias, sc, mu, var = synth.bn_random(43, n)
    if not bn:
        sc = mu = var = None
    kw = dict(n=n, size=size, stride=stride, pad=pad, groups=groups)
    name = bf16.conv_kernel_name(n, c, groups, size).decode()
    # a 3x3 layer packed tap-blocked but with padding other than 1 runs on the direct kernel
    reduced = name.count(",") == 5 and not (size == 3 and pad != 1)    # <BM,BN,WM,WN,mode,variant>
    got = run_conv(bf16, x, wt, bias, sc, mu, var, bn=bn, act=act, **kw)
    if reduced:
        want = orc.conv(round_bf16(x), round_bf16(wt), bias, sc, mu, var, batch_normalize=bn, activation=act, **kw)
    else:
        want = orc.conv(x, wt, bias, sc, mu, var, batch_normalize=bn, activation=act, **kw)
    assert norm_err(got, want) <= REL_TOL, (name, reduced)


@pytest.fixture
def bf16x3(dn):
    dn.conv_set_precision(2)
    yield dn
    dn.conv_set_precision(0)


@pytest.mark.parametrize("b,c,h,w,n,size,stride,pad,groups,act", BF16_SHAPES)
def test_three_piece_mode_meets_the_fp32_bar(bf16x3, orc, b, c, h, w, n, size, stride, pad, groups, act):
    """precision 2: operands split into three bf16 pieces, six piece-products summed in fp32.  No
    rounding of the operands survives (x = hi + mid + lo exactly), so the fp32 parity bar applies
    unchanged, with the fp64 convolution as referee: the mode must sit as close to it as the
    fp32 checker does (within a factor that leaves room for the three dropped 2^-24 terms)."""
    x = synth.uniform(11, b * c * h * w).reshape(b, c, h, w)
    wt = synth.conv_weights(12, n, c // groups, size)
    bias, sc, mu, var = synth.bn_random(13, n)
    kw = dict(n=n, size=size, stride=stride, pad=pad, groups=groups)
    name = bf16x3.conv_kernel_name(n, c, groups, size).decode()
    assert name.count(",") == 5 and name.endswith(",3>")
    got = run_conv(bf16x3, x, wt, bias, sc, mu, var, bn=1, act=act, **kw)
    want = orc.conv(x, wt, bias, sc, mu, var, batch_normalize=1, activation=act, **kw)
    ref64 = orc.conv_f64(x, wt, bias, sc, mu, var, batch_normalize=1, activation=act, **kw)
    e_cpu, e_64, cpu_64 = norm_err(got, want), norm_err(got, ref64), norm_err(want, ref64)
    print(f"three-piece mode {size}x{size}/{stride} {c}->{n} g{groups}: vs cpu {e_cpu:.2e}, vs fp64 {e_64:.2e}, "
          f"cpu vs fp64 {cpu_64:.2e}")
    assert e_cpu <= REL_TOL
    assert e_64 <= max(4 * cpu_64, 2e-6)


@pytest.mark.parametrize("b,c,h,w,n,size,stride,pad,groups,act,bn", __import__("test_gpu_conv").random_geometries(778, 24))
def test_three_piece_mode_random_geometries(bf16x3, orc, b, c, h, w, n, size, stride, pad, groups, act, bn):
    x = synth.uniform(51, b * c * h * w).reshape(b, c, h, w)
    wt = synth.conv_weights(52, n, c // groups, size)
    bias, sc, mu, var = synth.bn_random(53, n)
    if not bn:
        sc = mu = var = None
    kw = dict(n=n, size=size, stride=stride, pad=pad, groups=groups)
    got = run_conv(bf16x3, x, wt, bias, sc, mu, var, bn=bn, act=act, **kw)
    want = orc.conv(x, wt, bias, sc, mu, var, batch_normalize=bn, activation=act, **kw)
    assert norm_err(got, want) <= REL_TOL, bf16x3.conv_kernel_name(n, c, groups, size)


def test_three_piece_mode_whole_network(bf16x3):
    """yolov3 at 160 in the three-piece mode: per-layer <= 1e-4 and yolo heads <= 1e-3, the bar of
    the fp32 mode."""
    from test_gpu_network import check_network
    assert check_network(cfgs.yolov3(1, 160)) <= REL_TOL


def test_layers_on_other_kernels_stay_fp32(bf16, orc):
    """3 input channels -> reference-order kernel: the switch must not touch it."""
    b, c, h, w, n = 2, 3, 33, 35, 32
    x = synth.uniform(14, b * c * h * w).reshape(b, c, h, w)
    wt = synth.conv_weights(15, n, c, 3)
    bias, sc, mu, var = synth.bn_random(16, n)
    assert bf16.conv_kernel_name(n, c, 1, 3).decode().count(",") == 4
    got1 = run_conv(bf16, x, wt, bias, sc, mu, var, n=n, size=3, stride=1, pad=1, groups=1, bn=1, act="leaky")
    bf16.conv_set_precision(0)
    got0 = run_conv(bf16, x, wt, bias, sc, mu, var, n=n, size=3, stride=1, pad=1, groups=1, bn=1, act="leaky")
    assert np.array_equal(got0, got1)


def test_switch_round_trip_restores_fp32_bits(dn):
    b, c, h, w, n = 2, 64, 20, 20, 128
    x = synth.uniform(17, b * c * h * w).reshape(b, c, h, w)
    wt = synth.conv_weights(18, n, c, 3)
    bias, sc, mu, var = synth.bn_random(19, n)
    kw = dict(n=n, size=3, stride=1, pad=1, groups=1, bn=1, act="leaky")
    before = run_conv(dn, x, wt, bias, sc, mu, var, **kw)
    dn.conv_set_precision(1)
    try:
        mid = run_conv(dn, x, wt, bias, sc, mu, var, **kw)
    finally:
        dn.conv_set_precision(0)
    after = run_conv(dn, x, wt, bias, sc, mu, var, **kw)
    assert dn.conv_get_precision() == 0
    assert np.array_equal(before, after) and not np.array_equal(before, mid)


def test_yolov3_bf16_measured_error(bf16):
    """Whole network, bf16 operands in 74 of 75 convolutions: the error against the fp32 checker is
    measured per layer and at the yolo heads; the bounds are loose sanity limits, not parity."""
    text = cfgs.yolov3(1, 160)
    net = api.Network(cfg_text=text)
    ref = OracleNet(text)
    fill_params(net.set_conv, net.layers, bn="random")
    fill_params(ref.set_conv, ref.layers, bn="random")
    x = synth.uniform01(23, net.inputs)
    net.predict(x)
    outs = ref.forward(x)
    worst_conv = 0.0
    yolo_abs = 0.0
    for i, L in enumerate(net.layers):
        got, want = net.layer_output(i), outs[i]
        if L["type"] == "convolutional":
            worst_conv = max(worst_conv, norm_err(got, want))
        elif L["type"] == "yolo":
            yolo_abs = max(yolo_abs, float(np.max(np.abs(got - want))))
    print(f"yolov3-160 bf16 operands: worst conv layer {worst_conv:.2e} max-normalised, yolo heads {yolo_abs:.2e} abs")
    assert 1e-4 < worst_conv < 5e-2
    assert yolo_abs < 0.5
    net.free()
