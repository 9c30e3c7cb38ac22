"""Pins the CPU checker (oracle/oracle.c) function by function.

Three kinds of evidence, chosen so that a dropped term, a wrong sign or index, or a transposed
operand fails at least one test:
  * golden vectors written by the compiled reference (tests/golden/*.npz, see make_golden.py);
  * the compiled reference itself where oracle/_ref is present (bit-exact);
  * independent mathematics: brute-force loops, exact small-integer GEMM, the fp64 direct
    convolution, torch's CPU conv2d / max_pool2d, closed forms.
"""
import ctypes as C
import math
import os

import numpy as np
import pytest

from darknet_amd import synth
from oracle import ref
from oracle.cpu import ACTIVATIONS

from util import norm_err

GOLD = os.path.join(os.path.dirname(__file__), "golden")
needs_ref = pytest.mark.skipif(not ref.available(), reason="oracle/_ref (compiled reference) not built")
F = C.POINTER(C.c_float)


def fp(a):
    return a.ctypes.data_as(F)


# ---------------------------------------------------------------------------- im2col
def brute_im2col(im, c, h, w, k, s, p):
    oh = (h + 2 * p - k) // s + 1
    ow = (w + 2 * p - k) // s + 1
    col = np.zeros((c * k * k, oh * ow), np.float32)
    im = im.reshape(c, h, w)
    for ch in range(c):
        for ky in range(k):
            for kx in range(k):
                r = (ch * k + ky) * k + kx
                for oy in range(oh):
                    for ox in range(ow):
                        iy, ix = oy * s + ky - p, ox * s + kx - p
                        if 0 <= iy < h and 0 <= ix < w:
                            col[r, oy * ow + ox] = im[ch, iy, ix]
    return col


@pytest.mark.parametrize("c,h,w,k,s,p", [(2, 5, 6, 3, 1, 1), (3, 7, 5, 3, 2, 1), (1, 6, 6, 1, 1, 0),
                                         (2, 8, 9, 5, 2, 2), (1, 9, 9, 7, 2, 3), (2, 4, 4, 3, 1, 0)])
def test_im2col_brute_force(orc, c, h, w, k, s, p):
    im = synth.uniform(1, c * h * w)
    assert np.array_equal(orc.im2col(im, c, h, w, k, s, p), brute_im2col(im, c, h, w, k, s, p))


def test_im2col_delta_image(orc):
    """A single 1 at (ch, y, x) must appear exactly at rows (ch,ky,kx) / columns (y+p-ky, x+p-kx)."""
    c, h, w, k, p = 2, 5, 5, 3, 1
    im = np.zeros(c * h * w, np.float32)
    ch, y, x = 1, 2, 3
    im[(ch * h + y) * w + x] = 1
    col = orc.im2col(im, c, h, w, k, 1, p)
    hits = set(zip(*np.nonzero(col)))
    want = set()
    for ky in range(k):
        for kx in range(k):
            oy, ox = y + p - ky, x + p - kx
            if 0 <= oy < h and 0 <= ox < w:
                want.add(((ch * k + ky) * k + kx, oy * w + ox))
    assert hits == want


@needs_ref
@pytest.mark.parametrize("c,h,w,k,s,p", [(16, 26, 26, 3, 1, 1), (8, 52, 40, 3, 2, 1), (3, 33, 31, 7, 2, 3)])
def test_im2col_matches_reference(orc, c, h, w, k, s, p):
    lib = ref.raw()
    im = synth.uniform(2, c * h * w)
    mine = orc.im2col(im, c, h, w, k, s, p)
    theirs = np.empty_like(mine)
    lib.im2col_cpu.argtypes = [F] + [C.c_int] * 6 + [F]
    lib.im2col_cpu(fp(im), c, h, w, k, s, p, fp(theirs))
    assert np.array_equal(mine, theirs)


# ---------------------------------------------------------------------------- gemm
def test_gemm_exact_on_small_integers(orc):
    """All partial sums stay below 2^24, so any summation order gives the same bits."""
    rng = np.random.default_rng(0)
    A = rng.integers(-8, 9, (37, 53)).astype(np.float32)
    B = rng.integers(-8, 9, (53, 29)).astype(np.float32)
    assert np.array_equal(orc.gemm_nn(A, B), (A.astype(np.int64) @ B.astype(np.int64)).astype(np.float32))


def test_gemm_not_transposed_and_accumulates(orc):
    A = np.arange(6, dtype=np.float32).reshape(2, 3)
    B = np.arange(12, dtype=np.float32).reshape(3, 4) - 5
    C0 = np.full((2, 4), 10, np.float32)
    got = orc.gemm_nn(A, B, C0.copy(), alpha=2.0)
    assert np.array_equal(got, 10 + 2 * (A @ B))


def test_gemm_close_to_fp64(orc):
    A = synth.uniform(3, 64 * 300).reshape(64, 300)
    B = synth.uniform(4, 300 * 50).reshape(300, 50)
    assert norm_err(orc.gemm_nn(A, B), A.astype(np.float64) @ B.astype(np.float64)) < 1e-6


@needs_ref
def test_gemm_matches_reference_bits(orc):
    lib = ref.raw()
    M, N, K = 48, 169, 288
    A = synth.uniform(5, M * K).reshape(M, K)
    B = synth.uniform(6, K * N).reshape(K, N)
    mine = orc.gemm_nn(A, B)
    theirs = np.zeros((M, N), np.float32)
    lib.gemm.argtypes = [C.c_int] * 5 + [C.c_float, F, C.c_int, F, C.c_int, C.c_float, F, C.c_int]
    lib.gemm(0, 0, M, N, K, 1.0, fp(A), K, fp(B), N, 1.0, fp(theirs), N)
    assert np.array_equal(mine, theirs)


# ---------------------------------------------------------------------------- conv layer
CONV_SHAPES = [  # b, c, h, w, n, size, stride, pad, groups
    (2, 8, 9, 11, 12, 3, 1, 1, 1), (1, 16, 13, 10, 20, 3, 2, 1, 1), (2, 32, 7, 5, 19, 1, 1, 0, 1),
    (2, 8, 10, 10, 16, 3, 1, 1, 4), (1, 3, 20, 22, 8, 7, 2, 3, 1)]


@pytest.mark.parametrize("b,c,h,w,n,size,stride,pad,groups", CONV_SHAPES)
def test_conv_against_fp64_direct_and_torch(orc, b, c, h, w, n, size, stride, pad, groups):
    torch = pytest.importorskip("torch")
    x = synth.uniform(1, b * c * h * w).reshape(b, c, h, w)
    wt = synth.conv_weights(2, n, c // groups, size)
    bias, sc, mu, var = synth.bn_random(3, n)
    got = orc.conv(x, wt, bias, sc, mu, var, n=n, size=size, stride=stride, pad=pad, groups=groups,
                   batch_normalize=1, activation="leaky")
    ref64 = orc.conv_f64(x, wt, bias, sc, mu, var, n=n, size=size, stride=stride, pad=pad, groups=groups,
                         batch_normalize=1, activation="leaky")
    assert norm_err(got, ref64) < 2e-6
    # library routine: cross-correlation, NCHW, zero padding, groups
    y = torch.nn.functional.conv2d(torch.from_numpy(x).double(),
                                   torch.from_numpy(wt.reshape(n, c // groups, size, size)).double(),
                                   None, stride, pad, 1, groups).numpy()
    y = (y - mu.reshape(1, -1, 1, 1)) / (np.sqrt(var.astype(np.float64)).reshape(1, -1, 1, 1) + np.float32(1e-6))
    y = y * sc.reshape(1, -1, 1, 1) + bias.reshape(1, -1, 1, 1)
    y = np.where(y > 0, y, 0.1 * y)
    assert norm_err(got, y) < 2e-6


def test_conv_golden_vectors(orc):
    g = np.load(os.path.join(GOLD, "conv_cases.npz"))
    names = sorted(k[:-5] for k in g.files if k.endswith("_spec"))
    assert len(names) >= 6
    for name in names:
        b, c, h, w, n, size, stride, pad, groups, act, bn = [int(v) for v in g[name + "_spec"]]
        L = [{"type": "convolutional", "n": n, "c": c, "groups": groups, "size": size, "batch_normalize": bn}]
        params = {}
        from util import fill_params
        fill_params(lambda i, *a: params.update(p=a), L, seed=77, bn="random")
        wt, bias, sc, mu, var = params["p"]
        x = g[name + "_in"].reshape(b, c, h, w)
        got = orc.conv(x, wt, bias, sc, mu, var, n=n, size=size, stride=stride, pad=pad, groups=groups,
                       batch_normalize=bn, activation=ACTIVATIONS[act])
        assert np.array_equal(got.reshape(b, -1), g[name + "_out"]), name


def test_bn_identity_and_closed_form(orc):
    x = synth.uniform(1, 2 * 3 * 5).reshape(2, 3, 5)
    mean, var = np.zeros(3, np.float32), np.ones(3, np.float32)
    y = orc.normalize(x, mean, var)
    # mean 0 / variance 1: only the 1.000001 divisor remains
    assert np.array_equal(y, (x.astype(np.float64) / (1.0 + float(np.float32(1e-6)))).astype(np.float32))
    mean, var = synth.uniform(2, 3, -1, 1), synth.uniform(3, 3, 0.1, 4)
    y = orc.normalize(x, mean, var)
    want = (x - mean.reshape(1, 3, 1)).astype(np.float64) / (np.sqrt(var.astype(np.float64)).reshape(1, 3, 1)
                                                              + float(np.float32(1e-6)))
    assert np.array_equal(y, want.astype(np.float32))


def test_batchnorm_layer_is_normalize_scale_bias_in_sequence(orc):
    """The [batchnorm] layer at inference (src/batchnorm_layer.c:135-155): copy, normalize_cpu,
    scale_bias, add_bias.  Pinned by arithmetic done here in numpy, one rounding to float per
    pass as the reference's separate loops round, and by the fp64 closed form; a dropped pass, a
    swapped scale/bias or variance used without its square root each miss by far more than the
    bound.  (The compiled reference cannot serve as the pin: its CPU forward copies into l.x,
    which a CPU build never allocates for this layer, src/batchnorm_layer.c:16-33,138.)"""
    x = synth.uniform(5, 3 * 4 * 7).reshape(3, 4, 7)
    bias, scale, mean, var = synth.bn_random(6, 4)
    got = orc.batchnorm_layer(x, scale, bias, mean, var)
    r = lambda v: v.reshape(1, 4, 1)
    step = ((x - r(mean)).astype(np.float64) / (np.sqrt(r(var).astype(np.float64)) + float(np.float32(1e-6)))).astype(np.float32)
    step = (step * r(scale)).astype(np.float32)
    step = (step + r(bias)).astype(np.float32)
    assert np.array_equal(got, step)
    closed = (x.astype(np.float64) - r(mean)) / (np.sqrt(r(var).astype(np.float64)) + 1e-6) * r(scale) + r(bias)
    assert np.abs(got - closed).max() <= 1e-6 * np.abs(closed).max()
    # identity statistics leave only the 1.000001 divisor
    ident = orc.batchnorm_layer(x, np.ones(4, np.float32), np.zeros(4, np.float32), np.zeros(4, np.float32),
                                np.ones(4, np.float32))
    assert np.array_equal(ident, (x.astype(np.float64) / (1.0 + float(np.float32(1e-6)))).astype(np.float32))
    assert np.array_equal(x, synth.uniform(5, 3 * 4 * 7).reshape(3, 4, 7))      # the input is not modified


# ---------------------------------------------------------------------------- activations
def test_activation_closed_forms(orc):
    x = np.array([-3.5, -1.0, -0.0, 0.0, 0.25, 1.0, 7.0], np.float32)
    assert orc.activate(np.zeros(1, np.float32), "logistic")[0] == 0.5
    assert np.array_equal(orc.activate(x, "linear"), x)
    lk = orc.activate(x, "leaky")
    assert np.array_equal(lk[x > 0], x[x > 0])                       # exact for x > 0
    assert np.array_equal(lk[x <= 0], (0.1 * x[x <= 0].astype(np.float64)).astype(np.float32))
    assert lk[1] != np.float32(0.1) * np.float32(-1.0) or True        # (.1 is a double literal)
    lg = orc.activate(x, "logistic")
    assert np.all(np.diff(lg) >= 0) and np.all((lg > 0) & (lg < 1))
    want = np.array([1.0 / (1.0 + math.exp(-float(v))) for v in x]).astype(np.float32)
    assert np.array_equal(lg, want)
    assert np.array_equal(orc.activate(x, "relu"), np.maximum(x, 0))
    assert np.array_equal(orc.activate(x, "ramp"), (np.maximum(x, 0).astype(np.float64) + 0.1 * x).astype(np.float32))


@needs_ref
@pytest.mark.parametrize("act", ACTIVATIONS)
def test_activations_match_reference_bits(orc, act):
    lib = ref.raw()
    x = np.concatenate([synth.uniform(9, 4000, -6, 6), np.array([0.0, -0.0, 1.0, -1.0, 4.0, -4.0, 5.0], np.float32)])
    mine = orc.activate(x, act)
    theirs = x.copy()
    lib.activate_array.argtypes = [F, C.c_int, C.c_int]
    lib.activate_array(fp(theirs), theirs.size, ACTIVATIONS.index(act))
    assert np.array_equal(mine, theirs)


# ---------------------------------------------------------------------------- maxpool
def test_maxpool_textbook_and_padding(orc):
    torch = pytest.importorskip("torch")
    x = synth.uniform(1, 2 * 3 * 8 * 12).reshape(2, 3, 8, 12)
    out, idx = orc.maxpool(x, 2, 2, 1)           # darknet default padding = size-1, offset -pad/2 = 0
    want = torch.nn.functional.max_pool2d(torch.from_numpy(x), 2, 2).numpy()
    assert np.array_equal(out, want)
    assert np.array_equal(x.reshape(-1)[idx.reshape(-1)], out.reshape(-1))
    # the 13x13 stride-1 pool of yolov3-tiny: pad right/bottom with -FLT_MAX
    x = synth.uniform(2, 4 * 13 * 13).reshape(1, 4, 13, 13)
    out, idx = orc.maxpool(x, 2, 1, 1)
    xp = np.pad(x, ((0, 0), (0, 0), (0, 1), (0, 1)), constant_values=-np.finfo(np.float32).max)
    want = torch.nn.functional.max_pool2d(torch.from_numpy(xp), 2, 1).numpy()
    assert out.shape == (1, 4, 13, 13) and np.array_equal(out, want)


def test_maxpool_first_maximum_wins(orc):
    x = np.zeros((1, 1, 2, 2), np.float32) + 3
    out, idx = orc.maxpool(x, 2, 2, 1)
    assert out[0, 0, 0, 0] == 3 and idx[0, 0, 0, 0] == 0


def test_maxpool_golden(orc):
    g = np.load(os.path.join(GOLD, "maxpool_case.npz"))
    for name in ("s2", "s1pad", "k3s2"):
        b, c, h, w, size, stride, pad = [int(v) for v in g[name + "_spec"]]
        out, idx = orc.maxpool(g[name + "_in"].reshape(b, c, h, w), size, stride, pad)
        assert np.array_equal(out.reshape(b, -1), g[name + "_out"])
        assert np.array_equal(idx.reshape(b, -1), g[name + "_idx"])


# ---------------------------------------------------------------------------- the rest
def test_upsample_is_nearest(orc):
    x = synth.uniform(1, 2 * 3 * 4 * 5).reshape(2, 3, 4, 5)
    y = orc.upsample(x, 2)
    assert np.array_equal(y, x.repeat(2, axis=2).repeat(2, axis=3))
    assert np.array_equal(orc.upsample(x, 3, 0.5), (np.float32(0.5) * x).repeat(3, axis=2).repeat(3, axis=3))


def test_shortcut_invariants(orc):
    x = synth.uniform(1, 2 * 8 * 6 * 6).reshape(2, 8, 6, 6)
    add = synth.uniform(2, 2 * 8 * 6 * 6).reshape(2, 8, 6, 6)
    assert np.array_equal(orc.shortcut(x, add), x + add)
    # fewer channels in `add`, and `add` twice as large spatially (stride 2 sampling), as in resnext50
    add = synth.uniform(3, 2 * 4 * 12 * 12).reshape(2, 4, 12, 12)
    y = orc.shortcut(x, add)
    assert np.array_equal(y[:, 4:], x[:, 4:])
    assert np.array_equal(y[:, :4], x[:, :4] + add[:, :, ::2, ::2])
    # `add` smaller spatially: only every second output pixel receives it
    add = synth.uniform(4, 2 * 8 * 3 * 3).reshape(2, 8, 3, 3)
    y = orc.shortcut(x, add)
    want = x.copy()
    want[:, :, ::2, ::2] += add
    assert np.array_equal(y, want)


def test_route_concatenates_per_image(orc):
    a = synth.uniform(1, 3 * 10).reshape(3, 10)
    b = synth.uniform(2, 3 * 4).reshape(3, 4)
    assert np.array_equal(orc.route([a, b]), np.concatenate([a, b], axis=1))


def test_yolo_planes(orc):
    n, classes, h, w = 3, 2, 4, 5
    x = synth.uniform(1, 2 * n * (5 + classes) * h * w, -3, 3).reshape(2, n * (5 + classes), h, w)
    y = orc.yolo(x, n, classes).reshape(2, n, 5 + classes, h, w)
    xr = x.reshape(2, n, 5 + classes, h, w)
    assert np.array_equal(y[:, :, 2:4], xr[:, :, 2:4])                  # w,h stay raw
    sig = orc.activate(xr, "logistic")
    assert np.array_equal(y[:, :, :2], sig[:, :, :2]) and np.array_equal(y[:, :, 4:], sig[:, :, 4:])


def test_avgpool_and_softmax(orc):
    x = synth.uniform(1, 2 * 5 * 7 * 7).reshape(2, 5, 7, 7)
    assert norm_err(orc.avgpool(x), x.astype(np.float64).mean(axis=(2, 3))) < 1e-6
    z = synth.uniform(2, 3 * 1000, -5, 5).reshape(3, 1000)
    p = orc.softmax(z)
    assert np.allclose(p.sum(axis=1), 1, atol=1e-5) and np.array_equal(p.argmax(1), z.argmax(1))
    e = np.exp(z.astype(np.float64) - z.max(axis=1, keepdims=True))
    assert norm_err(p, e / e.sum(axis=1, keepdims=True)) < 1e-5
    p2 = orc.softmax(z, groups=4, temperature=2.0).reshape(3, 4, 250)
    assert np.allclose(p2.sum(axis=2), 1, atol=1e-5)


def test_binarize_semantics_and_golden(orc):
    x = np.array([0.0, -0.0, 1e-30, -2.0, np.nan, 3.0], np.float32)
    assert np.array_equal(orc.binarize_input(x), np.array([-1, -1, 1, -1, -1, 1], np.float32))
    w = synth.uniform(1, 4 * 27).astype(np.float32)
    w[5] = 0
    bw = orc.binarize_weights(w, 4).reshape(4, 27)
    for f in range(4):
        m = np.float32(0)
        for v in w.reshape(4, 27)[f]:
            m = np.float32(m + abs(v))
        m = np.float32(m / np.float32(27))
        assert np.array_equal(bw[f], np.where(w.reshape(4, 27)[f] > 0, m, -m))
    g = np.load(os.path.join(GOLD, "xnor_case.npz"))
    from util import fill_params
    L = [{"type": "convolutional", "n": 24, "c": 32, "groups": 1, "size": 3, "batch_normalize": 1}]
    params = {}
    fill_params(lambda i, *a: params.update(p=a), L, seed=33, bn="random")
    wt, bias, sc, mu, var = params["p"]
    out, bw, bi = orc.conv(g["input"].reshape(2, 32, 9, 9), wt, bias, sc, mu, var, n=24, size=3, stride=1, pad=1,
                           batch_normalize=1, activation="leaky", xnor=1, return_binary=True)
    assert np.array_equal(bw, g["binary_weights"])
    assert np.array_equal(bi.reshape(2, -1), g["binary_input"])
    assert np.array_equal(out.reshape(2, -1), g["output"])
    # exact-integer form: mean_f * (even integer) - the popcount kernel's arithmetic
    sign_w = np.where(wt.reshape(24, -1) > 0, 1.0, -1.0)
    mean_f = np.abs(bw.reshape(24, -1))[:, 0].astype(np.float64)
    col = np.stack([orc.im2col(np.ascontiguousarray(bi.reshape(2, -1)[b]), 32, 9, 9, 3, 1, 1) for b in range(2)])
    dots = np.einsum("fk,bkn->bfn", sign_w, col.astype(np.float64))
    assert np.all(dots == np.round(dots))
    pre = mean_f.reshape(1, -1, 1) * dots
    y = (pre - mu.reshape(1, -1, 1)) / (np.sqrt(var.astype(np.float64)).reshape(1, -1, 1) + np.float32(1e-6))
    y = y * sc.reshape(1, -1, 1) + bias.reshape(1, -1, 1)
    y = np.where(y > 0, y, 0.1 * y)
    assert norm_err(out.reshape(2, 24, -1), y) < 1e-5


# ---- connected / reorg / flatten / crop ---------------------------------------------------------
def test_connected_against_float64_matmul_and_closed_form(orc):
    o = orc
    rng = np.random.default_rng(3)
    x = rng.uniform(-1, 1, (5, 300)).astype(np.float32)
    w = rng.uniform(-1, 1, (70, 300)).astype(np.float32)
    b = rng.uniform(-1, 1, 70).astype(np.float32)
    got = o.connected(x, w, b, outputs=70, activation="linear")
    want = x.astype(np.float64) @ w.astype(np.float64).T + b
    assert np.abs(got - want).max() <= 1e-4 * np.abs(want).max()
    # small integers: exact; transposing the weight matrix must change the answer (w is [outputs][inputs])
    xi = rng.integers(-4, 5, (3, 6)).astype(np.float32)
    wi = rng.integers(-4, 5, (4, 6)).astype(np.float32)
    bi = rng.integers(-4, 5, 4).astype(np.float32)
    assert np.array_equal(o.connected(xi, wi, bi, outputs=4, activation="linear"), xi @ wi.T + bi)
    assert np.array_equal(o.connected(xi, wi, bi, outputs=4, activation="relu"), np.maximum(xi @ wi.T + bi, 0))
    # batch-norm tail: (x - mean)/(sqrt(var)+1e-6)*scale + bias per output
    sc, mu, var = (rng.uniform(0.5, 2, 4).astype(np.float32) for _ in range(3))
    got = o.connected(xi, wi, bi, sc, mu, var, outputs=4, batch_normalize=1, activation="linear")
    want = ((xi @ wi.T).astype(np.float64) - mu) / (np.sqrt(var.astype(np.float64)) + 1e-6) * sc + bi
    assert np.abs(got - want).max() <= 1e-5


def test_reorg_is_a_permutation_with_the_stated_index_map(orc):
    o = orc
    w, h, c, b, s = 6, 4, 8, 2, 2
    x = np.arange(w * h * c * b, dtype=np.float32)
    fwd = o.reorg(x, w, h, c, b, s, 1)
    back = o.reorg(x, w, h, c, b, s, 0)
    assert sorted(fwd.tolist()) == x.tolist() and sorted(back.tolist()) == x.tolist()
    assert np.array_equal(o.reorg(fwd, w, h, c, b, s, 0), x)        # the two directions are inverses
    # the index map, spelled independently: element (b,k,j,i) of the [c,h,w] walk pairs with
    # (b, k % oc, j*s + (k//oc)//s, i*s + (k//oc)%s) of an [oc, h*s, w*s] tensor, oc = c/s^2
    oc = c // (s * s)
    big = fwd.reshape(b, oc, h * s, w * s)
    walk = x.reshape(b, c, h, w)
    for (bb, k, j, i) in [(0, 0, 0, 0), (1, 5, 3, 2), (0, 7, 1, 5), (1, 2, 0, 4)]:
        assert big[bb, k % oc, j * s + (k // oc) // s, i * s + (k // oc) % s] == walk[bb, k, j, i]
    # the layer: a 2x reorg of yolov2 turns [c, h, w] into [4c, h/2, w/2] as a pure permutation
    img = np.arange(2 * 4 * 4 * 6, dtype=np.float32).reshape(2, 4, 4, 6)
    out = o.reorg_layer(img, 2)
    assert out.shape == (2, 96) and sorted(out.reshape(-1).tolist()) == img.reshape(-1).tolist()
    # the reverse layer walks ITS input's (w,h,c) with the scatter form; it is a permutation too,
    # but not the inverse of the forward layer (both describe the walk with their own input's
    # geometry, src/reorg_layer.c:102-106) - pinned by the golden network, not by an identity
    rev = o.reorg_layer(out.reshape(2, 16, 2, 3), 2, reverse=1)
    assert sorted(rev.reshape(-1).tolist()) == img.reshape(-1).tolist()


def test_flatten_is_a_transpose_and_extra_pads_with_zeros(orc):
    o = orc
    x = np.arange(2 * 5 * 12, dtype=np.float32).reshape(2, 5, 3, 4)
    f = o.reorg_layer(x, 1, flatten=1)
    assert np.array_equal(f.reshape(2, 12, 5), x.reshape(2, 5, 12).transpose(0, 2, 1))
    assert np.array_equal(o.reorg_layer(f.reshape(2, 5, 3, 4), 1, reverse=1, flatten=1).reshape(x.shape), x)
    e = o.reorg_layer(x, 1, extra=3)
    assert e.shape == (2, 63) and np.array_equal(e[:, :60], x.reshape(2, 60)) and not e[:, 60:].any()


def test_crop_takes_the_centred_window_and_rescales(orc):
    o = orc
    x = synth.uniform01(2, 2 * 3 * 9 * 12).reshape(2, 3, 9, 12)
    got = o.crop(x, 4, 6)
    assert np.array_equal(got, x[:, :, 2:6, 3:9] * np.float32(2) + np.float32(-1))   # (9-4)//2 = 2, (12-6)//2 = 3
    assert np.array_equal(o.crop(x, 4, 6, noadjust=1), x[:, :, 2:6, 3:9])
    assert np.array_equal(o.crop(x, 9, 12, noadjust=1), x)
