"""Parity of the memory-bound HIP kernels against the CPU checker, through the C-ABI.
Index / copy work (im2col, maxpool + indexes, upsample, route, shortcut, binarize) must be
bit-exact; arithmetic chains that the library evaluates exactly like the CPU (activations,
bias, scale) are also compared bit for bit; reductions (avgpool, softmax) within 1e-6."""
import ctypes as C
import os

import numpy as np
import pytest

from darknet_amd import api, cfgs, synth
from oracle.cpu import ACTIVATIONS

from util import fill_params, norm_err

pytestmark = pytest.mark.gpu
GOLD = os.path.join(os.path.dirname(__file__), "golden")
D = api.DeviceArray


@pytest.mark.parametrize("c,h,w,k,s,p", [(16, 26, 26, 3, 1, 1), (8, 52, 40, 3, 2, 1), (3, 33, 31, 7, 2, 3),
                                         (5, 9, 9, 1, 1, 0), (2, 8, 9, 5, 2, 2)])
def test_im2col_bit_exact(dn, orc, c, h, w, k, s, p):
    im = synth.uniform(2, c * h * w)
    want = orc.im2col(im, c, h, w, k, s, p)
    d_im, d_col = D(im), D(n=want.size)
    dn.im2col_gpu(d_im.ptr, c, h, w, k, s, p, d_col.ptr)
    assert np.array_equal(d_col.numpy(want.shape), want)


@pytest.mark.parametrize("b,c,h,w,size,stride,pad", [(2, 16, 416 // 8, 416 // 8, 2, 2, 1), (1, 4, 13, 13, 2, 1, 1),
                                                     (2, 3, 9, 7, 3, 2, 2), (1, 2, 10, 10, 3, 1, 0),
                                                     (3, 5, 7, 9, 2, 2, 1), (1, 1, 1, 1, 2, 2, 1)])
def test_maxpool_bit_exact_with_indexes(dn, orc, b, c, h, w, size, stride, pad):
    x = synth.uniform(5, b * c * h * w).reshape(b, c, h, w)
    x.reshape(-1)[3::7] = x.reshape(-1)[2::7][: x.reshape(-1)[3::7].size]      # ties
    out, idx = orc.maxpool(x, size, stride, pad)
    d_x, d_o, d_i = D(x), D(n=out.size), D(n=out.size, dtype=np.int32)
    dn.forward_maxpool_gpu(d_x.ptr, d_o.ptr, d_i.ptr, b, c, h, w, size, stride, pad)
    assert np.array_equal(d_o.numpy(out.shape), out)
    assert np.array_equal(d_i.numpy(out.shape), idx)
    dn.forward_maxpool_gpu(d_x.ptr, d_o.ptr, None, b, c, h, w, size, stride, pad)   # indexes are optional
    assert np.array_equal(d_o.numpy(out.shape), out)


def test_maxpool_golden(dn):
    g = np.load(os.path.join(GOLD, "maxpool_case.npz"))
    for name in ("s2", "s1pad", "k3s2"):
        b, c, h, w, size, stride, pad = [int(v) for v in g[name + "_spec"]]
        d_x, d_o, d_i = D(g[name + "_in"]), D(n=g[name + "_out"].size), D(n=g[name + "_out"].size, dtype=np.int32)
        dn.forward_maxpool_gpu(d_x.ptr, d_o.ptr, d_i.ptr, b, c, h, w, size, stride, pad)
        assert np.array_equal(d_o.numpy(g[name + "_out"].shape), g[name + "_out"])
        assert np.array_equal(d_i.numpy(g[name + "_idx"].shape), g[name + "_idx"])


@pytest.mark.parametrize("b,c,h,w,stride,scale", [(2, 128, 13, 13, 2, 1.0), (1, 3, 5, 7, 3, 1.0), (2, 4, 6, 6, 2, 0.5),
                                                  (1, 2, 3, 4, 1, 1.0)])
def test_upsample_bit_exact(dn, orc, b, c, h, w, stride, scale):
    x = synth.uniform(3, b * c * h * w).reshape(b, c, h, w)
    want = orc.upsample(x, stride, scale)
    d_x, d_o = D(x), D(n=want.size)
    dn.upsample_gpu(d_x.ptr, w, h, c, b, stride, 1, scale, d_o.ptr)
    assert np.array_equal(d_o.numpy(want.shape), want)


@pytest.mark.parametrize("sizes,batch", [([256 * 26 * 26, 512 * 26 * 26], 2), ([10, 4, 7], 3), ([128], 5),
                                         ([4, 8, 12, 16, 20, 24, 28, 32], 2)])
def test_route_bit_exact(dn, orc, sizes, batch):
    srcs = [synth.uniform(10 + i, batch * s).reshape(batch, s) for i, s in enumerate(sizes)]
    want = orc.route(srcs)
    d_srcs = [D(s) for s in srcs]
    d_o = D(n=want.size)
    ptrs = (C.c_void_p * len(sizes))(*[d.ptr for d in d_srcs])
    szs = (C.c_int * len(sizes))(*sizes)
    dn.forward_route_gpu(ptrs, szs, len(sizes), d_o.ptr, batch)
    assert np.array_equal(d_o.numpy(want.shape), want)


@pytest.mark.parametrize("shape_in,shape_add,alpha,beta,act", [
    ((2, 64, 26, 26), (2, 64, 26, 26), 1.0, 1.0, "linear"),      # darknet53 residual
    ((2, 256, 14, 14), (2, 64, 14, 14), 1.0, 1.0, "leaky"),      # resnext: fewer channels in `add`
    ((2, 32, 7, 7), (2, 16, 14, 14), 1.0, 1.0, "leaky"),         # resnext: `add` twice as large
    ((1, 8, 6, 6), (1, 8, 3, 3), 0.5, 2.0, "logistic"),          # `add` smaller, general scales
    ((1, 3, 5, 5), (1, 3, 5, 5), 1.0, 1.0, "relu"),              # odd size -> scalar path
    ((2, 16, 8, 8), (2, 64, 8, 8), 1.0, 1.0, "linear"),          # more channels in `add` than in the output
    ((1, 8, 7, 7), (1, 4, 7, 7), 1.0, 1.0, "leaky"),             # odd plane, fewer channels in `add`
    ((3, 20, 6, 10), (3, 12, 12, 20), 1.0, 0.5, "leaky"),        # `add` twice as large, not square
    ((2, 6, 12, 20), (2, 10, 6, 10), 1.0, 1.0, "linear")])       # `add` half as large, not square
def test_shortcut_bit_exact(dn, orc, shape_in, shape_add, alpha, beta, act):
    x = synth.uniform(1, int(np.prod(shape_in)), -2, 2).reshape(shape_in)
    add = synth.uniform(2, int(np.prod(shape_add)), -2, 2).reshape(shape_add)
    want = orc.shortcut(x, add, alpha, beta, act)
    d_x, d_a, d_o = D(x), D(add), D(n=want.size)
    b, c2, h2, w2 = shape_in
    _, c1, h1, w1 = shape_add
    dn.forward_shortcut_gpu(d_x.ptr, d_a.ptr, d_o.ptr, b, w1, h1, c1, w2, h2, c2, alpha, beta,
                            ACTIVATIONS.index(act))
    assert np.array_equal(d_o.numpy(want.shape), want)
    # the reference-named in-place helper (out already holds the layer input)
    if act == "linear":
        d_io = D(x)
        dn.shortcut_gpu(b, w1, h1, c1, d_a.ptr, w2, h2, c2, alpha, beta, d_io.ptr)
        assert np.array_equal(d_io.numpy(want.shape), want)


@pytest.mark.parametrize("b,w,h,n,classes", [(2, 13, 13, 3, 80), (1, 5, 4, 2, 1), (3, 7, 7, 3, 0)])
def test_yolo_logistic(dn, orc, b, w, h, n, classes):
    x = synth.uniform(4, b * n * (5 + classes) * h * w, -6, 6).reshape(b, n * (5 + classes), h, w)
    want = orc.yolo(x, n, classes)
    d_x, d_o = D(x), D(n=want.size)
    dn.forward_yolo_gpu(d_x.ptr, d_o.ptr, b, w, h, n, classes)
    got = d_o.numpy(want.shape)
    gr, xr = got.reshape(b, n, 5 + classes, h, w), x.reshape(b, n, 5 + classes, h, w)
    assert np.array_equal(gr[:, :, 2:4], xr[:, :, 2:4])          # raw planes byte-identical
    assert np.abs(got - want).max() <= 1e-6                      # logistic: device exp vs libm exp


@pytest.mark.parametrize("act", ACTIVATIONS)
def test_activate_array(dn, orc, act):
    x = np.concatenate([synth.uniform(9, 4093, -6, 6), np.array([0.0, -0.0, 1.0, -1.0, 4.0, -4.0, 5.0], np.float32)])
    want = orc.activate(x, act)
    d = D(x)
    dn.activate_array_gpu(d.ptr, x.size, ACTIVATIONS.index(act))
    got = d.numpy()
    if act in ("linear", "relu", "relie", "ramp", "plse", "leaky", "stair", "hardtan", "lhtan"):
        assert np.array_equal(got, want)                         # no transcendental involved
    else:
        assert norm_err(got, want) <= 2e-7


def test_bias_scale_normalize_fill_copy(dn, orc):
    b, f, sp = 2, 5, 33
    x = synth.uniform(1, b * f * sp).reshape(b, f, sp)
    bias, sc, mu, var = synth.bn_random(2, f)
    d, d_mu, d_var = D(x), D(mu), D(var)          # keep the device buffers alive across the call
    dn.normalize_gpu(d.ptr, d_mu.ptr, d_var.ptr, b, f, sp)
    want = orc.normalize(x, mu, var)
    assert norm_err(d.numpy(x.shape), want) <= 1.2e-7            # reciprocal-multiply vs divide
    d = D(x)
    keep = [D(sc), D(bias)]
    dn.scale_bias_gpu(d.ptr, keep[0].ptr, b, f, sp)
    dn.add_bias_gpu(d.ptr, keep[1].ptr, b, f, sp)
    assert np.array_equal(d.numpy(x.shape), x * sc.reshape(1, f, 1) + bias.reshape(1, f, 1))
    d = D(n=1001)
    dn.fill_gpu(1001, 2.5, d.ptr, 1)
    assert np.all(d.numpy() == 2.5)
    dn.fill_gpu(334, -1.0, d.ptr, 3)
    got = d.numpy()
    assert np.all(got[::3] == -1.0) and np.all(got[1::3] == 2.5)
    src, dst = D(np.arange(64, dtype=np.float32)), D(n=64)
    dn.copy_gpu(64, src.ptr, 1, dst.ptr, 1)
    assert np.array_equal(dst.numpy(), np.arange(64, dtype=np.float32))
    dn.copy_gpu_offset(10, src.ptr, 5, 2, dst.ptr, 1, 3)
    got = dst.numpy()
    assert np.array_equal(got[1:31:3], np.arange(5, 25, 2, dtype=np.float32))


def test_avgpool_softmax(dn, orc):
    x = synth.uniform(1, 4 * 100 * 7 * 7).reshape(4, 100, 7, 7)
    d_x, d_o = D(x), D(n=400)
    dn.forward_avgpool_gpu(d_x.ptr, d_o.ptr, 4, 100, 7, 7)
    assert norm_err(d_o.numpy((4, 100)), orc.avgpool(x)) <= 1e-6
    z = synth.uniform(2, 6 * 1000, -8, 8).reshape(6, 1000)
    d_z, d_p = D(z), D(n=z.size)
    dn.softmax_gpu(d_z.ptr, 1000, 6, 1000, 1, 1000, 1, 1.0, d_p.ptr)
    got = d_p.numpy(z.shape)
    # the CPU sums 1000 exponentials sequentially in fp32, the kernel as a 64-lane tree: both are
    # ~1e-6 from the exact sum, so they differ from each other by about as much
    assert norm_err(got, orc.softmax(z)) <= 5e-6 and np.array_equal(got.argmax(1), z.argmax(1))
    dn.softmax_gpu(d_z.ptr, 250, 6, 1000, 4, 250, 1, 2.0, d_p.ptr)
    assert norm_err(d_p.numpy(z.shape), orc.softmax(z, groups=4, temperature=2.0)) <= 5e-6


def test_binarize_bit_exact(dn, orc):
    x = synth.uniform(3, 5000, -1, 1)
    x[::13] = 0.0
    x[1::97] = -0.0
    d_x, d_b = D(x), D(n=x.size)
    dn.binarize_gpu(d_x.ptr, x.size, d_b.ptr)
    assert np.array_equal(d_b.numpy(), orc.binarize_input(x))
    w = synth.uniform(4, 24 * 288)
    w[7] = 0.0
    d_w, d_bw = D(w), D(n=w.size)
    dn.binarize_weights_gpu(d_w.ptr, 24, 288, d_bw.ptr)
    assert np.array_equal(d_bw.numpy(), orc.binarize_weights(w, 24))


@pytest.mark.parametrize("w,h,c,b,s", [(6, 4, 8, 2, 2), (13, 13, 64, 3, 2), (5, 7, 9, 1, 3), (8, 8, 4, 2, 1)])
def test_reorg_gpu_both_directions(dn, orc, w, h, c, b, s):
    x = synth.uniform(4, w * h * c * b, -1, 1)
    for forward in (1, 0):
        out = D(n=x.size)
        keep = D(x)
        dn.reorg_gpu(keep.ptr, w, h, c, b, s, forward, out.ptr)
        assert np.array_equal(out.numpy(), orc.reorg(x, w, h, c, b, s, forward))


def test_flatten_and_crop_gpu(dn, orc):
    x = synth.uniform(5, 3 * 10 * 6 * 7, -1, 1).reshape(3, 10, 6, 7)
    for forward in (1, 0):
        out, keep = D(n=x.size), D(x)
        dn.flatten_gpu(keep.ptr, 42, 10, 3, forward, out.ptr)
        assert np.array_equal(out.numpy(), orc.flatten(x.reshape(-1), 42, 10, 3, forward))
    for oh, ow, noadjust in [(4, 5, 0), (6, 7, 1), (1, 1, 0), (3, 2, 1)]:
        out, keep = D(n=3 * 10 * oh * ow), D(x)
        dn.forward_crop_gpu(keep.ptr, out.ptr, 3, 10, 6, 7, oh, ow, noadjust)
        assert np.array_equal(out.numpy((3, 10, oh, ow)), orc.crop(x, oh, ow, noadjust))


@pytest.mark.parametrize("n", [(4 << 20) // 4 - 1, (4 << 20) // 4, (16 << 20) // 4 + 123, (48 << 20) // 4 + 5,
                               (16 << 20) // 4 * 2])
def test_large_copies_round_trip_through_the_staging_buffers(dn, n):
    """Copies of 4 MB and more are cut into 16 MB chunks that alternate between two pinned buffers;
    sizes sit on and around the chunk and threshold boundaries."""
    x = synth.uniform(n % 97, n, -1, 1)
    d = D(x)                       # hip_make_array: plain copy
    back = np.empty_like(x)
    dn.hip_pull_array(d.ptr, api._fp(back), n)
    assert np.array_equal(back, x)
    y = synth.uniform(7, n, -1, 1)
    dn.hip_push_array(d.ptr, api._fp(y), n)
    dn.hip_pull_array(d.ptr, api._fp(back), n)
    assert np.array_equal(back, y)
    # a kernel queued before the pull must be seen by it
    dn.fill_gpu(1000, 3.5, d.ptr, 1)
    dn.hip_pull_array(d.ptr, api._fp(back), n)
    assert np.all(back[:1000] == 3.5) and np.array_equal(back[1000:], y[1000:])


def test_pinned_host_buffers_copy_directly_and_predict_the_same(dn):
    """hip_host_alloc memory is zero-filled, moves with push/pull like any host buffer (also from the
    middle of the block and across the staging threshold), and a batch built in it gives the bits
    network_predict gives for the same batch in pageable memory."""
    n = (8 << 20) // 4 + 77
    a = api.pinned_array(n)
    assert a.dtype == np.float32 and not a.any()
    x = synth.uniform(5, n, -1, 1)
    a[:] = x
    d = D(n=n)
    dn.hip_push_array(d.ptr, api._fp(a), n)
    dn.fill_gpu(500, -2.0, d.ptr, 1)                # queued work is seen by the pull
    b = api.pinned_array(n + 10)
    dn.hip_pull_array(d.ptr, api._fp(b[10:]), n)    # inside the pinned block, offset start
    assert np.all(b[10:510] == -2.0) and np.array_equal(b[510:], x[500:]) and not b[:10].any()
    api.free_pinned_array(a)
    api.free_pinned_array(b)

    net = api.Network(cfg_text=cfgs.yolov3_tiny(2, 96))
    fill_params(net.set_conv, net.layers)
    xin = synth.uniform01(9, net.inputs * 2)
    want = net.predict(xin)
    p = api.pinned_array(xin.size)
    p[:] = xin
    got = net.predict(p)
    assert np.array_equal(got, want)
    api.free_pinned_array(p)
    net.free()


def test_forward_batchnorm_gpu_bit_exact(dn, orc):
    """The standalone batch-norm forward: one pass, the bits of the reference's four."""
    x = synth.uniform(5, 5 * 13 * 33).reshape(5, 13, 33)
    bias, scale, mean, var = synth.bn_random(6, 13)
    want = orc.batchnorm_layer(x, scale, bias, mean, var)
    d = [api.DeviceArray(a) for a in (x, scale, bias, mean, var)]
    out = api.DeviceArray(n=x.size)
    dn.forward_batchnorm_gpu(d[0].ptr, out.ptr, d[1].ptr, d[2].ptr, d[3].ptr, d[4].ptr, 5, 13, 33)
    assert np.array_equal(out.numpy(x.shape), want)
    dn.forward_batchnorm_gpu(d[0].ptr, d[0].ptr, d[1].ptr, d[2].ptr, d[3].ptr, d[4].ptr, 5, 13, 33)   # in place
    assert np.array_equal(d[0].numpy(x.shape), want)


def test_cuda_random_fills_the_unit_interval(dn):
    """cuda_random (src/cuda.c:106): uniform floats in (0, 1], a new stream on every call."""
    n = 1 << 20
    a, b = api.DeviceArray(n=n), api.DeviceArray(n=n)
    dn.cuda_random(a.ptr, n)
    dn.cuda_random(b.ptr, n)
    x, y = a.numpy(), b.numpy()
    for v in (x, y):
        assert v.min() > 0 and v.max() <= 1 and abs(v.mean() - 0.5) < 2e-3 and abs(v.var() - 1 / 12) < 1e-3
    assert (x != y).mean() > 0.99
