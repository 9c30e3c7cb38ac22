"""ctypes bindings to liboracle.so (strict build) and liboracle_fast.so (timing build)."""
from __future__ import annotations

import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_F = C.POINTER(C.c_float)
_D = C.POINTER(C.c_double)
_I = C.POINTER(C.c_int)

ACTIVATIONS = ["logistic", "relu", "relie", "linear", "ramp", "tanh", "plse", "leaky", "elu",
               "loggy", "stair", "hardtan", "lhtan", "selu"]


def build(force: bool = False) -> None:
    """Compile the restatement (both builds) with the committed Makefile."""
    args = ["make", "-C", _HERE, "oracle"]
    if force:
        args.insert(1, "-B")
    subprocess.run(args, check=True, stdout=subprocess.DEVNULL)


def _fp(a: np.ndarray):
    assert a.dtype == np.float32 and a.flags.c_contiguous
    return a.ctypes.data_as(_F)


def _opt(a):
    return None if a is None else _fp(a)


class Oracle:
    def __init__(self, fast: bool = False):
        name = "liboracle_fast.so" if fast else "liboracle.so"
        path = os.path.join(_HERE, name)
        if not os.path.exists(path):
            build()
        self.lib = C.CDLL(path)
        L = self.lib
        L.orc_im2col.argtypes = [_F] + [C.c_int] * 6 + [_F]
        L.orc_gemm_nn.argtypes = [C.c_int] * 3 + [C.c_float, _F, C.c_int, _F, C.c_int, _F, C.c_int]
        L.orc_normalize.argtypes = [_F, _F, _F] + [C.c_int] * 3
        L.orc_scale_bias.argtypes = [_F, _F] + [C.c_int] * 3
        L.orc_add_bias.argtypes = [_F, _F] + [C.c_int] * 3
        L.orc_activate_array.argtypes = [_F, C.c_long, C.c_int]
        L.orc_binarize_weights.argtypes = [_F, C.c_int, C.c_int, _F]
        L.orc_binarize_input.argtypes = [_F, C.c_long, _F]
        L.orc_conv_forward.argtypes = [_F] * 10 + [C.c_int] * 12
        L.orc_conv_forward_f64.argtypes = [_F] * 6 + [_D] + [C.c_int] * 11
        L.orc_maxpool.argtypes = [_F, _F, _I] + [C.c_int] * 7
        L.orc_upsample.argtypes = [_F, _F] + [C.c_int] * 5 + [C.c_float]
        L.orc_shortcut.argtypes = [C.c_int] * 4 + [_F] + [C.c_int] * 3 + [C.c_float, C.c_float, _F]
        L.orc_route_copy.argtypes = [_F, C.c_int, _F, C.c_int, C.c_int, C.c_int]
        L.orc_yolo.argtypes = [_F, _F] + [C.c_int] * 5
        L.orc_avgpool.argtypes = [_F, _F] + [C.c_int] * 4
        L.orc_softmax.argtypes = [_F] + [C.c_int] * 6 + [C.c_float, _F]
        for f in ("orc_im2col", "orc_gemm_nn", "orc_normalize", "orc_scale_bias", "orc_add_bias",
                  "orc_activate_array", "orc_binarize_weights", "orc_binarize_input",
                  "orc_conv_forward", "orc_conv_forward_f64", "orc_maxpool", "orc_upsample",
                  "orc_shortcut", "orc_route_copy", "orc_yolo", "orc_avgpool", "orc_softmax"):
            getattr(L, f).restype = None

    # -- primitives -------------------------------------------------------------------------
    def im2col(self, im, channels, h, w, ksize, stride, pad):
        oh = (h + 2 * pad - ksize) // stride + 1
        ow = (w + 2 * pad - ksize) // stride + 1
        col = np.empty((channels * ksize * ksize, oh * ow), np.float32)
        self.lib.orc_im2col(_fp(im), channels, h, w, ksize, stride, pad, _fp(col))
        return col

    def gemm_nn(self, A, B, Cm=None, alpha=1.0):
        M, K = A.shape
        K2, N = B.shape
        assert K == K2
        if Cm is None:
            Cm = np.zeros((M, N), np.float32)
        self.lib.orc_gemm_nn(M, N, K, alpha, _fp(A), K, _fp(B), N, _fp(Cm), N)
        return Cm

    def activate(self, x, activation):
        y = np.ascontiguousarray(x, np.float32).copy()
        a = ACTIVATIONS.index(activation) if isinstance(activation, str) else activation
        self.lib.orc_activate_array(_fp(y.reshape(-1)), y.size, a)
        return y

    def normalize(self, x, mean, var):
        y = x.copy()
        b, f = y.shape[0], y.shape[1]
        self.lib.orc_normalize(_fp(y), _fp(mean), _fp(var), b, f, y.size // (b * f))
        return y

    def batchnorm_layer(self, x, scales, biases, mean, var):
        """forward_batchnorm_layer at inference (src/batchnorm_layer.c:135-155 with net.train == 0):
        copy, normalize_cpu with the rolling statistics, scale_bias, add_bias, each a pass of its own
        over [batch, c, spatial]."""
        y = np.ascontiguousarray(x, np.float32).copy()
        b, f = y.shape[0], y.shape[1]
        sp = y.size // (b * f)
        self.lib.orc_normalize(_fp(y), _fp(np.ascontiguousarray(mean, np.float32)),
                               _fp(np.ascontiguousarray(var, np.float32)), b, f, sp)
        self.lib.orc_scale_bias(_fp(y), _fp(np.ascontiguousarray(scales, np.float32)), b, f, sp)
        self.lib.orc_add_bias(_fp(y), _fp(np.ascontiguousarray(biases, np.float32)), b, f, sp)
        return y

    def binarize_weights(self, w, n):
        out = np.empty_like(w)
        self.lib.orc_binarize_weights(_fp(w), n, w.size // n, _fp(out))
        return out

    def binarize_input(self, x):
        out = np.empty_like(x)
        self.lib.orc_binarize_input(_fp(x), x.size, _fp(out))
        return out

    # -- layers -----------------------------------------------------------------------------
    def conv(self, x, weights, biases, scales=None, mean=None, var=None, *, n, size, stride, pad,
             groups=1, batch_normalize=0, activation="linear", xnor=0, return_binary=False):
        b, c, h, w = x.shape
        oh = (h + 2 * pad - size) // stride + 1
        ow = (w + 2 * pad - size) // stride + 1
        out = np.empty((b, n, oh, ow), np.float32)
        ws = np.empty(max(1, oh * ow * size * size * (c // groups)), np.float32)
        bw = np.empty(weights.size if xnor else 1, np.float32)
        bi = np.empty(x.size if xnor else 1, np.float32)
        a = ACTIVATIONS.index(activation) if isinstance(activation, str) else activation
        self.lib.orc_conv_forward(_fp(x), _fp(weights), _fp(biases), _opt(scales), _opt(mean),
                                  _opt(var), _fp(out), _fp(ws), _fp(bw), _fp(bi),
                                  b, c, h, w, n, groups, size, stride, pad, batch_normalize, a, xnor)
        if return_binary:
            return out, bw, bi
        return out

    def conv_f64(self, x, weights, biases, scales=None, mean=None, var=None, *, n, size, stride,
                 pad, groups=1, batch_normalize=0, activation="linear"):
        b, c, h, w = x.shape
        oh = (h + 2 * pad - size) // stride + 1
        ow = (w + 2 * pad - size) // stride + 1
        out = np.empty((b, n, oh, ow), np.float64)
        a = ACTIVATIONS.index(activation) if isinstance(activation, str) else activation
        self.lib.orc_conv_forward_f64(_fp(x), _fp(weights), _fp(biases), _opt(scales), _opt(mean),
                                      _opt(var), out.ctypes.data_as(_D),
                                      b, c, h, w, n, groups, size, stride, pad, batch_normalize, a)
        return out

    def maxpool(self, x, size, stride, pad):
        b, c, h, w = x.shape
        oh = (h + pad - size) // stride + 1
        ow = (w + pad - size) // stride + 1
        out = np.empty((b, c, oh, ow), np.float32)
        idx = np.empty((b, c, oh, ow), np.int32)
        self.lib.orc_maxpool(_fp(x), _fp(out), idx.ctypes.data_as(_I), b, c, h, w, size, stride, pad)
        return out, idx

    def upsample(self, x, stride, scale=1.0):
        b, c, h, w = x.shape
        out = np.empty((b, c, h * stride, w * stride), np.float32)
        self.lib.orc_upsample(_fp(x), _fp(out), b, c, h, w, stride, scale)
        return out

    def shortcut(self, x, add, alpha=1.0, beta=1.0, activation="linear"):
        """x: layer input [b,c2,h2,w2]; add: earlier layer output [b,c1,h1,w1]."""
        out = x.copy()
        b, c2, h2, w2 = x.shape
        _, c1, h1, w1 = add.shape
        self.lib.orc_shortcut(b, w1, h1, c1, _fp(add), w2, h2, c2, alpha, beta, _fp(out))
        a = ACTIVATIONS.index(activation) if isinstance(activation, str) else activation
        self.lib.orc_activate_array(_fp(out.reshape(-1)), out.size, a)
        return out

    def route(self, sources):
        """sources: list of [b, ...] arrays; concatenated per image."""
        b = sources[0].shape[0]
        sizes = [s.size // b for s in sources]
        out = np.empty((b, sum(sizes)), np.float32)
        off = 0
        for s, sz in zip(sources, sizes):
            self.lib.orc_route_copy(_fp(s), sz, _fp(out), out.shape[1], off, b)
            off += sz
        return out

    def yolo(self, x, n_anchors, classes):
        b, c, h, w = x.shape
        assert c == n_anchors * (5 + classes)
        out = np.empty_like(x)
        self.lib.orc_yolo(_fp(x), _fp(out), b, w, h, n_anchors, classes)
        return out

    def connected(self, x, weights, biases, scales=None, mean=None, var=None, *, outputs, batch_normalize=0,
                  activation="logistic"):
        x = np.ascontiguousarray(x, np.float32)
        b, inputs = x.shape
        out = np.empty((b, outputs), np.float32)
        wt = np.ascontiguousarray(weights, np.float32)
        assert wt.size == inputs * outputs
        bi = np.ascontiguousarray(biases, np.float32)
        bn = [None if a is None else np.ascontiguousarray(a, np.float32) for a in (scales, mean, var)]
        self.lib.orc_connected_forward(_fp(x), _fp(wt), _fp(bi), _opt(bn[0]), _opt(bn[1]), _opt(bn[2]), _fp(out),
                                       b, inputs, outputs, int(batch_normalize), ACTIVATIONS.index(activation))
        return out

    def reorg(self, x, w, h, c, batch, stride, forward):
        """reorg_cpu on a flat array with the reference's own argument meaning."""
        x = np.ascontiguousarray(x, np.float32)
        out = np.zeros_like(x)
        self.lib.orc_reorg(_fp(x), w, h, c, batch, stride, int(forward), _fp(out))
        return out

    def flatten(self, x, size, layers, batch, forward):
        x = np.ascontiguousarray(x, np.float32)
        out = np.zeros_like(x)
        self.lib.orc_flatten(_fp(x), size, layers, batch, int(forward), _fp(out))
        return out

    def reorg_layer(self, x, stride, reverse=0, flatten=0, extra=0):
        """forward_reorg_layer (src/reorg_layer.c:88-107) on x [b, c, h, w] -> [b, outputs]."""
        x = np.ascontiguousarray(x, np.float32)
        b, c, h, w = x.shape
        if flatten:
            return self.flatten(x, w * h, c, b, 0 if reverse else 1).reshape(b, -1)
        if extra:
            out = np.zeros((b, c * h * w + extra), np.float32)
            out[:, :c * h * w] = x.reshape(b, -1)
            return out
        return self.reorg(x, w, h, c, b, stride, 1 if reverse else 0).reshape(b, -1)

    def crop(self, x, out_h, out_w, noadjust=0):
        x = np.ascontiguousarray(x, np.float32)
        b, c, h, w = x.shape
        out = np.empty((b, c, out_h, out_w), np.float32)
        self.lib.orc_crop(_fp(x), _fp(out), b, c, h, w, out_h, out_w, int(noadjust))
        return out

    def resize_image(self, im, ow, oh):
        im = np.ascontiguousarray(im, np.float32)
        c, h, w = im.shape
        out = np.empty((c, oh, ow), np.float32)
        self.lib.orc_resize_image(_fp(im), w, h, c, _fp(out), ow, oh)
        return out

    def letterbox_image(self, im, bw, bh):
        im = np.ascontiguousarray(im, np.float32)
        c, h, w = im.shape
        out = np.empty((c, bh, bw), np.float32)
        self.lib.orc_letterbox_image(_fp(im), w, h, c, _fp(out), bw, bh)
        return out

    def region(self, x, n_anchors, classes, coords=4, background=0, softmax=1):
        x = np.ascontiguousarray(x, np.float32)
        b, c, h, w = x.shape
        assert c == n_anchors * (coords + classes + 1)
        out = np.empty_like(x)
        self.lib.orc_region(_fp(x), _fp(out), b, w, h, n_anchors, classes, coords, background, softmax)
        return out

    def local(self, x, weights, biases, *, n, size, stride=1, pad=0, activation="logistic"):
        """forward_local_layer on x [b, c, h, w]; pad is the number of zero pixels per side."""
        x = np.ascontiguousarray(x, np.float32)
        b, c, h, w = x.shape
        oh = (h - (1 if pad else size)) // stride + 1
        ow = (w - (1 if pad else size)) // stride + 1
        assert (h + 2 * pad - size) // stride + 1 == oh and (w + 2 * pad - size) // stride + 1 == ow
        wt = np.ascontiguousarray(weights, np.float32)
        bi = np.ascontiguousarray(biases, np.float32)
        assert wt.size == oh * ow * n * size * size * c and bi.size == oh * ow * n
        out = np.empty((b, n, oh, ow), np.float32)
        work = np.empty(size * size * c * oh * ow, np.float32)
        a = ACTIVATIONS.index(activation) if isinstance(activation, str) else activation
        self.lib.orc_local_forward(_fp(x), _fp(wt), _fp(bi), _fp(out), b, c, h, w, n, size, stride, pad, a,
                                   _fp(work))
        return out

    def detection(self, x, side, classes, softmax=0):
        """forward_detection_layer at inference on x [b, inputs]."""
        x = np.ascontiguousarray(x, np.float32)
        out = np.empty_like(x)
        self.lib.orc_detection_forward(_fp(x), _fp(out), x.shape[0], x.shape[1], side, classes, int(softmax))
        return out

    def detection_detections(self, pred, side, n, classes, sqrt, w, h, thresh):
        """get_detection_detections on one image's layer output -> all side*side*n rows."""
        pred = np.ascontiguousarray(pred, np.float32).reshape(-1)
        assert pred.size == side * side * (5 * n + classes)
        rows = np.zeros((side * side * n, 5 + classes), np.float32)
        self.lib.orc_detection_detections(_fp(pred), side, n, classes, int(sqrt), w, h, C.c_float(thresh),
                                          _fp(rows))
        return rows

    def region_detections(self, pred, n_anchors, classes, coords, background, biases, netw, neth, w, h, relative,
                          thresh):
        """get_region_detections on image 0 of `pred` -> all lw*lh*n rows [*, 5 + classes]."""
        pred = np.ascontiguousarray(pred, np.float32)
        lh, lw = pred.shape[-2:]
        rows = np.zeros((lw * lh * n_anchors, 5 + classes), np.float32)
        bi = np.ascontiguousarray(biases, np.float32)
        self.lib.orc_region_detections(_fp(pred), lw, lh, n_anchors, classes, coords, background, _fp(bi), netw,
                                       neth, w, h, relative, C.c_float(thresh), _fp(rows))
        return rows

    def yolo_detections(self, pred, n_anchors, classes, biases, mask, netw, neth, w, h, relative, thresh):
        """get_yolo_detections on image 0 of `pred` [n*(5+classes), lh, lw] -> rows [count, 5+classes]."""
        pred = np.ascontiguousarray(pred, np.float32)
        lh, lw = pred.shape[-2:]
        rows = np.zeros((lw * lh * n_anchors, 5 + classes), np.float32)
        bi = np.ascontiguousarray(biases, np.float32)
        mk = np.ascontiguousarray(mask, np.int32)
        f = self.lib.orc_yolo_detections
        f.restype = C.c_int
        n = f(_fp(pred), lw, lh, n_anchors, classes, _fp(bi), mk.ctypes.data_as(C.POINTER(C.c_int)),
              netw, neth, w, h, relative, C.c_float(thresh), _fp(rows))
        return rows[:n].copy()

    def nms_sort(self, rows, classes, thresh):
        """do_nms_sort on rows [n, 5+classes]; returns the suppressed copy (row order kept)."""
        out = np.ascontiguousarray(rows, np.float32).copy()
        self.lib.orc_nms_sort(_fp(out), out.shape[0], classes, C.c_float(thresh))
        return out

    def box_iou(self, a, b):
        f = self.lib.orc_box_iou
        f.restype = C.c_float
        a = np.ascontiguousarray(a, np.float32)
        b = np.ascontiguousarray(b, np.float32)
        return float(f(_fp(a), _fp(b)))

    def avgpool(self, x):
        b, c, h, w = x.shape
        out = np.empty((b, c), np.float32)
        self.lib.orc_avgpool(_fp(x), _fp(out), b, c, h, w)
        return out

    def softmax(self, x, groups=1, temperature=1.0):
        b = x.shape[0]
        inputs = x.size // b
        out = np.empty_like(x)
        self.lib.orc_softmax(_fp(x), inputs // groups, b, inputs, groups, inputs // groups, 1,
                             temperature, _fp(out))
        return out
