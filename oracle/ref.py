"""Bindings to the compiled reference under oracle/_ref (test infrastructure, optional).

``make -C oracle ref`` builds it where the reference tree is present; the built libraries travel
with the working tree, the reference sources do not.  ``available()`` says whether it is there.
"""
from __future__ import annotations

import ctypes as C
import os

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_F = C.POINTER(C.c_float)
_I = C.POINTER(C.c_int)

# LAYER_TYPE enum order of the reference (include/darknet.h:60-91)
LAYER_TYPES = ["convolutional", "deconvolutional", "connected", "maxpool", "softmax", "detection",
               "dropout", "crop", "route", "cost", "normalization", "avgpool", "local", "shortcut",
               "active", "rnn", "gru", "lstm", "crnn", "batchnorm", "network", "xnor", "region",
               "yolo", "iseg", "reorg", "upsample", "logxent", "l2norm", "blank"]
ACTIVATIONS = ["logistic", "relu", "relie", "linear", "ramp", "tanh", "plse", "leaky", "elu",
               "loggy", "stair", "hardtan", "lhtan", "selu"]

_IV = ["type", "batch", "h", "w", "c", "out_h", "out_w", "out_c", "n", "size", "stride", "pad",
       "groups", "batch_normalize", "activation", "binary", "xnor", "index", "inputs", "outputs",
       "nweights", "classes", "total", "reverse", "workspace_floats", "nbiases", "truths",
       "max_boxes"]
_FV = ["alpha", "beta", "scale", "temperature"]


_HARNESS = {"fast": "librefh.so", "o2": "librefh_o2.so", "hip": "librefh_hip.so"}
_LIBRARY = {"fast": "libdarknet_ref.so", "o2": "libdarknet_ref_o2.so", "hip": "libdarknet_ref_hip.so"}


def _path(variant: str) -> str:
    """fast / o2: the reference's CPU build.  hip: the reference's own host files built with -DGPU
    and bound to darknet_amd/libdarknet_hip.so through integration/adapters.c - the same calls then
    run the reference's parse_network_cfg / network_predict / forward_network_gpu on the HIP kernels."""
    return os.path.join(_HERE, "_ref", _HARNESS[variant])


def available(variant: str = "o2") -> bool:
    return os.path.exists(_path(variant))


def raw(variant: str = "o2"):
    """The reference library itself (plain-pointer functions such as im2col_cpu, gemm)."""
    return C.CDLL(os.path.join(_HERE, "_ref", _LIBRARY[variant]))


def _harness(variant="o2"):
    raw(variant)
    return C.CDLL(_path(variant))


def resize_image(im, ow, oh, variant="o2"):
    """resize_image of the compiled reference on an array [c, h, w]."""
    im = np.ascontiguousarray(im, np.float32)
    c, h, w = im.shape
    out = np.empty((c, oh, ow), np.float32)
    _harness(variant).refh_resize_image(im.ctypes.data_as(_F), w, h, c, ow, oh, out.ctypes.data_as(_F))
    return out


def letterbox_image(im, bw, bh, variant="o2"):
    im = np.ascontiguousarray(im, np.float32)
    c, h, w = im.shape
    out = np.empty((c, bh, bw), np.float32)
    _harness(variant).refh_letterbox_image(im.ctypes.data_as(_F), w, h, c, bw, bh, out.ctypes.data_as(_F))
    return out


class RefNet:
    """A network parsed and run by the compiled reference (CPU build, or variant "hip")."""

    def __init__(self, cfg_path: str, variant: str = "o2", gpu: int | None = 0):
        self.lib = raw(variant)
        self.h = C.CDLL(_path(variant))
        H = self.h
        for f in (self.lib.load_weights, self.lib.save_weights):
            f.restype = None
            f.argtypes = [C.c_void_p, C.c_char_p]
        if variant == "hip" and gpu is not None:
            H.refh_set_gpu(gpu)
        H.refh_load.restype = C.c_void_p
        H.refh_load.argtypes = [C.c_char_p]
        H.refh_free.argtypes = [C.c_void_p]
        H.refh_nlayers.argtypes = [C.c_void_p]
        H.refh_net_info.argtypes = [C.c_void_p, _I]
        H.refh_layer_info.argtypes = [C.c_void_p, C.c_int, _I, _F]
        H.refh_route_inputs.argtypes = [C.c_void_p, C.c_int, _I, _I, C.c_int]
        H.refh_yolo_mask.argtypes = [C.c_void_p, C.c_int, _I, C.c_int, _F, C.c_int]
        H.refh_set_conv.argtypes = [C.c_void_p, C.c_int] + [_F] * 5
        H.refh_set_connected.argtypes = [C.c_void_p, C.c_int] + [_F] * 5
        H.refh_set_local.argtypes = [C.c_void_p, C.c_int] + [_F] * 2
        H.refh_set_batchnorm.argtypes = [C.c_void_p, C.c_int] + [_F] * 4
        H.refh_predict.restype = _F
        H.refh_predict.argtypes = [C.c_void_p, _F]
        for f in ("refh_layer_output", "refh_layer_weights", "refh_layer_binary_weights",
                  "refh_layer_binary_input"):
            getattr(H, f).restype = _F
            getattr(H, f).argtypes = [C.c_void_p, C.c_int]
        H.refh_layer_indexes.restype = _I
        H.refh_layer_indexes.argtypes = [C.c_void_p, C.c_int]
        H.refh_forward_layer.argtypes = [C.c_void_p, C.c_int, _F]
        H.refh_get_boxes.argtypes = [C.c_void_p, C.c_int, C.c_int, C.c_float, C.c_int, C.c_float, _F, C.c_int]
        H.refh_set_output.argtypes = [C.c_void_p, C.c_int, _F]
        self.net = H.refh_load(cfg_path.encode())
        if not self.net:
            raise RuntimeError("reference failed to parse " + cfg_path)
        iv = (C.c_int * 8)()
        H.refh_net_info(self.net, iv)
        self.n, self.batch, self.height, self.width, self.channels, self.inputs, self.outputs = list(iv)[:7]
        self.layers = [self._layer(i) for i in range(self.n)]

    def _layer(self, i):
        iv = (C.c_int * len(_IV))()
        fv = (C.c_float * len(_FV))()
        self.h.refh_layer_info(self.net, i, iv, fv)
        d = dict(zip(_IV, list(iv)))
        d.update(zip(_FV, [float(v) for v in fv]))
        d["type"] = LAYER_TYPES[d["type"]]
        d["activation"] = ACTIVATIONS[d["activation"]]
        if d["type"] == "route":
            a = (C.c_int * 16)()
            b = (C.c_int * 16)()
            k = self.h.refh_route_inputs(self.net, i, a, b, 16)
            d["input_layers"] = list(a)[:k]
            d["input_sizes"] = list(b)[:k]
        if d["type"] == "yolo":
            m = (C.c_int * 32)()
            an = (C.c_float * 64)()
            k = self.h.refh_yolo_mask(self.net, i, m, 32, an, 64)
            d["mask"] = list(m)[:k]
            d["anchors"] = [float(v) for v in an][:2 * d["total"]]
        return d

    def set_conv(self, i, weights, biases, scales=None, mean=None, var=None):
        p = lambda a: None if a is None else np.ascontiguousarray(a, np.float32).ctypes.data_as(_F)
        if self.layers[i]["type"] == "local":
            self.h.refh_set_local(self.net, i, p(weights), p(biases))
            return
        if self.layers[i]["type"] == "batchnorm":
            self.h.refh_set_batchnorm(self.net, i, p(biases), p(scales), p(mean), p(var))
            return
        f = self.h.refh_set_connected if self.layers[i]["type"] == "connected" else self.h.refh_set_conv
        f(self.net, i, p(weights), p(biases), p(scales), p(mean), p(var))

    def set_output(self, i, values):
        """Overwrite layer i's host output (drives get_boxes with chosen yolo tensors)."""
        v = np.ascontiguousarray(values, np.float32)
        assert v.size == self.layers[i]["outputs"] * self.batch
        self.h.refh_set_output(self.net, i, v.ctypes.data_as(_F))

    def get_boxes(self, w, h, thresh, relative=1, nms=0.0):
        """get_network_boxes (+ do_nms_sort when nms > 0) -> rows [n, 5 + classes]."""
        classes = self.layers[-1]["classes"]
        cap = sum(L["w"] * L["h"] * L["n"] for L in self.layers if L["type"] in ("yolo", "region", "detection"))
        rows = np.zeros((max(cap, 1), 5 + classes), np.float32)
        n = self.h.refh_get_boxes(self.net, w, h, thresh, relative, nms, rows.ctypes.data_as(_F), cap)
        return rows[:n].copy()

    def load_weights(self, path):
        """load_weights of the reference (src/parser.c:1308); its GPU build ends each layer's load with
        push_convolutional_layer (:1210-1214)."""
        self.lib.load_weights(self.net, path.encode())

    def save_weights(self, path):
        self.lib.save_weights(self.net, path.encode())

    def free(self):
        if self.net:
            self.h.refh_free(self.net)
            self.net = None

    def predict(self, x):
        x = np.ascontiguousarray(x, np.float32)
        assert x.size == self.inputs * self.batch
        self.h.refh_predict(self.net, x.ctypes.data_as(_F))
        return [self.layer_output(i) for i in range(self.n)]

    def layer_output(self, i):
        L = self.layers[i]
        p = self.h.refh_layer_output(self.net, i)
        return np.ctypeslib.as_array(p, shape=(L["batch"], L["outputs"])).copy()

    def layer_indexes(self, i):
        L = self.layers[i]
        p = self.h.refh_layer_indexes(self.net, i)
        return np.ctypeslib.as_array(p, shape=(L["batch"], L["outputs"])).copy()

    def forward_layer(self, i, x):
        """Run layer i alone on input x; returns its output."""
        x = np.ascontiguousarray(x, np.float32)
        self.h.refh_forward_layer(self.net, i, x.ctypes.data_as(_F))
        return self.layer_output(i)

    def binary_tensors(self, i):
        L = self.layers[i]
        bw = np.ctypeslib.as_array(self.h.refh_layer_binary_weights(self.net, i), shape=(L["nweights"],)).copy()
        bi = np.ctypeslib.as_array(self.h.refh_layer_binary_input(self.net, i), shape=(L["batch"], L["inputs"])).copy()
        return bw, bi
