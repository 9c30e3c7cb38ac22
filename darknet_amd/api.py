"""Python face of the native library, in the spirit of the reference's ``python/darknet.py``
(a ctypes wrapper over ``libdarknet.so``, python/darknet.py:48-115): ``load_net``, ``predict`` and
a small ``Network`` convenience class.  All arithmetic happens in the native library; numpy is
only the host-side container.
"""
from __future__ import annotations

import ctypes as C
import os
import tempfile

import numpy as np

from . import lib as _lib

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
_F = C.POINTER(C.c_float)


def _fp(a):
    return a.ctypes.data_as(_F)


class BOX(C.Structure):
    """python/darknet.py:22-26"""
    _fields_ = [("x", C.c_float), ("y", C.c_float), ("w", C.c_float), ("h", C.c_float)]


class DETECTION(C.Structure):
    """python/darknet.py:28-34"""
    _fields_ = [("bbox", BOX), ("classes", C.c_int), ("prob", _F), ("mask", _F),
                ("objectness", C.c_float), ("sort_class", C.c_int)]


class IMAGE(C.Structure):
    """python/darknet.py:36-40; data is [c][h][w] float32"""
    _fields_ = [("w", C.c_int), ("h", C.c_int), ("c", C.c_int), ("data", _F)]


def _image_of(arr):
    arr = np.ascontiguousarray(arr, np.float32)
    c, h, w = arr.shape
    return IMAGE(w, h, c, _fp(arr)), arr


def _bind_image_calls(L):
    if getattr(L, "_image_calls_bound", False):
        return
    for name in ("letterbox_image", "resize_image"):
        f = getattr(L, name)
        f.argtypes = [IMAGE, C.c_int, C.c_int]
        f.restype = IMAGE
    L.free_image.argtypes = [IMAGE]
    L.free_image.restype = None
    L.network_predict_image.argtypes = [C.c_void_p, IMAGE]
    L.network_predict_image.restype = _F
    L.network_letterbox_input.argtypes = [C.c_void_p, C.c_int, IMAGE]
    L.network_letterbox_input.restype = None
    L._image_calls_bound = True


def _image_call(name, arr, w, h):
    L = _lib.load()
    _bind_image_calls(L)
    im, keep = _image_of(arr)
    out = getattr(L, name)(im, w, h)
    res = np.ctypeslib.as_array(out.data, shape=(out.c, out.h, out.w)).copy()
    L.free_image(out)
    return res


def letterbox_image(arr, w, h):
    """letterbox_image (python/darknet.py:102-104) on an array [c, h, w]."""
    return _image_call("letterbox_image", arr, w, h)


def resize_image(arr, w, h):
    return _image_call("resize_image", arr, w, h)


def _rows_of(dets, n, classes):
    rows = np.zeros((n, 5 + classes), np.float32)
    for i in range(n):
        d = dets[i]
        rows[i, :5] = (d.bbox.x, d.bbox.y, d.bbox.w, d.bbox.h, d.objectness)
        rows[i, 5:] = np.ctypeslib.as_array(d.prob, shape=(classes,)) if classes else 0
    return rows


def do_nms_sort(rows: np.ndarray, classes: int, thresh: float) -> np.ndarray:
    """do_nms_sort (python/darknet.py:98-100) on rows [n, 5 + classes] = x, y, w, h, objectness,
    prob[classes]; returns the rows as the library leaves its detection array."""
    L = _lib.load()
    rows = np.ascontiguousarray(rows, np.float32)
    n = rows.shape[0]
    dets = (DETECTION * max(n, 1))()
    keep = [np.ascontiguousarray(rows[i, 5:]).copy() for i in range(n)]
    for i in range(n):
        dets[i].bbox = BOX(*[float(v) for v in rows[i, :4]])
        dets[i].classes = classes
        dets[i].prob = _fp(keep[i])
        dets[i].objectness = float(rows[i, 4])
    L.do_nms_sort(C.cast(dets, C.c_void_p), n, classes, thresh)
    return _rows_of(dets, n, classes)


def pinned_array(n: int):
    """A zero-filled float32 numpy array over pinned host memory (hip_host_alloc): push/pull and
    network_predict move it with one DMA.  Release it with free_pinned_array."""
    ptr = _lib.load().hip_host_alloc(n)
    return np.ctypeslib.as_array(ptr, shape=(n,))


def free_pinned_array(a):
    _lib.load().hip_host_free(a.ctypes.data_as(C.POINTER(C.c_float)))


def set_gpu(n: int = 0):
    _lib.load().cuda_set_device(n)


def load_net(cfg: str, weights: str = "", clear: int = 0):
    """python/darknet.py:78-80 - returns an opaque ``network *``."""
    return _lib.load().load_network(cfg.encode(), weights.encode() if weights else None, clear)


def predict(net, x: np.ndarray) -> np.ndarray:
    """python/darknet.py:56-58 - network_predict on a float32 array; the result is copied."""
    L = _lib.load()
    x = np.ascontiguousarray(x, np.float32)
    iv = (C.c_int * 8)()
    L.network_info(net, iv)
    out = L.network_predict(net, _fp(x))
    n = iv[1] * _last_outputs(net)
    return np.ctypeslib.as_array(out, shape=(n,)).copy()


def _last_outputs(net):
    L = _lib.load()
    iv = (C.c_int * len(_IV))()
    fv = (C.c_float * len(_FV))()
    L.network_layer_info(net, L.network_num_layers(net) - 1, iv, fv)
    return iv[_IV.index("outputs")]


class DeviceArray:
    """A float32 (or int32) device buffer made with the library's own allocator."""

    def __init__(self, data=None, n=None, dtype=np.float32):
        L = _lib.load()
        self.dtype = np.dtype(dtype)
        if data is not None:
            data = np.ascontiguousarray(data, self.dtype)
            n = data.size
        self.n = int(n)
        if self.dtype == np.float32:
            self.ptr = L.hip_make_array(_fp(data) if data is not None else None, self.n)
        else:
            p = data.ctypes.data_as(C.POINTER(C.c_int)) if data is not None else None
            self.ptr = L.hip_make_int_array(p, self.n)
            if data is None:
                L.fill_gpu(self.n, 0.0, self.ptr, 1)

    def numpy(self, shape=None):
        L = _lib.load()
        out = np.empty(self.n, self.dtype)
        if self.dtype == np.float32:
            L.hip_pull_array(self.ptr, _fp(out), self.n)
        else:
            L.hip_pull_int_array(self.ptr, out.ctypes.data_as(C.POINTER(C.c_int)), self.n)
        return out.reshape(shape) if shape is not None else out

    def free(self):
        if self.ptr:
            _lib.load().hip_free(self.ptr)
            self.ptr = None

    def __del__(self):
        try:
            self.free()
        except Exception:
            pass


class Network:
    """A parsed network living on the GPU."""

    def __init__(self, cfg_text: str = None, cfg_path: str = None, weights: str = ""):
        self.L = _lib.load()
        if cfg_path is None:
            with tempfile.NamedTemporaryFile("w", suffix=".cfg", delete=False) as f:
                f.write(cfg_text)
                cfg_path = f.name
            self._tmp = cfg_path
        else:
            self._tmp = None
        self.net = load_net(cfg_path, weights, 0)
        if self._tmp:
            os.unlink(self._tmp)
        iv = (C.c_int * 8)()
        self.L.network_info(self.net, iv)
        self.n, self.batch, self.h, self.w, self.c, self.inputs, self.outputs = list(iv)[:7]
        self.layers = [self._layer(i) for i in range(self.n)]

    def _layer(self, i):
        iv = (C.c_int * len(_IV))()
        fv = (C.c_float * len(_FV))()
        self.L.network_layer_info(self.net, i, iv, fv)
        d = dict(zip(_IV, list(iv)))
        d.update(zip(_FV, [float(v) for v in fv]))
        d["type"] = LAYER_TYPES[d["type"]]
        d["activation"] = ACTIVATIONS[d["activation"]]
        if d["type"] == "route":
            a = (C.c_int * 16)()
            b = (C.c_int * 16)()
            k = self.L.network_route_inputs(self.net, i, a, b, 16)
            d["input_layers"] = list(a)[:k]
            d["input_sizes"] = list(b)[:k]
        return d

    def set_conv(self, i, weights, biases, scales=None, mean=None, var=None):
        arrs = [None if a is None else np.ascontiguousarray(a, np.float32)
                for a in (weights, biases, scales, mean, var)]
        self.L.network_set_conv(self.net, i, *[None if a is None else _fp(a) for a in arrs])

    def predict(self, x):
        x = np.ascontiguousarray(x, np.float32)
        assert x.size == self.inputs * self.batch, (x.size, self.inputs, self.batch)
        out = self.L.network_predict(self.net, _fp(x))
        last = [L for L in self.layers if L["type"] != "cost"][-1]   # get_network_output_layer
        return np.ctypeslib.as_array(out, shape=(self.batch, last["outputs"])).copy()

    def submit(self, x):
        """network_predict_submit: queue upload, forward and download of one batch (two may be in
        flight).  A pinned array (pinned_array) is used where it is and must stay untouched until
        the batch is collected; anything else is copied before the call returns."""
        x = x if isinstance(x, np.ndarray) and x.dtype == np.float32 and x.flags.c_contiguous else \
            np.ascontiguousarray(x, np.float32)
        assert x.size == self.inputs * self.batch, (x.size, self.inputs, self.batch)
        self.L.network_predict_submit(self.net, _fp(x))

    def collect(self, copy=True):
        """network_predict_collect: the output layer of the oldest batch in flight, [batch, outputs]."""
        out = self.L.network_predict_collect(self.net)
        last = [L for L in self.layers if L["type"] != "cost"][-1]
        a = np.ctypeslib.as_array(out, shape=(self.batch, last["outputs"]))
        return a.copy() if copy else a

    def collected_output(self, i, copy=True):
        """Host copy of layer i (a yolo head or the output layer) of the batch collected last."""
        p = self.L.network_collected_output(self.net, i)
        a = np.ctypeslib.as_array(p, shape=(self.batch, self.layers[i]["outputs"]))
        return a.copy() if copy else a

    def push_input(self, x):
        """Place a batch in the network's device input buffer (for forward_device)."""
        x = np.ascontiguousarray(x, np.float32)
        assert x.size == self.inputs * self.batch
        self._in = x
        ptr = self.input_gpu()
        self.L.hip_push_array(ptr, _fp(x), x.size)

    def input_gpu(self):
        return self.L.network_input_gpu(self.net)

    def forward_device(self):
        self.L.forward_network_device(self.net)

    def forward_profiled(self):
        """One device-resident forward with per-layer HIP events -> (total_ms, [layer_ms])."""
        buf = (C.c_float * self.n)()
        total = self.L.forward_network_profiled(self.net, buf)
        return float(total), [float(v) for v in buf]

    def forward_profiled_kernels(self):
        """forward_profiled plus each convolution's main-kernel duration alone (ms, -1 = none)."""
        buf = (C.c_float * self.n)()
        kbuf = (C.c_float * self.n)()
        total = self.L.forward_network_profiled_kernels(self.net, buf, kbuf)
        return float(total), [float(v) for v in buf], [float(v) for v in kbuf]

    def synchronize(self):
        self.L.hip_synchronize()

    def layer_output(self, i):
        L = self.layers[i]
        p = self.L.layer_output_host(self.net, i)
        return np.ctypeslib.as_array(p, shape=(L["batch"], L["outputs"])).copy()

    def layer_indexes(self, i):
        L = self.layers[i]
        p = self.L.layer_indexes_host(self.net, i)
        return np.ctypeslib.as_array(p, shape=(L["batch"], L["outputs"])).copy()

    def set_batch(self, b):
        """set_batch_network: 1 .. the batch the cfg was parsed with (buffers are sized for that)."""
        self.L.set_batch_network(self.net, b)
        self._refresh_batch()

    def _refresh_batch(self):
        iv = (C.c_int * 8)()
        self.L.network_info(self.net, iv)
        self.batch = list(iv)[1]
        for L in self.layers:          # layer_output / layer_indexes shape their result from these
            L["batch"] = self.batch

    def predict_image(self, arr):
        """network_predict_image (python/darknet.py:106-108): letterbox on the device, batch 1
        (the network stays at batch 1 afterwards, as in the reference; set_batch() brings it back)."""
        _bind_image_calls(self.L)
        im, keep = _image_of(arr)
        out = self.L.network_predict_image(self.net, im)
        self._refresh_batch()
        last = [L for L in self.layers if L["type"] != "cost"][-1]
        return np.ctypeslib.as_array(out, shape=(1, last["outputs"])).copy()

    def letterbox_input(self, b, arr):
        """Letterbox an image [c, h, w] into slot b of the device input (no forward)."""
        _bind_image_calls(self.L)
        im, keep = _image_of(arr)
        self.L.network_letterbox_input(self.net, b, im)
        self.L.hip_synchronize()      # `keep` may be released once the frame has left the host

    def get_boxes(self, w, h, thresh, relative=1, nms=0.0, image=0):
        """get_network_boxes (python/darknet.py:86-88) for `image` of the batch, with the
        suppression of do_nms_sort when nms > 0 -> rows [n, 5 + classes]."""
        num = C.c_int(0)
        dets = self.L.get_network_boxes_image(self.net, image, w, h, thresh, relative, nms, C.byref(num))
        classes = max([L["classes"] for L in self.layers if L["type"] in ("yolo", "region", "detection")] + [0])
        rows = _rows_of(C.cast(dets, C.POINTER(DETECTION)), num.value, classes)
        self.L.free_detections(dets, num.value)
        return rows

    def get_network_boxes(self, w, h, thresh, relative=1):
        """The reference's own call (image 0, no suppression)."""
        num = C.c_int(0)
        dets = self.L.get_network_boxes(self.net, w, h, thresh, 0.5, None, relative, C.byref(num))
        classes = max([L["classes"] for L in self.layers if L["type"] in ("yolo", "region", "detection")] + [0])
        rows = _rows_of(C.cast(dets, C.POINTER(DETECTION)), num.value, classes)
        self.L.free_detections(dets, num.value)
        return rows

    def conv_flops(self):
        return float(self.L.network_conv_flops(self.net))

    def save_weights(self, path):
        self.L.save_weights(self.net, path.encode())

    def load_weights(self, path):
        self.L.load_weights(self.net, path.encode())

    def free(self):
        if self.net:
            self.L.free_network(self.net)
            self.net = None


