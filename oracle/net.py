"""forward_network over a parsed layer table, on the CPU restatement (test infrastructure).

Restates the CPU loop of src/network.c:188-211: each layer's forward reads the previous
layer's output (``net.input = l.output``), route and shortcut reach back into earlier outputs.
"""
from __future__ import annotations

import numpy as np

from . import cfg as _cfg
from .cpu import Oracle


class OracleNet:
    def __init__(self, cfg_text: str, fast: bool = False):
        self.net = _cfg.parse(cfg_text)
        self.orc = Oracle(fast=fast)
        self.params = {}

    @property
    def layers(self):
        return self.net["layers"]

    def set_conv(self, i, weights, biases, scales=None, mean=None, var=None):
        self.params[i] = tuple(None if a is None else np.ascontiguousarray(a, np.float32)
                               for a in (weights, biases, scales, mean, var))

    def forward_layer(self, i, x, outs):
        L = self.layers[i]
        o = self.orc
        t = L["type"]
        b = L["batch"]
        if t == "convolutional":
            w, bi, sc, mu, var = self.params[i]
            return o.conv(x.reshape(b, L["c"], L["h"], L["w"]), w, bi, sc, mu, var, n=L["n"],
                          size=L["size"], stride=L["stride"], pad=L["pad"], groups=L["groups"],
                          batch_normalize=L["batch_normalize"], activation=L["activation"],
                          xnor=L["xnor"])
        if t == "maxpool":
            return o.maxpool(x.reshape(b, L["c"], L["h"], L["w"]), L["size"], L["stride"], L["pad"])[0]
        if t == "upsample":
            return o.upsample(x.reshape(b, L["c"], L["h"], L["w"]), L["stride"], L["scale"])
        if t == "shortcut":
            add = outs[L["index"]].reshape(b, L["c"], L["h"], L["w"])
            return o.shortcut(x.reshape(b, L["out_c"], L["out_h"], L["out_w"]), add,
                              L["alpha"], L["beta"], L["activation"])
        if t == "route":
            return o.route([outs[j].reshape(b, -1) for j in L["input_layers"]])
        if t == "yolo":
            return o.yolo(x.reshape(b, L["c"], L["h"], L["w"]), L["n"], L["classes"])
        if t == "avgpool":
            return o.avgpool(x.reshape(b, L["c"], L["h"], L["w"]))
        if t == "softmax":
            return o.softmax(x.reshape(b, -1), L["groups"], L["temperature"])
        if t == "region":
            return o.region(x.reshape(b, L["c"], L["h"], L["w"]), L["n"], L["classes"], L["coords"],
                            L["background"], L["softmax"])
        if t == "local":
            w, bi = self.params[i][:2]
            return o.local(x.reshape(b, L["c"], L["h"], L["w"]), w, bi, n=L["n"], size=L["size"],
                           stride=L["stride"], pad=L["pad"], activation=L["activation"])
        if t == "detection":
            return o.detection(x.reshape(b, -1), L["side"], L["classes"], L["softmax"])
        if t == "connected":
            w, bi, sc, mu, var = self.params[i]
            return o.connected(x.reshape(b, -1), w, bi, sc, mu, var, outputs=L["outputs"],
                               batch_normalize=L["batch_normalize"], activation=L["activation"])
        if t == "batchnorm":
            _, bi, sc, mu, var = self.params[i]
            return o.batchnorm_layer(x.reshape(b, L["c"], L["h"] * L["w"]), sc, bi, mu, var)
        if t == "dropout":
            return x                                   # forward_dropout_layer returns at once when not training
        if t == "cost":
            return np.zeros((b, L["outputs"]), np.float32)   # no truth: the output buffer is never written
        if t == "crop":
            return o.crop(x.reshape(b, L["c"], L["h"], L["w"]), L["out_h"], L["out_w"], L["noadjust"])
        if t == "reorg":
            return o.reorg_layer(x.reshape(b, L["c"], L["h"], L["w"]), L["stride"], L["reverse"], L["flatten"],
                                 L["extra"])
        raise NotImplementedError(t)

    def forward(self, x, upto=None):
        """Returns the list of every layer's output (flattened per image: [batch, outputs])."""
        outs = []
        cur = np.ascontiguousarray(x, np.float32)
        n = self.net["n"] if upto is None else upto
        for i in range(n):
            y = self.forward_layer(i, cur, outs)
            y = np.ascontiguousarray(y).reshape(self.layers[i]["batch"], -1)
            outs.append(y)
            cur = y
        return outs

    def get_boxes(self, outs, w, h, thresh, relative=1, nms=0.0, image=0):
        """get_network_boxes (src/network.c:563, fill order :543-561) on layer outputs `outs`,
        then do_nms_sort when nms > 0.  Rows [n, 5 + classes] in the reference's fill order."""
        rows = []
        classes = 0
        for i, L in enumerate(self.layers):
            if L["type"] == "region":
                classes = L["classes"]
                pred = np.asarray(outs[i], np.float32).reshape(L["batch"], L["c"], L["h"], L["w"])[image]
                rows.append(self.orc.region_detections(pred, L["n"], classes, L["coords"], L["background"],
                                                       L["anchors"], self.net["w"], self.net["h"], w, h, relative,
                                                       thresh))
                continue
            if L["type"] == "detection":   # src/network.c:555-558: w, h as given, no letterbox correction
                classes = L["classes"]
                pred = np.asarray(outs[i], np.float32).reshape(L["batch"], -1)[image]
                rows.append(self.orc.detection_detections(pred, L["side"], L["n"], classes, L["sqrt"], w, h, thresh))
                continue
            if L["type"] != "yolo":
                continue
            classes = L["classes"]
            anchors = L.get("anchors", [0.5] * (2 * L["total"]))
            biases = np.full(2 * L["total"], 0.5, np.float32)
            biases[:min(len(anchors), biases.size)] = anchors[:biases.size]
            pred = np.asarray(outs[i], np.float32).reshape(L["batch"], L["c"], L["h"], L["w"])[image]
            rows.append(self.orc.yolo_detections(pred, L["n"], classes, biases, L["mask"], self.net["w"],
                                                 self.net["h"], w, h, relative, thresh))
        rows = np.concatenate(rows) if rows else np.zeros((0, 5), np.float32)
        if nms > 0 and len(rows):
            rows = self.orc.nms_sort(rows, classes, nms)
        return rows

