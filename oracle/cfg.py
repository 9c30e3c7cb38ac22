"""Restatement of the reference's cfg grammar and layer-geometry rules (test infrastructure).

Grammar: src/parser.c:891-924 (read_cfg), src/option_list.c:52-77 (read_option),
src/utils.c:302-313 (strip removes every blank, tab and newline before anything else).
Geometry: parse_net_options src/parser.c:655-679; parse_convolutional :179-207 with
convolutional_out_height/width src/convolutional_layer.c:66-74; parse_maxpool :483-498 with
make_maxpool_layer src/maxpool_layer.c:21-36; parse_route :601-640; parse_shortcut :539-556
with make_shortcut_layer src/shortcut_layer.c:9-24; parse_upsample :592-599 with
make_upsample_layer src/upsample_layer.c:7-29; parse_yolo :306-342 with make_yolo_layer
src/yolo_layer.c:13-32; parse_avgpool :500-511; parse_softmax :270-283; parse_local :161-177 with
make_local_layer src/local_layer.c:10-47; parse_detection :405-428 with make_detection_layer
src/detection_layer.c:14-33.

Pinned by tests/test_oracle_cfg.py against the layer table of the compiled reference.
"""
from __future__ import annotations

import re

SECTION_ALIASES = {
    "[conv]": "convolutional", "[convolutional]": "convolutional",
    "[max]": "maxpool", "[maxpool]": "maxpool",
    "[avg]": "avgpool", "[avgpool]": "avgpool",
    "[soft]": "softmax", "[softmax]": "softmax",
    "[route]": "route", "[shortcut]": "shortcut", "[upsample]": "upsample", "[yolo]": "yolo",
    "[conn]": "connected", "[connected]": "connected", "[dropout]": "dropout", "[reorg]": "reorg",
    "[crop]": "crop", "[cost]": "cost", "[region]": "region",
    "[local]": "local", "[detection]": "detection", "[batchnorm]": "batchnorm",
    "[net]": "net", "[network]": "net",
}


def _atoi(s: str) -> int:
    m = re.match(r"[+-]?\d+", s)
    return int(m.group(0)) if m else 0


def _atof(s: str) -> float:
    m = re.match(r"[+-]?(\d+\.?\d*([eE][+-]?\d+)?|\.\d+([eE][+-]?\d+)?)", s)
    return float(m.group(0)) if m else 0.0


def read_cfg(text: str):
    """-> list of (section_name_with_brackets, {key: value}) in file order."""
    sections = []
    for raw in text.split("\n"):
        line = raw.replace(" ", "").replace("\t", "").replace("\n", "")
        if not line or line[0] in "#;":
            continue
        if line[0] == "[":
            sections.append((line, {}))
            continue
        if "=" not in line:
            continue
        key, val = line.split("=", 1)
        if val == "" :
            continue
        # option_find returns the first matching key in insertion order
        sections[-1][1].setdefault(key, val)
    return sections


def parse(text: str) -> dict:
    sections = read_cfg(text)
    if not sections:
        raise ValueError("Config file has no sections")
    head, opts = sections[0]
    if SECTION_ALIASES.get(head) != "net":
        raise ValueError("First section must be [net] or [network]")
    gi = lambda o, k, d: _atoi(o[k]) if k in o else d
    gf = lambda o, k, d: _atof(o[k]) if k in o else d
    batch = gi(opts, "batch", 1) // gi(opts, "subdivisions", 1) * gi(opts, "time_steps", 1)
    net = {"batch": batch, "h": gi(opts, "height", 0), "w": gi(opts, "width", 0),
           "c": gi(opts, "channels", 0)}
    net["inputs"] = gi(opts, "inputs", net["h"] * net["w"] * net["c"])
    h, w, c, inputs = net["h"], net["w"], net["c"], net["inputs"]
    layers = []
    for index, (name, o) in enumerate(sections[1:]):
        kind = SECTION_ALIASES.get(name)
        if kind is None:
            raise NotImplementedError(f"layer type {name} is outside the checked path")
        L = {"type": kind, "batch": batch, "h": h, "w": w, "c": c, "inputs": inputs}
        if kind == "convolutional":
            n = gi(o, "filters", 1)
            size = gi(o, "size", 1)
            stride = gi(o, "stride", 1)
            padding = gi(o, "padding", 0)
            if gi(o, "pad", 0):
                padding = size // 2
            groups = gi(o, "groups", 1)
            L.update(n=n, size=size, stride=stride, pad=padding, groups=groups,
                     activation=o.get("activation", "logistic"),
                     batch_normalize=gi(o, "batch_normalize", 0),
                     binary=gi(o, "binary", 0), xnor=gi(o, "xnor", 0))
            L["out_h"] = (h + 2 * padding - size) // stride + 1
            L["out_w"] = (w + 2 * padding - size) // stride + 1
            L["out_c"] = n
            L["nweights"] = c // groups * n * size * size
        elif kind == "maxpool":
            stride = gi(o, "stride", 1)
            size = gi(o, "size", stride)
            padding = gi(o, "padding", size - 1)
            L.update(size=size, stride=stride, pad=padding)
            L["out_h"] = (h + padding - size) // stride + 1
            L["out_w"] = (w + padding - size) // stride + 1
            L["out_c"] = c
        elif kind == "avgpool":
            L.update(out_h=1, out_w=1, out_c=c)
        elif kind == "softmax":
            L.update(groups=gi(o, "groups", 1), temperature=gf(o, "temperature", 1.0),
                     out_h=0, out_w=0, out_c=0, outputs=inputs)
            # parse_softmax sets l.w/h/c from params but leaves out_* at zero
        elif kind == "connected":
            # parse_connected src/parser.c:259-268, make_connected_layer src/connected_layer.c:14-33
            outputs = gi(o, "output", 1)
            L.update(n=outputs, size=1, stride=1, pad=0, groups=1, h=1, w=1, c=inputs,
                     activation=o.get("activation", "logistic"),
                     batch_normalize=gi(o, "batch_normalize", 0), binary=0, xnor=0,
                     out_h=1, out_w=1, out_c=outputs, outputs=outputs, nweights=inputs * outputs)
        elif kind == "batchnorm":
            # parse_batchnorm src/parser.c:533-537, make_batchnorm_layer src/batchnorm_layer.c:6-19
            L.update(out_h=h, out_w=w, out_c=c, outputs=h * w * c, inputs=h * w * c)
        elif kind == "dropout":
            # parse_dropout src/parser.c:513-521: geometry passes through, output = input
            L.update(probability=gf(o, "probability", 0.5), out_h=h, out_w=w, out_c=c, outputs=inputs,
                     h=0, w=0, c=0)
        elif kind == "cost":
            L.update(out_h=0, out_w=0, out_c=0, outputs=inputs, h=0, w=0, c=0)
        elif kind == "crop":
            # parse_crop src/parser.c:441-463, make_crop_layer src/crop_layer.c:18-51
            ch, cw = gi(o, "crop_height", 1), gi(o, "crop_width", 1)
            L.update(out_h=ch, out_w=cw, out_c=c, noadjust=gi(o, "noadjust", 0), flip=gi(o, "flip", 0),
                     inputs=h * w * c)
        elif kind == "reorg":
            # parse_reorg src/parser.c:465-481, make_reorg_layer src/reorg_layer.c:8-35
            stride = gi(o, "stride", 1)
            reverse, flat, extra = gi(o, "reverse", 0), gi(o, "flatten", 0), gi(o, "extra", 0)
            if reverse:
                oh, ow, oc = h * stride, w * stride, c // (stride * stride)
            else:
                oh, ow, oc = h // stride, w // stride, c * stride * stride
            L.update(stride=stride, reverse=reverse, flatten=flat, extra=extra, out_h=oh, out_w=ow, out_c=oc,
                     inputs=h * w * c, outputs=oh * ow * oc)
            if extra:
                L.update(out_h=0, out_w=0, out_c=0, outputs=h * w * c + extra)
        elif kind == "region":
            # parse_region src/parser.c:353-403, make_region_layer src/region_layer.c:13-56
            if "tree" in o or "map" in o:
                raise NotImplementedError("region layer with tree/map")
            coords, classes, num = gi(o, "coords", 4), gi(o, "classes", 20), gi(o, "num", 1)
            anchors = [0.5] * (2 * num)
            if "anchors" in o:
                for i, t in enumerate(o["anchors"].split(",")):
                    if i < 2 * num:
                        anchors[i] = _atof(t)
            L.update(n=num, classes=classes, coords=coords, softmax=gi(o, "softmax", 0),
                     background=gi(o, "background", 0), anchors=anchors,
                     c=num * (classes + coords + 1), out_h=h, out_w=w, out_c=num * (classes + coords + 1))
            L["outputs"] = h * w * L["out_c"]
            if L["outputs"] != inputs:
                raise ValueError("region layer: outputs != inputs")
        elif kind == "local":
            # pad is the number of zero pixels itself; the output size is the layer's own rule
            n, size, stride, pad = gi(o, "filters", 1), gi(o, "size", 1), gi(o, "stride", 1), gi(o, "pad", 0)
            if not (h and w and c):
                raise ValueError("Layer before local layer must output image.")
            oh = (h - (1 if pad else size)) // stride + 1
            ow = (w - (1 if pad else size)) // stride + 1
            L.update(n=n, size=size, stride=stride, pad=pad, activation=o.get("activation", "logistic"),
                     out_h=oh, out_w=ow, out_c=n, inputs=h * w * c)
        elif kind == "detection":
            coords, classes, num, side = gi(o, "coords", 1), gi(o, "classes", 1), gi(o, "num", 1), gi(o, "side", 7)
            if side * side * ((1 + coords) * num + classes) != inputs:
                raise ValueError("detection layer: side*side*((1+coords)*num+classes) != inputs")
            L.update(n=num, classes=classes, coords=coords, side=side, rescore=gi(o, "rescore", 0),
                     softmax=gi(o, "softmax", 0), sqrt=gi(o, "sqrt", 0), max_boxes=gi(o, "max", 90),
                     truths=side * side * (1 + coords + classes),
                     h=side, w=side, c=0, out_h=0, out_w=0, out_c=0, outputs=inputs)
        elif kind == "upsample":
            stride = gi(o, "stride", 2)
            L.update(stride=stride, scale=gf(o, "scale", 1.0),
                     out_h=h * stride, out_w=w * stride, out_c=c)
        elif kind == "shortcut":
            frm = _atoi(o["from"])
            if frm < 0:
                frm = index + frm
            src = layers[frm]
            # make_shortcut_layer: (w,h,c) of the layer become those of `from`'s output, the
            # output geometry is that of the running input.
            L.update(index=frm, activation=o.get("activation", "linear"),
                     alpha=gf(o, "alpha", 1.0), beta=gf(o, "beta", 1.0),
                     h=src["out_h"], w=src["out_w"], c=src["out_c"],
                     out_h=h, out_w=w, out_c=c)
        elif kind == "route":
            ids = []
            for tok in o["layers"].split(","):
                i = _atoi(tok)
                ids.append(index + i if i < 0 else i)
            first = layers[ids[0]]
            oh, ow, oc = first["out_h"], first["out_w"], first["out_c"]
            for i in ids[1:]:
                nxt = layers[i]
                if nxt["out_w"] == first["out_w"] and nxt["out_h"] == first["out_h"]:
                    oc += nxt["out_c"]
                else:
                    oh = ow = oc = 0
            sizes = [layers[i]["outputs"] for i in ids]
            L.update(input_layers=ids, input_sizes=sizes, out_h=oh, out_w=ow, out_c=oc,
                     outputs=sum(sizes), n=len(ids), h=0, w=0, c=0)
            L["inputs"] = L["outputs"]  # make_route_layer leaves h/w/c at zero
        elif kind == "yolo":
            classes = gi(o, "classes", 20)
            total = gi(o, "num", 1)
            mask = [_atoi(t) for t in o["mask"].split(",")] if "mask" in o else list(range(total))
            L.update(classes=classes, total=total, mask=mask, n=len(mask),
                     c=len(mask) * (classes + 5), out_h=h, out_w=w,
                     out_c=len(mask) * (classes + 5))
            if "anchors" in o:
                L["anchors"] = [_atof(t) for t in o["anchors"].split(",")]
            L["outputs"] = h * w * L["out_c"]
            if L["outputs"] != inputs:
                raise ValueError("yolo layer: outputs != inputs")
        if "outputs" not in L:
            L["outputs"] = L["out_h"] * L["out_w"] * L["out_c"]
        layers.append(L)
        h, w, c, inputs = L["out_h"], L["out_w"], L["out_c"], L["outputs"]
    net["layers"] = layers
    net["n"] = len(layers)
    net["outputs"] = layers[-1]["outputs"]
    return net


def conv_flops(L: dict) -> float:
    """The reference's own operation count: examples/darknet.c:88, src/convolutional_layer.c:325."""
    return 2.0 * L["n"] * L["size"] * L["size"] * (L["c"] // L["groups"]) * L["out_h"] * L["out_w"]
