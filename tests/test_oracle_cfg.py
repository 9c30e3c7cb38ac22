"""Pins the cfg grammar + geometry restatement (oracle/cfg.py) and the cfg generators.

Golden layer tables (tests/golden/layer_tables.json) were printed by the compiled reference's
parse_network_cfg; where the reference tree and oracle/_ref are present, every cfg the reference
ships that stays within the path's layer types is parsed by both and compared field by field.
"""
import glob
import json
import os
import re

import pytest

from darknet_amd import cfgs
from oracle import cfg as ocfg
from oracle import ref

from util import have_reference_tree, write_cfg

GOLD = os.path.join(os.path.dirname(__file__), "golden")
COMMON = ["type", "batch", "h", "w", "c", "out_h", "out_w", "out_c", "inputs", "outputs"]
PER_TYPE = {
    "convolutional": ["n", "size", "stride", "pad", "groups", "batch_normalize", "activation", "binary", "xnor",
                      "nweights"],
    "maxpool": ["size", "stride", "pad"],
    "route": ["input_layers", "input_sizes", "n"],
    "shortcut": ["index", "activation", "alpha", "beta"],
    "upsample": ["stride", "scale"],
    "yolo": ["classes", "total", "mask", "n"],
    "softmax": ["groups", "temperature"],
    "local": ["n", "size", "stride", "pad", "activation"],
    "detection": ["n", "classes", "truths", "max_boxes"],
}


def same_table(a, b, where=""):
    assert len(a) == len(b), where
    for i, (x, y) in enumerate(zip(a, b)):
        for k in COMMON + PER_TYPE.get(x["type"], []):
            assert x[k] == y[k], (where, i, x["type"], k, x[k], y[k])


@pytest.mark.parametrize("name,text", [("yolov3-tiny-416", cfgs.yolov3_tiny(1, 416)),
                                       ("yolov3-416", cfgs.yolov3(1, 416)),
                                       ("resnext50-224", cfgs.resnext50(1, 224)),
                                       ("small_net", open(os.path.join(GOLD, "small_net.cfg")).read()),
                                       ("small_net2", open(os.path.join(GOLD, "small_net2.cfg")).read()),
                                       ("yolov1_net", open(os.path.join(GOLD, "yolov1_net.cfg")).read()),
                                       ("bn_net", open(os.path.join(GOLD, "bn_net.cfg")).read())],
                         ids=["yolov3-tiny-416", "yolov3-416", "resnext50-224", "small_net", "small_net2", "yolov1_net",
                              "bn_net"])
def test_parser_matches_golden_layer_tables(name, text):
    gold = json.load(open(os.path.join(GOLD, "layer_tables.json")))[name]
    same_table(gold, ocfg.parse(text)["layers"], name)


def test_grammar_details():
    text = "[net]\n batch = 8 \nsubdivisions=4\n# comment\n;also\nwidth=32\nheight = 32\nchannels=3\n\n" \
           "[conv]\nfilters=4\nsize=3\npad=1\nstride=1\nactivation = leaky\nfilters=99\n"
    net = ocfg.parse(text)
    assert net["batch"] == 2                      # batch / subdivisions
    L = net["layers"][0]
    assert L["n"] == 4 and L["pad"] == 1          # first key wins; pad=1 -> size/2
    assert L["batch_normalize"] == 0 and L["activation"] == "leaky"
    with pytest.raises(ValueError):
        ocfg.parse("[convolutional]\nfilters=1\n")
    # maxpool default padding is size-1, default size is stride
    net = ocfg.parse("[net]\nwidth=13\nheight=13\nchannels=2\n[maxpool]\nstride=1\nsize=2\n")
    assert net["layers"][0]["pad"] == 1 and net["layers"][0]["out_w"] == 13


def test_flop_counts_match_published_table():
    """Per-image GFLOP of the benchmark configurations (the reference's own `ops` counter)."""
    for text, want in [(cfgs.yolov3_tiny(1, 416), 5.565), (cfgs.yolov3(1, 416), 65.864),
                       (cfgs.yolov3(1, 608), 140.692), (cfgs.resnext50(1, 224), 7.742)]:
        net = ocfg.parse(text)
        total = sum(ocfg.conv_flops(L) for L in net["layers"] if L["type"] == "convolutional")
        assert abs(total / 1e9 - want) < 6e-4


@pytest.mark.skipif(not (ref.available() and have_reference_tree()), reason="needs the reference tree + oracle/_ref")
def test_generated_cfgs_equal_the_reference_files():
    def edit(text, batch, size):
        t = re.sub(r"(?m)^batch\s*=.*$", f"batch={batch}", text)
        t = re.sub(r"(?m)^subdivisions\s*=.*$", "subdivisions=1", t)
        t = re.sub(r"(?m)^width\s*=.*$", f"width={size}", t)
        return re.sub(r"(?m)^height\s*=.*$", f"height={size}", t)

    for name, gen, size in [("yolov3-tiny", cfgs.yolov3_tiny, 416), ("yolov3", cfgs.yolov3, 608),
                            ("resnext50", cfgs.resnext50, 256), ("yolov1-tiny", cfgs.yolov1_tiny, 448),
                            ("yolov1", cfgs.yolov1, 448)]:
        p1 = write_cfg(edit(open(f"/root/reference/cfg/{name}.cfg").read(), 2, size))
        p2 = write_cfg(gen(2, size))
        a, b = ref.RefNet(p1).layers, ref.RefNet(p2).layers
        os.unlink(p1)
        os.unlink(p2)
        assert a == b, name


@pytest.mark.skipif(not (ref.available() and have_reference_tree()), reason="needs the reference tree + oracle/_ref")
def test_every_in_scope_reference_cfg_parses_identically():
    done = 0
    for path in sorted(glob.glob("/root/reference/cfg/*.cfg")):
        text = open(path).read()
        kinds = set(re.findall(r"(?m)^\s*(\[[a-z]+\])", text))
        if not kinds <= set(ocfg.SECTION_ALIASES):
            continue
        if re.search(r"(?m)^\s*(tree|map)\s*=", text):
            continue            # needs data files relative to the reference's working directory
        mine = ocfg.parse(text)["layers"]
        theirs = ref.RefNet(path).layers
        same_table(theirs, mine, os.path.basename(path))
        done += 1
    assert done >= 37
