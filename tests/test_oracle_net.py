"""Pins the CPU checker's forward_network loop (oracle/net.py) end to end."""
import json
import os

import numpy as np
import pytest

from darknet_amd import cfgs, synth
from oracle import ref
from oracle.net import OracleNet

from util import fill_params, write_cfg

GOLD = os.path.join(os.path.dirname(__file__), "golden")


def test_tiny_forward_matches_golden_checksums():
    gold = json.load(open(os.path.join(GOLD, "tiny416_b1.json")))
    net = OracleNet(cfgs.yolov3_tiny(1, 416))
    fill_params(net.set_conv, net.layers, seed=gold["seed"], bn="random")
    outs = net.forward(synth.uniform01(gold["input_seed"], net.net["inputs"]))
    for i, (o, g) in enumerate(zip(outs, gold["layers"])):
        flat = o.reshape(-1)
        step = max(1, flat.size // 16)
        assert [float(v) for v in flat[::step][:16]] == g["samples"], i
        assert float(flat.astype(np.float64).sum()) == g["sum"], i
        assert float(np.abs(flat.astype(np.float64)).sum()) == g["abssum"], i


def test_small_net_matches_golden_outputs_of_every_layer():
    g = np.load(os.path.join(GOLD, "small_net.npz"))
    net = OracleNet(open(os.path.join(GOLD, "small_net.cfg")).read())
    fill_params(net.set_conv, net.layers, seed=500, bn="random")
    outs = net.forward(g["input"])
    for i, o in enumerate(outs):
        assert np.array_equal(o, g[f"layer{i}"]), (i, net.layers[i]["type"])


def test_small_net2_matches_golden_outputs_of_every_layer():
    """crop, reorg (plain / reverse / flatten / extra), dropout, connected, softmax, cost."""
    g = np.load(os.path.join(GOLD, "small_net2.npz"))
    net = OracleNet(open(os.path.join(GOLD, "small_net2.cfg")).read())
    fill_params(net.set_conv, net.layers, seed=640, bn="random")
    outs = net.forward(g["input"])
    kinds = [L["type"] for L in net.layers]
    assert kinds.count("reorg") == 4 and kinds.count("connected") == 2 and "crop" in kinds and "cost" in kinds
    for i, o in enumerate(outs):
        assert np.array_equal(o, g[f"layer{i}"]), (i, net.layers[i]["type"])


@pytest.mark.skipif(not ref.available(), reason="oracle/_ref (compiled reference) not built")
@pytest.mark.parametrize("name,text", [("resnext50", cfgs.resnext50(2, 64)), ("yolov3", cfgs.yolov3(1, 96)),
                                       ("tiny-xnor", cfgs.yolov3_tiny(1, 96, xnor=True))])
def test_networks_match_compiled_reference_bit_for_bit(name, text):
    p = write_cfg(text)
    r = ref.RefNet(p)
    os.unlink(p)
    o = OracleNet(text)
    fill_params(r.set_conv, r.layers, seed=300)
    fill_params(o.set_conv, o.layers, seed=300)
    x = synth.uniform01(3, r.inputs * r.batch)
    for i, (a, b) in enumerate(zip(r.predict(x), o.forward(x))):
        assert np.array_equal(a, b), (name, i, o.layers[i]["type"])
