"""The reference's own host code on the HIP kernels.

oracle/_ref/libdarknet_ref_hip.so is the reference tree's src/*.c compiled with -DGPU where it lies
and linked with integration/adapters.c against libdarknet_hip.so (oracle/Makefile, target ref_hip;
built in the container that holds the reference, it travels as a binary).  Here the reference's
parse_network_cfg builds the by-value `layer` structs, its network_predict -> forward_network ->
forward_network_gpu loop (src/network.c:497-508, :188-195, :762-788) calls l.forward_gpu per layer,
and those land in the adapters and the exported helpers - nothing of this repository's own host
(cfg parser, network.c, layers.c) takes part.

Gates are the ones the library's own networks are held to, against the reference's CPU build
(oracle/_ref/libdarknet_ref_o2.so) on the same seeded weights and inputs: every conv layer <= 1e-4
max-normalised, maxpool / route / upsample / shortcut bit-exact given the same input, yolo tensors
<= 1e-3 absolute."""
import os

import numpy as np
import pytest

from darknet_amd import api, cfgs, lib, synth
from oracle import ref

from util import REL_TOL, YOLO_ABS_TOL, fill_params, norm_err, write_cfg

pytestmark = [pytest.mark.gpu,
              pytest.mark.skipif(not (ref.available("hip") and ref.available("o2")),
                                 reason="the compiled reference (CPU build and HIP-bound build) is not present")]
GOLD = os.path.join(os.path.dirname(__file__), "golden")
EXACT_GIVEN_INPUT = ("maxpool", "route", "upsample", "shortcut")


def run_both(text, input_seed=7, bn="random"):
    path = write_cfg(text)
    bound = ref.RefNet(path, "hip")          # reference host + adapters + HIP kernels
    cpu = ref.RefNet(path, "o2")             # reference CPU build
    os.unlink(path)
    assert bound.h.refh_is_gpu_build() == 1 and cpu.h.refh_is_gpu_build() == 0
    assert bound.layers == cpu.layers
    fill_params(bound.set_conv, bound.layers, bn=bn)
    fill_params(cpu.set_conv, cpu.layers, bn=bn)
    x = synth.uniform01(input_seed, bound.inputs * bound.batch)
    got = bound.predict(x)
    want = cpu.predict(x)
    return bound, cpu, x, got, want


def gate(bound, cpu, x, got, want):
    worst = 0.0
    for i, L in enumerate(cpu.layers):
        if L["type"] == "cost":
            continue
        e = norm_err(got[i], want[i])
        worst = max(worst, e)
        assert e <= REL_TOL, (i, L["type"], e)
        if L["type"] in EXACT_GIVEN_INPUT and L["type"] != "route" and L["type"] != "shortcut":
            # the CPU build's layer on the HIP-bound build's input: bit for bit
            prev = got[i - 1] if i else x.reshape(bound.batch, -1)
            again = cpu.forward_layer(i, prev)
            assert np.array_equal(got[i], again), (i, L["type"])
        if L["type"] == "shortcut" and L["activation"] == "linear" and got[L["index"]].shape == got[i].shape:
            assert np.array_equal(got[i], got[i - 1] + got[L["index"]]), i
        if L["type"] == "route":
            parts = [got[j].reshape(bound.batch, -1) for j in L["input_layers"]]
            assert np.array_equal(got[i], np.concatenate(parts, axis=1)), i
        if L["type"] == "yolo":
            assert np.abs(got[i] - want[i]).max() <= YOLO_ABS_TOL
    return worst


def test_yolov3_tiny_through_the_reference_driver_loop(dn):
    bound, cpu, x, got, want = run_both(cfgs.yolov3_tiny(1, 416))
    worst = gate(bound, cpu, x, got, want)
    print(f"yolov3-tiny-416 through the reference's forward_network_gpu: worst layer {worst:.3g}")
    # the convolutions are the library's kernels with the arguments the library's own host passes:
    # same bits as the library's own network object on the same parameters
    net = api.Network(cfg_text=cfgs.yolov3_tiny(1, 416))
    fill_params(net.set_conv, net.layers)
    net.predict(x)
    for i, L in enumerate(net.layers):
        if L["type"] in ("convolutional", "maxpool", "route", "upsample"):
            assert np.array_equal(net.layer_output(i), got[i]), (i, L["type"])
    net.free()
    bound.free()
    cpu.free()


def test_yolov3_residual_blocks_and_heads(dn):
    """75 convolutions, 23 shortcuts through the reference's own forward_shortcut_layer_gpu
    (copy_gpu + shortcut_gpu + activate_array_gpu of the library), upsample + route, three heads."""
    bound, cpu, x, got, want = run_both(cfgs.yolov3(1, 320))
    gate(bound, cpu, x, got, want)
    bound.free()
    cpu.free()


def test_resnext50_grouped_avgpool_softmax(dn):
    bound, cpu, x, got, want = run_both(cfgs.resnext50(1, 224))
    gate(bound, cpu, x, got, want)
    assert abs(float(got[-1].sum()) - 1.0) < 1e-4
    bound.free()
    cpu.free()


def test_batch_of_four_images(dn):
    bound, cpu, x, got, want = run_both(cfgs.yolov3_tiny(4, 224))
    gate(bound, cpu, x, got, want)
    bound.free()
    cpu.free()


def test_xnor_layer_with_the_network_input_as_its_input(dn):
    """One xnor=1 convolution fed by the network input, so both builds binarise the same bits (a
    whole XNOR network is ill-posed end to end: exact ties at zero flip signs in the next layer)."""
    bound, cpu, x, got, want = run_both(cfgs.single_conv(2, 64, 26, 26, 96, 3, 1, xnor=True))
    assert norm_err(got[0], want[0]) <= REL_TOL
    bound.free()
    cpu.free()


def test_reference_load_weights_reaches_the_device_and_repacks(dn, tmp_path):
    """The reference's load_weights ends every convolution with push_convolutional_layer
    (src/parser.c:1210-1214), here the adapter: the parameters reach the device and the library drops
    its packed copy of the old weights.  A forward with other weights first makes a stale copy show."""
    g = np.load(os.path.join(GOLD, "small_net.npz"))
    bound = ref.RefNet(os.path.join(GOLD, "small_net.cfg"), "hip")
    fill_params(bound.set_conv, bound.layers, seed=77)
    first = bound.predict(g["input"])
    assert norm_err(first[0], g["layer0"]) > 1e-2
    bound.load_weights(os.path.join(GOLD, "small_net.weights"))
    got = bound.predict(g["input"])
    for i, L in enumerate(bound.layers):
        assert norm_err(got[i], g[f"layer{i}"]) <= REL_TOL, (i, L["type"])
    assert np.array_equal(bound.layer_indexes(1), g["indexes1"])
    out = str(tmp_path / "roundtrip.weights")
    bound.save_weights(out)                      # pull_convolutional_layer adapter, then the file
    assert open(out, "rb").read() == open(os.path.join(GOLD, "small_net.weights"), "rb").read()
    bound.free()


def test_packed_copies_follow_the_weights_lifetime(dn):
    L = lib.load()
    before = L.conv_packed_cached_count()
    path = write_cfg(cfgs.yolov3_tiny(1, 160))
    bound = ref.RefNet(path, "hip")
    os.unlink(path)
    fill_params(bound.set_conv, bound.layers)
    bound.predict(synth.uniform01(3, bound.inputs))
    held = L.conv_packed_cached_count() - before
    convs = [l for l in bound.layers if l["type"] == "convolutional"]
    assert held == sum(1 for l in convs if L.conv_packed_floats(l["n"], l["c"], l["groups"], l["size"])) >= 12
    bound.predict(synth.uniform01(4, bound.inputs))
    assert L.conv_packed_cached_count() - before == held
    bound.free()                 # the reference's free_network -> free_layer -> cuda_free(weights_gpu)
    assert L.conv_packed_cached_count() == before
