"""End-to-end parity of whole networks: parse_network_cfg -> network_predict through the native
library against the CPU checker on the same seeded weights and inputs.

Gates: every conv layer <= 1e-4 (max-normalised), index/copy layers bit-exact *given the same
input* (checked by feeding the library's own previous-layer output to the CPU checker), final
yolo tensors <= 1e-3 absolute.  Batch-64 runs use size-independent properties."""
import json
import os

import numpy as np
import pytest

from darknet_amd import api, cfgs, synth
from oracle.net import OracleNet

from util import REL_TOL, YOLO_ABS_TOL, fill_params, norm_err

pytestmark = pytest.mark.gpu
GOLD = os.path.join(os.path.dirname(__file__), "golden")
EXACT_GIVEN_INPUT = ("maxpool", "route", "upsample", "shortcut")


def build_pair(text, seed=1000, bn="random"):
    net = api.Network(cfg_text=text)
    orc = OracleNet(text)
    def both(i, *arrays):            # one pass of the generator feeds both networks
        net.set_conv(i, *arrays)
        orc.set_conv(i, *arrays)

    assert [(L["type"], L["outputs"]) for L in net.layers] == [(L["type"], L["outputs"]) for L in orc.layers]
    fill_params(both, orc.layers, seed=seed, bn=bn)
    return net, orc


def check_network(text, input_seed=7, bn="random"):
    net, orc = build_pair(text, bn=bn)
    x = synth.uniform01(input_seed, net.inputs * net.batch)
    final = net.predict(x)
    want = orc.forward(x)
    got = [net.layer_output(i) for i in range(net.n)]
    worst = 0.0
    for i, L in enumerate(orc.layers):
        e = norm_err(got[i], want[i])
        worst = max(worst, e)
        assert e <= REL_TOL, (i, L["type"], e)
        if L["type"] in EXACT_GIVEN_INPUT:
            # re-run the CPU checker's layer on the LIBRARY's inputs: must match bit for bit
            prev = got[i - 1] if i else x.reshape(net.batch, -1)
            again = np.ascontiguousarray(orc.forward_layer(i, prev, got)).reshape(net.batch, -1)
            assert np.array_equal(got[i], again), (i, L["type"])
        if L["type"] == "yolo":
            assert np.abs(got[i] - want[i]).max() <= YOLO_ABS_TOL
    assert np.array_equal(final, got[-1])
    net.free()
    return worst


def test_parser_matches_golden_layer_tables(dn):
    gold = json.load(open(os.path.join(GOLD, "layer_tables.json")))
    for name, text in [("yolov3-tiny-416", cfgs.yolov3_tiny(1, 416)), ("yolov3-416", cfgs.yolov3(1, 416)),
                       ("resnext50-224", cfgs.resnext50(1, 224)),
                       ("small_net", open(os.path.join(GOLD, "small_net.cfg")).read())]:
        net = api.Network(cfg_text=text)
        assert len(net.layers) == len(gold[name])
        for i, (a, b) in enumerate(zip(net.layers, gold[name])):
            for k, v in b.items():
                if k in ("mask",):
                    continue
                if k in ("h", "w", "c") and b["type"] == "route":
                    continue
                assert a[k] == v or (isinstance(v, float) and abs(a[k] - v) < 1e-7), (name, i, k, a[k], v)
        assert abs(net.conv_flops() - {"yolov3-tiny-416": 5.565e9, "yolov3-416": 65.864e9,
                                       "resnext50-224": 7.742e9}.get(name, net.conv_flops())) < 1e6
        net.free()


def test_small_net_golden_outputs_and_reference_weights_file(dn, tmp_path):
    """The library loads the weights file the REFERENCE saved and reproduces the reference's
    per-layer outputs; saving it back yields the identical file."""
    g = np.load(os.path.join(GOLD, "small_net.npz"))
    net = api.Network(cfg_path=os.path.join(GOLD, "small_net.cfg"),
                      weights=os.path.join(GOLD, "small_net.weights"))
    net.predict(g["input"])
    for i, L in enumerate(net.layers):
        got = net.layer_output(i)
        assert norm_err(got, g[f"layer{i}"]) <= REL_TOL, (i, L["type"])
    assert np.array_equal(net.layer_indexes(1), g["indexes1"])
    out = str(tmp_path / "roundtrip.weights")
    net.save_weights(out)
    assert open(out, "rb").read() == open(os.path.join(GOLD, "small_net.weights"), "rb").read()
    net.free()


def test_yolov3_tiny_416(dn):
    assert check_network(cfgs.yolov3_tiny(1, 416)) <= REL_TOL


def test_yolov3_tiny_golden_checksums(dn):
    gold = json.load(open(os.path.join(GOLD, "tiny416_b1.json")))
    net = api.Network(cfg_text=cfgs.yolov3_tiny(1, 416))
    fill_params(net.set_conv, net.layers, seed=gold["seed"], bn="random")
    net.predict(synth.uniform01(gold["input_seed"], net.inputs))
    for i, g in enumerate(gold["layers"]):
        flat = net.layer_output(i).reshape(-1)
        step = max(1, flat.size // 16)
        assert np.abs(flat[::step][:16] - np.array(g["samples"], np.float32)).max() <= REL_TOL * g["max"], i
        assert abs(float(np.abs(flat.astype(np.float64)).sum()) - g["abssum"]) <= 1e-5 * g["abssum"] + 1e-6, i
    net.free()


def test_yolov3_tiny_benchmark_init(dn):
    """The initialisation the benchmark configurations name: BN mean 0, variance 1, scale 1."""
    assert check_network(cfgs.yolov3_tiny(1, 416), bn="identity") <= REL_TOL


def test_yolov3_416(dn):
    assert check_network(cfgs.yolov3(1, 416)) <= REL_TOL


def test_yolov3_608_small_batch(dn):
    assert check_network(cfgs.yolov3(1, 608), bn="identity") <= REL_TOL


def test_resnext50_224(dn):
    assert check_network(cfgs.resnext50(2, 224)) <= REL_TOL


def test_batch_64_images_are_independent(dn):
    """At the benchmark batch the CPU checker would take minutes; instead: image k of a batch-64
    forward equals the batch-1 forward of that image (already checked against the CPU above)."""
    text64, text1 = cfgs.yolov3_tiny(64, 416), cfgs.yolov3_tiny(1, 416)
    net64, net1 = api.Network(cfg_text=text64), api.Network(cfg_text=text1)
    fill_params(net64.set_conv, net64.layers)
    fill_params(net1.set_conv, net1.layers)
    x = synth.uniform01(3, net64.inputs * 64).reshape(64, -1)
    net64.predict(x)
    heads = [i for i, L in enumerate(net64.layers) if L["type"] == "yolo"]
    for k in (0, 31, 63):
        net1.predict(x[k])
        for i in heads + [12, 20]:
            a, b = net64.layer_output(i)[k], net1.layer_output(i)[0]
            # not bit-equal: the K-split of partial tile rounds depends on the batch size
            assert norm_err(a, b) <= 1e-5, (k, i)
    net64.free()
    net1.free()


def test_yolov3_batch_64_runs_and_is_consistent(dn):
    net64 = api.Network(cfg_text=cfgs.yolov3(64, 416))
    net1 = api.Network(cfg_text=cfgs.yolov3(1, 416))
    fill_params(net64.set_conv, net64.layers, bn="identity")
    fill_params(net1.set_conv, net1.layers, bn="identity")
    x = synth.uniform01(5, net64.inputs * 64).reshape(64, -1)
    out64 = net64.predict(x)
    out1 = net1.predict(x[40])
    assert np.abs(out64[40] - out1[0]).max() <= YOLO_ABS_TOL
    for i in (82, 94):
        assert np.abs(net64.layer_output(i)[40] - net1.layer_output(i)[0]).max() <= YOLO_ABS_TOL
    # device-resident forward (what the benchmark times) gives the same result as network_predict
    net64.push_input(x)
    net64.forward_device()
    net64.synchronize()
    assert np.array_equal(net64.layer_output(net64.n - 1), out64)
    net64.free()
    net1.free()


def test_set_batch_network_shrinks_and_grows_back(dn):
    net = api.Network(cfg_text=cfgs.yolov3_tiny(4, 160))
    fill_params(net.set_conv, net.layers)
    x = synth.uniform01(9, net.inputs * 4).reshape(4, -1)
    full = net.predict(x)
    net.set_batch(1)
    one = net.predict(x[0])
    assert np.abs(one[0] - full[0]).max() <= 1e-5 * max(np.abs(full[0]).max(), 1.0)   # another K-split, same values
    assert net.layer_output(3).shape[0] == 1          # shaped from the current batch, not the parse-time one
    # and back up to the batch the buffers were allocated for
    net.set_batch(4)
    again = net.predict(x)
    assert np.array_equal(again, full)
    assert net.layer_output(3).shape[0] == 4
    net.free()


ROUTE_VIEWS = """[net]
batch=2
subdivisions=1
width=12
height=10
channels=4

[convolutional]
filters=8
size=3
stride=1
pad=1
activation=leaky

[route]
layers=-1

[route]
layers=-1

[dropout]
probability=.5

[convolutional]
filters=6
size=1
stride=1
pad=1
activation=linear

[route]
layers=3

[route]
layers=-1,1

[route]
layers=4
"""


def test_views_of_views_and_of_dropout_layers(dn):
    """A route of a route, a dropout behind a view, a route whose source is a dropout layer, a
    two-source route that concatenates two views, and a view as the network's last layer: every
    layer equals the checker's, and building and freeing the network three times returns the memory."""
    import ctypes as C
    hip = C.CDLL("libamdhip64.so")

    def free_bytes():
        free, total = C.c_size_t(), C.c_size_t()
        assert hip.hipMemGetInfo(C.byref(free), C.byref(total)) == 0
        return free.value

    assert check_network(ROUTE_VIEWS) <= REL_TOL
    before = free_bytes()
    for _ in range(3):
        check_network(ROUTE_VIEWS)
    assert free_bytes() == before
    net = api.Network(cfg_text=ROUTE_VIEWS)
    kinds = [L["type"] for L in net.layers]
    assert kinds == ["convolutional", "route", "route", "dropout", "convolutional", "route", "route", "route"]
    net.free()


@pytest.mark.parametrize("pin", ["algo3", "ksplit1"])
def test_same_image_same_bits_at_any_batch_without_the_k_split(dn, pin):
    """With the cut along K switched off every output sums K in one fixed order, whatever tile it
    falls into: an image then gives the same bits at batch 1 and inside a batch of five, as the
    reference's per-image GEMM does at any batch size."""
    if pin == "algo3":
        dn.conv_set_algo(3)
    else:
        dn.conv_set_ksplit(1, 0)
        dn.conv_set_bands(1)
    try:
        net5 = api.Network(cfg_text=cfgs.yolov3(5, 160))
        net1 = api.Network(cfg_text=cfgs.yolov3(1, 160))
        fill_params(net5.set_conv, net5.layers)
        fill_params(net1.set_conv, net1.layers)
        x = synth.uniform01(9, net5.inputs * 5).reshape(5, -1)
        net5.predict(x)
        for k in (0, 3):
            net1.predict(x[k])
            for i in range(net5.n):
                assert np.array_equal(net5.layer_output(i)[k], net1.layer_output(i)[0]), (pin, k, i)
        net5.free()
        net1.free()
    finally:
        dn.conv_set_algo(0)
        dn.conv_set_ksplit(0, 0)
        dn.conv_set_bands(0)


def test_one_source_route_is_a_view_of_its_source(dn):
    """`[route] layers=-4` copies one layer in the reference (src/route_layer.c:74-87); here the
    route's output is the source's buffer: the same bits, no launch, and the two-source routes of the
    same network still concatenate."""
    net = api.Network(cfg_text=cfgs.yolov3(2, 160))
    fill_params(net.set_conv, net.layers)
    x = synth.uniform01(23, net.inputs * 2)
    net.predict(x)
    seen = 0
    for i, L in enumerate(net.layers):
        if L["type"] != "route":
            continue
        parts = [net.layer_output(j).reshape(2, -1) for j in L["input_layers"]]
        assert np.array_equal(net.layer_output(i).reshape(2, -1), np.concatenate(parts, axis=1)), i
        seen += len(parts) == 1
    assert seen == 2
    net.free()


def test_shortcut_fusion_changes_no_bit(dn):
    """forward_network_device folds each residual add into the convolution before it; with the
    fusion switched off every layer output must hold the same bits."""
    net = api.Network(cfg_text=cfgs.yolov3(2, 160))
    fill_params(net.set_conv, net.layers)
    x = synth.uniform01(21, net.inputs * 2)
    net.predict(x)
    fused = [net.layer_output(i) for i in range(net.n)]
    net.forward_profiled()      # the event-timed loop folds the same pairs
    for i in range(net.n):
        assert np.array_equal(net.layer_output(i), fused[i]), i
    assert sum(L["type"] == "shortcut" for L in net.layers) == 23
    net.L.network_set_fusion(0)
    try:
        net.predict(x)
        for i in range(net.n):
            assert np.array_equal(net.layer_output(i), fused[i]), i
    finally:
        net.L.network_set_fusion(1)
    net.free()


def test_kernel_stamped_timing(dn):
    """forward_network_profiled_kernels: every MFMA convolution's main kernel carries its own
    start/stop events; the stamped duration is positive, no longer than the interval between the
    events around its layer (plus timer slack), other layers report -1, and no output bit changes."""
    net = api.Network(cfg_text=cfgs.yolov3(2, 160))
    fill_params(net.set_conv, net.layers)
    x = synth.uniform01(22, net.inputs * 2)
    net.predict(x)
    want = [net.layer_output(i) for i in range(net.n)]
    for _ in range(2):
        total, layer_ms, kernel_ms = net.forward_profiled_kernels()
    assert dn.conv_profile_pending() == 0
    for i, L in enumerate(net.layers):
        assert np.array_equal(net.layer_output(i), want[i]), i
        if L["type"] == "convolutional":
            assert 0 < kernel_ms[i] <= layer_ms[i] + 0.25, (i, kernel_ms[i], layer_ms[i])   # slack: two timers
        else:
            assert kernel_ms[i] == -1.0, (i, L["type"], kernel_ms[i])
    assert sum(k for k in kernel_ms if k > 0) < total
    net.free()


def test_small_net2_crop_reorg_dropout_connected_cost(dn, tmp_path):
    """The layer types beyond the yolo family (crop, the four reorg modes, dropout, connected with
    and without batch-norm, cost): layer table, reference-written weights file, per-layer outputs
    (index/copy layers bit-exact, connected <= 1e-4), and the weights file round trip."""
    text = open(os.path.join(GOLD, "small_net2.cfg")).read()
    gold = json.load(open(os.path.join(GOLD, "layer_tables.json")))["small_net2"]
    g = np.load(os.path.join(GOLD, "small_net2.npz"))
    net = api.Network(cfg_text=text, weights=os.path.join(GOLD, "small_net2.weights"))
    assert [L["type"] for L in net.layers] == [L["type"] for L in gold]
    for i, (a, b) in enumerate(zip(net.layers, gold)):
        for k in ("batch", "out_h", "out_w", "out_c", "inputs", "outputs"):
            assert a[k] == b[k], (i, a["type"], k, a[k], b[k])
    final = net.predict(g["input"])
    exact = ("crop", "reorg", "dropout", "cost")
    prev = g["input"].reshape(net.batch, -1)
    for i, L in enumerate(net.layers):
        got, want = net.layer_output(i), g[f"layer{i}"].reshape(net.batch, -1)
        assert norm_err(got, want) <= REL_TOL or (L["type"] == "cost" and not got.any()), (i, L["type"])
        if L["type"] in exact:
            # bit-exact on the library's own input: re-run the CPU checker's layer on it
            again = OracleNet(text).forward_layer(i, prev, None)
            assert np.array_equal(got, np.ascontiguousarray(again).reshape(net.batch, -1)), (i, L["type"])
        prev = got
    # the network's output layer skips the trailing cost layer (src/network.c:689-697)
    assert net.layers[-1]["type"] == "cost" and np.array_equal(final, net.layer_output(net.n - 2))
    out = str(tmp_path / "roundtrip.weights")
    net.save_weights(out)
    assert open(out, "rb").read() == open(os.path.join(GOLD, "small_net2.weights"), "rb").read()
    net.free()


def test_batchnorm_layer_network_and_weights_file(dn, tmp_path):
    """[batchnorm] as a layer of its own (after a plain and after a batch-normalised convolution):
    layer table, the weights file the reference saved for it (scales, mean, variance of those
    layers; byte-identical round trip), and every layer against the checker."""
    text = open(os.path.join(GOLD, "bn_net.cfg")).read()
    gold = json.load(open(os.path.join(GOLD, "layer_tables.json")))["bn_net"]
    net = api.Network(cfg_text=text, weights=os.path.join(GOLD, "bn_net.weights"))
    assert [L["type"] for L in net.layers] == [L["type"] for L in gold] and net.layers[1]["type"] == "batchnorm"
    orc = OracleNet(text)
    fill_params(orc.set_conv, orc.layers, seed=710, bn="random")   # what the fixture's weights file holds
    x = synth.uniform01(17, net.inputs * net.batch)
    final = net.predict(x)
    want = orc.forward(x)
    for i, L in enumerate(net.layers):
        assert norm_err(net.layer_output(i), want[i]) <= REL_TOL, (i, L["type"])
    assert np.array_equal(final, net.layer_output(net.n - 1))
    out = str(tmp_path / "roundtrip.weights")
    net.save_weights(out)
    assert open(out, "rb").read() == open(os.path.join(GOLD, "bn_net.weights"), "rb").read()
    # with non-zero biases too (a weights file never carries them for this layer)
    fill_params(net.set_conv, net.layers, seed=33, bn="random")
    fill_params(orc.set_conv, orc.layers, seed=33, bn="random")
    b4 = synth.uniform(91, net.layers[4]["c"], -0.5, 0.5)
    p = orc.params[4]
    orc.set_conv(4, None, b4, p[2], p[3], p[4])
    net.set_conv(4, None, b4, p[2], p[3], p[4])
    net.predict(x)
    want = orc.forward(x)
    for i, L in enumerate(net.layers):
        assert norm_err(net.layer_output(i), want[i]) <= REL_TOL, (i, L["type"])
    net.free()


def test_connected_layers_at_classifier_sizes(dn):
    """vgg/alexnet-like heads: K = 9216 and 4096, batch 64; K-split tails and ragged M (1000)."""
    text = ("[net]\nbatch=64\nsubdivisions=1\nwidth=6\nheight=6\nchannels=256\n"
            "[connected]\noutput=4096\nactivation=relu\n[dropout]\nprobability=.5\n"
            "[connected]\noutput=1000\nbatch_normalize=1\nactivation=linear\n[softmax]\n")
    net, orc = build_pair(text, seed=77)
    x = synth.uniform(3, net.inputs * net.batch, -1, 1)
    net.predict(x)
    want = orc.forward(x)
    for i in range(net.n):
        assert norm_err(net.layer_output(i), want[i]) <= REL_TOL, i
    assert abs(net.conv_flops() - 2.0 * (9216 * 4096 + 4096 * 1000)) < 1
    net.free()


def device_free_bytes():
    """Free device memory as the HIP runtime (already loaded by the library) reports it."""
    import ctypes
    rt = ctypes.CDLL("libamdhip64.so")
    free, total = ctypes.c_size_t(), ctypes.c_size_t()
    assert rt.hipMemGetInfo(ctypes.byref(free), ctypes.byref(total)) == 0
    return free.value


def test_free_network_returns_its_device_memory(dn):
    """A serving process that loads and frees networks must not grow: after a first cycle has
    sized the library's process-wide work buffers, every later parse -> set weights -> predict ->
    detect -> free cycle gives back all the device memory it took."""
    def cycle(text):
        net = api.Network(cfg_text=text)
        fill_params(net.set_conv, net.layers, seed=5, bn="random")
        net.predict(synth.uniform01(3, net.inputs * net.batch))
        net.free()

    texts = [cfgs.yolov3(2, 416), cfgs.yolov3_tiny(2, 416, xnor=True), cfgs.resnext50(2, 224)]
    for t in texts:
        cycle(t)
    base = device_free_bytes()
    for _ in range(3):
        for t in texts:
            cycle(t)
    assert device_free_bytes() >= base - (4 << 20), (base, device_free_bytes())


def test_pipelined_predict_gives_the_bits_of_network_predict(dn):
    """network_predict_submit / _collect with two batches in flight: five different batches, pageable
    and pinned inputs mixed, every yolo head and the output layer bit-equal to network_predict on the
    same batch; the pointers of a collected batch stay intact while the next one is in flight."""
    net = api.Network(cfg_text=cfgs.yolov3_tiny(8, 224))
    fill_params(net.set_conv, net.layers)
    heads = [i for i, L in enumerate(net.layers) if L["type"] == "yolo"]
    xs = [synth.uniform01(100 + k, net.inputs * 8) for k in range(5)]
    want = []
    for x in xs:
        final = net.predict(x)
        want.append({i: net.layer_output(i) for i in heads})
        assert np.array_equal(final, want[-1][heads[-1]])
    pinned = api.pinned_array(xs[1].size)
    pinned[:] = xs[1]
    feed = [xs[0], pinned, xs[2], xs[3], xs[4]]
    net.submit(feed[0])
    assert dn.network_predict_in_flight(net.net) == 1
    for k in range(1, 5):
        net.submit(feed[k])                          # batch k uploads and computes ...
        assert dn.network_predict_in_flight(net.net) == 2
        final = net.collect()                        # ... while batch k-1 comes back
        got = {i: net.collected_output(i) for i in heads}
        for i in heads:
            assert np.array_equal(got[i], want[k - 1][i]), (k - 1, i)
        assert np.array_equal(final, want[k - 1][heads[-1]])
    net.collect()
    for i in heads:
        assert np.array_equal(net.collected_output(i), want[4][i]), (4, i)
    assert dn.network_predict_in_flight(net.net) == 0
    # the synchronous call still works on the same network afterwards
    assert np.array_equal(net.predict(xs[0]), want[0][heads[-1]])
    api.free_pinned_array(pinned)
    net.free()


def test_pipelined_predict_on_a_classifier_and_at_a_smaller_batch(dn):
    net = api.Network(cfg_text=cfgs.resnext50(4, 64))
    fill_params(net.set_conv, net.layers)
    xs = [synth.uniform01(300 + k, net.inputs * 4) for k in range(3)]
    want = [net.predict(x) for x in xs]
    net.submit(xs[0])
    net.submit(xs[1])
    assert np.array_equal(net.collect(), want[0])
    net.submit(xs[2])
    assert np.array_equal(net.collect(), want[1])
    assert np.array_equal(net.collect(), want[2])
    net.set_batch(2)
    small = net.predict(xs[0][:net.inputs * 2])
    net.submit(xs[0][:net.inputs * 2])
    assert np.array_equal(net.collect(), small)
    net.free()


@pytest.mark.parametrize("misuse,message", [
    ("net.submit(x); net.submit(x); net.submit(x)", "two batches are in flight already"),
    ("net.collect()", "no batch is in flight"),
    ("net.submit(x); net.predict(x)", "collect them first"),
    ("net.submit(x); net.set_batch(1)", "collect them first"),
])
def test_pipelined_predict_misuse_ends_with_a_message(misuse, message):
    """A third submit, a collect with nothing in flight, and the synchronous calls that would write the
    buffers a batch in flight is still being copied out of end the process with a message, as every
    argument the library cannot honour does (a process of its own: the library exits)."""
    import os
    import subprocess
    import sys
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    code = ("from darknet_amd import api, cfgs, synth\napi.set_gpu(0)\n"
            "net = api.Network(cfg_text=cfgs.yolov3_tiny(2, 96))\n"
            "x = synth.uniform01(1, net.inputs * 2)\nnet.predict(x)\nprint('ready', flush=True)\n"
            + "\n".join(part.strip() for part in misuse.split(";")) + "\nprint('survived', flush=True)\n")
    r = subprocess.run([sys.executable, "-c", code], cwd=root, capture_output=True, text=True, timeout=100)
    assert "ready" in r.stdout and "survived" not in r.stdout and r.returncode != 0, (r.stdout, r.stderr[-400:])
    assert message in r.stderr, r.stderr[-400:]

