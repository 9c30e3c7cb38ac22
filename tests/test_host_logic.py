"""The library's host logic without a GPU: cfg reader + parser (layer geometry) and the weights
file reader/writer, through the C-ABI in parse-only mode (hip_set_parse_only: no device memory, no
launches, and anything that would compute ends the process).

The parser is checked against the golden layer tables the compiled reference printed and, where
the reference tree is present, against the CPU checker's parse of every cfg the reference ships
within the supported layer types (that parse is itself pinned to the compiled reference in
test_oracle_cfg.py)."""
import glob
import json
import os
import re
import subprocess
import sys

import numpy as np
import pytest

from darknet_amd import api, cfgs, lib
from oracle import cfg as ocfg

from test_oracle_cfg import COMMON, PER_TYPE
from util import have_reference_tree

GOLD = os.path.join(os.path.dirname(__file__), "golden")
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.fixture
def parse_only():
    L = lib.load()
    L.hip_set_parse_only(1)
    yield L
    L.hip_set_parse_only(0)


def same_table(want, got, where):
    assert len(want) == len(got), where
    for i, (x, y) in enumerate(zip(want, got)):
        for k in COMMON + PER_TYPE.get(x["type"], []):
            if k == "mask":
                continue                      # not part of the library's layer query
            if x["type"] == "route" and k in ("h", "w", "c"):
                continue                      # the reference leaves them unset for routes
            a, b = x[k], y[k]
            assert a == b or (isinstance(a, float) and abs(a - b) < 1e-6), (where, i, x["type"], k, a, b)


@pytest.mark.parametrize("name,text", [("yolov3-tiny-416", cfgs.yolov3_tiny(1, 416)),
                                       ("yolov3-416", cfgs.yolov3(1, 416)),
                                       ("resnext50-224", cfgs.resnext50(1, 224)),
                                       ("small_net", open(os.path.join(GOLD, "small_net.cfg")).read()),
                                       ("small_net2", open(os.path.join(GOLD, "small_net2.cfg")).read()),
                                       ("yolov1_net", open(os.path.join(GOLD, "yolov1_net.cfg")).read()),
                                       ("bn_net", open(os.path.join(GOLD, "bn_net.cfg")).read())],
                         ids=["yolov3-tiny-416", "yolov3-416", "resnext50-224", "small_net", "small_net2", "yolov1_net",
                              "bn_net"])
def test_library_parser_matches_golden_layer_tables(parse_only, name, text):
    gold = json.load(open(os.path.join(GOLD, "layer_tables.json")))[name]
    net = api.Network(cfg_text=text)
    same_table(gold, net.layers, name)
    if name == "yolov3-416":
        assert abs(net.conv_flops() - 65.864e9) < 1e6
    net.free()


def test_library_parser_grammar_details(parse_only):
    text = "[net]\n batch = 8 \nsubdivisions=4\n# comment\n;also\nwidth=32\nheight = 32\nchannels=3\n\n" \
           "[conv]\nfilters=4\nsize=3\npad=1\nstride=1\nactivation = leaky\nfilters=99\n" \
           "[maxpool]\nstride=1\nsize=2\n"
    net = api.Network(cfg_text=text)
    assert net.batch == 2                                     # batch / subdivisions
    L = net.layers[0]
    assert L["n"] == 4 and L["pad"] == 1                      # first key wins; pad=1 -> size/2
    assert L["batch_normalize"] == 0 and L["activation"] == "leaky"
    assert net.layers[1]["pad"] == 1 and net.layers[1]["out_w"] == 32   # maxpool padding defaults to size-1
    net.free()


@pytest.mark.skipif(not have_reference_tree(), reason="needs the reference's cfg directory")
def test_library_parses_every_in_scope_reference_cfg(parse_only):
    done = 0
    for path in sorted(glob.glob("/root/reference/cfg/*.cfg")):
        text = open(path).read()
        kinds = set(re.findall(r"(?m)^\s*(\[[a-z]+\])", text))
        if not kinds <= set(ocfg.SECTION_ALIASES):
            continue
        if re.search(r"(?m)^\s*(tree|map)\s*=", text):
            continue            # needs data files relative to the reference's working directory
        want = ocfg.parse(text)["layers"]
        net = api.Network(cfg_path=path)
        same_table(want, net.layers, os.path.basename(path))
        net.free()
        done += 1
    assert done >= 40


def test_weights_file_round_trip_on_the_host(parse_only, tmp_path):
    """The file the REFERENCE saved for small_net is read into host arrays and written back byte
    for byte; a truncated file is noticed."""
    src = os.path.join(GOLD, "small_net.weights")
    net = api.Network(cfg_path=os.path.join(GOLD, "small_net.cfg"), weights=src)
    out = str(tmp_path / "again.weights")
    net.save_weights(out)
    assert open(out, "rb").read() == open(src, "rb").read()
    net.free()
    src2 = os.path.join(GOLD, "small_net2.weights")     # connected layers, batch-normalised and plain
    net = api.Network(cfg_path=os.path.join(GOLD, "small_net2.cfg"), weights=src2)
    net.save_weights(out)
    assert open(out, "rb").read() == open(src2, "rb").read()
    net.free()
    src3 = os.path.join(GOLD, "yolov1_net.weights")     # a local layer's block: biases per output, weights per location
    net = api.Network(cfg_path=os.path.join(GOLD, "yolov1_net.cfg"), weights=src3)
    net.save_weights(out)
    assert open(out, "rb").read() == open(src3, "rb").read()
    net.free()
    src4 = os.path.join(GOLD, "bn_net.weights")         # [batchnorm] layers: scales, mean, variance (no biases)
    net = api.Network(cfg_path=os.path.join(GOLD, "bn_net.cfg"), weights=src4)
    net.save_weights(out)
    assert open(out, "rb").read() == open(src4, "rb").read()
    net.free()


VARIANT_CFG = ("[net]\nbatch=1\nheight=4\nwidth=4\nchannels=2\n"
               "[convolutional]\nfilters=3\nsize=3\npad=1\nstride=1\nactivation=linear\n{flip}"
               "[connected]\noutput=5\nactivation=linear\n")


def _variant_payload(conv_w, fc_w):
    """biases, weights of the conv layer, then biases, weights of the connected one (no batch-norm)."""
    f32 = lambda a: np.asarray(a, np.float32).tobytes()
    return f32(np.arange(3) + 0.5) + f32(conv_w) + f32(np.arange(5) - 2.25) + f32(fc_w)


def test_weights_file_header_and_layout_variants(parse_only, tmp_path):
    """The branches no reference-written fixture reaches, on hand-built files (format from
    src/parser.c:1227-1246, 1098-1104, 1164-1209): the old header with an `int seen`, the
    transposed connected weights of files whose major or minor version exceeds 1000, and the
    `flipped` convolution weights.  Each file is read in and saved again; the saved file always has
    the current header (0, 2, 0, size_t seen) and the library's own weight order."""
    conv = np.arange(3 * 2 * 9, dtype=np.float32).reshape(3, 18) * 0.25          # [n][c*size*size]
    fc = (np.arange(5 * 48, dtype=np.float32).reshape(5, 48) - 100) * 0.125      # [outputs][inputs]
    canonical = (np.array([0, 2, 0], np.int32).tobytes() + np.array([12345], np.uint64).tobytes()
                 + _variant_payload(conv, fc))
    out = str(tmp_path / "saved.weights")

    def round_trip(name, header, payload, flip=""):
        cfgp, wp = str(tmp_path / (name + ".cfg")), str(tmp_path / (name + ".weights"))
        open(cfgp, "w").write(VARIANT_CFG.format(flip=flip))
        open(wp, "wb").write(header + payload)
        net = api.Network(cfg_path=cfgp, weights=wp)
        net.save_weights(out)
        net.free()
        return open(out, "rb").read()

    new_header = np.array([0, 2, 0], np.int32).tobytes() + np.array([12345], np.uint64).tobytes()
    assert round_trip("current", new_header, _variant_payload(conv, fc)) == canonical
    # version 0.1: `seen` is a 4-byte int
    old_header = np.array([0, 1, 0, 12345], np.int32).tobytes()
    assert round_trip("old_header", old_header, _variant_payload(conv, fc)) == canonical
    # major > 1000 (and so an int `seen`): connected weights are stored [inputs][outputs]
    t_header = np.array([1001, 0, 0, 12345], np.int32).tobytes()
    assert round_trip("transposed", t_header, _variant_payload(conv, fc.T.copy())) == canonical
    # minor > 1000 selects the same transpose
    t2_header = np.array([0, 1001, 0, 12345], np.int32).tobytes()
    assert round_trip("transposed_minor", t2_header, _variant_payload(conv, fc.T.copy())) == canonical
    # flipped=1 on the convolution: its weights are stored [c*size*size][n]
    assert round_trip("flipped", new_header, _variant_payload(conv.T.copy(), fc), flip="flipped=1\n") == canonical
    # a file that ends inside a layer is an error, not a silent partial load
    cfgp, wp = str(tmp_path / "short.cfg"), str(tmp_path / "short.weights")
    open(cfgp, "w").write(VARIANT_CFG.format(flip=""))
    open(wp, "wb").write((new_header + _variant_payload(conv, fc))[:-40])
    code = ("from darknet_amd import api, lib\nL = lib.load(); L.hip_set_parse_only(1)\n"
            f"api.Network(cfg_path={cfgp!r}, weights={wp!r})\nprint('loaded')\n")
    r = subprocess.run([sys.executable, "-c", code], cwd=ROOT, capture_output=True, text=True, timeout=120)
    assert r.returncode != 0 and "loaded" not in r.stdout


def test_numload_reads_only_the_first_filters(parse_only, tmp_path):
    """numload=2 on a 3-filter convolution: the file holds two filters' worth of every vector
    (src/parser.c:1166); the third keeps its initial values and the layer keeps its geometry."""
    cfgp, wp, out = str(tmp_path / "n.cfg"), str(tmp_path / "n.weights"), str(tmp_path / "o.weights")
    open(cfgp, "w").write("[net]\nbatch=1\nheight=4\nwidth=4\nchannels=2\n"
                          "[convolutional]\nfilters=3\nsize=3\npad=1\nstride=1\nactivation=linear\nnumload=2\n")
    w2 = np.arange(2 * 18, dtype=np.float32) + 1
    header = np.array([0, 2, 0], np.int32).tobytes() + np.array([7], np.uint64).tobytes()
    open(wp, "wb").write(header + np.array([1.5, 2.5], np.float32).tobytes() + w2.tobytes())
    net = api.Network(cfg_path=cfgp, weights=wp)
    assert net.layers[0]["n"] == 3 and net.layers[0]["nweights"] == 54
    net.save_weights(out)
    net.free()
    want = header + np.array([1.5, 2.5, 0], np.float32).tobytes() + np.concatenate([w2, np.zeros(18, np.float32)]).tobytes()
    assert open(out, "rb").read() == want


def test_strided_1x1_convolution_is_refused_when_the_network_is_built():
    """A 1x1 kernel with stride 2 (or padding): refused at parse time with a message, not at the
    first forward (the reference computes a misread image for it, src/convolutional_layer.c:468-469)."""
    code = ("from darknet_amd import api, lib\n"
            "L = lib.load(); L.hip_set_parse_only(1)\n"
            "api.Network(cfg_text='[net]\\nbatch=1\\nheight=8\\nwidth=8\\nchannels=16\\n"
            "[convolutional]\\nfilters=32\\nsize=1\\nstride=2\\nactivation=linear\\n')\n"
            "print('built', flush=True)\n")
    r = subprocess.run([sys.executable, "-c", code], cwd=ROOT, capture_output=True, text=True, timeout=120)
    assert r.returncode != 0 and "built" not in r.stdout and "1x1 kernel needs stride 1" in r.stderr


def test_parse_only_mode_computes_nothing():
    """network_predict in parse-only mode ends the process with a message (no host fallback)."""
    code = ("import numpy as np\n"
            "from darknet_amd import api, cfgs, lib\n"
            "L = lib.load(); L.hip_set_parse_only(1)\n"
            "net = api.Network(cfg_text=cfgs.yolov3_tiny(1, 64))\n"
            "print('parsed', net.n, flush=True)\n"
            "net.predict(np.zeros(net.inputs, np.float32))\n"
            "print('computed', flush=True)\n")
    r = subprocess.run([sys.executable, "-c", code], cwd=ROOT, capture_output=True, text=True, timeout=120)
    assert "parsed 24" in r.stdout and "computed" not in r.stdout
    assert r.returncode != 0 and "parse-only" in r.stderr


def test_which_layers_run_inside_the_convolution_in_front_of_them(parse_only):
    """network_layer_runs_fused / network_layer_output_skipped are host decisions over the parsed layer table:
    yolov3's 23 residual adds and 3 yolo heads; in yolov3-tiny the maxpools behind the two first-layer
    convolutions and the two heads; with xnor=1 also the maxpools behind the xnor convolutions (not the
    stride-1 pool), and no yolo head behind an xnor convolution; nothing at level 0; at level 2 the maps only
    a fused maxpool reads are reported as not written."""
    L = parse_only
    cases = [(cfgs.yolov3(1, 416), None, []),
             (cfgs.yolov3_tiny(2, 416), [1, 3, 16, 23], [0, 2]),
             (cfgs.yolov3_tiny(2, 416, xnor=True), [1, 3, 5, 7, 9, 23], [0, 2, 4, 6])]
    try:
        for text, fused, skipped in cases:
            net = api.Network(cfg_text=text)
            types = [Ly["type"] for Ly in net.layers]
            L.network_set_fusion(0)
            assert not any(L.network_layer_runs_fused(net.net, i) for i in range(net.n))
            L.network_set_fusion(1)
            got = [i for i in range(net.n) if L.network_layer_runs_fused(net.net, i)]
            if fused is None:
                assert sorted(types[i] for i in got) == ["shortcut"] * 23 + ["yolo"] * 3
            else:
                assert got == fused
            assert not any(L.network_layer_output_skipped(net.net, i) for i in range(net.n))
            L.network_set_fusion(2)
            assert [i for i in range(net.n) if L.network_layer_output_skipped(net.net, i)] == skipped
            assert not L.network_layer_runs_fused(net.net, 0) and not L.network_layer_runs_fused(net.net, net.n)
            net.free()
    finally:
        L.network_set_fusion(1)

