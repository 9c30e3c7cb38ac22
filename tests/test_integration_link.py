"""The reference's own host files bound to the HIP library (no GPU needed).

`make -C oracle ref_hip` compiles every src/*.c of the reference tree with -DGPU where it lies
(minus src/cuda.c, which the library replaces), against the two headers the binding changes, and
links them with integration/adapters.c + integration/training_stubs.c and libdarknet_hip.so under
-Wl,--no-undefined.  These tests hold the claims made about that link:

* it succeeds, i.e. nothing the tree needs is missing;
* the list of not-served symbols in training_stubs.c is exactly what the tree needs beyond the
  adapters and the library - no more, no less;
* no function that takes a by-value `layer` / `network` crosses from the tree into the library
  (the library's structs are a subset at other offsets: such a call would link and misbehave);
* the reference's parser, built with -DGPU, runs on the library's device shim: in parse-only mode
  it produces the reference's own layer table.
"""
import os
import re
import subprocess

import pytest

from darknet_amd import cfgs, lib
from oracle import ref

from util import have_reference_tree, write_cfg

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
REF_OUT = os.path.join(ROOT, "oracle", "_ref")
OBJ = os.path.join(REF_OUT, "hip_tree", "obj")
needs_tree = pytest.mark.skipif(not have_reference_tree(), reason="needs the reference tree to compile")
needs_built = pytest.mark.skipif(not os.path.exists(os.path.join(REF_OUT, "librefh_hip.so")),
                                 reason="oracle/_ref/librefh_hip.so is not built")


def nm(path, *flags):
    out = subprocess.run(["nm", *flags, path], check=True, capture_output=True, text=True).stdout
    return {line.split()[-1].split("@")[0] for line in out.splitlines() if line.strip()}


def stub_names():
    text = open(os.path.join(ROOT, "integration", "training_stubs.c")).read()
    return set(re.findall(r"^DN_NOT_SERVED\((\w+)\)", text, flags=re.M))


@needs_tree
def test_reference_tree_links_against_the_library():
    r = subprocess.run(["make", "-j8", "-C", os.path.join(ROOT, "oracle"), "ref_hip"], capture_output=True, text=True)
    assert r.returncode == 0, r.stdout[-3000:] + r.stderr[-3000:]
    for name in ("libdarknet_ref_hip.so", "librefh_hip.so"):
        assert os.path.exists(os.path.join(REF_OUT, name)), name
    # the link line asks the linker to refuse undefined symbols
    mk = open(os.path.join(ROOT, "oracle", "Makefile")).read()
    rule = mk[mk.index("$(OUT)/libdarknet_ref_hip.so:"):]
    assert "--no-undefined" in rule[:rule.index("\n\n")]


@needs_tree
def test_stub_list_is_exactly_what_the_tree_needs():
    objs = [os.path.join(OBJ, f) for f in sorted(os.listdir(OBJ)) if f.endswith(".o")]
    tree = [o for o in objs if os.path.basename(o) not in ("adapters.o", "training_stubs.o")]
    assert len(tree) >= 40
    defined, undefined = set(), set()
    for o in tree:
        defined |= nm(o, "--defined-only", "-g")
        undefined |= nm(o, "-u")
    needed = undefined - defined
    adapters = nm(os.path.join(OBJ, "adapters.o"), "--defined-only", "-g")
    stubs = nm(os.path.join(OBJ, "training_stubs.o"), "--defined-only", "-g")
    library = nm(lib.LIB_PATH, "-D", "--defined-only")
    assert stubs == stub_names()
    assert stubs <= needed, sorted(stubs - needed)                 # no stub the tree does not ask for
    assert adapters <= needed, sorted(adapters - needed)            # no adapter the tree does not ask for
    assert not (stubs & library), sorted(stubs & library)           # nothing stubbed that the library serves
    from_library = (needed - adapters - stubs) & library
    system = needed - adapters - stubs - library                    # libc, libm, libgomp, pthread
    assert all(not s.endswith("_gpu") and not s.startswith(("cuda", "cublas", "curand", "cudnn")) for s in system), \
        sorted(system)
    by_value = set(lib.STRUCT_BY_VALUE)
    assert not (from_library & by_value), sorted(from_library & by_value)
    assert from_library <= set(lib.SIGNATURES) | {"gpu_index"}, sorted(from_library - set(lib.SIGNATURES))
    # the functions of the CUDA translation units that inference reaches are all adapters
    assert {"forward_convolutional_layer_gpu", "push_convolutional_layer", "pull_convolutional_layer",
            "forward_maxpool_layer_gpu", "forward_avgpool_layer_gpu", "forward_crop_layer_gpu",
            "forward_dropout_layer_gpu"} == adapters


@needs_built
def test_built_tree_imports_only_plain_pointer_entry_points():
    imports = nm(os.path.join(REF_OUT, "libdarknet_ref_hip.so"), "-D", "-u")
    library = nm(lib.LIB_PATH, "-D", "--defined-only")
    crossing = imports & library
    assert "cuda_make_array" in crossing and "forward_convolutional_gpu" in crossing
    assert not (crossing & set(lib.STRUCT_BY_VALUE)), sorted(crossing & set(lib.STRUCT_BY_VALUE))
    exports = nm(os.path.join(REF_OUT, "libdarknet_ref_hip.so"), "-D", "--defined-only")
    assert {"parse_network_cfg", "network_predict", "forward_network_gpu", "forward_yolo_layer_gpu"} <= exports
    assert stub_names() <= exports


@needs_built
def test_reference_parser_runs_on_the_shim_in_parse_only_mode():
    L = lib.load()
    L.hip_set_parse_only(1)
    try:
        path = write_cfg(cfgs.yolov3_tiny(1, 416))
        bound = ref.RefNet(path, "hip", gpu=None)
        assert bound.h.refh_is_gpu_build() == 1
        cpu = ref.RefNet(path, "o2")
        assert cpu.h.refh_is_gpu_build() == 0
        assert bound.layers == cpu.layers
        bound.free()
        cpu.free()
        os.unlink(path)
    finally:
        L.hip_set_parse_only(0)
