"""The drop-in boundary against the reference's own headers, as text (nothing of the reference is
compiled or run): every function this library declares under a name the reference also declares
has the reference's return type and argument types; the ACTIVATION / LAYER_TYPE enums have the
reference's members in the reference's order; every member of this library's `layer` / `network`
exists in the reference's structs with the same type (apart from the documented additions); and
the adapter stubs of the integration guide only touch struct members and device-layer functions
that exist.  Skipped where the reference tree is not mounted."""
import glob
import os
import re

import pytest

from util import have_reference_tree

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
REF = "/root/reference"
GUIDE = "INTEGRATION.md"   # the guide for binders at the repository root
pytestmark = pytest.mark.skipif(not have_reference_tree(), reason="needs the reference's headers")

# typedefs of the reference that stand for `layer` (include/darknet.h and src/*_layer.h)
LAYER_ALIASES = {"convolutional_layer", "maxpool_layer", "route_layer", "avgpool_layer", "softmax_layer",
                 "dropout_layer", "crop_layer", "cost_layer", "local_layer", "detection_layer", "connected_layer"}
# members this library adds to the reference's structs (the integration guide tells a binder to add them)
LAYER_ADDITIONS = {"weights_packed_gpu", "xnor_wbits_gpu", "xnor_xbits_gpu", "xnor_wmean_gpu", "output_gpu_is_view"}
NETWORK_ADDITIONS = {"det_rows_gpu", "det_count_gpu", "det_max_rows", "max_batch", "pipeline"}
# same name, deliberately another signature
SIGNATURE_EXCEPTIONS = {
    "check_error": "takes cudaError_t in the reference; the library's is hip_check_error(int)",
}


def strip_comments(text):
    text = re.sub(r"/\*.*?\*/", " ", text, flags=re.S)
    return re.sub(r"//[^\n]*", " ", text)


def norm_type(t):
    t = re.sub(r"\b(const|struct|extern)\b", " ", t)
    t = re.sub(r"\s*\*\s*", "*", " ".join(t.split()))
    words = t.replace("*", " * ").split()
    words = ["layer" if w in LAYER_ALIASES else w for w in words]
    words = ["int" if w in ("ACTIVATION", "COST_TYPE") else w for w in words]   # an enum passes as an int in the C ABI
    return " ".join(words).replace(" *", "*").replace("* ", "*")


def split_arg(arg):
    """'float *x_gpu' -> 'float*'; 'size_t n' -> 'size_t'; 'void' -> ''."""
    arg = arg.strip()
    if arg in ("", "void"):
        return None
    m = re.match(r"^(.*?)(\b[A-Za-z_]\w*)?\s*(\[\s*\d*\s*\])?$", arg, flags=re.S)
    head, name, arr = m.group(1), m.group(2), m.group(3)
    if not head.strip():          # a bare type without a name
        head, name = arg, None
    t = norm_type(head)
    return t + ("*" if arr else "")


def prototypes(text):
    """{name: (return type, [argument types])} of the function declarations in a header."""
    text = strip_comments(text)
    text = re.sub(r"#[^\n]*", " ", text)
    out = {}
    for stmt in text.split(";"):
        stmt = " ".join(stmt.split("}")[-1].split("{")[-1].split())
        m = re.match(r"^((?:[A-Za-z_]\w*[\s\*]+)+?)\s*([A-Za-z_]\w*)\s*\(([^()]*)\)$", stmt)
        if not m:
            continue
        ret, name, args = m.group(1), m.group(2), m.group(3)
        if "typedef" in ret.split() or "return" in ret.split():
            continue
        argv = [split_arg(a) for a in args.split(",")]
        out[name] = (norm_type(ret), [a for a in argv if a is not None])
    return out


def enum_members(text, name):
    m = re.search(r"typedef\s+enum\s*\{([^}]*)\}\s*" + name + r"\s*;", strip_comments(text), flags=re.S)
    assert m, name
    return [w.strip().split("=")[0].strip() for w in m.group(1).split(",") if w.strip()]


def struct_members(text, opener):
    """{member: type} of the struct whose definition starts with `opener`; function pointers keep
    the text of their declaration as the type."""
    text = strip_comments(text)
    start = text.index(opener)
    body = text[text.index("{", start) + 1:]
    depth, end = 1, 0
    for end, ch in enumerate(body):
        depth += ch == "{"
        depth -= ch == "}"
        if depth == 0:
            break
    body = re.sub(r"#[^\n]*", " ", body[:end])
    out = {}
    for decl in body.split(";"):
        decl = " ".join(decl.split())
        if not decl:
            continue
        fp = re.match(r"^(.*?)\(\s*\*\s*(\w+)\s*\)\s*\((.*)\)$", decl)
        if fp:
            out[fp.group(2)] = norm_type(fp.group(1)) + "(*)(" + ",".join(norm_type(a) for a in fp.group(3).split(",")) + ")"
            continue
        m = re.match(r"^(.*?)((?:\**\s*\w+\s*,\s*)*\**\s*\w+)$", decl)
        base, names = m.group(1), m.group(2)
        for nm in names.split(","):
            nm = nm.strip()
            stars = len(nm) - len(nm.lstrip("* "))
            out[nm.lstrip("* ")] = norm_type(base + "*" * nm[:stars].count("*"))
    return out


@pytest.fixture(scope="module")
def ref_headers():
    return {p: open(p).read() for p in sorted(glob.glob(REF + "/src/*.h")) + [REF + "/include/darknet.h"]}


@pytest.fixture(scope="module")
def own_headers():
    return {p: open(os.path.join(ROOT, "include", p)).read() for p in ("darknet_hip.h", "darknet_amd.h")}


def test_shared_function_names_have_the_reference_signatures(ref_headers, own_headers):
    ref = {}
    for path, text in ref_headers.items():
        for name, sig in prototypes(text).items():
            ref.setdefault(name, (sig, path))
    own = {}
    for text in own_headers.values():
        own.update(prototypes(text))
    shared = sorted(set(own) & set(ref))
    # the boundary the path needs: the device shim, the element-wise helpers, the per-layer forwards
    for must in ("cuda_make_array", "cuda_push_array", "cuda_pull_array", "cuda_free", "cuda_set_device", "cuda_random",
                 "cuda_mag_array", "cuda_compare", "cuda_make_int_array",
                 "fill_gpu", "copy_gpu", "activate_array_gpu", "normalize_gpu", "scale_bias_gpu", "add_bias_gpu",
                 "shortcut_gpu", "upsample_gpu", "softmax_gpu", "im2col_gpu",
                 "forward_convolutional_layer_gpu", "push_convolutional_layer", "pull_convolutional_layer",
                 "forward_batchnorm_layer_gpu", "push_batchnorm_layer", "pull_batchnorm_layer", "make_batchnorm_layer",
                 "forward_maxpool_layer_gpu", "forward_upsample_layer_gpu", "forward_shortcut_layer_gpu",
                 "forward_route_layer_gpu", "forward_yolo_layer_gpu", "forward_avgpool_layer_gpu",
                 "forward_softmax_layer_gpu", "parse_network_cfg", "network_predict", "forward_network",
                 "forward_network_gpu", "load_weights", "save_weights", "get_network_boxes", "do_nms_sort",
                 "letterbox_image", "network_predict_image", "set_batch_network", "make_convolutional_layer"):
        assert must in shared, must + " is not declared on both sides"
    bad = []
    for name in shared:
        if name in SIGNATURE_EXCEPTIONS:
            continue
        (rret, rargs), path = ref[name]
        oret, oargs = own[name]
        if (rret, rargs) != (oret, oargs):
            bad.append(f"{name}: reference {rret}({', '.join(rargs)}) [{os.path.relpath(path, REF)}] "
                       f"vs library {oret}({', '.join(oargs)})")
    assert not bad, "\n".join(bad)
    assert len(shared) >= 90


def test_enums_have_the_reference_members_in_order(ref_headers, own_headers):
    ref, own = ref_headers[REF + "/include/darknet.h"], own_headers["darknet_amd.h"]
    for name in ("ACTIVATION", "LAYER_TYPE"):
        assert enum_members(own, name) == enum_members(ref, name), name
    codes = re.search(r"enum\s*\{([^}]*)\}", strip_comments(own_headers["darknet_hip.h"]), flags=re.S).group(1)
    plain = [w.strip().split("=")[0].strip()[3:] for w in codes.split(",") if w.strip()]
    assert plain == enum_members(ref, "ACTIVATION")           # DN_LOGISTIC .. DN_SELU: the same order


def test_struct_members_exist_in_the_reference_with_the_same_type(ref_headers, own_headers):
    ref, own = ref_headers[REF + "/include/darknet.h"], own_headers["darknet_amd.h"]
    for opener, additions in (("struct layer{", LAYER_ADDITIONS), ("typedef struct network{", NETWORK_ADDITIONS)):
        want = struct_members(ref, opener)
        got = struct_members(own, opener.replace("{", " {"))
        assert len(got) > 20
        for member, typ in got.items():
            if member in additions:
                assert member not in want, member
                continue
            assert member in want, f"{opener} {member}: not a member of the reference's struct"
            assert want[member] == typ, f"{opener} {member}: {typ} here, {want[member]} in the reference"


def test_integration_adapters_use_members_and_functions_that_exist(ref_headers, own_headers):
    doc = open(os.path.join(ROOT, GUIDE)).read()
    code = "\n".join(re.findall(r"```c\n(.*?)```", doc, flags=re.S))
    # the adapters a tree needs are a compiled file (tests/test_integration_link.py links it into the
    # reference tree); the guide's own blocks are the optional replacements, checked here as text
    adapters = open(os.path.join(ROOT, "integration", "adapters.c")).read()
    assert "forward_convolutional_layer_gpu" in adapters and "forward_maxpool_layer_gpu" in adapters
    assert "forward_connected_layer_gpu" in code and "forward_route_layer_gpu" in code
    code = code + "\n" + adapters
    ref = ref_headers[REF + "/include/darknet.h"]
    layer = set(struct_members(ref, "struct layer{")) | LAYER_ADDITIONS
    network = set(struct_members(ref, "typedef struct network{")) | NETWORK_ADDITIONS
    code_nc = strip_comments(code)
    for var, member in re.findall(r"\b(l|s)\.(\w+)", code_nc):
        assert member in layer, f"{var}.{member} is not a member of the reference's struct layer"
    for member in re.findall(r"\bnet(?:\.|->)(\w+)", code_nc):
        assert member in network, f"net.{member} is not a member of the reference's struct network"
    for member in re.findall(r"\bnet(?:\.|->)layers\[[^\]]*\]\.(\w+)", code_nc):
        assert member in layer, member
    # every device-layer function the stubs call is declared by darknet_hip.h with that many arguments
    own = prototypes(own_headers["darknet_hip.h"])
    called = re.findall(r"\b(\w+_gpu|cuda_\w+|conv_\w+)\s*\(", code_nc)
    defined_in_doc = set(re.findall(r"^void\s+(\w+)\s*\(", code_nc, flags=re.M))
    checked = 0
    for name in set(called) - defined_in_doc:
        assert name in own, name + " is called by a stub of the integration guide but not declared in darknet_hip.h"
        checked += 1
    assert checked >= 15
    # argument counts of the calls written out in full
    for name, args in re.findall(r"\b(forward_\w+_gpu|upsample_gpu|softmax_gpu|copy_gpu|conv_pack_weights_gpu|cuda_push_array)"
                                 r"\s*\(([^;{}]*?)\)\s*;", code_nc, flags=re.S):
        if name in defined_in_doc or "<" in args:
            continue
        depth, count = 0, 1
        for ch in args:
            depth += ch in "(["
            depth -= ch in ")]"
            count += ch == "," and depth == 0
        assert count == len(own[name][1]), f"{name}: {count} arguments in the integration guide, {len(own[name][1])} declared"
