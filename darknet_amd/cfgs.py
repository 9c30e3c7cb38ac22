"""Generators for the network descriptions (cfg text) the benchmark configurations name.

The cfg grammar is the reference's (``[section]`` lines followed by ``key=value`` lines,
src/parser.c:891-924); the text produced here parses to the same layer table as the
reference's own ``cfg/yolov3-tiny.cfg``, ``cfg/yolov3.cfg`` and ``cfg/resnext50.cfg`` with the
``[net]`` edits those configurations require (``batch=N subdivisions=1``, ``width/height``).
tests/test_oracle_cfg.py checks that equivalence layer by layer where the reference tree is
present.  Batch size is fixed at parse time (src/parser.c:657-666), hence the ``batch`` argument.
"""
from __future__ import annotations


def _net(batch: int, width: int, height: int, channels: int = 3) -> str:
    return (f"[net]\nbatch={batch}\nsubdivisions=1\nwidth={width}\nheight={height}\n"
            f"channels={channels}\n")


def _conv(filters: int, size: int, stride: int = 1, bn: bool = True, act: str = "leaky",
          groups: int = 1, extra: str = "") -> str:
    s = "[convolutional]\n"
    if bn:
        s += "batch_normalize=1\n"
    s += f"filters={filters}\nsize={size}\nstride={stride}\npad=1\n"
    if groups != 1:
        s += f"groups={groups}\n"
    s += f"activation={act}\n{extra}"
    return s


def _yolo(mask, anchors, classes: int = 80) -> str:
    num = len(anchors) // 2
    return ("[yolo]\nmask=" + ",".join(map(str, mask)) + "\nanchors=" +
            ",".join(map(str, anchors)) + f"\nclasses={classes}\nnum={num}\n")


TINY_ANCHORS = [10, 14, 23, 27, 37, 58, 81, 82, 135, 169, 344, 319]
V3_ANCHORS = [10, 13, 16, 30, 33, 23, 30, 61, 62, 45, 59, 119, 116, 90, 156, 198, 373, 326]


def yolov3_tiny(batch: int = 1, size: int = 416, xnor: bool = False,
                xnor_skip=(0, 22)) -> str:
    """13 conv / 6 maxpool / upsample / 2 route / 2 yolo.  With ``xnor`` every conv except the
    layer indices in ``xnor_skip`` carries ``binary=1 xnor=1`` (src/parser.c:199-200)."""
    out = [_net(batch, size, size)]
    idx = [0]

    def conv(*a, **k):
        extra = "binary=1\nxnor=1\n" if (xnor and idx[0] not in xnor_skip) else ""
        out.append(_conv(*a, extra=extra, **k))
        idx[0] += 1

    def other(text):
        out.append(text)
        idx[0] += 1

    for i, f in enumerate([16, 32, 64, 128, 256, 512]):
        conv(f, 3)
        other(f"[maxpool]\nsize=2\nstride={2 if i < 5 else 1}\n")
    conv(1024, 3)
    conv(256, 1)
    conv(512, 3)
    conv(255, 1, bn=False, act="linear")
    other(_yolo([3, 4, 5], TINY_ANCHORS))
    other("[route]\nlayers=-4\n")
    conv(128, 1)
    other("[upsample]\nstride=2\n")
    other("[route]\nlayers=-1,8\n")
    conv(256, 3)
    conv(255, 1, bn=False, act="linear")
    other(_yolo([0, 1, 2], TINY_ANCHORS))
    return "\n".join(out)


def yolov3(batch: int = 1, size: int = 416) -> str:
    """darknet53 backbone + 3-scale head: 75 conv, 23 shortcut, 2 upsample, 4 route, 3 yolo."""
    out = [_net(batch, size, size), _conv(32, 3)]

    def stage(filters: int, blocks: int):
        out.append(_conv(filters, 3, stride=2))
        for _ in range(blocks):
            out.append(_conv(filters // 2, 1))
            out.append(_conv(filters, 3))
            out.append("[shortcut]\nfrom=-3\nactivation=linear\n")

    for f, nb in [(64, 1), (128, 2), (256, 8), (512, 8), (1024, 4)]:
        stage(f, nb)

    def head(filters: int, mask):
        for _ in range(3):
            out.append(_conv(filters, 1))
            out.append(_conv(filters * 2, 3))
        out.append(_conv(255, 1, bn=False, act="linear"))
        out.append(_yolo(mask, V3_ANCHORS))

    head(512, [6, 7, 8])
    out.append("[route]\nlayers=-4\n")
    out.append(_conv(256, 1))
    out.append("[upsample]\nstride=2\n")
    out.append("[route]\nlayers=-1,61\n")
    head(256, [3, 4, 5])
    out.append("[route]\nlayers=-4\n")
    out.append(_conv(128, 1))
    out.append("[upsample]\nstride=2\n")
    out.append("[route]\nlayers=-1,36\n")
    head(128, [0, 1, 2])
    return "\n".join(out)


def resnext50(batch: int = 1, size: int = 224) -> str:
    """ResNeXt-50 32x4d classifier: 7x7/2 stem, maxpool, 16 grouped bottlenecks with shortcuts,
    global avgpool, a 1x1 conv as 1000-way classifier, softmax."""
    out = [_net(batch, size, size), _conv(64, 7, stride=2), "[maxpool]\nsize=2\nstride=2\n"]
    for width, blocks, first_stride in [(128, 3, 1), (256, 4, 2), (512, 6, 2), (1024, 3, 2)]:
        for b in range(blocks):
            out.append(_conv(width, 1))
            out.append(_conv(width, 3, stride=first_stride if b == 0 else 1, groups=32))
            out.append(_conv(width * 2, 1, act="linear"))
            out.append("[shortcut]\nfrom=-4\nactivation=leaky\n")
    out.append("[avgpool]\n")
    out.append(_conv(1000, 1, bn=False, act="linear"))
    out.append("[softmax]\ngroups=1\n")
    return "\n".join(out)


def single_conv(batch: int, c: int, h: int, w: int, filters: int, size: int, stride: int,
                pad: int = 1, groups: int = 1, bn: bool = True, act: str = "leaky",
                xnor: bool = False) -> str:
    """A one-layer network, for the single-layer sweep."""
    s = f"[net]\nbatch={batch}\nsubdivisions=1\nwidth={w}\nheight={h}\nchannels={c}\n\n[convolutional]\n"
    if bn:
        s += "batch_normalize=1\n"
    s += f"filters={filters}\nsize={size}\nstride={stride}\npad={pad}\n"
    if groups != 1:
        s += f"groups={groups}\n"
    if xnor:
        s += "binary=1\nxnor=1\n"
    s += f"activation={act}\n"
    return s


# The single-layer sweep of the benchmark configurations: name -> (c, h, w, filters, size, stride)
SWEEP = {
    "3x3s1_256to512_26": (256, 26, 26, 512, 3, 1),
    "1x1_512to256_52": (512, 52, 52, 256, 1, 1),
    "3x3s2_128to256_104": (128, 104, 104, 256, 3, 2),
}


def _detection(num: int, side: int = 7, classes: int = 20) -> str:
    return (f"[detection]\nclasses={classes}\ncoords=4\nrescore=1\nside={side}\nnum={num}\nsoftmax=0\nsqrt=1\n"
            "jitter=.2\nobject_scale=1\nnoobject_scale=.5\nclass_scale=1\ncoord_scale=5\n")


def yolov1_tiny(batch: int = 1, size: int = 448) -> str:
    """cfg/yolov1-tiny.cfg: 8 conv / 6 maxpool, a connected layer onto the 7x7x(2*5+20) grid, detection.
    The connected layer fixes the input size: side * 64 pixels."""
    out = [_net(batch, size, size)]
    for f in [16, 32, 64, 128, 256, 512]:
        out.append(_conv(f, 3))
        out.append("[maxpool]\nsize=2\nstride=2\n")
    out.append(_conv(1024, 3))
    out.append(_conv(256, 3))
    out.append("[connected]\noutput=1470\nactivation=linear\n")
    out.append(_detection(2))
    return "\n".join(out)


def yolov1(batch: int = 1, size: int = 448) -> str:
    """cfg/yolov1.cfg: 24 conv / 4 maxpool, the locally connected layer on the 7x7x1024 map,
    dropout, a connected layer onto the 7x7x(3*5+20) grid, detection."""
    out = [_net(batch, size, size)]
    pool = "[maxpool]\nsize=2\nstride=2\n"
    out += [_conv(64, 7, 2), pool, _conv(192, 3), pool,
            _conv(128, 1), _conv(256, 3), _conv(256, 1), _conv(512, 3), pool]
    for _ in range(4):
        out += [_conv(256, 1), _conv(512, 3)]
    out += [_conv(512, 1), _conv(1024, 3), pool]
    for _ in range(2):
        out += [_conv(512, 1), _conv(1024, 3)]
    out += [_conv(1024, 3), _conv(1024, 3, 2), _conv(1024, 3), _conv(1024, 3)]
    out.append("[local]\nsize=3\nstride=1\npad=1\nfilters=256\nactivation=leaky\n")
    out.append("[dropout]\nprobability=.5\n")
    out.append("[connected]\noutput=1715\nactivation=linear\n")
    out.append(_detection(3))
    return "\n".join(out)
