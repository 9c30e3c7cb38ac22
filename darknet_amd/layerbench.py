"""Single-layer timing of the convolution kernel through the C-ABI:
``python -m darknet_amd.layerbench --c 256 --hw 26 --n 512 --size 3 --stride 1 --batch 64``.

Times ``forward_convolutional_gpu`` (packed weights prepared once, as a network does at load
time) with HIP events on the library's stream and prints achieved TFLOP/s against the fp32
MFMA peak and the algorithmic GB/s.  ``--sweep`` runs the three single-layer shapes of the
benchmark configurations at batch 1 and 64.
"""
from __future__ import annotations

import argparse
import json

import numpy as np

from . import api, cfgs, synth
from . import lib as _lib

PEAK = 157.3


def time_layer(batch, c, h, w, n, size, stride, pad=None, groups=1, bn=1, act=7, iters=20, warmup=3,
               data="random"):
    L = _lib.load()
    if pad is None:
        pad = size // 2
    oh = (h + 2 * pad - size) // stride + 1
    ow = (w + 2 * pad - size) // stride + 1
    xh = synth.uniform(1, batch * c * h * w)
    wh = synth.conv_weights(2, n, c // groups, size)
    if data == "zeros":          # same instruction stream, no operand bits toggling: shows what the
        xh[:] = 0                # part's clock management costs on real data
        wh[:] = 0
    x = api.DeviceArray(xh)
    wt = api.DeviceArray(wh)
    b, s, m, v = [api.DeviceArray(a) for a in synth.bn_random(3, n)]
    out = api.DeviceArray(n=batch * n * oh * ow)
    pf = L.conv_packed_floats(n, c, groups, size)
    packed = api.DeviceArray(n=pf) if pf else None
    if packed:
        L.conv_pack_weights_gpu(wt.ptr, packed.ptr, n, c, groups, size)

    def run():
        L.forward_convolutional_gpu(x.ptr, wt.ptr, packed.ptr if packed else None, b.ptr, s.ptr, m.ptr,
                                    v.ptr, out.ptr, batch, c, h, w, n, groups, size, stride, pad, bn, act)

    for _ in range(warmup):
        run()
    L.hip_synchronize()
    e0, e1 = L.hip_event_create(), L.hip_event_create()
    L.hip_event_record(e0)
    for _ in range(iters):
        run()
    L.hip_event_record(e1)
    ms = L.hip_event_elapsed_ms(e0, e1) / iters
    flops = 2.0 * n * size * size * (c // groups) * oh * ow * batch
    byts = 4.0 * (batch * c * h * w + batch * n * oh * ow + n * (c // groups) * size * size)
    return {"batch": batch, "shape": f"{size}x{size}/{stride} {c}->{n} @{w}x{h} g{groups}",
            "kernel": L.conv_kernel_name_geometry(batch, c, h, w, n, groups, size, stride, pad).decode(), "ms": round(ms, 4),
            "tflops": round(flops / ms / 1e9, 2), "frac_of_fp32_mfma_peak": round(flops / ms / 1e9 / PEAK, 4),
            "algorithmic_gbs": round(byts / ms / 1e6, 1)}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--batch", type=int, default=64)
    ap.add_argument("--c", type=int, default=256)
    ap.add_argument("--hw", type=int, default=26)
    ap.add_argument("--n", type=int, default=512)
    ap.add_argument("--size", type=int, default=3)
    ap.add_argument("--stride", type=int, default=1)
    ap.add_argument("--groups", type=int, default=1)
    ap.add_argument("--iters", type=int, default=20)
    ap.add_argument("--sweep", action="store_true")
    ap.add_argument("--algo", type=int, default=0)
    ap.add_argument("--data", default="random", choices=["random", "zeros"])
    ap.add_argument("--precision", default="fp32", choices=["fp32", "bf16", "bf16x3"])
    a = ap.parse_args()
    api.set_gpu(0)
    _lib.load().conv_set_algo(a.algo)
    _lib.load().conv_set_precision({"fp32": 0, "bf16": 1, "bf16x3": 2}[a.precision])
    if a.sweep:
        for name, (c, h, w, n, size, stride) in cfgs.SWEEP.items():
            for batch in (1, 64):
                r = time_layer(batch, c, h, w, n, size, stride, pad=size // 2 if size > 1 else 0, iters=a.iters)
                r["name"] = name
                print(json.dumps(r), flush=True)
    else:
        print(json.dumps(time_layer(a.batch, a.c, a.hw, a.hw, a.n, a.size, a.stride,
                                    pad=a.size // 2 if a.size > 1 else 0, groups=a.groups, iters=a.iters,
                                    data=a.data)),
              flush=True)


if __name__ == "__main__":
    main()
