"""The allocation-free convolution entry point against the ordinary one, through the C-ABI.

`forward_convolutional_noalloc_gpu` shares the kernels of `forward_convolutional_gpu` and keeps
its K-split accumulators in a fixed device array instead of a buffer grown with hipMalloc, so the
two must agree bit for bit.  Two calls in a row share that array, the second with a smaller input:
nothing the first call left behind may leak into the second result.  The shapes are batch-1 layers
of yolov3 whose tiles are cut along K (that is what uses the array), plus one without a K-split.
The free-memory reading of the device must not move across the calls (no allocation)."""
import ctypes as C

import numpy as np
import pytest

from darknet_amd import api, synth
from oracle.cpu import ACTIVATIONS

from util import REL_TOL, norm_err

pytestmark = pytest.mark.gpu
D = api.DeviceArray


class Case:
    def __init__(self, dn, seed, b, c, h, w, n, size, stride, pad, act="leaky", bn=1):
        self.dn = dn
        self.geom = (b, c, h, w, n, 1, size, stride, pad, bn, ACTIVATIONS.index(act))
        self.act, self.bn = act, bn
        self.x = synth.uniform(seed, b * c * h * w).reshape(b, c, h, w)
        self.wt = synth.conv_weights(seed + 1, n, c, size)
        self.bias, self.sc, self.mu, self.var = synth.bn_random(seed + 2, n)
        self.oh = (h + 2 * pad - size) // stride + 1
        self.ow = (w + 2 * pad - size) // stride + 1
        self.dev = [D(a) for a in (self.x, self.wt, self.bias, self.sc, self.mu, self.var)]
        self.packed = D(n=dn.conv_packed_floats(n, c, 1, size))
        dn.conv_pack_weights_gpu(self.dev[1].ptr, self.packed.ptr, n, c, 1, size)
        # poisoned outputs: every element must be written by the call under test
        self.out_a = D(np.full(b * n * self.oh * self.ow, np.nan, np.float32))
        self.out_b = D(np.full(b * n * self.oh * self.ow, np.nan, np.float32))

    def args(self, out, packed=True):
        d = self.dev
        return ([d[0].ptr, d[1].ptr, self.packed.ptr if packed else None, d[2].ptr, d[3].ptr, d[4].ptr, d[5].ptr,
                 out.ptr] + list(self.geom))

    def shape(self):
        b, _, _, _, n = self.geom[:5]
        return (b, n, self.oh, self.ow)


def free_bytes():
    hip = C.CDLL("libamdhip64.so")
    free, total = C.c_size_t(), C.c_size_t()
    assert hip.hipMemGetInfo(C.byref(free), C.byref(total)) == 0
    return free.value


def test_noalloc_matches_allocating_entry_point(dn, orc):
    big = Case(dn, 11, 1, 256, 26, 26, 512, 3, 1, 1)      # 3x3 256->512 @26, batch 1: K-split tail
    small = Case(dn, 21, 1, 512, 13, 13, 255, 1, 1, 0, act="linear", bn=0)  # smaller, ragged M
    whole = Case(dn, 31, 2, 16, 9, 9, 48, 3, 1, 1)        # a grid without K-split
    # reference results from the existing entry point (this may allocate; it runs first)
    for cs in (big, small, whole):
        dn.forward_convolutional_gpu(*cs.args(cs.out_a))
    dn.hip_synchronize()
    before = free_bytes()
    # two calls in a row through the allocation-free entry point, the second one smaller
    assert dn.forward_convolutional_noalloc_gpu(*big.args(big.out_b)) == 0
    assert dn.forward_convolutional_noalloc_gpu(*small.args(small.out_b)) == 0
    assert dn.forward_convolutional_noalloc_gpu(*whole.args(whole.out_b)) == 0
    dn.hip_synchronize()
    assert free_bytes() == before, "the allocation-free entry point changed the device's free memory"
    for cs in (big, small, whole):
        got, want = cs.out_b.numpy(cs.shape()), cs.out_a.numpy(cs.shape())
        assert not np.isnan(got).any()
        assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
    # and the shared result is the checker's, to the convolution bar
    ref = orc.conv(big.x, big.wt, big.bias, big.sc, big.mu, big.var, n=512, size=3, stride=1, pad=1, groups=1,
                   batch_normalize=1, activation="leaky")
    assert norm_err(big.out_b.numpy(big.shape()), ref) <= REL_TOL
    # the same pair again in the opposite order: the array keeps the last call's contents
    small.out_b = D(np.full(small.out_b.n, np.nan, np.float32))
    big.out_b = D(np.full(big.out_b.n, np.nan, np.float32))
    assert dn.forward_convolutional_noalloc_gpu(*small.args(small.out_b)) == 0
    assert dn.forward_convolutional_noalloc_gpu(*big.args(big.out_b)) == 0
    for cs in (big, small):
        assert np.array_equal(cs.out_b.numpy(cs.shape()).view(np.uint32), cs.out_a.numpy(cs.shape()).view(np.uint32))


def test_noalloc_refuses_what_would_allocate(dn, capfd):
    cs = Case(dn, 41, 1, 32, 8, 8, 64, 3, 1, 1)
    sentinel = np.full(cs.out_b.n, 7.0, np.float32)
    cs.out_b = D(sentinel)
    # without the packed copy the call would have to allocate a repack buffer: refused, nothing launched
    assert dn.forward_convolutional_noalloc_gpu(*cs.args(cs.out_b, packed=False)) == -1
    dn.hip_synchronize()
    assert "packed" in capfd.readouterr().err
    assert np.array_equal(cs.out_b.numpy((cs.out_b.n,)), sentinel)
    # and the entry point keeps working afterwards
    assert dn.forward_convolutional_noalloc_gpu(*cs.args(cs.out_b)) == 0
    dn.forward_convolutional_gpu(*cs.args(cs.out_a))
    assert np.array_equal(cs.out_b.numpy(cs.shape()).view(np.uint32), cs.out_a.numpy(cs.shape()).view(np.uint32))


def test_noalloc_refusals_decided_on_the_host(dn, capfd):
    """A K-split that needs more than the fixed array, and the bf16 staging mode on a 3x3 layer: both
    are refused before anything is launched, and a timing pair armed for the refused call does not
    stay armed for the next one."""
    cs = Case(dn, 51, 1, 128, 52, 52, 256, 3, 1, 1)       # 86 tiles of 128x64 at batch 1: all of them tail
    sentinel = np.full(cs.out_b.n, 5.0, np.float32)
    cs.out_b = D(sentinel)
    e0, e1 = dn.hip_event_create(), dn.hip_event_create()
    dn.conv_set_ksplit(32, 64)                            # 86 tiles x 32 slices x 128x64 floats = 90 MB > 64 MiB
    try:
        dn.conv_profile_next(e0, e1)
        assert dn.forward_convolutional_noalloc_gpu(*cs.args(cs.out_b)) == -1
    finally:
        dn.conv_set_ksplit(0, 0)
    assert "scratch" in capfd.readouterr().err
    assert dn.conv_profile_pending() == 0
    dn.conv_set_precision(1)
    try:
        assert dn.forward_convolutional_noalloc_gpu(*cs.args(cs.out_b)) == -1
    finally:
        dn.conv_set_precision(0)
    assert "bf16" in capfd.readouterr().err
    dn.hip_synchronize()
    assert np.array_equal(cs.out_b.numpy((cs.out_b.n,)), sentinel)
    dn.hip_event_destroy(e0)
    dn.hip_event_destroy(e1)
    # the same layer under the library's own choice of split fits and agrees with the allocating entry
    assert dn.forward_convolutional_noalloc_gpu(*cs.args(cs.out_b)) == 0
    dn.forward_convolutional_gpu(*cs.args(cs.out_a))
    assert np.array_equal(cs.out_b.numpy(cs.shape()).view(np.uint32), cs.out_a.numpy(cs.shape()).view(np.uint32))
