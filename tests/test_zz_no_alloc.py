"""The entry point that allocates nothing (m26s_b1_ffn_static): its workspace is a fixed array inside the
library's device image. Checked against the allocating entry it is a variant of (m26s_b1_ffn_dev), bit for
bit, on two calls in a row, the second smaller than the first, so that whatever the first call left in the
shared array would show; then its limits and its status words."""
import numpy as np
import pytest

from helpers import DeviceLayer
from mimo26f_afd_amd import b1, synth

pytestmark = pytest.mark.gpu


def device_inputs(wl):
    return [b1.DeviceBuffer.from_host(a) for a in (wl.payload, wl.scales, wl.ids, wl.weights)]


def run_static(layer, wl, ids=None):
    bufs = device_inputs(wl)
    if ids is not None:
        bufs[2] = b1.DeviceBuffer.from_host(ids)
    fill = np.full(wl.rows * 4096, 0x5A5A, np.uint16)
    out, status = b1.DeviceBuffer.from_host(fill), b1.DeviceBuffer.from_host(np.full(8, 0xDEAD, np.uint32))
    b1.ffn_static(layer, bufs[0].ptr, 4096, bufs[1].ptr, 128, bufs[2].ptr, bufs[3].ptr, wl.rows, out.ptr, status.ptr)
    # the call only launches (on the default stream here); these copies are synchronous on that stream
    return out.to_host(np.uint16).reshape(wl.rows, 4096), status.to_host(np.uint32)


def run_dev(layer, scratch, wl):
    bufs = device_inputs(wl)
    out = b1.DeviceBuffer(wl.rows * 4096 * 2)
    stats = b1.ffn_dev(layer, scratch, bufs[0].ptr, 4096, bufs[1].ptr, 128, bufs[2].ptr, bufs[3].ptr, wl.rows, out.ptr)
    return out.to_host(np.uint16).reshape(wl.rows, 4096), stats


def test_static_workspace_call_equals_the_allocating_call():
    wl = synth.make(2)                                               # 128 tokens, 256 experts x I 2048: the entry's largest call
    layer = DeviceLayer(wl.pools(wl.touched())).layer
    pick = np.arange(37) * 3 % wl.rows                               # then 37 tokens: the one-tile-pair schedule, fewer groups
    small = synth.Workload("small", 2, wl.seed, 4, len(pick), wl.ids[pick], wl.weights[pick], wl.x[pick], wl.payload[pick], wl.scales[pick])
    tiny = synth.Workload("tiny", 2, wl.seed, 4, 5, wl.ids[:5], wl.weights[:5], wl.x[:5], wl.payload[:5], wl.scales[:5])
    scratch = b1.Scratch()
    for w_ in (wl, small, tiny, wl):                                 # two calls in a row, the second smaller; then smaller still, then large again
        got, status = run_static(layer, w_)
        want, stats = run_dev(layer, scratch, w_)
        assert np.array_equal(got, want), w_.name
        assert status[0] == stats.groups and status[2] > 0 and not status[[1, 3, 4, 6, 7]].any() and status[5] == 0xFFFFFFFF, status


def test_static_workspace_call_allocates_nothing():
    """The GPU's free memory reads the same before and after calls of the entry, the first call on this GPU
    included when this test runs alone (the workspace is part of the loaded code object, not an allocation),
    and the array needs no initialising call: its constants are rewritten by every call's first kernel."""
    wl = synth.make(2)
    layer = DeviceLayer(wl.pools(wl.touched())).layer
    bufs = device_inputs(wl)
    out, status = b1.DeviceBuffer(wl.rows * 4096 * 2), b1.DeviceBuffer(32)
    out.to_host(np.uint16)                                           # the library is loaded and the device initialised by now
    free_before = b1.device_memory()[0]
    for rows in (wl.rows, 16):
        b1.ffn_static(layer, bufs[0].ptr, 4096, bufs[1].ptr, 128, bufs[2].ptr, bufs[3].ptr, rows, out.ptr, status.ptr)
        assert b1.device_memory()[0] == free_before
    words = status.to_host(np.uint32)
    assert words[0] > 0 and not words[[1, 3, 4, 6, 7]].any()
    assert b1.device_memory()[0] == free_before


def test_static_workspace_limits_and_status_words():
    wl = synth.make(2)
    layer = DeviceLayer(wl.pools(wl.touched())).layer
    big = synth.make(3, rows=129)
    bufs = device_inputs(big)
    out = b1.DeviceBuffer(big.rows * 4096 * 2)
    with pytest.raises(b1.B1Error, match="129 rows exceed the 128 rows") as e:
        b1.ffn_static(layer, bufs[0].ptr, 4096, bufs[1].ptr, 128, bufs[2].ptr, bufs[3].ptr, big.rows, out.ptr)
    assert e.value.code == 1
    with pytest.raises(b1.B1Error, match="bad rows/handles/pitch"):
        b1.ffn_static(layer, bufs[0].ptr, 4096, bufs[1].ptr, 128, bufs[2].ptr, bufs[3].ptr, 0, out.ptr)
    with pytest.raises(b1.B1Error, match="bad rows/handles/pitch"):
        b1.ffn_static(layer, bufs[0].ptr + 8, 4096, bufs[1].ptr, 128, bufs[2].ptr, bufs[3].ptr, 16, out.ptr)
    ids = wl.ids.copy()
    ids[7, 5] = ids[7, 4]                                            # an expert twice in one token
    got, status = run_static(layer, wl, ids)
    assert status[1] == 7 and status[0] == 0 and (got == 0x5A5A).all()   # plan rejected (metadata), nothing computed
    got, status = run_static(layer, wl)                              # and the next call is clean
    assert status[1] == 0 and status[0] > 0 and not (got == 0x5A5A).all()
