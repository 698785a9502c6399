"""The red zones themselves: a byte written past an array, by anybody, is found. Here the stray byte comes from
a host copy, so no kernel misbehaves; the switches of a scratch are exercised beside it."""
import ctypes as C

import numpy as np
import pytest

from helpers import DeviceLayer, GuardedDeviceBuffer, check_all_guards, run_ffn_dev
from mimo26f_afd_amd import b1, synth

pytestmark = pytest.mark.gpu


def poke(address: int, value: int) -> None:
    byte = np.array([value], np.uint8)
    assert b1.load().m26s_b1_copy_to_device(address, byte.ctypes.data, 1) == 0


def peek(address: int) -> int:
    byte = np.zeros(1, np.uint8)
    assert b1.load().m26s_b1_copy_to_host(byte.ctypes.data, address, 1) == 0
    return int(byte[0])


def test_a_guarded_buffer_reports_a_byte_written_either_side():
    buf = b1.DeviceBuffer(1000)
    assert isinstance(buf, GuardedDeviceBuffer)
    buf.check()
    for where in (buf.ptr + 1000, buf.ptr - 1, buf.ptr + 1000 + 255, buf.ptr - 256):
        old = peek(where)
        poke(where, 0x00)
        with pytest.raises(AssertionError, match="red zone"):
            buf.check()
        poke(where, old)
        buf.check()
    buf.free()


def test_a_guarded_scratch_reports_a_byte_written_behind_an_internal_array():
    wl = synth.make(1)
    layer = DeviceLayer(wl.pools(wl.touched())).layer
    scratch = b1.Scratch()
    with pytest.raises(b1.B1Error) as e:                      # no call made yet: nothing to read back
        super(type(scratch), scratch).check_guards()             # the library's own answer (the helper's wrapper lets it pass)
    assert e.value.code == 1
    run_ffn_dev(layer, scratch, wl)
    scratch.check_guards()
    for which in ("original_routes", "mid_scales", "y"):
        ptr, size = C.c_void_p(), C.c_size_t()
        assert b1.load().m26s_b1_scratch_view(scratch._h, b1.Scratch.VIEW[which], C.byref(ptr), C.byref(size)) == 0
        behind = ptr.value + ((size.value + 3) & ~3)          # the first byte behind the array's last word
        old = peek(behind)
        assert old == 0xA5
        poke(behind, 0x5A)
        with pytest.raises(b1.B1Error, match="red zone") as e:
            scratch.check_guards()
        assert e.value.code == 4
        poke(behind, old)
        scratch.check_guards()
    check_all_guards()


def test_scratch_switches():
    wl = synth.make(1)
    layer = DeviceLayer(wl.pools(wl.touched())).layer
    scratch = b1.Scratch()
    assert b1.load().m26s_b1_scratch_set_option(scratch._h, 99, 1) == 1 and b1.load().m26s_b1_scratch_set_option(None, 0, 1) == 1
    stats, bf, _ = run_ffn_dev(layer, scratch, wl, want_partial=False)
    assert stats.phase_ms[0] > 0 and stats.phase_ms[2] > 0
    scratch.set_option("scope_timing", True)                   # FC1 + FC2 as one interval, the gate's scope
    scoped, bf2, _ = run_ffn_dev(layer, scratch, wl, want_partial=False)
    assert scoped.phase_ms[2] == 0 and scoped.phase_ms[0] > 0.7 * (stats.phase_ms[0] + stats.phase_ms[2]) - 0.01
    assert np.array_equal(bf, bf2)
    scratch.set_option("guards", False)                         # back to the plain layout: a fresh slab, same results
    _, bf3, _ = run_ffn_dev(layer, scratch, wl, want_partial=False)
    assert np.array_equal(bf, bf3)
    with pytest.raises(b1.B1Error):
        super(type(scratch), scratch).check_guards()
    free, total = b1.device_memory()
    assert 0 < free <= total
