"""Shared pieces of the GPU parity tests: device staging through the library's own helpers and the
parity metrics the benchmark contract states."""
from __future__ import annotations

import weakref

import numpy as np

from mimo26f_afd_amd import b1, synth

# ---- red zones (the reference guards every device buffer of its tests and checks the guards after every run:
# crates/mimo26-expert/tests/b1_core/primitive.cu:23-40, bench_connected.cuh:62) ---------------------------
GUARD_BYTES, GUARD_FILL = 256, 0xA5
_PlainDeviceBuffer, _PlainScratch = b1.DeviceBuffer, b1.Scratch


class GuardedDeviceBuffer(_PlainDeviceBuffer):
    """A device buffer with 256 bytes of 0xa5 either side (256 keeps the alignment the plain allocation has).
    check() reads both zones back; free() checks first."""
    live = weakref.WeakSet()

    def __init__(self, nbytes: int):
        super().__init__(int(nbytes) + 2 * GUARD_BYTES)
        self._base, self.ptr, self.nbytes = self.ptr, self.ptr + GUARD_BYTES, int(nbytes)
        zone = np.full(GUARD_BYTES, GUARD_FILL, np.uint8)
        for at in (self._base, self.ptr + self.nbytes):
            if b1.load().m26s_b1_copy_to_device(at, zone.ctypes.data, GUARD_BYTES):
                raise b1.B1Error(2, "b1: guard upload failed")
        GuardedDeviceBuffer.live.add(self)

    def check(self) -> None:
        if not getattr(self, "_base", None):
            return
        zone = np.empty(GUARD_BYTES, np.uint8)
        for name, at in (("front", self._base), ("back", self.ptr + self.nbytes)):
            if b1.load().m26s_b1_copy_to_host(zone.ctypes.data, at, GUARD_BYTES):
                raise b1.B1Error(2, "b1: guard download failed")
            hit = np.flatnonzero(zone != GUARD_FILL)
            assert hit.size == 0, f"{name} red zone of a {self.nbytes}-byte device buffer written at byte {int(hit[0])}"

    def free(self) -> None:
        if getattr(self, "_base", None) and b1.load is not None:
            try:
                self.check()
            finally:
                b1.load().m26s_b1_device_free(self._base)
                self._base = self.ptr = None

    __del__ = free


class GuardedScratch(_PlainScratch):
    """A scratch whose internal arrays lie between red zones (the library's own test switch)."""
    live = weakref.WeakSet()

    def __init__(self, stream=None):
        super().__init__(stream)
        self.set_option("guards", True)
        GuardedScratch.live.add(self)

    def check_guards(self) -> None:
        try:
            super().check_guards()
        except b1.B1Error as e:
            if e.code != 1:  # 1: no call made on it yet
                raise


def install_guards() -> None:
    """Every DeviceBuffer and Scratch made from here on, by the tests or by the package's own host code, is guarded."""
    b1.DeviceBuffer, b1.Scratch = GuardedDeviceBuffer, GuardedScratch


def check_all_guards() -> None:
    for s in list(GuardedScratch.live):
        if getattr(s, "_h", None) and s._h.value:
            s.check_guards()
    for buf in list(GuardedDeviceBuffer.live):
        buf.check()


def bf16_to_f32(bits: np.ndarray) -> np.ndarray:
    return (bits.astype(np.uint32) << 16).view(np.float32)


def parity(got: np.ndarray, ref: np.ndarray):
    """(max-abs error / max|ref|, mean relative error) as the north star defines them."""
    got = got.astype(np.float64)
    ref = ref.astype(np.float64)
    scale = np.max(np.abs(ref))
    max_abs = np.max(np.abs(got - ref)) / scale
    mean_rel = np.sum(np.abs(got - ref)) / np.sum(np.abs(ref))
    return max_abs, mean_rel


class DeviceLayer:
    """Uploads canonical rank pools, prepares a layer, frees the canonical copies."""

    def __init__(self, pools):
        bufs = [b1.DeviceBuffer.from_host(p) for p in pools]
        if len(bufs) == 1:
            self.layer = b1.Layer(bufs[0].ptr, bufs[0].nbytes, 0)
        else:
            self.layer = b1.Layer.full([b.ptr for b in bufs], bufs[0].nbytes)
        for b in bufs:
            b.free()


def run_ffn_dev(layer: b1.Layer, scratch: b1.Scratch, wl: synth.Workload, want_partial=True):
    """Device-resident call; returns (stats, bf16 bits [rows,4096], fp32 partial or None)."""
    dp = b1.DeviceBuffer.from_host(wl.payload)
    ds = b1.DeviceBuffer.from_host(wl.scales)
    di = b1.DeviceBuffer.from_host(wl.ids)
    dw = b1.DeviceBuffer.from_host(wl.weights)
    out = b1.DeviceBuffer(wl.rows * 4096 * 2)
    part = b1.DeviceBuffer(wl.rows * 4096 * 4) if want_partial else None
    stats = b1.ffn_dev(layer, scratch, dp.ptr, 4096, ds.ptr, 128, di.ptr, dw.ptr, wl.rows, out.ptr,
                       part.ptr if part else None)
    bf = out.to_host(np.uint16).reshape(wl.rows, 4096)
    pf = part.to_host(np.float32).reshape(wl.rows, 4096) if part else None
    check_all_guards()  # after every run, like the reference's gate: inputs, outputs and the scratch's own arrays
    return stats, bf, pf


def stack_reference_rows(seed: int, layer: int, payload: np.ndarray, scales: np.ndarray, ids: np.ndarray,
                         weights: np.ndarray):
    """The CPU rule's BF16 rows for a few tokens of one layer of the resident stack, with that layer's
    touched experts regenerated on the host from the stack's seeded streams."""
    import b1_oracle as O
    touched = np.unique(ids)
    pools = []
    for r in range(4):
        pool = np.full(synth.EXPERTS * synth.IMAGE_BYTES, 0x22, np.uint8)
        for e in touched:
            pool[e * synth.IMAGE_BYTES:(e + 1) * synth.IMAGE_BYTES] = synth.expert_image(seed, r, int(e), layer)
        pools.append(pool)
    rc, _, bits, _ = O.layer_ffn(pools, payload, scales, ids, weights)
    return rc, bits
