"""Host side of the B1 path: the mirror of the reference's Rust wrapper.

Same names, argument meaning and error behaviour as crates/mimo26-spark/src/b1.rs (Layer:63-91,
Scratch:94-118, FfnStats:120-129, ffn:131-152, ffn_strided:154-176): a failing call raises
B1Error carrying the library's message where the Rust side returns Err(String). Arrays are numpy
on the host; the *_dev variants take raw device addresses (for example torch tensor data_ptr()).
"""
from __future__ import annotations

import ctypes as C
from dataclasses import dataclass, field

import numpy as np

from ._lib import load

HIDDEN = 4096
EXPERTS = 256
QUARTER_SLICE_BYTES = 3342336
ERRLEN = 256  # b1.rs:75,199


class B1Error(RuntimeError):
    def __init__(self, code: int, message: str):
        super().__init__(message)
        self.code = code


def _err():
    return C.create_string_buffer(ERRLEN)


def _raise(rc: int, buf) -> None:
    if rc != 0:
        raise B1Error(rc, buf.value.decode("utf-8", "replace"))


@dataclass
class FfnStats:
    """b1.rs:120-129."""
    upload_plan_ms: float = 0.0
    gpu_ms: float = 0.0
    tail_ms: float = 0.0
    groups: int = 0
    phase_ms: list = field(default_factory=lambda: [0.0] * 4)  # FC1(+quantizer), quantizer (0), FC2, reduce

    @classmethod
    def from_ms(cls, ms) -> "FfnStats":
        return cls(float(ms[0]), float(ms[1]), float(ms[2]), int(ms[3]), [float(v) for v in ms[4:8]])


class Layer:
    """One MoE layer's prepared pool (256 experts). b1.rs:63-91."""

    def __init__(self, canonical_dev: int, nbytes: int, rank: int):
        self._h = C.c_void_p()
        buf = _err()
        _raise(load().m26s_b1_layer_new(canonical_dev, nbytes, rank, C.byref(self._h), buf, ERRLEN), buf)

    @classmethod
    def full(cls, rank_images_dev, bytes_each: int) -> "Layer":
        """All four TP4 rank pools fused on one GPU (intermediate 2048)."""
        self = cls.__new__(cls)
        self._h = C.c_void_p()
        arr = (C.c_void_p * 4)(*[int(p) for p in rank_images_dev])
        buf = _err()
        _raise(load().m26s_b1_layer_new_full(arr, bytes_each, C.byref(self._h), buf, ERRLEN), buf)
        return self

    def all_scales_normal(self) -> bool:
        return load().m26s_b1_layer_all_normal(self._h) != 0

    @property
    def intermediate(self) -> int:
        return int(load().m26s_b1_layer_intermediate(self._h))

    def prepared_view(self) -> tuple[int, int, int]:
        """(device pointer of the prepared pool, bytes per expert image, layout tag)."""
        ptr, nbytes, tag = C.c_void_p(), C.c_uint64(), C.c_uint32()
        if load().m26s_b1_layer_view(self._h, C.byref(ptr), C.byref(nbytes), C.byref(tag)) != 0:
            raise B1Error(1, "b1 layer view: bad handle")
        return int(ptr.value), int(nbytes.value), int(tag.value)

    def close(self) -> None:
        if getattr(self, "_h", None) and self._h.value and load is not None:  # load is gone at interpreter exit
            load().m26s_b1_layer_free(self._h)
            self._h = C.c_void_p()

    __del__ = close


class Scratch:
    """Per-request device scratch and the B1 stream. b1.rs:94-118."""

    VIEW = dict(inverse=0, original_routes=1, grouped_weights=2, groups=3, meta=4, mid_payload=5, mid_scales=6,
                y=7, gate=8, up=9, h=10, chunks=11, clock=12)

    def __init__(self, stream: int | None = None):
        self._h = C.c_void_p()
        buf = _err()
        if stream is None:
            _raise(load().m26s_b1_scratch_new(C.byref(self._h), buf, ERRLEN), buf)
        else:
            _raise(load().m26s_b1_scratch_new_on(stream, C.byref(self._h), buf, ERRLEN), buf)

    OPTION = dict(taps=0, fused_combine=1, bf16_route_rows=2, guards=3, scope_timing=4)

    def set_taps(self, on: bool) -> None:
        load().m26s_b1_scratch_set_taps(self._h, 1 if on else 0)

    def set_option(self, name: str, on: bool) -> None:
        """Switches for the calls that follow: 'fused_combine' (the combine inside FC2 instead of as a launch of its
        own; same bits, not faster), 'bf16_route_rows' (the reference's opt-in MIMO26_B1_Y=bf16 numerical mode),
        'guards' (red zones around every internal array, read back by check_guards), 'scope_timing' (the timed
        entries report FC1 + FC2 as one interval in phase_ms[0]), 'taps'."""
        rc = load().m26s_b1_scratch_set_option(self._h, self.OPTION[name], 1 if on else 0)
        if rc:
            raise B1Error(rc, f"b1 scratch: option {name} refused")

    def check_guards(self) -> None:
        """Waits for the stream and raises when a red zone of the last call's workspace was written to."""
        buf = _err()
        _raise(load().m26s_b1_scratch_check_guards(self._h, buf, ERRLEN), buf)

    @property
    def stream(self) -> int:
        """The HIP stream the scratch launches on (0 for the default stream)."""
        return int(load().m26s_b1_scratch_stream(self._h) or 0)

    def sync(self) -> None:
        buf = _err()
        _raise(load().m26s_b1_scratch_sync(self._h, buf, ERRLEN), buf)

    def view(self, name: str, dtype, count: int) -> np.ndarray:
        """Copy `count` items of an internal device buffer to the host."""
        ptr, size = C.c_void_p(), C.c_size_t()
        if load().m26s_b1_scratch_view(self._h, self.VIEW[name], C.byref(ptr), C.byref(size)):
            raise B1Error(1, f"b1 scratch: no buffer {name}")
        out = np.empty(count, dtype)
        if out.nbytes > size.value:
            raise B1Error(1, f"b1 scratch: {name} holds {size.value} bytes, asked for {out.nbytes}")
        if out.nbytes and load().m26s_b1_copy_to_host(out.ctypes.data, ptr, out.nbytes):
            raise B1Error(2, "b1 scratch: copy failed")
        return out

    def close(self) -> None:
        if getattr(self, "_h", None) and self._h.value and load is not None:
            load().m26s_b1_scratch_free(self._h)
            self._h = C.c_void_p()

    __del__ = close


def _ffn_raw(layer, scratch, payload_ptr, payload_pitch, scales_ptr, scales_pitch, ids, weights, rows, bf16_out):
    if rows == 0 or ids.size != rows * 8 or weights.size != rows * 8 or bf16_out.size != rows * HIDDEN:
        raise B1Error(1, f"b1 ffn: extents do not match {rows} rows")
    ms = (C.c_float * 8)()
    buf = _err()
    rc = load().m26s_b1_ffn(layer._h, scratch._h, payload_ptr, payload_pitch, scales_ptr, scales_pitch,
                            ids.ctypes.data, weights.ctypes.data, rows, bf16_out.ctypes.data, ms, buf, ERRLEN)
    _raise(rc, buf)
    return FfnStats.from_ms(ms)


def ffn(layer: Layer, scratch: Scratch, payload: np.ndarray, scales: np.ndarray, ids: np.ndarray,
        weights: np.ndarray, rows: int, bf16_out: np.ndarray) -> FfnStats:
    """One rank's FFN for `rows` tokens on host arrays. b1.rs:131-152."""
    payload = np.ascontiguousarray(payload, np.uint8)
    scales = np.ascontiguousarray(scales, np.uint8)
    ids = np.ascontiguousarray(ids, np.int32)
    weights = np.ascontiguousarray(weights, np.float32)
    if rows == 0 or payload.size != rows * HIDDEN or scales.size != rows * HIDDEN // 32:
        raise B1Error(1, f"b1 ffn: extents do not match {rows} rows")
    assert bf16_out.dtype == np.uint16 and bf16_out.flags.c_contiguous
    return _ffn_raw(layer, scratch, payload.ctypes.data, HIDDEN, scales.ctypes.data, HIDDEN // 32, ids, weights, rows, bf16_out)


def ffn_strided(layer: Layer, scratch: Scratch, hidden: np.ndarray, row_stride: int, ids: np.ndarray,
                weights: np.ndarray, rows: int, bf16_out: np.ndarray) -> FfnStats:
    """ffn on a request frame's interleaved rows (4,096 payload bytes then 128 scales), read in
    place. b1.rs:154-176."""
    hidden = np.ascontiguousarray(hidden, np.uint8).reshape(-1)
    ids = np.ascontiguousarray(ids, np.int32)
    weights = np.ascontiguousarray(weights, np.float32)
    need = HIDDEN + HIDDEN // 32
    if rows == 0 or row_stride < need or hidden.size < (rows - 1) * row_stride + need:
        raise B1Error(1, f"b1 ffn: hidden rows do not match {rows} rows of {row_stride} B")
    assert bf16_out.dtype == np.uint16 and bf16_out.flags.c_contiguous
    base = hidden.ctypes.data
    return _ffn_raw(layer, scratch, base, row_stride, base + HIDDEN, row_stride, ids, weights, rows, bf16_out)


def ffn_dev(layer: Layer, scratch: Scratch, payload_dev: int, payload_pitch: int, scales_dev: int, scales_pitch: int,
            ids_dev: int, weights_dev: int, rows: int, bf16_out_dev: int, partial_dev: int | None = None) -> FfnStats:
    """Device-resident call, synchronous."""
    ms = (C.c_float * 8)()
    buf = _err()
    _raise(load().m26s_b1_ffn_dev(layer._h, scratch._h, payload_dev, payload_pitch, scales_dev, scales_pitch, ids_dev,
                                  weights_dev, rows, bf16_out_dev, partial_dev, ms, buf, ERRLEN), buf)
    return FfnStats.from_ms(ms)


def ffn_enqueue(layer: Layer, scratch: Scratch, payload_dev: int, payload_pitch: int, scales_dev: int,
                scales_pitch: int, ids_dev: int, weights_dev: int, rows: int, bf16_out_dev: int,
                partial_dev: int | None = None) -> None:
    """Device-resident call, launches only; faults surface at Scratch.sync()."""
    buf = _err()
    _raise(load().m26s_b1_ffn_enqueue(layer._h, scratch._h, payload_dev, payload_pitch, scales_dev, scales_pitch,
                                      ids_dev, weights_dev, rows, bf16_out_dev, partial_dev, buf, ERRLEN), buf)


STATIC_MAX_ROWS = 128


def ffn_static(layer: Layer, payload_dev: int, payload_pitch: int, scales_dev: int, scales_pitch: int, ids_dev: int,
               weights_dev: int, rows: int, bf16_out_dev: int, status_dev: int | None = None, stream: int | None = None) -> None:
    """Device-resident call of up to 128 rows that allocates nothing (the workspace is a fixed array inside
    the library); launches only. `status_dev`: 8 uint32 of device memory that receive the call's count and
    fault words. Calls that overlap on one GPU race."""
    buf = _err()
    _raise(load().m26s_b1_ffn_static(layer._h, payload_dev, payload_pitch, scales_dev, scales_pitch, ids_dev, weights_dev,
                                     rows, bf16_out_dev, status_dev, stream, buf, ERRLEN), buf)


# ---- stage-level entry points -----------------------------------------------------------------
def plan_dev(ids_dev, weights_dev, rows, capacity, resident_dev, inverse_dev, original_dev, gw_dev, groups_dev,
             count_dev, fault_dev) -> None:
    buf = _err()
    _raise(load().m26s_b1_plan_dev(ids_dev, weights_dev, rows, capacity, resident_dev, inverse_dev, original_dev,
                                   gw_dev, groups_dev, count_dev, fault_dev, buf, ERRLEN), buf)


def quantize_dev(h_dev, elements, payload_dev, scales_dev, faults_dev) -> None:
    buf = _err()
    _raise(load().m26s_b1_quantize_dev(h_dev, elements, payload_dev, scales_dev, faults_dev, buf, ERRLEN), buf)


def reduce_dev(y_dev, weights_dev, rows, partial_dev, bf16_dev, fault_dev) -> None:
    buf = _err()
    _raise(load().m26s_b1_reduce_dev(y_dev, weights_dev, rows, partial_dev, bf16_dev, fault_dev, buf, ERRLEN), buf)


def device_memory() -> tuple[int, int]:
    """(free, total) bytes of the current GPU's memory."""
    free, total = C.c_size_t(), C.c_size_t()
    if load().m26s_b1_device_memory(C.byref(free), C.byref(total)):
        raise B1Error(2, "b1: memory query failed")
    return int(free.value), int(total.value)


class DeviceBuffer:
    """A device allocation made through the library's own helpers (no other HIP binding needed)."""

    def __init__(self, nbytes: int):
        self.nbytes = int(nbytes)
        self.ptr = load().m26s_b1_device_alloc(self.nbytes)
        if not self.ptr:
            raise B1Error(2, f"b1: device allocation of {nbytes} bytes failed")

    @classmethod
    def from_host(cls, array: np.ndarray) -> "DeviceBuffer":
        array = np.ascontiguousarray(array)
        self = cls(max(array.nbytes, 1))
        if array.nbytes and load().m26s_b1_copy_to_device(self.ptr, array.ctypes.data, array.nbytes):
            raise B1Error(2, "b1: upload failed")
        return self

    def to_host(self, dtype, count: int | None = None) -> np.ndarray:
        dtype = np.dtype(dtype)
        count = self.nbytes // dtype.itemsize if count is None else count
        out = np.empty(count, dtype)
        if out.nbytes and load().m26s_b1_copy_to_host(out.ctypes.data, self.ptr, out.nbytes):
            raise B1Error(2, "b1: download failed")
        return out

    def free(self) -> None:
        if getattr(self, "ptr", None) and load is not None:
            load().m26s_b1_device_free(self.ptr)
            self.ptr = None

    __del__ = free
