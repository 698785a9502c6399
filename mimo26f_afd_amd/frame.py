"""Frame adapter of the expert rank: DS41RTE3 v3 request frame in, compact BF16 return frame out.

Mirrors, for the B1 path only, what the reference's daemon does around the FFN call:
  crates/mimo26-wire/src/layout.rs:27-118     constants, header / descriptor / route offsets
  crates/mimo26-wire/src/frame.rs:341-393     header parse (magic, version, kind, lengths)
  crates/mimo26-wire/src/frame.rs:406-457     L4 CRC32C over the frame with its CRC field zeroed
  crates/mimo26-wire/src/frame.rs:845-972     RequestView: a request validated where it lies
  crates/mimo26-wire/src/frame.rs:987-1041    return header for a frame assembled in place, seal
  crates/mimo26-spark/src/serve.rs:206-248    serve_b1_view: routes gathered from the frame, the hidden
                                              rows handed to the FFN in place at their 4,224-byte stride
  crates/mimo26-spark/src/main.rs:395-451     BF16 rows written straight behind the 128-byte header
`encode_request` (frame.rs:466-551) is here for the tests and for a coordinator that builds frames.

`serve_b1_view` works on host frames, as the reference does (its NIC lands frames in registered host
memory). `DeviceFrameAdapter` is this build's addition for frames that already lie in HBM: the
routes are gathered by a kernel, the hidden rows are read in place, and the BF16 rows are written
behind the return header in a device buffer; only the 128 header bytes cross to the host.
"""
from __future__ import annotations

import ctypes as C
import os
import struct

import numpy as np

from . import b1
from ._lib import load

MAGIC, VERSION, KIND_REQUEST, KIND_RETURN = b"DS41RTE3", 3, 1, 2
HEADER_LEN, ROW_DESCRIPTOR_LEN, ROUTE_ENTRY_LEN = 128, 40, 12
HIDDEN, TOPK, K32 = 4096, 8, 32
HIDDEN_ROW_BYTES = HIDDEN + HIDDEN // K32            # 4224
REQUEST_ROW_BYTES = ROW_DESCRIPTOR_LEN + HIDDEN_ROW_BYTES + TOPK * ROUTE_ENTRY_LEN  # 4360
RETURN_ROW_BYTES = HIDDEN * 2                        # 8192
DTYPE_BF16, DTYPE_FP8_ROW_SCALED, DTYPE_FP8_UE8M0_K32 = 1, 5, 7
SOURCE_DECODE, SOURCE_PREFILL, SOURCE_MTP_VERIFY, SOURCE_BENCHMARK = 1, 2, 3, 4
STATUS_OK, STATUS_ERROR = 0, 1
FLAG_SPARK_REDUCTION, FLAG_V41_COMPACT_BF16 = 1 << 9, 1 << 16
FLAG_RETURN_REQUIRED = FLAG_SPARK_REDUCTION | FLAG_V41_COMPACT_BF16

# header fields: name -> (offset, struct code)
HDR = dict(version=(8, "<H"), kind=(10, "<H"), header_len=(12, "<I"), request_id=(16, "<Q"), placement_version=(24, "<Q"),
           layer_id=(32, "<I"), row_count=(36, "<I"), dim=(40, "<I"), payload_dtype=(44, "<H"), source_kind=(46, "<H"),
           route_count=(48, "<I"), row_descriptor_bytes=(52, "<I"), route_bytes=(56, "<I"), payload_bytes=(60, "<Q"),
           logical_payload_bytes=(68, "<Q"), wire_bytes=(76, "<Q"), flags=(84, "<I"), row_stride_bytes=(88, "<I"),
           status=(92, "<I"), executor_id=(96, "<Q"), token_position=(104, "<Q"), seq=(112, "<Q"), crc32c=(120, "<I"),
           reserved=(124, "<I"))
CRC_OFFSET = 120
DESCRIPTOR = np.dtype({"names": ["row_id", "source_kind", "source_request_id", "token_position", "route_offset", "route_count"],
                       "formats": ["<u8", "<u2", "<u8", "<u8", "<u4", "<u4"], "offsets": [0, 8, 12, 20, 28, 32],
                       "itemsize": ROW_DESCRIPTOR_LEN})
ROUTE = np.dtype({"names": ["row_index", "expert_id", "gate_weight"], "formats": ["<u4", "<u4", "<f4"], "offsets": [0, 4, 8],
                  "itemsize": ROUTE_ENTRY_LEN})


class WireError(ValueError):
    """A frame that must not be served; `kind` names the reference's error variant."""

    def __init__(self, kind: str, message: str = ""):
        super().__init__(f"{kind}: {message}" if message else kind)
        self.kind = kind


def _bytes_view(buf) -> np.ndarray:
    a = buf if isinstance(buf, np.ndarray) else np.frombuffer(buf, np.uint8)
    if a.dtype != np.uint8 or a.ndim != 1 or not a.flags.c_contiguous:
        raise TypeError("a frame is a contiguous run of bytes")
    return a


def crc32c(data) -> int:
    a = _bytes_view(data)
    return load().m26w_crc32c_update(0xFFFFFFFF, a.ctypes.data, a.size) ^ 0xFFFFFFFF


def crc_disabled() -> bool:
    """Process configuration, never a frame bit: MIMO26_WIRE_NOCRC=1 neither seals nor verifies."""
    return os.environ.get("MIMO26_WIRE_NOCRC") == "1"


def compute_crc(frame) -> int:
    """CRC32C of the frame with its four CRC bytes taken as zero, streamed in three segments."""
    a = _bytes_view(frame)
    lib, zero = load(), np.zeros(4, np.uint8)
    c = lib.m26w_crc32c_update(0xFFFFFFFF, a.ctypes.data, CRC_OFFSET)
    c = lib.m26w_crc32c_update(c, zero.ctypes.data, 4)
    c = lib.m26w_crc32c_update(c, a.ctypes.data + CRC_OFFSET + 4, a.size - CRC_OFFSET - 4)
    return c ^ 0xFFFFFFFF


def seal_in_place(frame) -> None:
    """Writes the checksum of a frame assembled in place (its CRC field must be zero)."""
    if crc_disabled():
        return
    a = _bytes_view(frame)
    struct.pack_into("<I", a, CRC_OFFSET, compute_crc(a))


def _get(a: np.ndarray, name: str) -> int:
    off, code = HDR[name]
    return struct.unpack_from(code, a, off)[0]


def parse_header(frame) -> dict:
    a = _bytes_view(frame)
    if a.size < HEADER_LEN:
        raise WireError("TooShort", f"need {HEADER_LEN}, got {a.size}")
    if a[:8].tobytes() != MAGIC:
        raise WireError("BadMagic", repr(a[:8].tobytes()))
    if _get(a, "version") != VERSION:
        raise WireError("BadVersion", str(_get(a, "version")))
    kind = _get(a, "kind")
    if kind not in (KIND_REQUEST, KIND_RETURN):
        raise WireError("BadKind", str(kind))
    if _get(a, "header_len") != HEADER_LEN:
        raise WireError("BadHeaderLen", str(_get(a, "header_len")))
    declared = _get(a, "wire_bytes")
    if a.size < declared:
        raise WireError("Truncated", f"declared {declared}, got {a.size}")
    if a.size > declared:
        raise WireError("TrailingBytes", f"declared {declared}, got {a.size}")
    h = {name: _get(a, name) for name in HDR}
    if not 1 <= h["payload_dtype"] <= 7:
        raise WireError("BadCode", f"payload_dtype {h['payload_dtype']}")
    if not 1 <= h["source_kind"] <= 4:
        raise WireError("BadCode", f"source_kind {h['source_kind']}")
    if h["status"] not in (STATUS_OK, STATUS_ERROR):
        raise WireError("BadCode", f"status {h['status']}")
    return h


def verify_crc(frame, seq: int) -> None:
    if crc_disabled():
        return
    a = _bytes_view(frame)
    want, got = compute_crc(a), _get(a, "crc32c")
    if want != got:
        raise WireError("Corrupt", f"seq {seq}: want {want:#010x}, got {got:#010x}")


def _write_header(out: np.ndarray, **f) -> None:
    out[:HEADER_LEN] = 0
    out[:8] = np.frombuffer(MAGIC, np.uint8)
    f = dict(version=VERSION, header_len=HEADER_LEN, **f)
    for name, value in f.items():
        off, code = HDR[name]
        struct.pack_into(code, out, off, value)


class RequestView:
    """A request frame validated where it lies; nothing is copied."""

    def __init__(self, frame, header: dict):
        a = _bytes_view(frame)
        self.frame = a
        for k in ("request_id", "placement_version", "layer_id", "executor_id", "source_kind", "token_position", "flags", "seq"):
            setattr(self, k, header[k])
        self.rows, self.routes, self.row_stride = header["row_count"], header["route_count"], header["row_stride_bytes"]
        self.route_base = HEADER_LEN + self.rows * ROW_DESCRIPTOR_LEN
        self.hidden_base = self.route_base + self.routes * ROUTE_ENTRY_LEN
        self.descriptors = a[HEADER_LEN:self.route_base].view(DESCRIPTOR)
        self.route_entries = a[self.route_base:self.hidden_base].view(ROUTE)

    @classmethod
    def parse(cls, frame) -> "RequestView":
        a = _bytes_view(frame)
        h = parse_header(a)
        verify_crc(a, h["seq"])
        if h["kind"] != KIND_REQUEST:
            raise WireError("BadKind", str(h["kind"]))
        rows, routes = h["row_count"], h["route_count"]

        def want(field, expect, got):
            if expect != got:
                raise WireError("DimMismatch", f"{field}: want {expect}, got {got}")
        if rows == 0:
            raise WireError("DimMismatch", "row_count: want 1, got 0")
        want("row_descriptor_bytes", rows * ROW_DESCRIPTOR_LEN, h["row_descriptor_bytes"])
        want("route_bytes", routes * ROUTE_ENTRY_LEN, h["route_bytes"])
        want("hidden_dim", HIDDEN, h["dim"])
        if h["payload_dtype"] not in (DTYPE_FP8_UE8M0_K32, DTYPE_FP8_ROW_SCALED):
            raise WireError("DimMismatch", f"request_payload_dtype: want {DTYPE_FP8_UE8M0_K32}, got {h['payload_dtype']}")
        stride = h["row_stride_bytes"]
        if stride < HIDDEN:
            raise WireError("DimMismatch", f"row_stride_bytes: want {HIDDEN}, got {stride}")
        want("payload_bytes", rows * stride, h["payload_bytes"])
        want("body_len", rows * ROW_DESCRIPTOR_LEN + routes * ROUTE_ENTRY_LEN + rows * stride, a.size - HEADER_LEN)
        view = cls(a, h)
        d, r = view.descriptors, view.route_entries
        bad_kind = (d["source_kind"] < 1) | (d["source_kind"] > 4)
        bad_range = d["route_offset"].astype(np.uint64) + d["route_count"] > routes
        first = np.flatnonzero(bad_kind | bad_range)
        if first.size:
            i = int(first[0])
            raise WireError("BadCode", f"source_kind {int(d['source_kind'][i])}") if bad_kind[i] else WireError("RouteRangeBad", f"row {i}")
        stray = np.flatnonzero(r["row_index"] >= rows)
        if stray.size:
            j = int(stray[0])
            raise WireError("RouteRowMismatch", f"entry {j}: row_index {int(r['row_index'][j])}, rows {rows}")
        return view

    def hidden(self) -> np.ndarray:
        """rows * row_stride bytes: per row the E4M3 payload (4096 bytes) then its scales."""
        return self.frame[self.hidden_base:]


def b1_inputs(view: RequestView):
    """Token-major top-8 expert ids (i32) and route weights (f32) of a validated request, with the
    shape checks of serve.rs:219-232: every row carries 8 routes and every route names its row."""
    if view.row_stride != HIDDEN_ROW_BYTES:
        raise WireError("ServeB1", f"hidden row stride {view.row_stride} is not 4,096 E4M3 + 128 scales")
    d, r = view.descriptors, view.route_entries
    odd = np.flatnonzero(d["route_count"] != TOPK)
    if odd.size:
        i = int(odd[0])
        raise WireError("ServeB1", f"row {i} has {int(d['route_count'][i])} routes, want 8")
    index = d["route_offset"].astype(np.int64)[:, None] + np.arange(TOPK)
    picked = r[index]
    wrong = np.flatnonzero((picked["row_index"] != np.arange(view.rows, dtype=np.uint32)[:, None]).reshape(-1))
    if wrong.size:
        i = int(wrong[0]) // TOPK
        raise WireError("ServeB1", f"route row {int(picked['row_index'].reshape(-1)[wrong[0]])} under row {i}")
    return np.ascontiguousarray(picked["expert_id"].astype(np.int32)), np.ascontiguousarray(picked["gate_weight"])


def return_header(view, rows: int, seq: int, status: int = STATUS_OK) -> np.ndarray:
    """The 128 header bytes of a compact BF16 return of `rows` rows for `view`'s request."""
    if rows == 0:
        raise WireError("DimMismatch", "rows: want 1, got 0")
    out = np.zeros(HEADER_LEN, np.uint8)
    payload = rows * RETURN_ROW_BYTES
    _write_header(out, kind=KIND_RETURN, request_id=view.request_id, placement_version=view.placement_version,
                  layer_id=view.layer_id, row_count=rows, dim=HIDDEN, payload_dtype=DTYPE_BF16, source_kind=SOURCE_DECODE,
                  route_count=TOPK, row_descriptor_bytes=0, route_bytes=0, payload_bytes=payload,
                  logical_payload_bytes=payload, wire_bytes=HEADER_LEN + payload, flags=FLAG_RETURN_REQUIRED,
                  row_stride_bytes=RETURN_ROW_BYTES, status=status, executor_id=view.executor_id,
                  token_position=view.token_position, seq=seq)
    return out


def encode_request(payload: np.ndarray, scales: np.ndarray, ids: np.ndarray, weights: np.ndarray, *, request_id=1,
                   placement_version=1, layer_id=1, executor_id=0, source_kind=SOURCE_DECODE, token_position=0, flags=0,
                   seq=0) -> np.ndarray:
    """The request frame of `rows` tokens with their top-8 routes: row t has row id and token position
    t and routes 8t..8t+7 (the decode-kind frame the coordinator's fast path builds, frame.rs:569-657)."""
    rows = payload.shape[0]
    assert payload.shape == (rows, HIDDEN) and scales.shape == (rows, HIDDEN // K32) and ids.shape == (rows, TOPK) == weights.shape
    routes = rows * TOPK
    total = HEADER_LEN + rows * ROW_DESCRIPTOR_LEN + routes * ROUTE_ENTRY_LEN + rows * HIDDEN_ROW_BYTES
    out = np.zeros(total, np.uint8)
    _write_header(out, kind=KIND_REQUEST, request_id=request_id, placement_version=placement_version, layer_id=layer_id,
                  row_count=rows, dim=HIDDEN, payload_dtype=DTYPE_FP8_UE8M0_K32, source_kind=source_kind, route_count=routes,
                  row_descriptor_bytes=rows * ROW_DESCRIPTOR_LEN, route_bytes=routes * ROUTE_ENTRY_LEN,
                  payload_bytes=rows * HIDDEN_ROW_BYTES, logical_payload_bytes=rows * REQUEST_ROW_BYTES, wire_bytes=total,
                  flags=flags, row_stride_bytes=HIDDEN_ROW_BYTES, status=STATUS_OK, executor_id=executor_id,
                  token_position=token_position, seq=seq)
    route_base = HEADER_LEN + rows * ROW_DESCRIPTOR_LEN
    hidden_base = route_base + routes * ROUTE_ENTRY_LEN
    d = out[HEADER_LEN:route_base].view(DESCRIPTOR)
    d["row_id"] = np.arange(rows)
    d["source_kind"] = source_kind
    d["source_request_id"] = request_id
    d["token_position"] = np.arange(rows)
    d["route_offset"] = np.arange(rows) * TOPK
    d["route_count"] = TOPK
    r = out[route_base:hidden_base].view(ROUTE)
    r["row_index"] = np.repeat(np.arange(rows, dtype=np.uint32), TOPK)
    r["expert_id"] = ids.reshape(-1).astype(np.uint32)
    r["gate_weight"] = weights.reshape(-1)
    body = out[hidden_base:].reshape(rows, HIDDEN_ROW_BYTES)
    body[:, :HIDDEN], body[:, HIDDEN:] = payload, scales
    seal_in_place(out)
    return out


def serve_b1_view(view: RequestView, layer: b1.Layer, scratch: b1.Scratch, out_frame: np.ndarray, seq: int = 0) -> b1.FfnStats:
    """One request through the FFN into a return frame assembled in place: `out_frame` is the send
    buffer (at least 128 + rows * 8192 bytes, 2-byte aligned); on return its first
    128 + rows * 8192 bytes are the sealed return frame."""
    ids, weights = b1_inputs(view)
    rows = view.rows
    need = HEADER_LEN + rows * RETURN_ROW_BYTES
    out = _bytes_view(out_frame)
    if out.size < need:
        raise WireError("ServeB1", f"return frame {need} B exceeds the send buffer")
    body = out[HEADER_LEN:need].view(np.uint16)
    stats = b1.ffn_strided(layer, scratch, view.hidden(), view.row_stride, ids, weights, rows, body)
    out[:HEADER_LEN] = return_header(view, rows, seq)
    seal_in_place(out[:need])
    return stats


class DeviceFrameAdapter:
    """Request frames that already lie in device memory (a transport that lands them in HBM): routes
    gathered on the device, hidden rows read in place, BF16 rows written behind the return header in
    a device buffer. The host reads the 128 header bytes it is given and writes 128 back. The L4
    checksum of a device-resident frame is not computed here: run such lanes with the checksum off
    (MIMO26_WIRE_NOCRC=1, the reference's fast-path setting) or seal after the frame reaches the host."""

    def __init__(self, layer: b1.Layer, scratch: b1.Scratch, max_rows: int = 8192):
        """The route gathering and the staging copy launch on the scratch's own stream, ahead of the
        FFN that reads what they write; no other stream takes part."""
        self.layer, self.scratch, self.max_rows, self.stream = layer, scratch, max_rows, scratch.stream
        self.ids = b1.DeviceBuffer(max_rows * TOPK * 4)
        self.weights = b1.DeviceBuffer(max_rows * TOPK * 4)
        self.fault = b1.DeviceBuffer(4)
        self.staging = None  # hidden rows of frames whose rows do not start on a 16-byte boundary

    def serve(self, header, frame_dev: int, out_frame_dev: int, seq: int = 0) -> np.ndarray:
        """`header` = the request's first 128 bytes (host), `frame_dev` = the whole request frame in
        device memory (4-byte aligned), `out_frame_dev` = device buffer of 128 + rows * 8192 bytes.
        Launches on the scratch's stream, waits, and returns the 128 return-header bytes, which are
        also written to out_frame_dev."""
        a = _bytes_view(header)
        if a.size != HEADER_LEN:
            raise WireError("TooShort", f"need {HEADER_LEN} header bytes, got {a.size}")
        h = {name: _get(a, name) for name in HDR}
        if a[:8].tobytes() != MAGIC:
            raise WireError("BadMagic", repr(a[:8].tobytes()))
        if h["version"] != VERSION:
            raise WireError("BadVersion", str(h["version"]))
        if h["kind"] != KIND_REQUEST:
            raise WireError("BadKind", str(h["kind"]))
        if h["header_len"] != HEADER_LEN:
            raise WireError("BadHeaderLen", str(h["header_len"]))
        rows, routes, stride = h["row_count"], h["route_count"], h["row_stride_bytes"]
        if rows == 0 or rows > self.max_rows or h["dim"] != HIDDEN or stride != HIDDEN_ROW_BYTES \
                or h["row_descriptor_bytes"] != rows * ROW_DESCRIPTOR_LEN or h["route_bytes"] != routes * ROUTE_ENTRY_LEN \
                or h["payload_bytes"] != rows * stride or h["payload_dtype"] != DTYPE_FP8_UE8M0_K32 \
                or h["wire_bytes"] != HEADER_LEN + rows * ROW_DESCRIPTOR_LEN + routes * ROUTE_ENTRY_LEN + rows * stride:
            raise WireError("DimMismatch", "request header does not describe a B1 frame this adapter serves")
        if frame_dev & 3:
            raise WireError("ServeB1", "a device-resident frame must start on a 4-byte boundary")
        view = RequestView.__new__(RequestView)
        for k in ("request_id", "placement_version", "layer_id", "executor_id", "token_position"):
            setattr(view, k, h[k])
        route_base = HEADER_LEN + rows * ROW_DESCRIPTOR_LEN
        hidden = frame_dev + route_base + routes * ROUTE_ENTRY_LEN
        rc = load().m26w_request_routes_dev(frame_dev + HEADER_LEN, frame_dev + route_base, rows, routes, self.ids.ptr,
                                            self.weights.ptr, self.fault.ptr, self.stream)
        if rc:
            raise WireError("ServeB1", f"route gathering refused (rc {rc})")
        if hidden & 15:
            if self.staging is None:
                self.staging = b1.DeviceBuffer(self.max_rows * HIDDEN_ROW_BYTES)
            if load().m26w_stage_rows_dev(self.staging.ptr, hidden, rows * stride, self.stream) != 0:
                raise WireError("ServeB1", "staging copy failed")
            hidden = self.staging.ptr
        failed = None
        try:
            b1.ffn_enqueue(self.layer, self.scratch, hidden, stride, hidden + HIDDEN, stride, self.ids.ptr, self.weights.ptr,
                           rows, out_frame_dev + HEADER_LEN)
            self.scratch.sync()
        except b1.B1Error as e:  # a frame that breaks the route contract may also hand the planner bad ids
            failed = e
        fault = int(self.fault.to_host(np.uint32)[0])
        if fault:
            what = {1: "does not carry 8 routes", 2: "has a route range outside the route array", 3: "holds a route of another row"}
            raise WireError("ServeB1", f"row {fault >> 2} {what[fault & 3]}")
        if failed is not None:
            raise failed
        out = return_header(view, rows, seq)
        if load().m26s_b1_copy_to_device(out_frame_dev, out.ctypes.data, HEADER_LEN) != 0:
            raise WireError("ServeB1", "header upload failed")
        return out

    def close(self) -> None:
        for buf in (self.ids, self.weights, self.fault, self.staging):
            if buf is not None:
                buf.free()
