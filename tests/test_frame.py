"""The expert rank's frame adapter: wire bytes pinned to the reference's own vectors
(crates/mimo26-wire/tests/wire_layout.rs:82-133), the rejection cases of its in-place view
(tests/request_view.rs:96-140), the in-place return (tests/in_place_return.rs), and (GPU) a request
frame served from host memory and from device memory."""
import struct

import numpy as np
import pytest

from mimo26f_afd_amd import frame as F
from mimo26f_afd_amd import synth


def small_request(rows=4, seed=3, **kw):
    rng = np.random.default_rng(seed)
    payload = rng.integers(0, 256, (rows, 4096), dtype=np.uint8)
    scales = rng.integers(110, 130, (rows, 128), dtype=np.uint8)
    ids = np.stack([rng.permutation(256)[:8] for _ in range(rows)]).astype(np.int32)
    w = rng.random((rows, 8), dtype=np.float32)
    return F.encode_request(payload, scales, ids, w, **kw), payload, scales, ids, w


def test_wire_constants_and_pinned_entry_bytes():
    assert (F.HIDDEN_ROW_BYTES, F.REQUEST_ROW_BYTES, F.RETURN_ROW_BYTES, F.HEADER_LEN) == (4224, 4360, 8192, 128)
    d = np.zeros(1, F.DESCRIPTOR)
    d["row_id"], d["source_kind"], d["source_request_id"] = 0x0102030405060708, 1, 0x1112131415161718
    d["token_position"], d["route_offset"], d["route_count"] = 0x2122232425262728, 0x31323334, 0x41424344
    assert d.tobytes() == bytes([8, 7, 6, 5, 4, 3, 2, 1, 1, 0, 0, 0, 0x18, 0x17, 0x16, 0x15, 0x14, 0x13, 0x12, 0x11,
                                 0x28, 0x27, 0x26, 0x25, 0x24, 0x23, 0x22, 0x21, 0x34, 0x33, 0x32, 0x31, 0x44, 0x43, 0x42, 0x41, 0, 0, 0, 0])
    r = np.zeros(1, F.ROUTE)
    r["row_index"], r["expert_id"], r["gate_weight"] = 0x01020304, 0x11121314, 1.0
    assert r.tobytes() == bytes([4, 3, 2, 1, 0x14, 0x13, 0x12, 0x11, 0, 0, 0x80, 0x3F])
    assert F.crc32c(b"123456789") == 0xE3069283  # RFC 3720
    assert F.crc32c(b"") == 0 and F.crc32c(bytes(32)) == 0x8A9136AA  # RFC 3720 B.4: 32 zero bytes
    # the table path against a bit-by-bit evaluation, odd lengths and alignments
    rng = np.random.default_rng(0)
    data = rng.integers(0, 256, 1000, dtype=np.uint8)
    for lo, hi in ((0, 1000), (1, 999), (3, 14), (7, 8), (5, 5)):
        c = 0xFFFFFFFF
        for b in data[lo:hi]:
            c ^= int(b)
            for _ in range(8):
                c = (c >> 1) ^ (0x82F63B78 if c & 1 else 0)
        assert F.crc32c(data[lo:hi].copy()) == c ^ 0xFFFFFFFF and F.crc32c(data[lo:hi]) == c ^ 0xFFFFFFFF


def test_crc32c_instruction_path_equals_the_table_walk():
    """m26w_crc32c_update uses the host's CRC32C instruction where there is one, three stripes of 4096 bytes side
    by side joined by the x^(8 * 4096) map; m26w_crc32c_update_portable is the table walk. Same state for every
    length around the stripe and triple-stripe boundaries, at every alignment, chained across an arbitrary cut,
    from an arbitrary starting state, and on a buffer the size of a 4096-row request frame (the reference compares
    its two paths at 1 MiB and 17.86 MB, crates/mimo26-wire/src/crc32c.rs:203-216). Both paths also get the
    bit-by-bit value on a 13 KB run, so the joining of stripes is pinned independently of the tables."""
    from mimo26f_afd_amd._lib import load
    lib = load()
    rng = np.random.default_rng(1)
    buf = rng.integers(0, 256, 128 + 4096 * 4360 + 64, dtype=np.uint8)
    lengths = [0, 1, 7, 8, 9, 4095, 4096, 4097, 12287, 12288, 12289, 12296, 24576 + 5, 3 * 4096 * 5 + 13, 1 << 20, buf.size - 16]
    for n in lengths:
        for off in (0, 1, 3, 8):
            a = buf[off:off + n]
            for start in (0xFFFFFFFF, 0, 0x12345678):
                want = lib.m26w_crc32c_update_portable(start, a.ctypes.data, a.size)
                assert lib.m26w_crc32c_update(start, a.ctypes.data, a.size) == want, (n, off, start)
                cut = n // 3
                head = lib.m26w_crc32c_update(start, a.ctypes.data, cut)
                assert lib.m26w_crc32c_update(head, a.ctypes.data + cut, n - cut) == want, (n, off, start)
    run = buf[5:5 + 13000]
    c = 0xFFFFFFFF
    for b in run:
        c ^= int(b)
        for _ in range(8):
            c = (c >> 1) ^ (0x82F63B78 if c & 1 else 0)
    assert lib.m26w_crc32c_update(0xFFFFFFFF, run.ctypes.data, run.size) == c
    assert lib.m26w_crc32c_update_portable(0xFFFFFFFF, run.ctypes.data, run.size) == c


def test_request_round_trip_and_body_accounting():
    for rows in (1, 3, 16):
        frame, payload, scales, ids, w = small_request(rows, request_id=42, layer_id=5, executor_id=2, seq=9)
        assert frame.size - F.HEADER_LEN == rows * 4360
        v = F.RequestView.parse(frame)
        assert (v.rows, v.routes, v.row_stride, v.request_id, v.layer_id, v.executor_id, v.seq) == (rows, rows * 8, 4224, 42, 5, 2, 9)
        body = v.hidden().reshape(rows, 4224)
        assert np.array_equal(body[:, :4096], payload) and np.array_equal(body[:, 4096:], scales)
        got_ids, got_w = F.b1_inputs(v)
        assert np.array_equal(got_ids, ids) and np.array_equal(got_w, w) and got_ids.dtype == np.int32 and got_w.dtype == np.float32


def reseal(frame, edit):
    b = frame.copy()
    edit(b)
    struct.pack_into("<I", b, 120, 0)
    F.seal_in_place(b)
    return b


def test_view_rejects_what_the_reference_rejects():
    rows = 4
    good, *_ = small_request(rows, seq=5)
    route_at = 128 + rows * 40

    def put(off, code, value):
        return lambda b: struct.pack_into(code, b, off, value)
    cases = [(put(route_at + 5 * 12, "<I", rows), "RouteRowMismatch"), (put(128 + 2 * 40 + 32, "<I", 1000), "RouteRangeBad"),
             (put(128 + 8, "<H", 0xBEEF), "BadCode"), (put(40, "<I", 2048), "DimMismatch"), (put(36, "<I", 0), "DimMismatch"),
             (put(88, "<I", 100), "DimMismatch"), (put(10, "<H", 2), "BadKind"), (put(8, "<H", 2), "BadVersion"),
             (put(12, "<I", 64), "BadHeaderLen"), (put(44, "<H", 1), "DimMismatch"), (put(44, "<H", 9), "BadCode")]
    for edit, kind in cases:
        with pytest.raises(F.WireError) as e:
            F.RequestView.parse(reseal(good, edit))
        assert e.value.kind == kind, (kind, str(e.value))
    flipped = good.copy()
    flipped[128 + 3 * 40 + 1] ^= 0x10
    with pytest.raises(F.WireError, match="Corrupt"):
        F.RequestView.parse(flipped)
    with pytest.raises(F.WireError, match="Truncated"):
        F.RequestView.parse(good[:-1].copy())
    with pytest.raises(F.WireError, match="TrailingBytes"):
        F.RequestView.parse(np.concatenate([good, np.zeros(1, np.uint8)]))
    bad_magic = good.copy()
    bad_magic[0] ^= 1
    with pytest.raises(F.WireError, match="BadMagic"):
        F.RequestView.parse(bad_magic)
    F.RequestView.parse(good)


def test_b1_shape_checks_above_the_codec():
    rows = 3
    good, *_ = small_request(rows)
    route_at = 128 + rows * 40
    v = F.RequestView.parse(reseal(good, lambda b: struct.pack_into("<I", b, 128 + 40 + 32, 7)))  # row 1 carries 7 routes
    with pytest.raises(F.WireError, match="row 1 has 7 routes, want 8"):
        F.b1_inputs(v)
    v = F.RequestView.parse(reseal(good, lambda b: struct.pack_into("<I", b, route_at + 9 * 12, 2)))  # a route of row 2 under row 1
    with pytest.raises(F.WireError, match="route row 2 under row 1"):
        F.b1_inputs(v)


def test_return_assembled_in_place():
    good, *_ = small_request(3, request_id=42, placement_version=1, layer_id=5, executor_id=2)
    v = F.RequestView.parse(good)
    rows = 3
    codes = np.array([[(r * 7919 + i * 31) & 0xFFFF for i in range(4096)] for r in range(rows)], np.uint16)
    buf = np.zeros(128 + rows * 8192 + 64, np.uint8)
    buf[128:128 + rows * 8192] = codes.view(np.uint8).reshape(-1)
    buf[:128] = F.return_header(v, rows, 17)
    F.seal_in_place(buf[:128 + rows * 8192])
    h = F.parse_header(buf[:128 + rows * 8192])
    F.verify_crc(buf[:128 + rows * 8192], 17)
    assert (h["kind"], h["row_count"], h["dim"], h["payload_dtype"], h["source_kind"], h["route_count"]) == (2, 3, 4096, 1, 1, 8)
    assert (h["payload_bytes"], h["logical_payload_bytes"], h["wire_bytes"], h["row_stride_bytes"]) == (24576, 24576, 24704, 8192)
    assert (h["request_id"], h["placement_version"], h["layer_id"], h["executor_id"], h["seq"], h["status"]) == (42, 1, 5, 2, 17, 0)
    assert h["flags"] == (1 << 9) | (1 << 16) and h["row_descriptor_bytes"] == 0 and h["route_bytes"] == 0 and h["reserved"] == 0


@pytest.mark.gpu
def test_serve_request_frames_from_host_and_device_memory():
    """A request frame served from host memory and from device memory, against the CPU checker's BF16 rows
    (bars of the benchmark contract); the routes the device gathered are read back and compared with the
    host parse of the same frame, id for id and weight bit for weight bit."""
    import b1_oracle as O
    from helpers import DeviceLayer, bf16_to_f32, parity
    from mimo26f_afd_amd import b1
    wl = synth.make(1)
    pools = wl.pools(wl.touched())
    layer = DeviceLayer(pools).layer
    scratch = b1.Scratch()
    rc, _, ref_bf16, _ = O.layer_ffn(pools, wl.payload, wl.scales, wl.ids, wl.weights)
    assert rc == 0

    def check_rows(bits):
        ma, mr = parity(bf16_to_f32(bits), bf16_to_f32(ref_bf16))
        assert ma <= 1e-2 and mr <= 1e-3, (ma, mr)

    request = F.encode_request(wl.payload, wl.scales, wl.ids, wl.weights, request_id=7, layer_id=3, executor_id=1, seq=4)
    view = F.RequestView.parse(request)
    host_ids, host_w = F.b1_inputs(view)
    assert np.array_equal(host_ids, wl.ids) and np.array_equal(host_w.view(np.uint32), wl.weights.view(np.uint32))
    send = np.zeros(128 + wl.rows * 8192, np.uint8)
    stats = F.serve_b1_view(view, layer, scratch, send, seq=11)
    assert stats.groups > 0
    h = F.parse_header(send)
    F.verify_crc(send, 11)
    assert (h["kind"], h["row_count"], h["request_id"], h["layer_id"], h["executor_id"], h["seq"]) == (2, wl.rows, 7, 3, 1, 11)
    served = send[128:].view(np.uint16).reshape(wl.rows, 4096).copy()
    check_rows(served)

    # the same request lying in device memory, at both alignments of its hidden rows (16 rows: rows start
    # 128 + 136 * 16 bytes in, a multiple of 16; shifted by 8 they are not and get staged)
    adapter = F.DeviceFrameAdapter(layer, scratch, max_rows=64)
    assert adapter.stream == scratch.stream
    for shift in (0, 8):
        dev = b1.DeviceBuffer(request.size + 16)
        assert b1.load().m26s_b1_copy_to_device(dev.ptr + shift, request.ctypes.data, request.size) == 0
        out = b1.DeviceBuffer(128 + wl.rows * 8192)
        assert b1.load().m26s_b1_copy_to_device(adapter.ids.ptr, np.full(wl.rows * 8, -7, np.int32).ctypes.data, wl.rows * 32) == 0
        header = adapter.serve(request[:128], dev.ptr + shift, out.ptr, seq=12)
        got_ids = adapter.ids.to_host(np.int32, wl.rows * 8).reshape(wl.rows, 8)
        got_w = adapter.weights.to_host(np.float32, wl.rows * 8).reshape(wl.rows, 8)
        assert np.array_equal(got_ids, host_ids), shift                    # what the device gathered = the host parse
        assert np.array_equal(got_w.view(np.uint32), host_w.view(np.uint32)), shift
        back = out.to_host(np.uint8)
        assert np.array_equal(back[:128], header) and F.parse_header(np.concatenate([header, back[128:]]))["seq"] == 12
        rows = back[128:].view(np.uint16).reshape(wl.rows, 4096)
        check_rows(rows)
        assert np.array_equal(rows, served), shift                         # and the host-memory path's bits
        dev.free()
        out.free()
    # a frame that breaks the route contract is refused with the row named
    broken = request.copy()
    struct.pack_into("<I", broken, 128 + wl.rows * 40 + (5 * 8 + 2) * 12, 9)  # a route of row 9 under row 5
    dev = b1.DeviceBuffer(broken.size)
    assert b1.load().m26s_b1_copy_to_device(dev.ptr, broken.ctypes.data, broken.size) == 0
    out = b1.DeviceBuffer(128 + wl.rows * 8192)
    with pytest.raises(F.WireError, match="row 5 holds a route of another row"):
        adapter.serve(broken[:128], dev.ptr, out.ptr)
    adapter.close()
