"""ctypes binding of the CPU checker (oracle/liboracle.so) and, where it was built, of the
reference's own B1 host units (oracle/_ref/libb1ref.so).

TEST INFRASTRUCTURE ONLY: imported by tests/, the smoke check and the benchmark's
cpu_baseline leg; never by the product package.
"""
from __future__ import annotations

import ctypes as C
import os
import subprocess

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
HIDDEN, EXPERTS, TOPK, RANK_I, IMAGE_BYTES = 4096, 256, 8, 512, 3342336
GROUP_DTYPE = np.dtype([("expert", "<i4"), ("rows", "<i4"), ("route_base", "<i4"), ("input_rows", "<i4", (16,))])
assert GROUP_DTYPE.itemsize == 76

_u8p, _f32p, _i32p, _u32p, _u16p = (C.POINTER(t) for t in (C.c_uint8, C.c_float, C.c_int32, C.c_uint32, C.c_uint16))


def build(force: bool = False) -> None:
    """Compile the checker (and the reference units when /root/reference is present)."""
    if force or not os.path.exists(os.path.join(HERE, "liboracle.so")):
        subprocess.run(["make", "-C", HERE, "-B" if force else "-s", "all"], check=True)


def _p(a, t):
    return a.ctypes.data_as(t) if a is not None else None


class _Layer(C.Structure):
    _fields_ = [("pool", C.c_void_p * 4), ("ranks", C.c_uint32)]


def _load():
    build()
    # B1_ORACLE_LIB: another build of the same checker (the sanitized one of `make -C oracle asan`)
    lib = C.CDLL(os.environ.get("B1_ORACLE_LIB") or os.path.join(HERE, "liboracle.so"))
    lib.orc_mxfp4_bits.restype = C.c_uint32
    lib.orc_mxfp4_bits.argtypes = [C.c_uint32, C.c_uint32]
    lib.orc_e4m3_value.restype = C.c_float
    lib.orc_e4m3_value.argtypes = [C.c_uint8]
    lib.orc_bf16_rne.restype = C.c_uint16
    lib.orc_bf16_rne.argtypes = [C.c_float]
    lib.orc_e4m3_encode_half_up.restype = C.c_uint8
    lib.orc_e4m3_encode_half_up.argtypes = [C.c_double]
    lib.orc_silu_up.restype = C.c_float
    lib.orc_silu_up.argtypes = [C.c_float, C.c_float]
    lib.orc_quant_v1.restype = C.c_size_t
    lib.orc_activation_decode.restype = C.c_size_t
    lib.orc_plan.restype = C.c_uint32
    lib.orc_reduce.restype = C.c_uint32
    lib.orc_reduce_bf16y.restype = C.c_uint32
    lib.orc_bf16_store_rows.restype = None
    lib.orc_expert_ffn.restype = C.c_uint32
    lib.orc_layer_ffn.restype = C.c_uint32
    lib.orc_layer_ffn_efp32.restype = C.c_uint32
    lib.orc_hardware_threads.restype = C.c_int
    lib.orc_bf16_rne_nan.restype = C.c_uint16
    lib.orc_bf16_rne_nan.argtypes = [C.c_float]
    return lib


LIB = _load()


def hardware_threads() -> int:
    return int(LIB.orc_hardware_threads())


def mxfp4_bits(nibble: int, scale: int) -> int:
    return int(LIB.orc_mxfp4_bits(nibble, scale))


def mxfp4_rows(payload: np.ndarray, scales: np.ndarray) -> np.ndarray:
    """payload u8 [n, k/2], scales u8 [n, k/32] -> f32 [n, k]."""
    payload = np.ascontiguousarray(payload, np.uint8)
    scales = np.ascontiguousarray(scales, np.uint8)
    n, half = payload.shape
    out = np.empty((n, half * 2), np.float32)
    for r in range(n):
        LIB.orc_mxfp4_row(_p(payload[r], _u8p), _p(scales[r], _u8p), C.c_size_t(half * 2), _p(out[r], _f32p))
    return out


def e4m3_value(code: int) -> float:
    return float(LIB.orc_e4m3_value(code))


def activation_decode(payload: np.ndarray, scales: np.ndarray):
    payload = np.ascontiguousarray(payload, np.uint8)
    scales = np.ascontiguousarray(scales, np.uint8)
    rows, cols = payload.shape
    out = np.empty((rows, cols), np.float32)
    bad = LIB.orc_activation_decode(_p(payload, _u8p), C.c_size_t(cols), _p(scales, _u8p), C.c_size_t(cols // 32),
                                    C.c_size_t(rows), C.c_size_t(cols), _p(out, _f32p))
    return out, int(bad)


def q0_quantize(x: np.ndarray):
    x = np.ascontiguousarray(x, np.float32)
    rows, cols = x.shape
    payload = np.empty((rows, cols), np.uint8)
    scales = np.empty((rows, cols // 32), np.uint8)
    LIB.orc_q0_quantize(_p(x, _f32p), C.c_size_t(rows), C.c_size_t(cols), _p(payload, _u8p), _p(scales, _u8p))
    return payload, scales


def q0_scales(x: np.ndarray):
    """Scale bytes and 2^(127 - s) per K32 block of a flat f32 array."""
    x = np.ascontiguousarray(x, np.float32).reshape(-1)
    n = x.size // 32
    scales, inv = np.empty(n, np.uint8), np.empty(n, np.float32)
    LIB.orc_q0_scales(_p(x, _f32p), C.c_size_t(n), _p(scales, _u8p), _p(inv, _f32p))
    return scales, inv


def router_topk(logits: np.ndarray, bias: np.ndarray, top_k: int):
    logits = np.ascontiguousarray(logits, np.float32)
    bias = np.ascontiguousarray(bias, np.float32)
    rows, n = logits.shape
    idx, w = np.empty((rows, top_k), np.int32), np.empty((rows, top_k), np.float32)
    LIB.orc_router_topk(_p(logits, _f32p), _p(bias, _f32p), C.c_size_t(rows), C.c_size_t(n), C.c_size_t(top_k),
                        _p(idx, C.POINTER(C.c_int32)), _p(w, _f32p))
    return idx, w


def rank_sum_bf16(p0, p1, p2, p3) -> np.ndarray:
    ps = [np.ascontiguousarray(p, np.uint16).reshape(-1) for p in (p0, p1, p2, p3)]
    out = np.empty(ps[0].size, np.float32)
    u16p = C.POINTER(C.c_uint16)
    LIB.orc_rank_sum_bf16(*[_p(p, u16p) for p in ps], _p(out, _f32p), C.c_size_t(out.size))
    return out


def bf16_rne_nan(x: np.ndarray) -> np.ndarray:
    x = np.ascontiguousarray(x, np.float32).reshape(-1)
    return np.array([LIB.orc_bf16_rne_nan(C.c_float(float(v))) for v in x], np.uint16)


def quant_v1(h: np.ndarray, fill: int = 0xA5):
    """f32 [..., n] -> (payload, scales, faults); faulting blocks keep the fill byte."""
    h = np.ascontiguousarray(h, np.float32)
    n = h.size
    payload = np.full(h.shape, fill, np.uint8)
    scales = np.full(h.shape[:-1] + (h.shape[-1] // 32,), fill, np.uint8)
    faults = np.zeros(n // 32, np.uint32)
    LIB.orc_quant_v1(_p(h, _f32p), C.c_size_t(n), _p(payload, _u8p), _p(scales, _u8p), _p(faults, _u32p))
    return payload, scales, faults.reshape(scales.shape)


class Plan:
    def __init__(self, capacity: int):
        n = capacity * 8
        self.inverse = np.full(n, 0x5A5A5A5A, np.int32)
        self.original_routes = np.full(n, 0x5A5A5A5A, np.int32)
        self.grouped_weights = np.full(n, 123.0, np.float32)
        self.groups = np.zeros(n, GROUP_DTYPE)
        self.groups["expert"] = 0x5A5A5A5A
        self.group_count = np.full(1, 0x5A5A5A5A, np.uint32)
        self.fault = np.full(1, 0x5A5A5A5A, np.uint32)
        self.status = None


def _plan_call(fn, capacity, ids, weights, resident, out: Plan):
    ids = np.ascontiguousarray(ids, np.int32).reshape(-1)
    weights = np.ascontiguousarray(weights, np.float32).reshape(-1)
    rows = ids.size // 8
    if resident is None:
        resident = np.ones(256, np.uint8)
    resident = np.ascontiguousarray(resident, np.uint8)
    out.status = int(fn(C.c_uint32(capacity), C.c_uint32(rows), _p(ids, _i32p), _p(weights, _f32p), _p(resident, _u8p),
                        _p(out.inverse, _i32p), _p(out.original_routes, _i32p), _p(out.grouped_weights, _f32p),
                        out.groups.ctypes.data_as(C.c_void_p), _p(out.group_count, _u32p), _p(out.fault, _u32p)))
    return out


def plan(capacity, ids, weights, resident=None, out: Plan | None = None) -> Plan:
    return _plan_call(LIB.orc_plan, capacity, ids, weights, resident, out or Plan(capacity))


def prepared_g950(images) -> np.ndarray:
    """One expert's prepared image in the gfx950 operand order, from its one or four canonical
    quarter-slice images (crates/mimo26-expert/src/slice.rs:45-53), written as a forward map: every
    canonical byte (projection, row, byte of the row) computes where it goes. The library walks
    destination cells instead; the reference tests its own permutation the same two-sided way
    (crates/mimo26-expert/tests/b1/host.cpp:30-67). Raises if the map is not a bijection.

    Destination, I = 512 * len(images) intermediate columns, lane = 16 * (k-block % 4) + row % 16:
      gate/up payload  [I/256][32 k-steps][8 blocks][4 tiles][64 lanes][16 B], block = row // 32 (its set of
                       eight = block // 8, place in the set = block % 8), tile = (row % 32) // 16 + (2 for up)
      gate/up scales   [I/32][8][4 tiles][64 lanes][4 B], byte = k-step % 4 of quad k-step // 4
      down payload     [8][I/128 k-steps][8 blocks][4 tiles][64 lanes][16 B], block = row // 64,
                       tile = (row % 64) // 16
      down scales      [64][I/512][4 tiles][64 lanes][4 B]
    with k-block = k // 32 and k-step = k-block // 4; the down projection's K runs over the ranks."""
    ranks = len(images)
    inter = 512 * ranks
    w13, s13 = 0, inter * 4096
    w2 = s13 + inter * 256
    s2 = w2 + inter * 2048
    total = s2 + inter * 128
    out = np.zeros(total, np.uint8)
    hits = np.zeros(total, np.uint8)

    def put(dest, values):
        np.add.at(hits, dest.reshape(-1), 1)
        out[dest.reshape(-1)] = values.reshape(-1)

    for r, img in enumerate(images):
        img = np.ascontiguousarray(img, np.uint8)
        assert img.size == 3342336
        for up, (pay, sc) in enumerate(((0, 1048576), (1114112, 2162688))):
            n = (r * 512 + np.arange(512))[:, None]                      # intermediate column
            b = np.arange(2048)[None, :]                                # byte of the row, 16 per k-block
            kb, within = b // 16, b % 16
            lane = 16 * (kb % 4) + n % 16
            tile = (n % 32) // 16 + 2 * up
            put(w13 + ((((((n // 256) * 32 + kb // 4) * 8 + (n // 32) % 8) * 4 + tile) * 64 + lane) * 16 + within), img[pay:pay + 512 * 2048].reshape(512, 2048))
            kb = np.arange(128)[None, :]
            lane = 16 * (kb % 4) + n % 16
            step = kb // 4
            put(s13 + ((((n // 32) * 8 + step // 4) * 4 + tile) * 64 + lane) * 4 + step % 4, img[sc:sc + 512 * 128].reshape(512, 128))
        n = np.arange(4096)[:, None]                                    # output column
        b = np.arange(256)[None, :]
        kb, within = r * 16 + b // 16, b % 16
        lane = 16 * (kb % 4) + n % 16
        tile = (n % 64) // 16
        put(w2 + ((((((n // 512) * (inter // 128) + kb // 4) * 8 + (n // 64) % 8) * 4 + tile) * 64 + lane) * 16 + within), img[2228224:2228224 + 4096 * 256].reshape(4096, 256))
        kb = r * 16 + np.arange(16)[None, :]
        lane = 16 * (kb % 4) + n % 16
        step = kb // 4
        put(s2 + ((((n // 64) * (inter // 512) + step // 4) * 4 + tile) * 64 + lane) * 4 + step % 4, img[3276800:3276800 + 4096 * 16].reshape(4096, 16))
    if not np.all(hits == 1):
        raise AssertionError("prepared layout: the forward map is not a bijection")
    return out


def silu_up(g, u) -> np.ndarray:
    g = np.asarray(g, np.float32)
    u = np.asarray(u, np.float32)
    return np.array([LIB.orc_silu_up(float(a), float(b)) for a, b in zip(g.reshape(-1), u.reshape(-1))],
                    np.float32).reshape(g.shape)


def reduce(y: np.ndarray, w: np.ndarray):
    """y f32 [rows, 8, cols], w f32 [rows, 8] -> (status, partial f32 [rows, cols], bf16 u16)."""
    y = np.ascontiguousarray(y, np.float32)
    w = np.ascontiguousarray(w, np.float32)
    rows, _, cols = y.shape
    partial = np.zeros((rows, cols), np.float32)
    bf16 = np.zeros((rows, cols), np.uint16)
    st = LIB.orc_reduce(_p(y, _f32p), _p(w, _f32p), C.c_size_t(rows), C.c_size_t(cols), _p(partial, _f32p), _p(bf16, _u16p))
    return int(st), partial, bf16


def bf16_store_rows(y: np.ndarray) -> np.ndarray:
    """FC2's store rule of the BF16 per-route mode: FP32 -> BF16 bits (connected.cu:41-44)."""
    y = np.ascontiguousarray(y, np.float32)
    out = np.zeros(y.shape, np.uint16)
    LIB.orc_bf16_store_rows(_p(y, _f32p), C.c_size_t(y.size), _p(out, _u16p))
    return out


def reduce_bf16y(y16: np.ndarray, w: np.ndarray):
    """The combine over BF16 per-route rows [rows*8, cols] (b1_serve.cu:98-143): (status, bf16 [rows, cols])."""
    y16 = np.ascontiguousarray(y16, np.uint16)
    w = np.ascontiguousarray(w, np.float32).reshape(-1, 8)
    rows, cols = w.shape[0], y16.shape[-1]
    bf16 = np.zeros((rows, cols), np.uint16)
    st = LIB.orc_reduce_bf16y(_p(y16, _u16p), _p(w, _f32p), C.c_size_t(rows), C.c_size_t(cols), _p(bf16, _u16p))
    return int(st), bf16


def _layer(pools) -> _Layer:
    L = _Layer()
    for i, p in enumerate(pools):
        assert p.dtype == np.uint8 and p.flags.c_contiguous and p.size == EXPERTS * IMAGE_BYTES
        L.pool[i] = p.ctypes.data
    L.ranks = len(pools)
    return L


def expert_ffn(pools, expert: int, x_payload: np.ndarray, x_scales: np.ndarray):
    """One expert over the given activation rows. Returns a dict of every stage."""
    xp = np.ascontiguousarray(x_payload, np.uint8)
    xs = np.ascontiguousarray(x_scales, np.uint8)
    rows = xp.shape[0]
    inter = RANK_I * len(pools)
    out = dict(gate=np.zeros((rows, inter), np.float32), up=np.zeros((rows, inter), np.float32),
               h=np.zeros((rows, inter), np.float32), mid_payload=np.zeros((rows, inter), np.uint8),
               mid_scales=np.zeros((rows, inter // 32), np.uint8), y=np.zeros((rows, HIDDEN), np.float32))
    L = _layer(pools)
    out["fault"] = int(LIB.orc_expert_ffn(C.byref(L), C.c_uint32(expert), _p(xp, _u8p), C.c_size_t(xp.shape[1]),
                                          _p(xs, _u8p), C.c_size_t(xs.shape[1]), C.c_size_t(rows),
                                          _p(out["gate"], _f32p), _p(out["up"], _f32p), _p(out["h"], _f32p),
                                          _p(out["mid_payload"], _u8p), _p(out["mid_scales"], _u8p), _p(out["y"], _f32p)))
    return out


def layer_ffn(pools, x_payload, x_scales, ids, weights, threads: int = 0, want_routes: bool = False, efp32: bool = False):
    """Whole layer. Returns (rc, partial f32 [rows,4096], bf16 u16 [rows,4096], y_routes or None)."""
    xp = np.ascontiguousarray(x_payload, np.uint8)
    xs = np.ascontiguousarray(x_scales, np.uint8)
    ids = np.ascontiguousarray(ids, np.int32).reshape(-1)
    weights = np.ascontiguousarray(weights, np.float32).reshape(-1)
    rows = xp.shape[0]
    partial = np.zeros((rows, HIDDEN), np.float32)
    bf16 = np.zeros((rows, HIDDEN), np.uint16)
    L = _layer(pools)
    if efp32:
        rc = LIB.orc_layer_ffn_efp32(C.byref(L), _p(xp, _u8p), C.c_size_t(xp.shape[1]), _p(xs, _u8p), C.c_size_t(xs.shape[1]),
                                     _p(ids, _i32p), _p(weights, _f32p), C.c_size_t(rows), _p(partial, _f32p),
                                     _p(bf16, _u16p), C.c_int(threads))
        return int(rc), partial, bf16, None
    yr = np.zeros((rows * 8, HIDDEN), np.float32) if want_routes else None
    rc = LIB.orc_layer_ffn(C.byref(L), _p(xp, _u8p), C.c_size_t(xp.shape[1]), _p(xs, _u8p), C.c_size_t(xs.shape[1]),
                           _p(ids, _i32p), _p(weights, _f32p), C.c_size_t(rows), _p(yr, _f32p), _p(partial, _f32p),
                           _p(bf16, _u16p), C.c_int(threads))
    return int(rc), partial, bf16, yr


# ---- the reference's own host units, where built (differential checks only) -------------------
_REF_PATH = os.path.join(HERE, "_ref", "libb1ref.so")


def ref_available() -> bool:
    """True where the reference's host units were built; asking does not load them."""
    return os.path.exists(_REF_PATH)


def _load_ref():
    if not ref_available():
        return None
    lib = C.CDLL(_REF_PATH)
    lib.ref_mxfp4_bits.restype = C.c_uint32
    lib.ref_mxfp4_bits.argtypes = [C.c_uint32, C.c_uint32]
    for f in (lib.ref_quant_v1, lib.ref_plan, lib.ref_reduce):
        f.restype = C.c_uint32
    return lib


_REF = None


def __getattr__(name):
    """`REF` is loaded on first use, so a process that only runs the GPU parity tests never maps it."""
    global _REF
    if name == "REF":
        if _REF is None:
            _REF = _load_ref()
        return _REF
    raise AttributeError(name)


def ref_quant_v1(h: np.ndarray, fill: int = 0xA5):
    h = np.ascontiguousarray(h, np.float32)
    n = h.size
    payload = np.full(h.shape, fill, np.uint8)
    scales = np.full(h.shape[:-1] + (h.shape[-1] // 32,), fill, np.uint8)
    faults = np.zeros(n // 32, np.uint32)
    st = __getattr__("REF").ref_quant_v1(_p(h, _f32p), C.c_uint64(n), _p(payload, _u8p), _p(scales, _u8p), _p(faults, _u32p))
    return payload, scales, faults.reshape(scales.shape), int(st)


def ref_plan(capacity, ids, weights, resident=None, out: Plan | None = None) -> Plan:
    return _plan_call(__getattr__("REF").ref_plan, capacity, ids, weights, resident, out or Plan(capacity))


def ref_reduce(y: np.ndarray, w: np.ndarray):
    y = np.ascontiguousarray(y, np.float32)
    w = np.ascontiguousarray(w, np.float32)
    rows = y.shape[0]
    partial = np.zeros((rows, HIDDEN), np.float32)
    bf16 = np.zeros((rows, HIDDEN), np.uint16)
    fault = np.zeros(1, np.uint32)
    st = __getattr__("REF").ref_reduce(_p(y, _f32p), _p(w, _f32p), C.c_uint32(rows), _p(partial, _f32p), _p(bf16, _u16p), _p(fault, _u32p))
    return int(st), partial, bf16
