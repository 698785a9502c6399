"""Seeded synthetic workloads of the routed-expert FFN (weights, activations, routing).

Everything derives from one counter-based splitmix64 stream (the generator the reference's GPU
step harness uses, crates/mimo26-expert/tests/gpu/step_hist.h:36-38), so any slice of any array
can be regenerated on its own: element i of stream `key` is mix(key + (i + 1) * GOLDEN).

Weights follow the quarter-slice image v2 of the reference (crates/mimo26-expert/src/slice.rs:33-53):
payload bytes uniform (two uniform E2M1 codes each), E8M0 scale bytes uniform in 119..123
(2^-8..2^-4). Activations are bf16-valued normals pushed through the coordinator's wire
quantizer (crates/mimo26-coordinator/src/wire.rs:53-78, crates/mimo26-load/src/e4m3.rs:50-81):
that quantizer sits upstream of the expert-rank boundary, so it lives here with the inputs.
"""
from __future__ import annotations

from dataclasses import dataclass

import numpy as np

HIDDEN, EXPERTS, TOPK, RANK_I = 4096, 256, 8, 512
IMAGE_BYTES = 3342336
GATE_SCALES, UP_PAYLOAD, UP_SCALES, DOWN_PAYLOAD, DOWN_SCALES = 1048576, 1114112, 2162688, 2228224, 3276800
SCALE_REGIONS = ((GATE_SCALES, UP_PAYLOAD), (UP_SCALES, DOWN_PAYLOAD), (DOWN_SCALES, IMAGE_BYTES))
BASE_SEED = 0x26AFD
_GOLDEN = np.uint64(0x9E3779B97F4A7C15)
_M1, _M2 = np.uint64(0xBF58476D1CE4E5B9), np.uint64(0x94D049BB133111EB)
# sub-streams by purpose
WEIGHTS, ACTIVATIONS, OUTLIERS, ROUTES, LOGITS, SHUFFLE = range(1, 7)


def _mix(z: np.ndarray) -> np.ndarray:
    z = (z ^ (z >> np.uint64(30))) * _M1
    z = (z ^ (z >> np.uint64(27))) * _M2
    return z ^ (z >> np.uint64(31))


def stream_key(seed: int, purpose: int, a: int = 0, b: int = 0) -> np.uint64:
    """A well-separated stream start for (purpose, a, b) under `seed`."""
    with np.errstate(over="ignore"):
        k = np.uint64(seed) ^ (np.uint64(purpose) * np.uint64(0xD1B54A32D192ED03))
        k = _mix(np.array([k], np.uint64))[0] ^ (np.uint64(a + 1) * _M2)
        k = _mix(np.array([k], np.uint64))[0] ^ (np.uint64(b + 1) * _M1)
        return _mix(np.array([k], np.uint64))[0]


def u64(key: np.uint64, count: int, start: int = 0) -> np.ndarray:
    with np.errstate(over="ignore"):
        i = np.arange(start + 1, start + count + 1, dtype=np.uint64)
        return _mix(key + i * _GOLDEN)


def uniform(key, count, start=0) -> np.ndarray:
    """Doubles in (0, 1]."""
    return ((u64(key, count, start) >> np.uint64(11)).astype(np.float64) + 1.0) * 2.0 ** -53


def normal(key, count) -> np.ndarray:
    """Box-Muller over consecutive pairs of the stream; float64."""
    u = uniform(key, 2 * count)
    return np.sqrt(-2.0 * np.log(u[0::2])) * np.cos(2.0 * np.pi * u[1::2])


def bf16_round(x: np.ndarray) -> np.ndarray:
    """float32 -> nearest-even bf16 -> float32."""
    b = np.ascontiguousarray(x, np.float32).view(np.uint32).astype(np.uint64)
    r = ((b + 0x7FFF + ((b >> 16) & 1)) & 0xFFFF0000).astype(np.uint32)
    return r.view(np.float32).reshape(np.shape(x))


# ---- weights ---------------------------------------------------------------------------------
def expert_image(seed: int, rank: int, expert: int, layer: int = 0) -> np.ndarray:
    """One quarter-slice image v2 (3,342,336 bytes) of `expert` of `layer` for TP4 rank `rank`."""
    raw = u64(stream_key(seed, WEIGHTS, rank, layer * EXPERTS + expert), IMAGE_BYTES // 8).view(np.uint8).copy()
    for lo, hi in SCALE_REGIONS:
        raw[lo:hi] = 119 + ((raw[lo:hi].astype(np.uint16) * 5) >> 8).astype(np.uint8)
    return raw


def rank_pool(seed: int, rank: int, experts=range(EXPERTS), out: np.ndarray | None = None) -> np.ndarray:
    """256 images back to back (855,638,016 bytes): what one rank hands to layer_new. Images of
    experts outside `experts` are left as they are in `out` (bytes 0x22 in a fresh pool: code 1.0,
    scale 2^-93, legal everywhere)."""
    pool = np.full(EXPERTS * IMAGE_BYTES, 0x22, np.uint8) if out is None else out
    for e in experts:
        pool[e * IMAGE_BYTES:(e + 1) * IMAGE_BYTES] = expert_image(seed, rank, e)
    return pool


# ---- the wire input quantizer ------------------------------------------------------------------
def q0_quantize(x: np.ndarray):
    """f32 [rows, cols] -> (E4M3 payload u8 [rows, cols], UE8M0 K32 scales u8 [rows, cols/32]).

    Per 32 values: s = 0 for an all-zero block, else clamp(ceil(log2(amax/448)) + 127, 0, 254);
    payload = nearest E4M3 of v * 2^(127-s), ties to the larger magnitude, saturating at 448,
    NaN -> 0, sign bit set when the value is below zero.
    """
    x = np.ascontiguousarray(x, np.float32)
    rows, cols = x.shape
    xb = x.reshape(rows, cols // 32, 32).astype(np.float64)
    amax = np.max(np.abs(np.nan_to_num(xb, nan=0.0)), axis=-1)
    m, e = np.frexp(amax)
    s = np.where(amax > 0, np.where(m <= 0.875, e - 9, e - 8) + 127, 0)
    s = np.clip(np.where(np.isinf(amax), 254, s), 0, 254).astype(np.int64)
    y = np.ldexp(np.nan_to_num(xb, nan=0.0), (127 - s)[..., None])
    mag = np.minimum(np.abs(y), 448.0)
    sign = np.where(y < 0, 0x80, 0)
    sub = mag < 2.0 ** -6
    m_sub = np.minimum(np.floor(mag * 512.0 + 0.5), 8).astype(np.int64)  # 8 is the first normal code
    f, g = np.frexp(np.where(sub, 1.0, mag))
    ef = g.astype(np.int64) + 6
    mant = np.floor((2.0 * f - 1.0) * 8.0 + 0.5).astype(np.int64)
    carry = mant >= 8
    ef = np.clip(np.where(carry, ef + 1, ef), 1, 15)
    mant = np.clip(np.where(carry, 0, mant), 0, 7)
    code = np.where(sub, m_sub, (ef << 3) | mant)
    code = np.where(mag == 0, 0, code) | sign
    return code.astype(np.uint8).reshape(rows, cols), s.astype(np.uint8)


# ---- routing -------------------------------------------------------------------------------------
def _softmax_weights(seed: int, rows: int) -> np.ndarray:
    z = normal(stream_key(seed, LOGITS), rows * TOPK).reshape(rows, TOPK)
    z = np.exp(z - z.max(axis=1, keepdims=True))
    return (z / z.sum(axis=1, keepdims=True)).astype(np.float32)


def _uniform_keys(seed, purpose, rows, a=0) -> np.ndarray:
    return u64(stream_key(seed, purpose, a), rows * EXPERTS).reshape(rows, EXPERTS)


def routes_uniform(seed: int, rows: int) -> np.ndarray:
    """Per token 8 distinct experts, uniform."""
    return np.argsort(_uniform_keys(seed, ROUTES, rows), axis=1, kind="stable")[:, :TOPK].astype(np.int32)


def routes_streams(seed: int, streams: int, positions: int, shared: int = 6) -> np.ndarray:
    """Tokens of one stream share `shared` experts; each token adds distinct others; slots shuffled."""
    rows = streams * positions
    per_stream = np.argsort(_uniform_keys(seed, ROUTES, streams), axis=1, kind="stable")[:, :shared]
    order = np.argsort(_uniform_keys(seed, ROUTES, rows, 1), axis=1, kind="stable")
    ids = np.empty((rows, TOPK), np.int32)
    for t in range(rows):
        mine = per_stream[t // positions]
        extra = [e for e in order[t] if e not in mine][:TOPK - shared]
        ids[t] = np.concatenate([mine, extra])
    shuffle = np.argsort(u64(stream_key(seed, SHUFFLE), rows * TOPK).reshape(rows, TOPK), axis=1, kind="stable")
    return np.take_along_axis(ids, shuffle, axis=1)


def routes_zipf(seed: int, rows: int, s: float = 1.1) -> np.ndarray:
    """Zipf(s) popularity over a random permutation of expert ids, 8 without replacement per token
    (exponential-key sampling: the 8 smallest of -ln(u)/p)."""
    perm = np.argsort(u64(stream_key(seed, ROUTES, 2), EXPERTS), kind="stable")
    p = 1.0 / np.arange(1, EXPERTS + 1, dtype=np.float64) ** s
    p /= p.sum()
    keys = -np.log(uniform(stream_key(seed, ROUTES), rows * EXPERTS)).reshape(rows, EXPERTS) / p
    ranks = np.argsort(keys, axis=1, kind="stable")[:, :TOPK]
    return perm[ranks].astype(np.int32)


# ---- configurations -------------------------------------------------------------------------------
@dataclass
class Workload:
    name: str
    config: int
    seed: int
    ranks: int            # 1 = one TP4 rank's share (I = 512), 4 = full intermediate
    rows: int
    ids: np.ndarray       # i32 [rows, 8]
    weights: np.ndarray   # f32 [rows, 8]
    x: np.ndarray         # f32 [rows, 4096], bf16-valued
    payload: np.ndarray   # u8  [rows, 4096]
    scales: np.ndarray    # u8  [rows, 128]

    @property
    def intermediate(self) -> int:
        return RANK_I * self.ranks

    def touched(self) -> np.ndarray:
        return np.unique(self.ids)

    def pools(self, experts=None):
        """Canonical rank pools (list of `ranks` arrays); only `experts` are filled when given."""
        experts = range(EXPERTS) if experts is None else experts
        return [rank_pool(self.seed, r, experts) for r in range(self.ranks)]

    def algorithmic_bytes(self) -> int:
        """Unique weight bytes of the touched experts + input rows + ids/weights + BF16 output rows."""
        per_expert = IMAGE_BYTES * self.ranks
        return int(self.touched().size * per_expert + self.rows * (4224 + 64 + 8192))

    def flops(self) -> int:
        return 6 * self.rows * TOPK * HIDDEN * self.intermediate


def _activations(seed: int, rows: int, sigma: float = 1.0, outliers: float = 0.0) -> np.ndarray:
    x = normal(stream_key(seed, ACTIVATIONS), rows * HIDDEN) * sigma
    if outliers:
        u = uniform(stream_key(seed, OUTLIERS), rows * HIDDEN)
        x = np.where(u <= outliers, np.where(u <= outliers / 2, 40.0, -40.0), x)
    return bf16_round(x.astype(np.float32)).reshape(rows, HIDDEN)


def make(config: int, rows: int | None = None) -> Workload:
    """The benchmark configurations 0..3 (rows can be overridden for reduced parity cases)."""
    seed = BASE_SEED + config
    if config == 0:  # one expert, one rank's share, 16 rows: every token's slot 0 is expert 0
        rows = rows or 16
        ids = np.tile(np.arange(TOPK, dtype=np.int32), (rows, 1))
        w = np.zeros((rows, TOPK), np.float32)
        w[:, 0] = 1.0
        x = _activations(seed, rows)
        name, ranks = "single expert, rank share, 16 rows", 1
    elif config == 1:
        rows = rows or 16
        ids, w, x = routes_uniform(seed, rows), _softmax_weights(seed, rows), _activations(seed, rows)
        name, ranks = "decode, 256 experts x rank share, 16 tokens", 1
    elif config == 2:
        rows = rows or 128
        ids, w, x = routes_streams(seed, rows // 8, 8), _softmax_weights(seed, rows), _activations(seed, rows)
        name, ranks = "decode/verify, 256 experts x I 2048, 128 tokens", 4
    elif config == 3:
        rows = rows or 8192
        ids, w = routes_zipf(seed, rows), _softmax_weights(seed, rows)
        x = _activations(seed, rows, sigma=1.5, outliers=1e-3)
        name, ranks = "prefill chunk, 256 experts x I 2048, 8192 tokens, Zipf(1.1)", 4
    else:
        raise ValueError(f"unknown config {config}")
    payload, scales = q0_quantize(x)
    return Workload(name, config, seed, ranks, rows, ids, w, x, payload, scales)
