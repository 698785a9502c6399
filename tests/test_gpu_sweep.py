"""Sizes and routings between the benchmark configurations, every row against the CPU reference.

The configurations fix a handful of shapes; a schedule can be right on all of them and wrong on a chunk
class they happen not to hold (a chunk of exactly four groups at the full intermediate was, for a while).
Each case here draws its experts, its skew and its row count from a seeded generator, names the chunk
classes it produced, and checks every row of the output (and a second run, bit for bit), at the full
intermediate and at one rank's share."""
import numpy as np
import pytest

import b1_oracle as O
from helpers import DeviceLayer, parity, run_ffn_dev
from mimo26f_afd_amd import b1, synth

pytestmark = pytest.mark.gpu
MAX_ABS, MEAN_REL = 1e-2, 1e-3

# (rows, experts in use, Zipf exponent of the routing)
FULL = [(200, 40, 1.1), (333, 20, 1.6), (520, 8, 1.6), (150, 12, 0.0), (1000, 256, 1.1)]
RANK = [(129, 100, 0.6), (777, 20, 0.6), (2500, 40, 1.6)]


@pytest.fixture(scope="module")
def pools():
    return synth.make(2).pools()


def routed(seed, rows, count, alpha):
    rng = np.random.default_rng(seed)
    experts = np.sort(rng.choice(256, count, replace=False)).astype(np.int32)
    p = 1.0 / np.arange(1, count + 1) ** alpha
    order = np.argsort(-np.log(rng.random((rows, count))) / p, axis=1, kind="stable")[:, :8]
    return experts[order]


def chunk_classes(ids):
    groups = (np.bincount(ids.reshape(-1), minlength=256) + 15) // 16
    return sorted({int(c) for g in groups[groups > 0] for c in [8] * (g // 8) + ([g % 8] if g % 8 else [])})


DOWN, DOWN_SCALES = 2228224, 3276800  # the down projection inside a quarter-slice image: u8[4096][256], u8[4096][16]


def down_weights(pools, expert):
    """The expert's decoded down projection, f64 [4096, 512 * ranks] (each rank image holds 512 of the K columns)."""
    parts = []
    for pool in pools:
        img = pool[expert * synth.IMAGE_BYTES:(expert + 1) * synth.IMAGE_BYTES]
        parts.append(O.mxfp4_rows(img[DOWN:DOWN + 4096 * 256].reshape(4096, 256),
                                  img[DOWN_SCALES:DOWN_SCALES + 4096 * 16].reshape(4096, 16)))
    return np.concatenate(parts, axis=1).astype(np.float64)


def one_code_apart(a, b):
    """E4M3 codes that are neighbours on the grid (same sign, magnitude codes differing by one)."""
    return (a ^ b) & 0x80 == 0 and abs(int(a & 0x7f) - int(b & 0x7f)) == 1


def explained_by_boundary_flips(scratch, stats, wl, pools, row, inter):
    """A row beyond the max-abs bar is accepted when it is this and nothing else: the requantised intermediate
    of one of its routes differs from the CPU rule's in a few bytes, each by one E4M3 code (an h on a rounding
    boundary went the other way: gate and up carry the FP32 accumulation error), the scales are identical, and
    every route's row is the exact product of the GPU's own intermediate bytes with the expert's decoded down
    weights. Returns the number of differing bytes over the row's eight routes, or raises."""
    n = wl.rows * 8
    groups = scratch.view("groups", O.GROUP_DTYPE, stats.groups)
    inverse = scratch.view("inverse", np.int32, n)
    rows_all = stats.groups * 16
    mp = scratch.view("mid_payload", np.uint8, rows_all * inter).reshape(rows_all, inter)
    ms = scratch.view("mid_scales", np.uint8, rows_all * inter // 32).reshape(rows_all, inter // 32)
    y = scratch.view("y", np.float32, n * 4096).reshape(wl.rows, 8, 4096)
    flipped = 0
    for slot in range(8):
        pos = int(inverse[row * 8 + slot])
        gi = int(np.searchsorted(groups["route_base"], pos, side="right") - 1)
        grow = gi * 16 + pos - int(groups["route_base"][gi])
        expert = int(wl.ids[row, slot])
        assert int(groups["expert"][gi]) == expert
        want = O.expert_ffn(pools, expert, wl.payload[row:row + 1], wl.scales[row:row + 1])
        assert want["fault"] == 0 and np.array_equal(ms[grow], want["mid_scales"][0]), (row, slot, "scales differ")
        differ = np.nonzero(mp[grow] != want["mid_payload"][0])[0]
        assert len(differ) <= 4 and all(one_code_apart(mp[grow][k], want["mid_payload"][0][k]) for k in differ), \
            (row, slot, "intermediate differs by more than neighbouring codes", differ[:8])
        flipped += len(differ)
        own = O.activation_decode(mp[grow:grow + 1], ms[grow:grow + 1])[0][0].astype(np.float64)
        exact = down_weights(pools, expert) @ own
        got = y[row, slot].astype(np.float64)
        assert np.max(np.abs(got - exact)) <= 1e-4 * np.max(np.abs(exact)), (row, slot, "FC2 is not the product of its own inputs")
    return flipped


def every_row(layer, ranks, pools, rows, count, alpha, seed, flips=None):
    ids = routed(seed, rows, count, alpha)
    w, x = synth._softmax_weights(seed, rows), synth._activations(seed, rows)
    payload, scales = synth.q0_quantize(x)
    wl = synth.Workload(f"sweep {rows}x{count}", 3 if ranks == 4 else 1, seed, ranks, rows, ids, w, x, payload, scales)
    scratch = b1.Scratch()
    stats, bf, pf = run_ffn_dev(layer, scratch, wl)
    rc, ref_partial, _, _ = O.layer_ffn(pools, wl.payload, wl.scales, wl.ids, wl.weights)
    assert rc == 0
    ma, mr = parity(pf, ref_partial)
    worst = np.abs(pf - ref_partial).max(axis=1) / np.abs(ref_partial).max()
    what = (rows, count, alpha, chunk_classes(ids))
    assert mr <= MEAN_REL, (what, ma, mr)
    beyond = np.nonzero(worst > MAX_ABS)[0]
    assert len(beyond) <= 2 and ma <= 2 * MAX_ABS, (what, ma, mr, beyond[:8])
    for row in beyond:  # rare: about one case in a hundred holds one such row
        found = explained_by_boundary_flips(scratch, stats, wl, pools, int(row), 512 * ranks)
        assert found >= 1, (what, int(row), "beyond the bar with an intermediate identical to the CPU rule's")
        if flips is not None:
            flips.append((what, int(row), float(worst[row]), found))
    _, bf2, pf2 = run_ffn_dev(layer, scratch, wl)
    assert np.array_equal(bf2, bf) and np.array_equal(pf2.view(np.uint32), pf.view(np.uint32)), what
    return chunk_classes(ids)


def test_full_intermediate_every_row(pools):
    layer = DeviceLayer(pools).layer
    seen = set()
    for n, (rows, count, alpha) in enumerate(FULL):
        seen |= set(every_row(layer, 4, pools, rows, count, alpha, synth.BASE_SEED + 300 + n))
    assert seen == set(range(1, 9)), seen  # chunks of every size from one group to eight


def test_rank_share_every_row(pools):
    one = [pools[1]]
    layer = DeviceLayer(one).layer
    seen = set()
    for n, (rows, count, alpha) in enumerate(RANK):
        seen |= set(every_row(layer, 1, one, rows, count, alpha, synth.BASE_SEED + 400 + n))
    assert seen == set(range(1, 9)), seen


def test_a_row_beyond_the_bar_is_a_boundary_flip_or_a_failure(pools):
    """Routings found by longer sweeps (989 cases) that hold one row between 1.0e-2 and 1.4e-2 of max|ref|: the
    sweep accepts such a row only after showing what it is. Between 128 and 256 the E4M3 step is 16 and the largest
    down weight 0.375: one code of one intermediate element moves its route's row by up to 6.0, and a route weighted
    above a third carries that past a hundredth of max|ref|. Prefill size at the full intermediate, decode size at one
    rank's share."""
    flips = []
    every_row(DeviceLayer(pools).layer, 4, pools, 1200, 8, 2.2, 105450157, flips)
    one = [pools[2]]
    every_row(DeviceLayer(one).layer, 1, one, 33, 64, 2.2, 291852939, flips)
    assert len(flips) == 2 and all(MAX_ABS < worst < 2 * MAX_ABS and 1 <= found <= 16 for _, _, worst, found in flips), flips  # found: bytes over the row's eight routes

