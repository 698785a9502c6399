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


def every_row(layer, ranks, pools, rows, count, alpha, seed):
    ids = routed(seed, rows, count, alpha)
    w, x = synth._softmax_weights(seed, rows), synth._activations(seed, rows)
    payload, scales = synth.q0_quantize(x)
    wl = synth.Workload(f"sweep {rows}x{count}", 3 if ranks == 4 else 1, seed, ranks, rows, ids, w, x, payload, scales)
    scratch = b1.Scratch()
    _, bf, pf = run_ffn_dev(layer, scratch, wl)
    _, bf2, pf2 = run_ffn_dev(layer, scratch, wl)
    rc, ref_partial, _, _ = O.layer_ffn(pools, wl.payload, wl.scales, wl.ids, wl.weights)
    assert rc == 0
    ma, mr = parity(pf, ref_partial)
    worst = np.abs(pf - ref_partial).max(axis=1) / np.abs(ref_partial).max()
    what = (rows, count, alpha, chunk_classes(ids))
    assert ma <= MAX_ABS and mr <= MEAN_REL, (what, ma, mr, int(worst.argmax()))
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
