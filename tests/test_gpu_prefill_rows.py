"""configs[3] in full: every one of the 8192 rows of the prefill chunk against the CPU rule, as the reference's
gate checks every coordinate of its run (crates/mimo26-expert/tests/b1_core/bench_connected.cuh:56-63). The GPU
call runs once; the CPU rule takes the rows in eight blocks of 1024 so that no single test is silent for long.
A deterministic error on any row of any chunk fails here; the sampled test of test_gpu_ffn.py would not see it."""
import numpy as np
import pytest

import b1_oracle as O
from helpers import bf16_to_f32, parity

pytestmark = pytest.mark.gpu
MAX_ABS, MEAN_REL = 1e-2, 1e-3
BLOCK = 1024


@pytest.mark.parametrize("block", range(8192 // BLOCK))
def test_every_row_of_the_prefill_chunk(full_layer, prefill_chunk_on_gpu, block):
    _, pools, _ = full_layer
    wl, bf, pf = prefill_chunk_on_gpu
    rows = slice(block * BLOCK, (block + 1) * BLOCK)
    rc, ref_partial, ref_bf16, _ = O.layer_ffn(pools, wl.payload[rows], wl.scales[rows], wl.ids[rows], wl.weights[rows])
    assert rc == 0
    ma, mr = parity(pf[rows], ref_partial)
    assert ma <= MAX_ABS and mr <= MEAN_REL, ("fp32 sums", block, ma, mr)
    ma, mr = parity(bf16_to_f32(bf[rows]), bf16_to_f32(ref_bf16))
    assert ma <= MAX_ABS and mr <= MEAN_REL, ("bf16 rows", block, ma, mr)
    per_row = np.abs(pf[rows].astype(np.float64) - ref_partial).max(axis=1) / np.abs(ref_partial).max()
    assert per_row.max() <= MAX_ABS, ("worst row", block * BLOCK + int(per_row.argmax()), float(per_row.max()))
    row_rel = np.abs(pf[rows].astype(np.float64) - ref_partial).sum(axis=1) / np.abs(ref_partial).sum(axis=1)
    assert np.median(row_rel) <= MEAN_REL and np.mean(bf[rows] == ref_bf16) > 0.8, (block, float(np.median(row_rel)))
