"""The router-weighted combine on the GPU in its three forms, through the C ABI.

Default: a launch of its own behind FC2, as the reference runs it
(crates/mimo26-spark/kernels/b1_serve.cu:502-515). `fused_combine`: inside FC2 (the wave that writes a token's
eighth per-route row sums the eight, in slot order). The two must give the same bits everywhere: the sum's
order is fixed by the slots, and integer counts decide only which wave performs it.
`bf16_route_rows`: the reference's opt-in numerical mode MIMO26_B1_Y=bf16 (b1_serve.cu:98-143,400-405),
against the CPU rule for it (orc_bf16_store_rows, orc_reduce_bf16y), bit for bit on the GPU's own rows.
"""
import numpy as np
import pytest

import b1_oracle as O
from helpers import DeviceLayer, bf16_to_f32, parity, run_ffn_dev
from mimo26f_afd_amd import b1, synth

pytestmark = pytest.mark.gpu


def subset(wl, pick, name):
    return synth.Workload(name, wl.config, wl.seed, wl.ranks, len(pick), wl.ids[pick], wl.weights[pick], wl.x[pick],
                          wl.payload[pick], wl.scales[pick])


def both_forms(layer, wl):
    fused, apart = b1.Scratch(), b1.Scratch()
    fused.set_option("fused_combine", True)
    s1, bf1, pf1 = run_ffn_dev(layer, fused, wl)
    s2, bf2, pf2 = run_ffn_dev(layer, apart, wl)
    if wl.rows >= 4096:  # no combine launch in the fused form: nothing lies between the FC2 event and the end event
        assert s1.phase_ms[3] < 0.02 < s2.phase_ms[3], (s1.phase_ms, s2.phase_ms)
    y1 = fused.view("y", np.float32, wl.rows * 8 * 4096)
    y2 = apart.view("y", np.float32, wl.rows * 8 * 4096)
    return (bf1, pf1, y1), (bf2, pf2, y2), fused


def test_fused_combine_gives_the_separate_combine_bits_at_every_schedule(full_layer):
    """Decode schedule with one and two activation tiles, the tile schedule with every chunk class, and the planner
    over several compute units: BF16 rows, FP32 sums and per-route rows identical between the two forms, and the
    fused form's output is the CPU rule's combine of the GPU's own per-route rows."""
    wl, _, layer = full_layer
    big = synth.make(3)
    cases = [subset(wl, np.arange(5), "5 rows"), subset(wl, np.arange(37) * 3 % wl.rows, "37 rows"), wl,
             subset(big, np.arange(130), "130 rows"), subset(big, np.arange(700) * 11 % big.rows, "700 rows")]
    for case in cases:
        (bf1, pf1, y1), (bf2, pf2, y2), _ = both_forms(layer, case)
        assert np.array_equal(y1.view(np.uint32), y2.view(np.uint32)), case.name
        assert np.array_equal(bf1, bf2) and np.array_equal(pf1.view(np.uint32), pf2.view(np.uint32)), case.name
        st, want_p, want_b = O.reduce(y1.reshape(case.rows, 8, 4096), case.weights)
        assert st == 0 and np.array_equal(want_b, bf1) and np.array_equal(want_p.view(np.uint32), pf1.view(np.uint32)), case.name


def test_fused_combine_at_rank_share_and_without_the_fp32_sum():
    wl = synth.make(1)
    layer = DeviceLayer(wl.pools(wl.touched())).layer
    (bf1, pf1, y1), (bf2, pf2, _), fused = both_forms(layer, wl)
    assert np.array_equal(bf1, bf2) and np.array_equal(pf1.view(np.uint32), pf2.view(np.uint32))
    _, bf3, _ = run_ffn_dev(layer, fused, wl, want_partial=False)
    assert np.array_equal(bf3, bf1)


def test_fused_combine_on_the_whole_prefill_chunk(full_layer):
    """configs[3], all 8192 tokens: 65,536 per-route rows handed between workgroups on eight XCDs. Both forms bit for
    bit, the fused form twice."""
    _, _, layer = full_layer
    wl = synth.make(3)
    (bf1, pf1, y1), (bf2, pf2, y2), fused = both_forms(layer, wl)
    assert np.array_equal(y1.view(np.uint32), y2.view(np.uint32))
    assert np.array_equal(bf1, bf2) and np.array_equal(pf1.view(np.uint32), pf2.view(np.uint32))
    _, bf3, pf3 = run_ffn_dev(layer, fused, wl)
    assert np.array_equal(bf3, bf1) and np.array_equal(pf3.view(np.uint32), pf1.view(np.uint32))


def test_fused_combine_reports_the_combine_fault(full_layer):
    """A sum that leaves binary32's finite range raises the combine's fault word, from the separate launch and
    from inside FC2 alike (return code 4, 'reduce fault')."""
    wl, _, layer = full_layer
    few = subset(wl, np.arange(4), "overflowing weights")
    few.weights[:] = np.float32(3.0e38)                                  # legal weights (finite, non-negative) whose products overflow
    for fuse in (False, True):
        s = b1.Scratch()
        s.set_option("fused_combine", fuse)
        with pytest.raises(b1.B1Error, match="reduce fault") as e:
            run_ffn_dev(layer, s, few)
        assert e.value.code == 4


def test_bf16_route_rows_mode(full_layer):
    """The opt-in mode: per-route rows equal the store rule applied to the FP32 rows of the default mode, the output
    equals the CPU rule's BF16 combine of those rows bit for bit (fused and separate), and it stays inside the
    output bars of the full CPU rule while differing from the default mode."""
    wl, pools, layer = full_layer
    big = synth.make(3)
    for case in (wl, subset(big, np.arange(700) * 11 % big.rows, "700 rows")):
        plain = b1.Scratch()
        _, bf_plain, _ = run_ffn_dev(layer, plain, case)
        y32 = plain.view("y", np.float32, case.rows * 8 * 4096).reshape(case.rows * 8, 4096)
        want_rows = O.bf16_store_rows(y32)
        st, want = O.reduce_bf16y(want_rows, case.weights)
        assert st == 0
        for fuse in (False, True):
            s = b1.Scratch()
            s.set_option("bf16_route_rows", True)
            s.set_option("fused_combine", fuse)
            _, bf, _ = run_ffn_dev(layer, s, case, want_partial=False)
            rows16 = s.view("y", np.uint16, case.rows * 8 * 4096).reshape(case.rows * 8, 4096)
            assert np.array_equal(rows16, want_rows), (case.name, fuse)
            assert np.array_equal(bf, want), (case.name, fuse)
        assert not np.array_equal(bf, bf_plain)                              # a numerical-mode change, not the default
        rc, _, ref_bf16, _ = O.layer_ffn(pools, case.payload, case.scales, case.ids, case.weights)
        ma, mr = parity(bf16_to_f32(bf), bf16_to_f32(ref_bf16))
        assert rc == 0 and ma <= 1e-2 and mr <= 2e-3, (ma, mr)               # BF16 rows add up to 2^-9 relative per route


def test_bf16_route_rows_on_the_conforming_arm():
    """A layer with exceptional weight scales combines separately in either mode; BF16 rows there too."""
    wl = synth.make(1)
    pools = wl.pools(wl.touched())
    e = int(wl.ids[0, 0])
    pools[0][e * synth.IMAGE_BYTES + synth.GATE_SCALES] = 1                 # one scale byte outside [2, 252]
    layer = DeviceLayer(pools).layer
    assert not layer.all_scales_normal()
    plain, mode = b1.Scratch(), b1.Scratch()
    mode.set_option("bf16_route_rows", True)
    _, bf_plain, _ = run_ffn_dev(layer, plain, wl)
    y32 = plain.view("y", np.float32, wl.rows * 8 * 4096).reshape(wl.rows * 8, 4096)
    _, bf, _ = run_ffn_dev(layer, mode, wl, want_partial=False)
    st, want = O.reduce_bf16y(O.bf16_store_rows(y32), wl.weights)
    assert st == 0 and np.array_equal(bf, want)
