"""GPU parity of the whole path through the C ABI against the CPU checker.

Bars (the benchmark contract): bucketing and codec bytes bit-exact; outputs within
max-abs <= 1e-2 * max|ref| and mean-rel <= 1e-3 of the CPU W4A8 reference, because the MFMA's FP32
accumulation order differs from an FP64 dot. The requantised bytes are compared on the h the GPU
reports, the reference's own rule (crates/mimo26-repack/tests/lattice_compare.py:105-108).
"""
import numpy as np
import pytest

import b1_oracle as O
from helpers import DeviceLayer, bf16_to_f32, parity, run_ffn_dev
from mimo26f_afd_amd import b1, synth
from test_oracle_path import closed_form_image, closed_form_rows, exact_projection

pytestmark = pytest.mark.gpu
MAX_ABS, MEAN_REL = 1e-2, 1e-3
# FP32 accumulation bound for one output: one rounding per 128-wide k-step plus the MFMA's internal
# sum, against the FP64 ideal: a small multiple of 2^-24 times the sum of |products|.
SILU_ULPS = 8.0
ACC_EPS = 8 * 2.0 ** -24


def check_outputs(got_partial, got_bf16, ref_partial, ref_bf16):
    ma, mr = parity(got_partial, ref_partial)
    assert ma <= MAX_ABS and mr <= MEAN_REL, ("fp32 rank sum", ma, mr)
    ma, mr = parity(bf16_to_f32(got_bf16), bf16_to_f32(ref_bf16))
    assert ma <= MAX_ABS and mr <= MEAN_REL, ("bf16 rows", ma, mr)
    return ma, mr


def check_stages(scratch, layer, wl, pools, stats, experts=3):
    """Plan bit-exact; per expert: gate/up/h within the accumulation bound, codec bytes exact on the
    reported h, y within the output bars."""
    n, inter = wl.rows * 8, layer.intermediate
    ref = O.plan(max(256, wl.rows), wl.ids, wl.weights)
    assert stats.groups == int(ref.group_count[0])
    assert np.array_equal(scratch.view("original_routes", np.int32, n), ref.original_routes[:n])
    assert np.array_equal(scratch.view("inverse", np.int32, n), ref.inverse[:n])
    assert np.array_equal(scratch.view("grouped_weights", np.float32, n), ref.grouped_weights[:n])
    groups = scratch.view("groups", O.GROUP_DTYPE, stats.groups)
    assert np.array_equal(groups, ref.groups[:stats.groups])
    rows_all = stats.groups * 16
    taps = {k: scratch.view(k, np.float32, rows_all * inter).reshape(rows_all, inter) for k in ("gate", "up", "h")}
    mp = scratch.view("mid_payload", np.uint8, rows_all * inter).reshape(rows_all, inter)
    ms = scratch.view("mid_scales", np.uint8, rows_all * inter // 32).reshape(rows_all, inter // 32)
    y = scratch.view("y", np.float32, n * 4096).reshape(n, 4096)
    for gi in np.linspace(0, stats.groups - 1, experts).astype(int):
        g = groups[gi]
        r, toks = int(g["rows"]), g["input_rows"][:int(g["rows"])]
        sl = slice(gi * 16, gi * 16 + r)
        want = O.expert_ffn(pools, int(g["expert"]), wl.payload[toks], wl.scales[toks])
        assert want["fault"] == 0
        x = np.abs(O.activation_decode(wl.payload[toks], wl.scales[toks])[0].astype(np.float64))
        for k in ("gate", "up"):
            err = np.abs(taps[k][sl].astype(np.float64) - want[k])
            assert np.max(err) <= ACC_EPS * 4096 * np.max(x) * 6 * 2.0 ** -4, (k, np.max(err))
            assert parity(taps[k][sl], want[k])[1] < 1e-5
        assert parity(taps["h"][sl], want["h"])[1] < 1e-4
        # The activation on its own inputs: the CPU rule rounds every step once, the kernel uses the
        # hardware 2^x and a refined reciprocal (the reference's kernels call expf): a few binary32 ulp.
        rule = O.silu_up(taps["gate"][sl], taps["up"][sl])
        ulps = np.abs(taps["h"][sl].astype(np.float64) - rule) / np.spacing(np.maximum(np.abs(rule), np.float32(2.0 ** -100)))
        assert np.max(ulps) <= SILU_ULPS, np.max(ulps)
        qp, qs, qf = O.quant_v1(taps["h"][sl])
        assert not qf.any() and np.array_equal(qp, mp[sl]) and np.array_equal(qs, ms[sl])       # codec bytes on the reported h
        assert np.mean(mp[sl] == want["mid_payload"]) > 0.995
        routes = ref.original_routes[int(g["route_base"]):int(g["route_base"]) + r]
        ma, mr = parity(y[routes], want["y"])
        assert ma <= MAX_ABS and mr <= MEAN_REL, ("y", ma, mr)


@pytest.fixture(scope="module")
def scratch():
    s = b1.Scratch()
    s.set_taps(True)
    yield s
    s.close()


def test_closed_form_projections(scratch):
    """The reference's synthetic projection fixture (tests/b1_core/compute_test.cuh:4-8,66-81) at the real
    shapes N512/K4096 and N4096/K512, M in {1, 2, 4, 8, 16}, against exact sums; padded rows stay out."""
    pool = np.full(synth.EXPERTS * synth.IMAGE_BYTES, 0x22, np.uint8)
    imgs = {e: closed_form_image(e % 3) for e in (3, 77, 200)}
    for e, img in imgs.items():
        pool[e * synth.IMAGE_BYTES:(e + 1) * synth.IMAGE_BYTES] = img
    layer = DeviceLayer([pool]).layer
    assert layer.all_scales_normal() and layer.intermediate == 512
    for m in (1, 2, 4, 8, 16):
        payload, scales = closed_form_rows(m)
        ids = np.tile(np.array([3, 77, 200, 1, 2, 4, 5, 6], np.int32), (m, 1))
        w = np.tile(np.array([1, .5, .25, 0, 0, 0, 0, 0], np.float32), (m, 1))
        wl = synth.Workload("closed form", -1, 0, 1, m, ids, w, np.zeros((m, 4096), np.float32), payload, scales)
        stats, bf, pf = run_ffn_dev(layer, scratch, wl)
        assert stats.groups == 8
        groups = scratch.view("groups", O.GROUP_DTYPE, 8)
        x64 = O.activation_decode(payload, scales)[0].astype(np.float64)
        inter = 512
        gate = scratch.view("gate", np.float32, 8 * 16 * inter).reshape(8 * 16, inter)
        up = scratch.view("up", np.float32, 8 * 16 * inter).reshape(8 * 16, inter)
        y = scratch.view("y", np.float32, m * 8 * 4096).reshape(m, 8, 4096)
        mp = scratch.view("mid_payload", np.uint8, 8 * 16 * inter).reshape(8 * 16, inter)
        ms = scratch.view("mid_scales", np.uint8, 8 * 16 * 16).reshape(8 * 16, 16)
        for gi, g in enumerate(groups):
            e = int(g["expert"])
            if e not in imgs:
                continue
            assert int(g["rows"]) == m and g["input_rows"][:m].tolist() == list(range(m))
            wg = exact_projection(imgs[e], 0, synth.GATE_SCALES, 512, 4096, x64)
            wu = exact_projection(imgs[e], synth.UP_PAYLOAD, synth.UP_SCALES, 512, 4096, x64)
            for got, want in ((gate[gi * 16:gi * 16 + m], wg), (up[gi * 16:gi * 16 + m], wu)):
                assert np.all(np.abs(got.astype(np.float64) - want) <= 1e-5 + 1e-5 * np.abs(want) + ACC_EPS * np.max(np.abs(want)))
            mid64 = O.activation_decode(mp[gi * 16:gi * 16 + m], ms[gi * 16:gi * 16 + m])[0].astype(np.float64)
            wy = exact_projection(imgs[e], synth.DOWN_PAYLOAD, synth.DOWN_SCALES, 4096, 512, mid64)
            slot = [3, 77, 200].index(e)
            assert np.all(np.abs(y[:, slot].astype(np.float64) - wy) <= 1e-5 + 1e-5 * np.abs(wy) + ACC_EPS * np.max(np.abs(wy)))


@pytest.mark.parametrize("cfg", [0, 1])
def test_rank_share_configs(scratch, cfg):
    """configs[0] (one expert: slot 0 carries weight 1) and configs[1] (256 experts, 16 tokens)."""
    wl = synth.make(cfg)
    pools = wl.pools(wl.touched())
    layer = DeviceLayer(pools).layer
    stats, bf, pf = run_ffn_dev(layer, scratch, wl)
    rc, ref_partial, ref_bf16, ref_y = O.layer_ffn(pools, wl.payload, wl.scales, wl.ids, wl.weights, want_routes=True)
    assert rc == 0
    check_outputs(pf, bf, ref_partial, ref_bf16)
    check_stages(scratch, layer, wl, pools, stats)
    if cfg == 0:  # FP32 unweighted FC2 output of the single expert
        y = scratch.view("y", np.float32, wl.rows * 8 * 4096).reshape(wl.rows, 8, 4096)[:, 0]
        one = O.expert_ffn(pools, 0, wl.payload, wl.scales)["y"]
        ma, mr = parity(y, one)
        assert ma <= MAX_ABS and mr <= MEAN_REL
    # the reference's host-pointer entry, separate arrays and in-frame rows of 4224 bytes
    out = np.zeros((wl.rows, 4096), np.uint16)
    st = b1.ffn(layer, scratch, wl.payload, wl.scales, wl.ids, wl.weights, wl.rows, out)
    assert np.array_equal(out, bf) and st.groups == stats.groups and st.gpu_ms > 0
    frame = np.zeros((wl.rows, 4224 + 64), np.uint8)
    frame[:, :4096], frame[:, 4096:4224] = wl.payload, wl.scales
    out2 = np.zeros((wl.rows, 4096), np.uint16)
    b1.ffn_strided(layer, scratch, frame.reshape(-1), 4288, wl.ids, wl.weights, wl.rows, out2)
    assert np.array_equal(out2, bf)


def test_tile_schedule_at_rank_share_stage_by_stage(scratch):
    """More than 128 rows at one rank's share (I = 512): the prefill schedule with chunks of every class
    (1, 2, 3-4 and 5-8 groups under Zipf routing) and an FC2 of a single quad of k-steps, checked stage
    by stage like the decode configurations: plan, gate/up/h taps, codec bytes, per-route rows, outputs."""
    rows, seed = 1200, synth.BASE_SEED + 7
    ids, w, x = synth.routes_zipf(seed, rows), synth._softmax_weights(seed, rows), synth._activations(seed, rows)
    payload, scales = synth.q0_quantize(x)
    wl = synth.Workload("tile schedule, rank share", 1, seed, 1, rows, ids, w, x, payload, scales)
    groups_of = (np.bincount(ids.reshape(-1), minlength=256) + 15) // 16
    assert (groups_of == 1).any() and (groups_of == 2).any() and ((groups_of % 8 == 3) | (groups_of % 8 == 4)).any() \
        and (groups_of >= 5).any()
    pools = wl.pools(wl.touched())
    layer = DeviceLayer(pools).layer
    stats, bf, pf = run_ffn_dev(layer, scratch, wl)
    rc, ref_partial, ref_bf16, _ = O.layer_ffn(pools, wl.payload, wl.scales, wl.ids, wl.weights)
    assert rc == 0
    check_outputs(pf, bf, ref_partial, ref_bf16)
    check_stages(scratch, layer, wl, pools, stats, experts=12)


def _skewed_routes(seed, rows, experts):
    """8 distinct experts per token out of `experts`, Zipf(1.1) popularity (exponential-key sampling)."""
    p = 1.0 / np.arange(1, len(experts) + 1, dtype=np.float64) ** 1.1
    u = synth.uniform(synth.stream_key(seed, synth.ROUTES, 5), rows * len(experts)).reshape(rows, len(experts))
    ranks = np.argsort(-np.log(u) / p, axis=1, kind="stable")[:, :8]
    return np.asarray(experts, np.int32)[ranks]


def test_ragged_sizes_across_the_schedules(scratch):
    """Row counts either side of every switch of schedule (one and two activation tiles per wave up to
    32 and 128 rows, the tile kernels above, the planner over several compute units above 512) with
    skewed routing, so chunks are ragged: plan bit-exact, stages and outputs to the bars."""
    seed = synth.BASE_SEED + 11
    experts = list(range(3, 256, 11))  # 23 experts
    pools = [synth.rank_pool(seed, 0, experts)]
    layer = DeviceLayer(pools).layer
    for rows in (1, 31, 33, 127, 129, 130, 191, 513):
        ids, w, x = _skewed_routes(seed + rows, rows, experts), synth._softmax_weights(seed + rows, rows), synth._activations(seed + rows, rows)
        payload, scales = synth.q0_quantize(x)
        wl = synth.Workload(f"ragged {rows}", 1, seed, 1, rows, ids, w, x, payload, scales)
        stats, bf, pf = run_ffn_dev(layer, scratch, wl)
        rc, ref_partial, ref_bf16, _ = O.layer_ffn(pools, wl.payload, wl.scales, wl.ids, wl.weights)
        assert rc == 0, rows
        check_outputs(pf, bf, ref_partial, ref_bf16)
        check_stages(scratch, layer, wl, pools, stats, experts=2)


def test_decode_layer_full_intermediate(scratch, full_layer):
    """configs[2]: 256 experts x I 2048 on one GPU, 128 tokens, every row against the CPU reference."""
    wl, pools, layer = full_layer
    assert layer.intermediate == 2048
    stats, bf, pf = run_ffn_dev(layer, scratch, wl)
    rc, ref_partial, ref_bf16, _ = O.layer_ffn(pools, wl.payload, wl.scales, wl.ids, wl.weights)
    assert rc == 0
    check_outputs(pf, bf, ref_partial, ref_bf16)
    check_stages(scratch, layer, wl, pools, stats)


def test_tile_schedule_at_full_intermediate_every_row(scratch, full_layer):
    """The prefill schedule at I = 2048, where FC2 runs several quads of k-steps: a few experts under skewed
    routing so that chunks of three and four groups (the four-tile bodies, last tile in use) and of five to
    eight occur, every row against the CPU reference and two runs bit for bit. (With one quad, as at one
    rank's share, the k-loop is not a loop, and what the compiler places behind a loop's last MFMA never runs.)"""
    _, pools, layer = full_layer
    seed, rows = synth.BASE_SEED + 13, 312
    experts = list(range(5, 256, 21))  # 12 experts
    ids, w, x = _skewed_routes(seed, rows, experts), synth._softmax_weights(seed, rows), synth._activations(seed, rows)
    groups_of = (np.bincount(ids.reshape(-1), minlength=256) + 15) // 16
    assert (groups_of % 8 == 4).any() and (groups_of % 8 == 3).any() and (groups_of >= 5).any(), groups_of[groups_of > 0]
    payload, scales = synth.q0_quantize(x)
    wl = synth.Workload("tile schedule, full intermediate", 3, seed, 4, rows, ids, w, x, payload, scales)
    stats, bf, pf = run_ffn_dev(layer, scratch, wl)
    rc, ref_partial, ref_bf16, _ = O.layer_ffn(pools, wl.payload, wl.scales, wl.ids, wl.weights)
    assert rc == 0
    check_outputs(pf, bf, ref_partial, ref_bf16)
    per_row = np.abs(pf - ref_partial).max(axis=1) / np.abs(ref_partial).max()
    assert per_row.max() <= MAX_ABS, ("worst row", int(per_row.argmax()), float(per_row.max()))
    _, bf2, pf2 = run_ffn_dev(layer, scratch, wl)
    assert np.array_equal(bf2, bf) and np.array_equal(pf2.view(np.uint32), pf.view(np.uint32))
    # The clock record of the two tile launches: ticks of the shader clock and of the fixed 100 MHz counter over
    # one work item each (the middle chunk's); an item lasts microseconds to tens of them and the clock lies
    # between 1 and 2.4 GHz.
    ticks = scratch.view("clock", np.uint64, 4)
    for shader, fixed in (ticks[:2], ticks[2:]):
        assert 200 < fixed < 100_000 and 1.0 < float(shader) / float(fixed) * 0.1 < 2.6, ticks


def test_prefill_chunk_properties_and_sampled_parity(full_layer):
    """configs[3] at its full 8192 tokens: some 390 sampled rows against the CPU reference, and size-independent
    properties over all rows: each row depends on its own routes only (a subset run alone reproduces
    its rows bit for bit, a permuted batch permutes the rows), and the plan is a stable bijection."""
    _, pools, layer = full_layer  # the same seeded weights serve both configurations
    wl = synth.make(3)
    s = b1.Scratch()
    stats, bf, pf = run_ffn_dev(layer, s, wl)
    n = wl.rows * 8
    orig, inv = s.view("original_routes", np.int32, n), s.view("inverse", np.int32, n)
    assert np.array_equal(np.sort(orig), np.arange(n)) and np.array_equal(inv[orig], np.arange(n))
    ref = O.plan(8192, wl.ids, wl.weights)                                 # the planner spread over several compute units
    assert ref.status == 0 and stats.groups == int(ref.group_count[0])
    assert np.array_equal(orig, ref.original_routes[:n]) and np.array_equal(inv, ref.inverse[:n])
    assert np.array_equal(s.view("groups", O.GROUP_DTYPE, stats.groups), ref.groups[:stats.groups])
    experts = wl.ids.reshape(-1)[orig]
    assert np.all(np.diff(experts) >= 0)
    same = np.diff(experts) == 0
    assert np.all(np.diff(orig)[same] > 0)                                 # stable inside every expert
    sample = np.unique(np.concatenate([[0, 1, 777, 4095, 4096, 8191], np.random.default_rng(3).integers(0, wl.rows, 394)]))
    sub = synth.Workload("sample", 3, wl.seed, 4, len(sample), wl.ids[sample], wl.weights[sample], wl.x[sample],
                         wl.payload[sample], wl.scales[sample])
    rc, ref_partial, ref_bf16, _ = O.layer_ffn(pools, sub.payload, sub.scales, sub.ids, sub.weights)
    assert rc == 0
    check_outputs(pf[sample], bf[sample], ref_partial, ref_bf16)
    _, bf_again, pf_again = run_ffn_dev(layer, s, wl)                     # every row, bit for bit, run after run
    assert np.array_equal(bf_again, bf) and np.array_equal(pf_again.view(np.uint32), pf.view(np.uint32))
    _, bf_sub, pf_sub = run_ffn_dev(layer, s, sub)
    assert np.array_equal(bf_sub, bf[sample]) and np.array_equal(pf_sub.view(np.uint32), pf[sample].view(np.uint32))
    perm = np.random.default_rng(1).permutation(wl.rows)
    pw = synth.Workload("permuted", 3, wl.seed, 4, wl.rows, wl.ids[perm], wl.weights[perm], wl.x[perm], wl.payload[perm], wl.scales[perm])
    _, bf_p, _ = run_ffn_dev(layer, s, pw, want_partial=False)
    assert np.array_equal(bf_p, bf[perm])


def test_two_scratches_in_flight_on_one_layer(full_layer):
    """One scratch is one call in flight; two scratches (two streams) may run at once on the same layer.
    Calls of three sizes (decode schedule, tile schedule) are enqueued alternately without a wait in
    between; every output equals the one the same call gives alone, bit for bit."""
    wl, _, layer = full_layer
    big = synth.make(3)
    pick = np.arange(700) * 11 % big.rows
    tile = synth.Workload("tile", 3, big.seed, 4, len(pick), big.ids[pick], big.weights[pick], big.x[pick],
                          big.payload[pick], big.scales[pick])
    few = synth.Workload("few", 2, wl.seed, 4, 5, wl.ids[:5], wl.weights[:5], wl.x[:5], wl.payload[:5], wl.scales[:5])
    calls = [wl, tile, few, tile, wl, few]
    alone = b1.Scratch()
    want = [run_ffn_dev(layer, alone, w, want_partial=False)[1] for w in calls]
    scratches = [b1.Scratch(), b1.Scratch()]
    held = []
    for n, w in enumerate(calls):
        bufs = [b1.DeviceBuffer.from_host(a) for a in (w.payload, w.scales, w.ids, w.weights)]
        out = b1.DeviceBuffer(w.rows * 4096 * 2)
        if n >= 2:
            scratches[n % 2].sync()                                        # the scratch's previous call, not the other's
        b1.ffn_enqueue(layer, scratches[n % 2], bufs[0].ptr, 4096, bufs[1].ptr, 128, bufs[2].ptr, bufs[3].ptr, w.rows, out.ptr)
        held.append((bufs, out))
    for s in scratches:
        s.sync()
    for (bufs, out), w, ref in zip(held, calls, want):
        assert np.array_equal(out.to_host(np.uint16).reshape(w.rows, 4096), ref)


def test_maximum_rows_on_eight_experts():
    """The largest call (8192 rows) with every token routed to the same eight experts: 8192 rows per
    expert, 64 full chunks each, the collision the planner's counters and the tile schedule see at most.
    Plan bit-exact; sampled rows to the bars; rows of identical input and routes come out identical."""
    seed, rows = synth.BASE_SEED + 21, 8192
    experts = [5, 40, 77, 101, 130, 188, 200, 255]
    rng = np.random.default_rng(21)
    ids = np.stack([rng.permutation(experts) for _ in range(rows)]).astype(np.int32)
    w, x = synth._softmax_weights(seed, rows), synth._activations(seed, rows)
    x[4096:] = x[:4096]                                                     # second half repeats the first ...
    ids[4096:], w[4096:] = ids[:4096], w[:4096]                             # ... routes and weights included
    payload, scales = synth.q0_quantize(x)
    wl = synth.Workload("eight experts", 1, seed, 1, rows, ids, w, x, payload, scales)
    pools = [synth.rank_pool(seed, 0, experts)]
    layer = DeviceLayer(pools).layer
    s = b1.Scratch()
    stats, bf, pf = run_ffn_dev(layer, s, wl)
    n = rows * 8
    ref = O.plan(8192, ids, w)
    assert ref.status == 0 and stats.groups == int(ref.group_count[0]) == 8 * 512
    assert np.array_equal(s.view("original_routes", np.int32, n), ref.original_routes[:n])
    assert np.array_equal(s.view("inverse", np.int32, n), ref.inverse[:n])
    assert np.array_equal(s.view("groups", O.GROUP_DTYPE, stats.groups), ref.groups[:stats.groups])
    assert np.array_equal(bf[4096:], bf[:4096]) and np.array_equal(pf[4096:].view(np.uint32), pf[:4096].view(np.uint32))
    sample = np.array([0, 1, 2047, 4095, 4096, 6000, 8190, 8191])
    rc, ref_partial, ref_bf16, _ = O.layer_ffn(pools, payload[sample], scales[sample], ids[sample], w[sample])
    assert rc == 0
    check_outputs(pf[sample], bf[sample], ref_partial, ref_bf16)


def test_errors_and_faults(full_layer):
    """Return codes and messages of the reference entry (b1_serve.cu:315-317,365,551-562)."""
    wl, pools, layer = full_layer
    s = b1.Scratch()
    out = np.zeros((wl.rows, 4096), np.uint16)
    ids = wl.ids.copy(); ids[5, 3] = ids[5, 2]
    with pytest.raises(b1.B1Error, match="invalid routes") as e:
        b1.ffn(layer, s, wl.payload, wl.scales, ids, wl.weights, wl.rows, out)
    assert e.value.code == 3
    w = wl.weights.copy(); w[0, 0] = np.nan
    with pytest.raises(b1.B1Error, match="invalid routes"):
        b1.ffn(layer, s, wl.payload, wl.scales, wl.ids, w, wl.rows, out)
    pay = wl.payload.copy(); pay[17, 100] = 0x7F                         # an E4M3 NaN code in one row
    with pytest.raises(b1.B1Error, match="quantizer fault 1") as e:
        b1.ffn(layer, s, pay, wl.scales, wl.ids, wl.weights, wl.rows, out)
    assert e.value.code == 4 and O.layer_ffn(pools, pay[16:18], wl.scales[16:18], wl.ids[16:18], wl.weights[16:18])[0] == 4
    sc = wl.scales.copy(); sc[3, 9] = 104                                # activation scale below the legal window
    with pytest.raises(b1.B1Error, match="quantizer fault 1"):
        b1.ffn(layer, s, wl.payload, sc, wl.ids, wl.weights, wl.rows, out)
    from mimo26f_afd_amd._lib import load
    import ctypes as C
    buf = C.create_string_buffer(256)
    lib = load()
    args = (wl.payload.ctypes.data, 4096, wl.scales.ctypes.data, 128, wl.ids.ctypes.data, wl.weights.ctypes.data)
    assert lib.m26s_b1_ffn(layer._h, s._h, *args, 0, out.ctypes.data, None, buf, 256) == 1
    assert lib.m26s_b1_ffn(layer._h, s._h, *args, 8193, out.ctypes.data, None, buf, 256) == 1
    assert lib.m26s_b1_ffn(layer._h, s._h, args[0], 4095, *args[2:], 16, out.ctypes.data, None, buf, 256) == 1
    assert lib.m26s_b1_ffn(None, s._h, *args, 16, out.ctypes.data, None, buf, 256) == 1 and b"bad rows/handles/pitch" in buf.value
    assert lib.m26s_b1_layer_new(1, 5, 0, C.byref(C.c_void_p()), buf, 256) == 1 and b"bad canonical extent/rank" in buf.value
    st = b1.ffn(layer, s, wl.payload, wl.scales, wl.ids, wl.weights, wl.rows, out)   # the scratch recovers after faults
    assert st.groups > 0 and out.any()


def test_wide_planner_faults_and_recovery(full_layer):
    """Above 512 rows the planner runs as three launches over several compute units: the same faults in
    the same order of precedence, nothing written by a rejected plan, and the next call is clean."""
    _, pools, layer = full_layer
    wl = synth.make(3, rows=1536)
    s = b1.Scratch()
    s.set_taps(True)                                                     # also fills grouped_weights
    out = np.zeros((wl.rows, 4096), np.uint16)
    n = wl.rows * 8
    b1.ffn(layer, s, wl.payload, wl.scales, wl.ids, wl.weights, wl.rows, out)
    ref = O.plan(2048, wl.ids, wl.weights)
    good = [s.view(k, np.int32, n).copy() for k in ("original_routes", "inverse")]
    assert np.array_equal(good[0], ref.original_routes[:n]) and np.array_equal(good[1], ref.inverse[:n])
    assert np.array_equal(s.view("grouped_weights", np.float32, n), ref.grouped_weights[:n])
    cases = []
    ids = wl.ids.copy(); ids[1400, 7] = ids[1400, 0]; cases.append((ids, wl.weights))          # repeat inside a token
    ids = wl.ids.copy(); ids[700, 2] = 256; cases.append((ids, wl.weights))                     # id out of range
    ids = wl.ids.copy(); ids[3, 1] = -1; cases.append((ids, wl.weights))
    w = wl.weights.copy(); w[1535, 7] = -1.0; cases.append((wl.ids, w))                         # negative weight
    w = wl.weights.copy(); w[600, 0] = np.inf; cases.append((wl.ids, w))
    for bad_ids, bad_w in cases:
        with pytest.raises(b1.B1Error, match="invalid routes") as e:
            b1.ffn(layer, s, wl.payload, wl.scales, bad_ids, bad_w, wl.rows, out)
        assert e.value.code == 3
        assert np.array_equal(s.view("original_routes", np.int32, n), good[0])   # the rejected plan wrote nothing
        assert np.array_equal(s.view("inverse", np.int32, n), good[1])
    out2 = np.zeros_like(out)
    st = b1.ffn(layer, s, wl.payload, wl.scales, wl.ids, wl.weights, wl.rows, out2)
    assert st.groups == int(ref.group_count[0]) and np.array_equal(out2, out)


def test_rejected_plan_is_remembered_until_the_sync(full_layer):
    """Faults of every call enqueued since the last sync accumulate: a call whose routes are rejected,
    followed by good calls on the same scratch, still makes the sync return code 3, and the later calls
    compute nothing (their outputs keep the bytes they held); after the sync the scratch is clean. Both
    planners (one workgroup up to 512 rows, several above)."""
    wl, _, layer = full_layer
    big = synth.make(3, rows=640)
    for w_ in (wl, big):
        s = b1.Scratch()
        bad_ids = w_.ids.copy()
        bad_ids[3, 1] = bad_ids[3, 0]
        bufs = [b1.DeviceBuffer.from_host(a) for a in (w_.payload, w_.scales, w_.ids, w_.weights, bad_ids)]
        fill = np.full(w_.rows * 4096, 0xABCD, np.uint16)
        outs = [b1.DeviceBuffer.from_host(fill) for _ in range(3)]
        args = (bufs[0].ptr, 4096, bufs[1].ptr, 128)
        b1.ffn_enqueue(layer, s, *args, bufs[4].ptr, bufs[3].ptr, w_.rows, outs[0].ptr)      # rejected
        b1.ffn_enqueue(layer, s, *args, bufs[2].ptr, bufs[3].ptr, w_.rows, outs[1].ptr)      # good, but behind a fault
        with pytest.raises(b1.B1Error, match="invalid routes") as e:
            s.sync()
        assert e.value.code == 3
        assert np.array_equal(outs[0].to_host(np.uint16), fill) and np.array_equal(outs[1].to_host(np.uint16), fill)
        s.sync()                                                                             # nothing pending: clean
        b1.ffn_enqueue(layer, s, *args, bufs[2].ptr, bufs[3].ptr, w_.rows, outs[2].ptr)
        s.sync()
        _, want, _ = run_ffn_dev(layer, b1.Scratch(), w_, want_partial=False)
        assert np.array_equal(outs[2].to_host(np.uint16).reshape(w_.rows, 4096), want)


def test_four_rank_composition_is_the_reference_sum():
    """The reference's system: four TP4 ranks each return the BF16 rounding of their own partial row, and
    the coordinator adds the four planes in rank order in FP32 (crates/mimo26-repack/tests/lattice_oracle.py:94-113,
    crates/mimo26-coordinator/kernels/glue.cu:200-213). One GPU plays the four ranks in turn (four
    single-pool layers, configs[2] routing and inputs) and then the coordinator: the rank sum is bit for
    bit the CPU rule's sum of the GPU's own planes, every plane and the sum meet the bars against the CPU
    rule's planes and their sum, and the fused layer (one FP32 sum over I = 2048, one BF16 rounding) stays
    within the wire bound of that sum."""
    from mimo26f_afd_amd import glue
    wl = synth.make(2)
    pools = wl.pools(wl.touched())
    scratch = b1.Scratch()
    planes, ref_planes, held = [], [], []
    for r in range(4):
        one = synth.Workload(f"rank {r}", 2, wl.seed, 1, wl.rows, wl.ids, wl.weights, wl.x, wl.payload, wl.scales)
        buf = b1.DeviceBuffer.from_host(pools[r])
        layer = b1.Layer(buf.ptr, buf.nbytes, r)
        buf.free()
        assert layer.intermediate == 512
        bufs = [b1.DeviceBuffer.from_host(a) for a in (one.payload, one.scales, one.ids, one.weights)]
        out = b1.DeviceBuffer(wl.rows * 4096 * 2)
        b1.ffn_dev(layer, scratch, bufs[0].ptr, 4096, bufs[1].ptr, 128, bufs[2].ptr, bufs[3].ptr, wl.rows, out.ptr)
        held.append(out)
        planes.append(out.to_host(np.uint16).reshape(wl.rows, 4096))
        rc, _, ref_bf16, _ = O.layer_ffn([pools[r]], wl.payload, wl.scales, wl.ids, wl.weights)
        assert rc == 0
        ref_planes.append(ref_bf16)
        ma, mr = parity(bf16_to_f32(planes[r]), bf16_to_f32(ref_bf16))
        assert ma <= MAX_ABS and mr <= MEAN_REL, (r, ma, mr)
        layer.close()
    total = b1.DeviceBuffer(wl.rows * 4096 * 4)
    glue.rank_sum_bf16(*[h.ptr for h in held], total.ptr, wl.rows * 4096, scratch.stream)
    scratch.sync()
    got = total.to_host(np.float32).reshape(wl.rows, 4096)
    assert np.array_equal(got.view(np.uint32), O.rank_sum_bf16(*planes).reshape(wl.rows, 4096).view(np.uint32))
    want = O.rank_sum_bf16(*ref_planes).reshape(wl.rows, 4096)
    ma, mr = parity(got, want)
    assert ma <= MAX_ABS and mr <= MEAN_REL, (ma, mr)
    # the fused layer against the four-plane sum: each plane carries one BF16 rounding (2^-9 relative)
    full = DeviceLayer(pools).layer
    _, _, pf = run_ffn_dev(full, scratch, wl)
    bound = 2.4e-6 + np.sum([np.abs(bf16_to_f32(p).astype(np.float64)) for p in planes], axis=0) * 2.0 ** -8
    bound += 1e-4 * np.max(np.abs(want))                                     # FP32 accumulation order (K = 2048 at once against four sums of 512)
    assert np.all(np.abs(pf.astype(np.float64) - got) <= bound)
