"""Pins the CPU checker's planner, combine, activation and FFN composition: vectors from the
reference's compiled host units (committed fixture, and live where oracle/_ref was built), the
reference's closed-form vectors, an independent stable sort, exact integer dots on closed-form
weights, brute force on one row, and the identities / mutation detectors of the reference's
lattice self-test (crates/mimo26-repack/tests/lattice_oracle.py:116-176)."""
import os

import numpy as np
import pytest

import b1_oracle as O
from mimo26f_afd_amd import synth

FIX = np.load(os.path.join(os.path.dirname(__file__), "golden", "b1_host_units.npz"))
needs_ref = pytest.mark.skipif(not O.ref_available(), reason="oracle/_ref not built (reference tree absent)")


# ---- planner -------------------------------------------------------------------------------------
def stable_sort_plan(ids):
    """Independent statement: stable sort of routes by expert, cut into runs of at most 16
    (crates/mimo26-expert/tests/b1/plan.cpp:33-57)."""
    flat = np.asarray(ids).reshape(-1)
    order = np.argsort(flat, kind="stable")
    groups = []
    begin = 0
    while begin < len(order):
        end = begin
        while end < len(order) and flat[order[end]] == flat[order[begin]] and end - begin < 16:
            end += 1
        rows = [int(order[i]) // 8 for i in range(begin, end)] + [-1] * (16 - (end - begin))
        groups.append([int(flat[order[begin]]), end - begin, begin] + rows)
        begin = end
    return order.astype(np.int32), np.array(groups, np.int32).reshape(-1, 19)


@pytest.mark.parametrize("name", ["a", "b", "c", "d"])
def test_plan_committed_reference_vectors(name):
    ids, w, cap = FIX[f"plan_{name}_ids"], FIX[f"plan_{name}_w"], int(FIX[f"plan_{name}_cap"][0])
    resident = None
    if name == "d":
        resident = np.zeros(256, np.uint8)
        resident[[255, 0, 7, 63, 128, 32, 254, 1]] = 1
    p = O.plan(cap, ids, w, resident)
    n, ng = ids.size, int(FIX[f"plan_{name}_count"][0])
    assert p.status == 0 and p.fault[0] == 0 and p.group_count[0] == ng
    assert np.array_equal(p.inverse[:n], FIX[f"plan_{name}_inverse"])
    assert np.array_equal(p.original_routes[:n], FIX[f"plan_{name}_original"])
    assert np.array_equal(p.grouped_weights[:n], FIX[f"plan_{name}_gw"])
    assert np.array_equal(p.groups[:ng].view(np.int32).reshape(ng, 19), FIX[f"plan_{name}_groups"])
    # tails are reset exactly as the serial planner leaves them
    assert (p.inverse[n:] == -1).all() and (p.original_routes[n:] == -1).all() and (p.grouped_weights[n:] == 0).all()
    tail = p.groups[ng:]
    assert (tail["expert"] == -1).all() and (tail["rows"] == 0).all() and (tail["route_base"] == -1).all() and (tail["input_rows"] == -1).all()


@pytest.mark.parametrize("rows,cap", [(0, 256), (1, 256), (17, 256), (256, 256), (700, 2048), (4096, 4096)])
def test_plan_against_independent_stable_sort(rows, cap):
    rng = np.random.default_rng(rows + 1)
    ids = np.stack([rng.permutation(256)[:8] for _ in range(max(rows, 1))])[:rows].astype(np.int32).reshape(rows, 8)
    if rows >= 256:
        ids[:, 0] = 5  # one hot expert: many full groups
        ids[:, 1:] = np.where(ids[:, 1:] == 5, 6, ids[:, 1:])
        ids[:, 1] = 250
        ids[:, 2:] = np.where(ids[:, 2:] == 250, 251, ids[:, 2:])
        ids[:, 2:] = np.where(ids[:, 2:] == 6, 252, ids[:, 2:])
        bad = [len(set(r)) != 8 for r in ids.tolist()]
        ids = ids[~np.array(bad)]
        rows = len(ids)
    w = rng.random((rows, 8)).astype(np.float32)
    p = O.plan(cap, ids, w)
    order, groups = stable_sort_plan(ids)
    assert p.status == 0 and int(p.group_count[0]) == len(groups)
    assert np.array_equal(p.original_routes[:rows * 8], order)
    assert np.array_equal(p.inverse[:rows * 8][order], np.arange(rows * 8))
    assert np.array_equal(p.grouped_weights[:rows * 8], w.reshape(-1)[order])
    assert np.array_equal(p.groups[:len(groups)].view(np.int32).reshape(-1, 19), groups)


def test_plan_negatives():
    """crates/mimo26-expert/tests/b1/plan.cpp:96-117: statuses, and nothing but the fault is written."""
    ids = np.arange(8, dtype=np.int32).reshape(1, 8)
    w = np.full((1, 8), 0.125, np.float32)
    good = O.plan(256, ids, w)
    assert good.status == 0

    def rejected(ids_, w_, resident=None):
        out = O.Plan(256)
        O.plan(256, ids_, w_, resident, out=out)
        fresh = O.Plan(256)
        assert np.array_equal(out.inverse, fresh.inverse) and np.array_equal(out.groups, fresh.groups)
        assert out.fault[0] == out.status
        return out.status

    for bad_id in (256, -1):
        i = ids.copy(); i[0, 7] = bad_id
        assert rejected(i, w) == 7
    i = ids.copy(); i[0, 7] = 0
    assert rejected(i, w) == 7                                  # duplicate expert in the token
    res = np.ones(256, np.uint8); res[7] = 0
    assert rejected(ids, w, res) == 7                           # not resident
    res = np.ones(256, np.uint8); res[3] = 2
    assert rejected(ids, w, res) == 7                           # non-binary mask
    for bad_w in (np.nan, -0.125, np.inf):
        ww = w.copy(); ww[0, 0] = bad_w
        assert rejected(ids, ww) == 8
    ww = w.copy(); ww[0, 0] = np.nan
    i = ids.copy(); i[0, 1] = 0                                 # weight fault at route 0 comes first
    assert rejected(i, ww) == 8


@needs_ref
def test_plan_live_differential():
    rng = np.random.default_rng(77)
    for rows, cap in ((1, 256), (64, 256), (255, 256), (2048, 2048), (3000, 4096)):
        ids = np.stack([rng.choice(rng.integers(8, 257), 8, replace=False) for _ in range(rows)]).astype(np.int32)
        w = rng.random((rows, 8)).astype(np.float32)
        a, b = O.plan(cap, ids, w), O.ref_plan(cap, ids, w)
        for k in ("inverse", "original_routes", "grouped_weights", "groups", "group_count", "fault"):
            assert np.array_equal(getattr(a, k), getattr(b, k)), (rows, k)
    ids = np.arange(8, dtype=np.int32).reshape(1, 8); w = np.full((1, 8), .5, np.float32)
    for mutate in (lambda i, w: i.__setitem__((0, 7), 256), lambda i, w: i.__setitem__((0, 7), 0),
                   lambda i, w: w.__setitem__((0, 3), np.nan), lambda i, w: w.__setitem__((0, 0), -1.0)):
        i2, w2 = ids.copy(), w.copy(); mutate(i2, w2)
        assert O.plan(256, i2, w2).status == O.ref_plan(256, i2, w2).status != 0


# ---- combine -------------------------------------------------------------------------------------
def test_reduce_committed_reference_vectors():
    st, part, bf = O.reduce(FIX["reduce_y"], FIX["reduce_w"])
    assert st == 0 and np.array_equal(part.view(np.uint32), FIX["reduce_partial"]) and np.array_equal(bf, FIX["reduce_bf16"])


def _one(zs, ws):
    y = np.zeros((1, 8, 4), np.float32); w = np.ones((1, 8), np.float32)
    y[0, :len(zs), 0] = zs
    w[0, :len(ws)] = ws
    return O.reduce(y, w)


def test_reduce_closed_form_vectors():
    """crates/mimo26-expert/tests/b1/route.cpp:69-96,120-133."""
    st, p, _ = _one([1e8, 1.0, -1e8, 3.0], [])
    assert st == 0 and p[0, 0] == 3.0                                            # slot order, not reassociated
    st, p, _ = _one([-1.0, 1.0 + 2.0 ** -23], [1.0, 1.0 - 2.0 ** -23])
    assert st == 0 and p[0, 0] == 0.0                                            # separate multiply and add, no FMA
    st, p, b = _one([2.0 ** -126], [0.5])
    assert st == 0 and p[0, 0] == np.float32(2.0 ** -127) and b[0, 0] == 0x0040  # subnormal product kept
    st, p, b = _one([1.0 + 1.0 / 256], [])
    assert b[0, 0] == 0x3F80
    st, p, b = _one([1.0 + 3.0 / 256], [])
    assert b[0, 0] == 0x3F82
    st, p, b = _one([-(1.0 + 1.0 / 256)], [])
    assert b[0, 0] == 0xBF80
    for bad in (np.nan, np.inf, -np.inf, -1.0):
        assert _one([1.0], [bad])[0] == 8
    assert _one([np.nan], [])[0] == 8
    assert _one([3.4028235e38], [])[0] == 8                                      # BF16 rounding overflows
    assert _one([3.4028235e38], [2.0])[0] == 8                                   # product overflows
    assert _one([3.4028235e38, 3.4028235e38], [])[0] == 8                        # running sum overflows
    y = np.stack([np.full((8, 4096), j + 1, np.float32) for j in range(2)])
    w = np.tile(np.arange(1, 9, dtype=np.float32) / 36, (2, 1))
    st, p, _ = O.reduce(y, w)
    expect = np.zeros(2, np.float32)
    for t in range(2):
        for j in range(8):
            expect[t] = np.float32(expect[t] + np.float32(np.float32(t + 1) * w[t, j]))
    assert st == 0 and (p == expect[:, None]).all()


@needs_ref
def test_reduce_live_differential():
    rng = np.random.default_rng(8)
    y = (rng.standard_normal((3, 8, 4096)) * np.exp2(rng.integers(-60, 60, (3, 8, 1)))).astype(np.float32)
    w = rng.random((3, 8)).astype(np.float32)
    a, b = O.reduce(y, w), O.ref_reduce(y, w)
    assert a[0] == b[0] == 0 and np.array_equal(a[1], b[1]) and np.array_equal(a[2], b[2])


# ---- the opt-in BF16 per-route mode (crates/mimo26-spark/kernels/b1_serve.cu:98-143, connected.cu:41-44) ----
def _one16(z_bits, ws):
    y = np.zeros((8, 4), np.uint16); w = np.ones((1, 8), np.float32)
    y[:len(z_bits), 0] = z_bits
    w[0, :len(ws)] = ws
    return O.reduce_bf16y(y, w)


def test_bf16_store_rule_hand_worked():
    """FC2's store in that mode: nearest BF16, ties to even, by the integer formula (no special cases)."""
    v = np.array([1.0, 1.0 + 2.0 ** -8, 1.0 + 3 * 2.0 ** -8, 1.0 + 2.0 ** -8 + 2.0 ** -20, -(1.0 + 2.0 ** -8), 0.0, -0.0,
                  2.0 ** -133, 3.3895314e38, np.inf], np.float32)
    want = [0x3F80, 0x3F80, 0x3F82, 0x3F81, 0xBF80, 0x0000, 0x8000, 0x0001, 0x7F7F, 0x7F80]
    assert O.bf16_store_rows(v).tolist() == want
    assert O.bf16_store_rows(np.array([3.4028235e38], np.float32))[0] == 0x7F80      # FLT_MAX rounds up into the exponent of all ones
    rng = np.random.default_rng(4)
    x = (rng.standard_normal(20000) * np.exp2(rng.integers(-100, 100, 20000))).astype(np.float32)
    got = O.bf16_store_rows(x).astype(np.uint32) << 16
    lo, hi = x.view(np.uint32) & 0xFFFF0000, (x.view(np.uint32) & 0xFFFF0000) + 0x10000   # the two neighbours on the BF16 grid
    d_lo = np.abs(x.astype(np.float64) - lo.view(np.float32)); d_hi = np.abs(hi.view(np.float32).astype(np.float64) - x)
    nearest = np.where(d_lo < d_hi, lo, np.where(d_hi < d_lo, hi, np.where((lo >> 16) & 1, hi, lo)))
    assert np.array_equal(got, nearest)


def test_reduce_bf16y_hand_worked_vectors():
    one, big = 0x3F80, 0x4CBF                                                    # 1.0 and 1.0e8 rounded to BF16 (100139008)
    st, b = _one16([big, one, big | 0x8000, 0x4040], [])                         # (big + 1 - big) + 3 = 3 only in slot order
    assert st == 0 and b[0, 0] == 0x4040
    st, b = _one16([0x3F81, 0x3F81], [0.5, 0.5])                                 # 1.0078125: exact in binary32, a BF16 midpoint at the output
    assert st == 0 and b[0, 0] == 0x3F81
    st, b = _one16([0x3F80, 0x3B80], [1.0, 1.0])                                 # 1 + 2^-8: tie, to even
    assert st == 0 and b[0, 0] == 0x3F80
    st, b = _one16([0x3F80, 0x3B80, 0x3B80, 0x3B80], [1.0, 1.0, 1.0, 1.0])       # 1 + 3 * 2^-8: tie, to even, upwards
    assert st == 0 and b[0, 0] == 0x3F82
    st, b = _one16([0x0080], [0.5])                                              # 2^-126 * 0.5: the subnormal product is kept
    assert st == 0 and b[0, 0] == 0x0040
    for bad in (np.nan, np.inf, -1.0):
        assert _one16([one], [bad])[0] == 5
    assert _one16([0x7F80], [])[0] == 5 and _one16([0x7FC0], [])[0] == 5 and _one16([0xFF80], [])[0] == 5
    assert _one16([0x7F7F, 0x7F7F], [])[0] == 5                                  # running sum overflows
    assert _one16([0x7F7F], [2.0])[0] == 5                                       # product overflows


def test_reduce_bf16y_is_the_pinned_combine_on_widened_rows():
    """Different code, same contract: orc_reduce (pinned by the reference's reduce_host and its vectors) on the
    rows widened to binary32 gives the same BF16 bits."""
    rng = np.random.default_rng(12)
    y = (rng.standard_normal((5, 8, 512)) * np.exp2(rng.integers(-40, 40, (5, 8, 1)))).astype(np.float32)
    w = rng.random((5, 8)).astype(np.float32)
    y16 = O.bf16_store_rows(y)
    wide = (y16.astype(np.uint32) << 16).view(np.float32)
    st, _, want = O.reduce(wide, w)
    st16, got = O.reduce_bf16y(y16.reshape(40, 512), w)
    assert st == 0 and st16 == 0 and np.array_equal(got, want)
    assert not np.array_equal(got, O.reduce(y, w)[2])                             # and it is a different numerical mode


# ---- activation ------------------------------------------------------------------------------------
def test_silu_reference_witnesses():
    """crates/mimo26-expert/tests/gpu/silu_exp_gpu.cu:21-22,44 and mimo26-repack/tests/step_oracle.py:10-13."""
    g = np.array([-0.19146597385406494, 0.327481746673584, -0.1987401247024536, 0.23654770851135254], np.float32)
    u = np.array([-0.17092028260231018, 0.14912837743759155, 0.5958439111709595, 0.2174588441848755], np.float32)
    h = np.array([0.014801025390625, 0.02838134765625, -0.0533447265625, 0.02874755673110485], np.float32)
    assert np.array_equal(O.silu_up(g, u).view(np.uint32), h.view(np.uint32))


def test_silu_specials():
    """lattice_oracle.py:166-175."""
    a = O.silu_up(np.array([-100.0, -0.0, 0.0, 100.0], np.float32), np.ones(4, np.float32))
    assert np.isfinite(a).all() and a[0] < 0 and np.signbit(a[1]) and not np.signbit(a[2]) and a[3] == 100.0
    x = np.linspace(-20, 20, 4001).astype(np.float32)
    want = (x.astype(np.float64) / (1 + np.exp(-x.astype(np.float64)))).astype(np.float32)
    got = O.silu_up(x, np.ones_like(x))
    assert np.max(np.abs(got.astype(np.float64) - want) / np.maximum(np.abs(want), 1e-30)) < 3e-7


# ---- FFN composition ----------------------------------------------------------------------------------
def closed_form_image(p_base: int) -> np.ndarray:
    """A quarter-slice image from the reference's closed-form fixture
    (crates/mimo26-expert/tests/b1_core/compute_test.cuh:4-8): codes (7n + 3k + 5(k/32) + 3p) % 16,
    scales 124 + (n + 2kb + p) % 7, p = 0 up, 1 gate, 2 down."""
    img = np.zeros(synth.IMAGE_BYTES, np.uint8)

    def region(rows, cols, p, payload_off, scale_off):
        n = np.arange(rows)[:, None]
        k = np.arange(cols)[None, :]
        codes = ((7 * n + 3 * k + 5 * (k // 32) + 3 * (p + p_base)) % 16).astype(np.uint8)
        img[payload_off:payload_off + rows * cols // 2] = (codes[:, 0::2] | (codes[:, 1::2] << 4)).reshape(-1)
        kb = np.arange(cols // 32)[None, :]
        img[scale_off:scale_off + rows * cols // 32] = (124 + (n + 2 * kb + p + p_base) % 7).astype(np.uint8).reshape(-1)
        return codes

    region(512, 4096, 1, 0, synth.GATE_SCALES)
    region(512, 4096, 0, synth.UP_PAYLOAD, synth.UP_SCALES)
    region(4096, 512, 2, synth.DOWN_PAYLOAD, synth.DOWN_SCALES)
    return img


def closed_form_rows(rows: int):
    """Activation rows of the same fixture: codes through the normal E4M3 values, scales 119 + (m+kb)%5."""
    norm = np.array([0, 0x30, 0x38, 0x3C, 0x40, 0x44, 0x48, 0x4C, 0x80, 0xB0, 0xB8, 0xBC, 0xC0, 0xC4, 0xC8, 0xCC], np.uint8)
    m = np.arange(rows)[:, None]
    k = np.arange(4096)[None, :]
    payload = norm[(3 * m + 5 * k + 7 * (k // 32)) % 16]
    scales = (119 + (m + np.arange(128)[None, :]) % 5).astype(np.uint8)
    return payload, scales


E2M1 = np.array([0, .5, 1, 1.5, 2, 3, 4, 6, -0.0, -.5, -1, -1.5, -2, -3, -4, -6])


def exact_projection(img, poff, soff, nrows, ncols, x64):
    """Independent scalar statement: integer-exact products, Python-int accumulation, one rounding."""
    pay = img[poff:poff + nrows * ncols // 2].reshape(nrows, ncols // 2)
    codes = np.empty((nrows, ncols), np.uint8)
    codes[:, 0::2], codes[:, 1::2] = pay & 15, pay >> 4
    sc = img[soff:soff + nrows * ncols // 32].reshape(nrows, ncols // 32).astype(np.int64)
    w = np.ldexp(E2M1[codes], np.repeat(sc - 127, 32, axis=1))
    # every term is a multiple of 2^-40 far below 2^53 in magnitude: int64 sums are exact
    wi = np.rint(np.ldexp(w, 24)).astype(np.int64)
    xi = np.rint(np.ldexp(x64, 24)).astype(np.int64)
    assert np.array_equal(np.ldexp(wi.astype(np.float64), -24), w) and np.array_equal(np.ldexp(xi.astype(np.float64), -24), x64)
    return np.ldexp((xi @ wi.T).astype(np.float64), -48).astype(np.float32)


def test_expert_ffn_closed_form_projections():
    img = closed_form_image(0)
    pool = np.full(synth.EXPERTS * synth.IMAGE_BYTES, 0x22, np.uint8)
    pool[3 * synth.IMAGE_BYTES:4 * synth.IMAGE_BYTES] = img
    payload, scales = closed_form_rows(5)
    out = O.expert_ffn([pool], 3, payload, scales)
    assert out["fault"] == 0
    x64 = O.activation_decode(payload, scales)[0].astype(np.float64)
    gate = exact_projection(img, 0, synth.GATE_SCALES, 512, 4096, x64)
    up = exact_projection(img, synth.UP_PAYLOAD, synth.UP_SCALES, 512, 4096, x64)
    assert np.array_equal(out["gate"], gate) and np.array_equal(out["up"], up)
    assert np.array_equal(out["h"], O.silu_up(gate, up))
    p, s, f = O.quant_v1(out["h"])
    assert not f.any() and np.array_equal(p, out["mid_payload"]) and np.array_equal(s, out["mid_scales"])
    mid64 = O.activation_decode(p, s)[0].astype(np.float64)
    assert np.array_equal(out["y"], exact_projection(img, synth.DOWN_PAYLOAD, synth.DOWN_SCALES, 4096, 512, mid64))


@pytest.fixture(scope="module")
def tiny_layer():
    wl = synth.make(1, rows=4)
    pools4 = [synth.rank_pool(wl.seed, r, wl.touched()[:3]) for r in range(4)]
    return wl, pools4


def test_expert_ffn_brute_force_one_row(tiny_layer):
    wl, pools4 = tiny_layer
    e = int(wl.touched()[0])
    out = O.expert_ffn(pools4[:1], e, wl.payload[:1], wl.scales[:1])
    x = O.activation_decode(wl.payload[:1], wl.scales[:1])[0][0]
    img = pools4[0][e * synth.IMAGE_BYTES:(e + 1) * synth.IMAGE_BYTES]
    gw = O.mxfp4_rows(img[:synth.GATE_SCALES].reshape(512, 2048), img[synth.GATE_SCALES:synth.UP_PAYLOAD].reshape(512, 128))
    for n in (0, 1, 255, 511):
        acc = 0.0
        for k in range(4096):
            acc += float(x[k]) * float(gw[n, k])
        assert out["gate"][0, n] == np.float32(acc)
    dw = O.mxfp4_rows(img[synth.DOWN_PAYLOAD:synth.DOWN_SCALES].reshape(4096, 256), img[synth.DOWN_SCALES:].reshape(4096, 16))
    mid = O.activation_decode(out["mid_payload"], out["mid_scales"])[0][0]
    for c in (0, 17, 4095):
        acc = 0.0
        for k in range(512):
            acc += float(mid[k]) * float(dw[c, k])
        assert out["y"][0, c] == np.float32(acc)


def test_rank_split_and_prefix_identities(tiny_layer):
    """lattice_oracle.py:78-88 (rank-local K32 bytes equal the full-row bytes; four rank partials sum to
    the full product) and :205-209 (M-prefix identity)."""
    wl, pools4 = tiny_layer
    e = int(wl.touched()[1])
    full = O.expert_ffn(pools4, e, wl.payload, wl.scales)
    assert full["fault"] == 0
    ysum = np.zeros((wl.rows, 4096), np.float64)
    for r in range(4):
        part = O.expert_ffn([pools4[r]], e, wl.payload, wl.scales)
        sl = slice(512 * r, 512 * (r + 1))
        for k in ("gate", "up", "h", "mid_payload"):
            assert np.array_equal(part[k], full[k][:, sl]), (r, k)
        assert np.array_equal(part["mid_scales"], full["mid_scales"][:, 16 * r:16 * (r + 1)])
        ysum += part["y"].astype(np.float64)
    # each rank partial and the full product were rounded to FP32 once: five half-ulp roundings at most
    assert np.max(np.abs(ysum - full["y"])) <= 5 * 2.0 ** -24 * np.max(np.abs(full["y"]))
    for m in (1, 2):
        pre = O.expert_ffn(pools4, e, wl.payload[:m], wl.scales[:m])
        for k in ("gate", "up", "h", "mid_payload", "mid_scales", "y"):
            assert np.array_equal(pre[k], full[k][:m]), (m, k)


def test_layer_ffn_is_plan_plus_experts_plus_reduce(tiny_layer):
    wl, _ = tiny_layer
    pools = [synth.rank_pool(wl.seed, 0, wl.touched())]
    rc, partial, bf16, y = O.layer_ffn(pools, wl.payload, wl.scales, wl.ids, wl.weights, want_routes=True)
    assert rc == 0
    for t in range(wl.rows):
        for s in range(8):
            one = O.expert_ffn(pools, int(wl.ids[t, s]), wl.payload[t:t + 1], wl.scales[t:t + 1])
            assert np.array_equal(one["y"][0], y[t * 8 + s])
    st, p2, b2 = O.reduce(y.reshape(wl.rows, 8, 4096), wl.weights)
    assert st == 0 and np.array_equal(p2, partial) and np.array_equal(b2, bf16)
    # mutation detectors: weight applied twice, intermediate rounding dropped, per-route BF16 return
    twice = O.reduce(y.reshape(wl.rows, 8, 4096) * wl.weights[:, :, None], wl.weights)[1]
    assert not np.allclose(twice, partial, rtol=1e-5, atol=1e-5)
    one = O.expert_ffn(pools, int(wl.ids[0, 0]), wl.payload[:1], wl.scales[:1])
    img = pools[0][int(wl.ids[0, 0]) * synth.IMAGE_BYTES:][:synth.IMAGE_BYTES]
    dw = O.mxfp4_rows(img[synth.DOWN_PAYLOAD:synth.DOWN_SCALES].reshape(4096, 256), img[synth.DOWN_SCALES:].reshape(4096, 16))
    dropped = (one["h"].astype(np.float64) @ dw.astype(np.float64).T).astype(np.float32)
    assert not np.allclose(dropped, one["y"], rtol=1e-5, atol=1e-5)
    rc2, p_e, _, _ = O.layer_ffn(pools, wl.payload, wl.scales, wl.ids, wl.weights, efp32=True)
    assert rc2 == 0 and np.max(np.abs(p_e - partial)) / np.max(np.abs(partial)) < 0.05  # same routing, looser numerics


def test_layer_ffn_rejects_bad_routes_and_inputs(tiny_layer):
    wl, _ = tiny_layer
    pools = [synth.rank_pool(wl.seed, 0, wl.touched())]
    ids = wl.ids.copy(); ids[1, 3] = ids[1, 2]
    assert O.layer_ffn(pools, wl.payload, wl.scales, ids, wl.weights)[0] == 3
    pay = wl.payload.copy(); pay[2, 100] = 0x7F
    assert O.layer_ffn(pools, pay, wl.scales, wl.ids, wl.weights)[0] == 4
    sc = wl.scales.copy(); sc[0, 5] = 104
    assert O.layer_ffn(pools, wl.payload, sc, wl.ids, wl.weights)[0] == 4
