"""What the GPU decodes: the MXFP4 weight format as the block-scaled MFMA reads it, for every E2M1 code
under every ordinary scale byte, and the conforming arm for the exceptional bytes 0, 1, 253, 254, 255.

The reference gates its MMA primitive the same way before anything else runs on it (all code x scale
container pairs, crates/mimo26-expert/tests/b1_core/primitive.cu:74-82,107-120) and probes its
exceptional arm with crates/mimo26-expert/tests/b1_core/compute_test.cuh:100-128. Here both go through
the library's own C ABI (m26s_b1_ffn_dev with the stage taps on).

The pin isolates single products. A pinned weight row holds one nonzero code, so each of its outputs is
one product x * w plus exact zeros, and that product of an E4M3 value at a power-of-two scale and an
E2M1 value at a power-of-two scale has at most eight significant bits: wherever it lies in binary32's
range (subnormals included) it is representable, the accumulation order cannot matter, and the GPU
has to return exactly the checker's decode of w times the checker's decode of x.
"""
import numpy as np
import pytest

import b1_oracle as O
from helpers import DeviceLayer, bf16_to_f32, parity, run_ffn_dev
from mimo26f_afd_amd import b1, synth

pytestmark = pytest.mark.gpu

NONZERO = np.array([1, 2, 3, 4, 5, 6, 7, 9, 10, 11, 12, 13, 14, 15], np.uint8)  # every code but +0 and -0
MXFP4 = np.array([[O.mxfp4_bits(c, s) for s in range(256)] for c in range(16)], np.uint32).view(np.float32)
E4M3 = np.array([O.e4m3_value(c) for c in range(256)], np.float32)
GATE_SET, UP_SET, DOWN_EXPERT = range(0, 8), range(8, 16), 16


def sparse_region(rows, k_len, first_pair, s_lo, s_hi):
    """Weight rows with one nonzero code each: row n holds pair first_pair + n of the walk over
    (code, scale byte), at column (131 n + 7 (pair / 512)) % K. Every other block of the row carries zero
    codes under some legal scale byte. Returns payload [rows, K/2], scales [rows, K/32] and the per-row
    column, code and scale byte."""
    n = np.arange(rows)
    pair = first_pair + n
    span = s_hi - s_lo + 1
    code = NONZERO[pair % 14]
    sc = (s_lo + (pair // 14) % span).astype(np.uint8)
    k = (n * 131 + 7 * (pair // 512)) % k_len
    payload = np.zeros((rows, k_len // 2), np.uint8)
    payload[n, k // 2] = np.where(k % 2 == 0, code, code << 4)           # low nibble = even k
    scales = (s_lo + (n[:, None] * 3 + np.arange(k_len // 32)[None, :] * 5) % span).astype(np.uint8)
    scales[n, k // 32] = sc
    return payload, scales, k, code, sc


def blank_image():
    img = np.zeros(synth.IMAGE_BYTES, np.uint8)                           # every code +0 ...
    for lo, hi in synth.SCALE_REGIONS:
        img[lo:hi] = 127                                                  # ... under the unit scale
    return img


def pin_pool(s_hi):
    """Experts 0..7: gate rows pinned (up zero), 8..15: up rows pinned (gate zero), both over scale bytes
    2..s_hi; expert 16: dense gate/up at scale byte 115 and pinned down rows over 2..252."""
    pool = np.full(synth.EXPERTS * synth.IMAGE_BYTES, 0x22, np.uint8)
    rows_of = {}
    for e in list(GATE_SET) + list(UP_SET):
        img = blank_image()
        pay, sc, k, code, s = sparse_region(512, 4096, (e % 8) * 512, 2, s_hi)
        poff, soff = (0, synth.GATE_SCALES) if e in GATE_SET else (synth.UP_PAYLOAD, synth.UP_SCALES)
        img[poff:poff + pay.size] = pay.reshape(-1)
        img[soff:soff + sc.size] = sc.reshape(-1)
        pool[e * synth.IMAGE_BYTES:(e + 1) * synth.IMAGE_BYTES] = img
        rows_of[e] = (k, code, s)
    img = synth.expert_image(synth.BASE_SEED + 40, 0, DOWN_EXPERT)
    img[synth.GATE_SCALES:synth.UP_PAYLOAD] = 115
    img[synth.UP_SCALES:synth.DOWN_PAYLOAD] = 115
    pay, sc, k, code, s = sparse_region(4096, 512, 0, 2, 252)
    img[synth.DOWN_PAYLOAD:synth.DOWN_PAYLOAD + pay.size] = pay.reshape(-1)
    img[synth.DOWN_SCALES:] = sc.reshape(-1)
    pool[DOWN_EXPERT * synth.IMAGE_BYTES:(DOWN_EXPERT + 1) * synth.IMAGE_BYTES] = img
    rows_of[DOWN_EXPERT] = (k, code, s)
    return pool, rows_of


def pin_rows(per_set, sx):
    """2 * per_set rows whose codes walk every finite E4M3 code (subnormals, both zeros, 448) under the
    one scale byte sx (at 247 only the codes whose value stays finite in binary32), then 16 rows of
    N(0,1) through the wire quantizer for the down pin."""
    finite = np.array([c for c in range(256) if (c & 0x7F) != 0x7F and (sx < 247 or (c & 0x7F) <= 0x77)], np.uint8)
    m = np.arange(2 * per_set)[:, None]
    k = np.arange(4096)[None, :]
    payload = finite[(5 * k + 37 * m + 3 * (k // 32)) % finite.size]
    scales = np.full((2 * per_set, 128), sx, np.uint8)
    x = synth._activations(synth.BASE_SEED + 41, 16)
    qp, qs = synth.q0_quantize(x)
    ids = np.concatenate([np.tile(np.array(GATE_SET, np.int32), (per_set, 1)), np.tile(np.array(UP_SET, np.int32), (per_set, 1)),
                          np.tile(np.arange(DOWN_EXPERT, DOWN_EXPERT + 8, dtype=np.int32), (16, 1))])
    rows = ids.shape[0]
    w = synth._softmax_weights(synth.BASE_SEED + 41, rows)
    return synth.Workload(f"decode pin, scale byte {sx}", -1, 0, 1, rows, ids, w, np.zeros((rows, 4096), np.float32),
                          np.concatenate([payload, qp]), np.concatenate([scales, qs]))


def single_products(x64, w32):
    """Elementwise x (binary64, exact) times w (the checker's binary32 decode): the binary32 value the GPU
    must return wherever the product is representable, and where that is."""
    with np.errstate(over="ignore", under="ignore"):
        p = x64 * w32.astype(np.float64)
        as32 = p.astype(np.float32)
        exact = np.isfinite(as32) & (as32.astype(np.float64) == p)
    return as32, exact


# (activation scale byte, highest weight scale byte that keeps every product below 2^128)
PIN_CLASSES = [(105, 252), (127, 242), (247, 122)]


@pytest.mark.parametrize("per_set", [16, 80])
def test_mfma_decodes_every_code_under_every_ordinary_scale(per_set):
    """All 14 nonzero E2M1 codes x scale bytes 2..252, on gate rows, up rows and down rows, against E4M3
    activations of every finite code at the ends and the middle of the legal activation window. 32 + 16
    rows take the one-tile direct schedule, 160 + 16 the tile schedule (chunks of five groups)."""
    covered = {"gate": set(), "up": set(), "down": set()}
    for sx, s_hi in PIN_CLASSES:
        pool, rows_of = pin_pool(s_hi)
        layer = DeviceLayer([pool]).layer
        assert layer.all_scales_normal() and layer.intermediate == 512
        scratch = b1.Scratch()
        scratch.set_taps(True)
        wl = pin_rows(per_set, sx)
        stats, _, _ = run_ffn_dev(layer, scratch, wl, want_partial=False)
        groups = scratch.view("groups", O.GROUP_DTYPE, stats.groups)
        n_rows = stats.groups * 16
        taps = {k: scratch.view(k, np.float32, n_rows * 512).reshape(n_rows, 512) for k in ("gate", "up")}
        mid_p = scratch.view("mid_payload", np.uint8, n_rows * 512).reshape(n_rows, 512)
        mid_s = scratch.view("mid_scales", np.uint8, n_rows * 16).reshape(n_rows, 16)
        y = scratch.view("y", np.float32, wl.rows * 8 * 4096).reshape(wl.rows, 8, 4096)
        x64 = np.ldexp(E4M3[wl.payload].astype(np.float64), wl.scales.astype(np.int64).repeat(32, axis=1) - 127)
        seen = set()
        for gi, g in enumerate(groups):
            e, r = int(g["expert"]), int(g["rows"])
            if e not in rows_of:
                continue
            seen.add(e)
            tokens = g["input_rows"][:r]
            k, code, s = rows_of[e]
            w32 = MXFP4[code, s]
            for j, t in enumerate(tokens):
                if e == DOWN_EXPERT:                                   # on the intermediate bytes the GPU itself wrote
                    mid64 = np.ldexp(E4M3[mid_p[gi * 16 + j]].astype(np.float64), mid_s[gi * 16 + j].astype(np.int64).repeat(32) - 127)
                    want, exact = single_products(mid64[k], w32)
                    name, got = "down", y[t, 0]
                else:
                    want, exact = single_products(x64[t, k], w32)
                    name = "gate" if e in GATE_SET else "up"
                    got = taps[name][gi * 16 + j]
                    other = taps["up" if name == "gate" else "gate"][gi * 16 + j]
                    assert not other.any(), (sx, e, "the unpinned projection is all zero codes")
                bad = exact & (got.view(np.uint32) != want.view(np.uint32)) & ~((got == 0) & (want == 0))
                assert not bad.any(), (name, sx, e, int(t), [(int(code[i]), int(s[i]), float(got[i]), float(want[i])) for i in np.flatnonzero(bad)[:4]])
                hit = exact & (want != 0)
                covered[name].update(zip(code[hit].tolist(), s[hit].tolist()))
        assert seen == set(rows_of), seen
    every = {(int(c), sb) for c in NONZERO for sb in range(2, 253)}
    for name, pairs in covered.items():
        assert every <= pairs, (name, sorted(every - pairs)[:8])


def test_swiglu_on_deeply_negative_gates():
    """Gates between -16 and -360 fed as exact single products. Down to about -87.3 the exponential is a normal
    binary32 number and the activation stays within the usual few ulp of the CPU rule. Below that the CPU rule's
    exp (and the expf of the reference's kernels, crates/mimo26-expert/kernels/b1/grouped.cu:89) is a subnormal,
    which the hardware 2^x returns as zero: the kernel's h is a signed zero where the rule's is at most
    104 * 2^-126 |u| in magnitude, twenty orders of magnitude under the quantizer's floor, and the bytes of the
    requantised intermediate are the same either way."""
    pool = np.full(synth.EXPERTS * synth.IMAGE_BYTES, 0x22, np.uint8)
    n = np.arange(512)
    img = blank_image()
    gate_pay, up_pay = np.zeros((512, 2048), np.uint8), np.zeros((512, 2048), np.uint8)
    gate_pay[:, 0] = np.array([0xF, 0xE, 0xD, 0xC], np.uint8)[n % 4]          # -6, -4, -3, -2 at k = 0 ...
    gate_sc, up_sc = np.full((512, 128), 127, np.uint8), np.full((512, 128), 127, np.uint8)
    gate_sc[:, 0] = 127 + (n // 4) % 2                                          # ... times 1 or 2
    up_pay[:, 0] = 0x2                                                          # +1.0 at k = 0 ...
    up_sc[:, 0] = 127 - n % 8                                                   # ... times 2^-(n % 8)
    img[0:gate_pay.size] = gate_pay.reshape(-1)
    img[synth.GATE_SCALES:synth.UP_PAYLOAD] = gate_sc.reshape(-1)
    img[synth.UP_PAYLOAD:synth.UP_PAYLOAD + up_pay.size] = up_pay.reshape(-1)
    img[synth.UP_SCALES:synth.DOWN_PAYLOAD] = up_sc.reshape(-1)
    pool[:synth.IMAGE_BYTES] = img
    for e in range(1, 8):
        pool[e * synth.IMAGE_BYTES:(e + 1) * synth.IMAGE_BYTES] = blank_image()
    layer = DeviceLayer([pool]).layer
    assert layer.all_scales_normal()
    rows = 16
    payload = np.zeros((rows, 4096), np.uint8)
    payload[:, 0] = np.array([0x50 + i for i in range(8)] + [0x58 + i for i in range(8)], np.uint8)   # 8..15, 16..30
    scales = np.full((rows, 128), 127, np.uint8)
    x0 = E4M3[payload[:, 0]].astype(np.float64)
    assert x0.tolist() == [8, 9, 10, 11, 12, 13, 14, 15, 16, 18, 20, 22, 24, 26, 28, 30]
    ids = np.tile(np.arange(8, dtype=np.int32), (rows, 1))
    w = np.full((rows, 8), 0.125, np.float32)
    wl = synth.Workload("deep negative gates", -1, 0, 1, rows, ids, w, np.zeros((rows, 4096), np.float32), payload, scales)
    scratch = b1.Scratch()
    scratch.set_taps(True)
    stats, _, _ = run_ffn_dev(layer, scratch, wl, want_partial=False)
    groups = scratch.view("groups", O.GROUP_DTYPE, stats.groups)
    gi = int(np.flatnonzero(groups["expert"] == 0)[0])
    sl = slice(gi * 16, gi * 16 + rows)
    taps = {k: scratch.view(k, np.float32, stats.groups * 16 * 512).reshape(-1, 512)[sl] for k in ("gate", "up", "h")}
    mid = scratch.view("mid_payload", np.uint8, stats.groups * 16 * 512).reshape(-1, 512)[sl]
    wg = MXFP4[gate_pay[:, 0] & 15, gate_sc[:, 0]].astype(np.float64)
    wu = MXFP4[up_pay[:, 0] & 15, up_sc[:, 0]].astype(np.float64)
    assert np.array_equal(taps["gate"].astype(np.float64), x0[:, None] * wg[None, :])        # exact single products
    assert np.array_equal(taps["up"].astype(np.float64), x0[:, None] * wu[None, :])
    g, u = taps["gate"], taps["up"]
    assert g.min() == -360 and ((g <= -80) & (g >= -104)).sum() > 500 and ((g > -87) & (g <= -16)).sum() > 1000
    rule = O.silu_up(g, u)
    diff = np.abs(taps["h"].astype(np.float64) - rule.astype(np.float64))
    normal_exp = g > -87.0                                                       # exp(g) is a normal binary32 number
    assert np.all(diff[normal_exp] <= 8 * np.spacing(np.abs(rule[normal_exp])))
    assert np.all(diff[~normal_exp] <= 2.0 ** -119 * np.abs(u[~normal_exp]))
    assert np.all(np.signbit(taps["h"]))                                         # negative gate, positive up: the sign survives a flushed zero
    qp, _, qf = O.quant_v1(rule)
    assert not qf.any() and np.array_equal(qp[~normal_exp], mid[~normal_exp])    # the requantised bytes do not see it
    assert np.mean(qp == mid) > 0.995


def exceptional_pool(wl, seed):
    """A rank pool of wl's touched experts with exceptional weight scale bytes sown over all three
    projections of every touched expert: bytes 0 and 1 in about one block in 64 (decoded weights down to
    the binary32 subnormals; the saturating bytes 253..255 would overflow every sum against N(0,1)
    activations and have the probe test below to themselves)."""
    pool = synth.rank_pool(seed, 0, wl.touched())
    rng = np.random.default_rng(seed)
    for e in wl.touched():
        base = int(e) * synth.IMAGE_BYTES
        for lo, hi in synth.SCALE_REGIONS:
            region = pool[base + lo:base + hi]
            where = rng.random(region.size) < 1 / 64
            region[where] = rng.choice(np.array([0, 1], np.uint8), int(where.sum()))
    return pool


def test_conforming_arm_matches_the_cpu_rule_bit_for_bit_on_subnormal_scales():
    """Weight scale bytes 0 and 1 (decoded weights are binary32 subnormals and near-subnormals): the layer
    is flagged, served by the conforming arm, and its gate / up / per-route rows are the CPU rule's
    binary64 dots bit for bit (same decode, same order of summation); the activation and everything
    behind it to the usual bars."""
    wl = synth.make(1)
    pool = exceptional_pool(wl, synth.BASE_SEED + 50)
    layer = DeviceLayer([pool]).layer
    assert not layer.all_scales_normal()
    scratch = b1.Scratch()
    scratch.set_taps(True)
    stats, bf, pf = run_ffn_dev(layer, scratch, wl)
    rc, ref_partial, ref_bf16, _ = O.layer_ffn([pool], wl.payload, wl.scales, wl.ids, wl.weights)
    assert rc == 0
    ma, mr = parity(pf, ref_partial)
    assert ma <= 1e-2 and mr <= 1e-3, (ma, mr)
    ma, mr = parity(bf16_to_f32(bf), bf16_to_f32(ref_bf16))
    assert ma <= 1e-2 and mr <= 1e-3, (ma, mr)
    groups = scratch.view("groups", O.GROUP_DTYPE, stats.groups)
    n_rows = stats.groups * 16
    taps = {k: scratch.view(k, np.float32, n_rows * 512).reshape(n_rows, 512) for k in ("gate", "up", "h")}
    mid_p = scratch.view("mid_payload", np.uint8, n_rows * 512).reshape(n_rows, 512)
    mid_s = scratch.view("mid_scales", np.uint8, n_rows * 16).reshape(n_rows, 16)
    y = scratch.view("y", np.float32, wl.rows * 8 * 4096).reshape(wl.rows * 8, 4096)
    plan = O.plan(256, wl.ids, wl.weights)
    for gi in (0, stats.groups // 2, stats.groups - 1):
        g = groups[gi]
        r, toks = int(g["rows"]), g["input_rows"][:int(g["rows"])]
        sl = slice(gi * 16, gi * 16 + r)
        want = O.expert_ffn([pool], int(g["expert"]), wl.payload[toks], wl.scales[toks])
        assert want["fault"] == 0
        assert np.array_equal(taps["gate"][sl].view(np.uint32), want["gate"].view(np.uint32))
        assert np.array_equal(taps["up"][sl].view(np.uint32), want["up"].view(np.uint32))
        qp, qs, qf = O.quant_v1(taps["h"][sl])
        assert not qf.any() and np.array_equal(qp, mid_p[sl]) and np.array_equal(qs, mid_s[sl])
        # FC2 on the bytes the GPU itself wrote: the checker's dot over the same decoded intermediate
        img = pool[int(g["expert"]) * synth.IMAGE_BYTES:][:synth.IMAGE_BYTES]
        dw = O.mxfp4_rows(img[synth.DOWN_PAYLOAD:synth.DOWN_SCALES].reshape(4096, 256), img[synth.DOWN_SCALES:].reshape(4096, 16))
        mid = O.activation_decode(mid_p[sl], mid_s[sl])[0]
        routes = plan.original_routes[int(g["route_base"]):int(g["route_base"]) + r]
        for j in range(r):
            acc = np.zeros(4096, np.float64)
            for k in range(512):                                        # ascending k, binary64, one rounding
                acc += float(mid[j, k]) * dw[:, k].astype(np.float64)
            assert np.array_equal(y[routes[j]].view(np.uint32), acc.astype(np.float32).view(np.uint32)), (gi, j)


def test_conforming_arm_on_the_reference_probe_of_every_exceptional_byte():
    """The reference's exceptional-scale probe (compute_test.cuh:100-128), through the whole FFN entry: one
    gate block per pinned row under scale byte 0, 1, 253, 254 or 255, codes (n + k) % 8 signed by n % 2,
    activations 256 or 2 at scale bytes 239/240 (small weights) or 105/106 (saturating weights) with -0
    at every eighth place; expected = the binary64 sum over the saturated decode, rounded once."""
    byte_of = [0, 1, 253, 254, 255]
    pool = np.full(synth.EXPERTS * synth.IMAGE_BYTES, 0x22, np.uint8)
    img = blank_image()
    n = np.arange(512)
    kb = (n * 7) % 128                                                     # the pinned block of gate row n
    t = n % 5                                                             # which exceptional byte it carries
    codes = ((n[:, None] + np.arange(32)[None, :]) % 8 | np.where(n % 2, 8, 0)[:, None]).astype(np.uint8)
    pay = np.zeros((512, 2048), np.uint8)
    for j in range(16):
        pay[n, kb * 16 + j] = codes[:, 2 * j] | (codes[:, 2 * j + 1] << 4)
    sc = np.full((512, 128), 127, np.uint8)
    sc[n, kb] = np.array(byte_of, np.uint8)[t]
    img[:pay.size] = pay.reshape(-1)
    img[synth.GATE_SCALES:synth.UP_PAYLOAD] = sc.reshape(-1)
    pool[3 * synth.IMAGE_BYTES:4 * synth.IMAGE_BYTES] = img
    layer = DeviceLayer([pool]).layer
    assert not layer.all_scales_normal()
    scratch = b1.Scratch()
    scratch.set_taps(True)
    got_by_class = {}
    for small in (True, False):                                          # bytes 0/1 against big activations, 253..255 against small ones
        rows = 16
        k = np.arange(4096)
        payload = np.tile(np.where(k % 8 == 0, 0x80, 0x78 if small else 0x40).astype(np.uint8), (rows, 1))
        scales = np.tile(((239 if small else 105) + np.arange(rows) % 2).astype(np.uint8)[:, None], (1, 128))
        ids = np.tile(np.array([3, 1, 2, 4, 5, 6, 7, 8], np.int32), (rows, 1))
        w = np.full((rows, 8), 0.125, np.float32)
        wl = synth.Workload("exceptional probe", -1, 0, 1, rows, ids, w, np.zeros((rows, 4096), np.float32), payload, scales)
        try:
            run_ffn_dev(layer, scratch, wl, want_partial=False)
        except b1.B1Error as err:                                        # sums past FLT_MAX are a numerical fault, as in the CPU rule
            assert err.code == 4, err
        groups = scratch.view("groups", O.GROUP_DTYPE, 8)
        gi = int(np.flatnonzero(groups["expert"] == 3)[0])
        gate = scratch.view("gate", np.float32, 8 * 16 * 512).reshape(8 * 16, 512)[gi * 16:gi * 16 + rows]
        x64 = np.ldexp(E4M3[payload].astype(np.float64), scales.astype(np.int64).repeat(32, axis=1) - 127)
        w_dec = MXFP4[codes, sc[n, kb][:, None]].astype(np.float64)      # [512, 32], saturated decode
        for row in range(rows):
            xb = x64[row].reshape(128, 32)[kb]                           # [512, 32]: the activations of each row's pinned block
            want = np.sum(xb * w_dec, axis=1)                            # 32 terms of at most 11 significant bits: exact in binary64
            with np.errstate(over="ignore"):
                want32 = want.astype(np.float32)
            use = (t < 2) if small else (t >= 2)
            assert np.array_equal(gate[row][use].view(np.uint32), want32[use].view(np.uint32)), (small, row)
            got_by_class[small] = True
    assert got_by_class == {True: True, False: True}
