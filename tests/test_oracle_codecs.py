"""Pins the CPU checker's codecs (oracle/b1_oracle.c) before anything is compared with it:
the reference's own golden data files, vectors produced by the reference's compiled host units
(committed fixture, and live where oracle/_ref was built), closed forms and exact-rational
referees."""
import json
import math
import os
from fractions import Fraction

import numpy as np
import pytest

import b1_oracle as O

GOLD = os.path.join(os.path.dirname(__file__), "golden")
FIX = np.load(os.path.join(GOLD, "b1_host_units.npz"))
needs_ref = pytest.mark.skipif(not O.ref_available(), reason="oracle/_ref not built (reference tree absent)")
CODEBOOK = [0.0, 0.5, 1.0, 1.5, 2.0, 3.0, 4.0, 6.0]
F32MAX = float(np.finfo(np.float32).max)


def f32_bits(v: float) -> int:
    return int(np.array([v], np.float32).view(np.uint32)[0])


# ---- MXFP4 ---------------------------------------------------------------------------------------
def test_mxfp4_reference_golden_file():
    """The reference's 64x64 pack/unpack golden (oracle/goldens/mxfp4_golden.json)."""
    g = json.load(open(os.path.join(GOLD, "ref_mxfp4_golden.json")))
    packed = np.frombuffer(bytes.fromhex(g["packed_u8_hex"]), np.uint8).reshape(g["packed_shape"])
    scales = np.frombuffer(bytes.fromhex(g["scales_u8_hex"]), np.uint8).reshape(g["scale_shape"])
    want = np.frombuffer(bytes.fromhex(g["unpacked_f32_hex"]), np.uint32).reshape(64, 64)
    assert np.array_equal(O.mxfp4_rows(packed, scales).view(np.uint32), want)
    assert [f32_bits(v) for v in g["e2m1_codebook_by_nibble"]] == [O.mxfp4_bits(n, 127) for n in range(16)]


def test_mxfp4_hand_vector():
    """crates/mimo26-expert/tests/unpack_fixture.rs:12-22: byte 0x71, scales 127 then 128."""
    row = O.mxfp4_rows(np.full((1, 32), 0x71, np.uint8), np.array([[127, 128]], np.uint8)).view(np.uint32)[0]
    assert [int(row[i]) for i in (0, 1, 32, 33)] == [0x3F000000, 0x40C00000, 0x3F800000, 0x41400000]


def test_mxfp4_closed_form_all_pairs():
    """codebook[n] * 2^(min(s,254)-127) as an exact rational, saturated; -0 kept; s = 0 is 2^-127."""
    for n in range(16):
        for s in range(256):
            exact = Fraction(CODEBOOK[n & 7]) * Fraction(2) ** (min(s, 254) - 127)
            want = min(float(exact), F32MAX) if exact <= Fraction(F32MAX) else F32MAX
            bits = f32_bits(want) | (0x80000000 if n & 8 else 0)
            assert O.mxfp4_bits(n, s) == bits, (n, s)
            if exact <= Fraction(F32MAX):
                assert Fraction(float(np.array([bits & 0x7FFFFFFF], np.uint32).view(np.float32)[0])) == exact
    assert O.mxfp4_bits(8, 3) == 0x80000000 and O.mxfp4_bits(1, 0) == f32_bits(2.0 ** -128)


def test_mxfp4_committed_reference_decoder_table():
    got = np.array([[O.mxfp4_bits(n, s) for s in range(256)] for n in range(16)], np.uint32)
    assert np.array_equal(got, FIX["mxfp4_bits"])


@needs_ref
def test_mxfp4_live_reference_decoder():
    assert all(O.mxfp4_bits(n, s) == O.REF.ref_mxfp4_bits(n, s) for n in range(16) for s in range(256))


# ---- E4M3FN ---------------------------------------------------------------------------------------
def test_e4m3_reference_decode_table():
    table = json.load(open(os.path.join(GOLD, "ref_e4m3_decode_table.json")))["table"]
    for code, want in enumerate(table):
        got = O.e4m3_value(code)
        if want is None:
            assert math.isnan(got)
        else:
            assert got == want and math.copysign(1, got) == math.copysign(1, want), code
    assert O.e4m3_value(0x38) == 1.0  # crates/mimo26-spark/src/serve.rs:362-370


def test_activation_decode_scale_window():
    p = np.full((1, 64), 0x38, np.uint8)
    for s, ok in ((104, False), (105, True), (127, True), (247, True), (248, False), (255, False)):
        out, bad = O.activation_decode(p, np.array([[s, 127]], np.uint8))
        assert (bad == 0) == ok
        if ok:
            assert out[0, 0] == 2.0 ** (s - 127) and out[0, 40] == 1.0
    p[0, 5] = 0x7F
    assert O.activation_decode(p, np.array([[127, 127]], np.uint8))[1] == 1


# ---- Q0, the wire input quantizer --------------------------------------------------------------------
def _nearest_ties_up(mag: np.ndarray) -> np.ndarray:
    """Direct search of the decode table: nearest code, ties to the larger code
    (the reference's own referee, crates/mimo26-load/src/e4m3.rs:151-168)."""
    tab = np.array([O.e4m3_value(c) for c in range(0x7F)], np.float64)
    mag = np.minimum(mag, 448.0)
    hi = np.searchsorted(tab, mag, side="left")
    hi = np.minimum(hi, 0x7E)
    lo = np.maximum(hi - 1, 0)
    pick_lo = (mag - tab[lo]) < (tab[hi] - mag)
    return np.where((hi > 0) & pick_lo, lo, hi)


def test_q0_encoder_brute_force_all_bf16_and_scales():
    bf16 = (np.arange(65536, dtype=np.uint32) << 16).view(np.float32)
    vals = bf16[np.isfinite(bf16)].astype(np.float64)
    for shift in range(-12, 13):  # the scaled value v * 2^(127-s) for every plausible block scale
        v = np.ldexp(vals, shift)
        got = np.array([O.LIB.orc_e4m3_encode_half_up(float(x)) for x in v[::7]], np.uint8)
        want = _nearest_ties_up(np.abs(v[::7])).astype(np.uint8) | np.where(v[::7] < 0, 0x80, 0).astype(np.uint8)
        assert np.array_equal(got, want), shift


def test_q0_encoder_stated_vectors():
    """crates/mimo26-load/src/e4m3.rs:180-208."""
    enc = lambda v: int(O.LIB.orc_e4m3_encode_half_up(float(v)))
    for c in range(0x7F):
        assert enc(O.e4m3_value(c)) == c
    assert enc(7.5 / 512) == 0x08 and enc(7.0 / 512) == 0x07 and enc(2.0 ** -6) == 0x08
    assert enc(1e9) == 0x7E and enc(-1e9) == 0xFE and enc(float("nan")) == 0 and enc(-0.0) == 0x00
    assert enc(-1e-9) == 0x80  # below zero, rounds to magnitude 0, keeps the sign bit


def test_q0_scale_formula_on_boundary_neighbours():
    """s = clamp(ceil(log2(amax/448)) + 127, 0, 254) as the reference writes it
    (crates/mimo26-coordinator/src/wire.rs:66-71), on both sides of every 448 * 2^k."""
    cases = []
    for k in range(-140, 125):
        b = np.float32(np.ldexp(448.0, k))
        if not np.isfinite(b) or b == 0:
            continue
        cases += [b, np.nextafter(b, np.float32(0)), np.nextafter(b, np.float32(np.inf)), np.float32(b * 1.3)]
    cases += [np.float32(1e-45), np.float32(F32MAX), np.float32(1.0), np.float32(0.875), np.float32(0.8750001)]
    for a in cases:
        if not np.isfinite(a) or a == 0:
            continue
        x = np.zeros((1, 32), np.float32)
        x[0, 11] = -a
        want = int(min(max(math.ceil(math.log2(float(a) / 448.0)) + 127, 0), 254))
        assert int(O.q0_quantize(x)[1][0, 0]) == want, float(a)
    assert int(O.q0_quantize(np.zeros((1, 32), np.float32))[1][0, 0]) == 0


def test_q0_block_matches_definition_on_random_rows():
    rng = np.random.default_rng(5)
    x = (rng.standard_normal((40, 256)) * np.exp2(rng.integers(-30, 30, (40, 1)))).astype(np.float32)
    x = (x.view(np.uint32) & 0xFFFF0000).view(np.float32)  # bf16-valued like the serving inputs
    payload, scales = O.q0_quantize(x)
    amax = np.abs(x.reshape(40, 8, 32)).max(-1).astype(np.float64)
    want_s = np.clip(np.ceil(np.log2(amax / 448.0)) + 127, 0, 254).astype(np.uint8)
    assert np.array_equal(scales, want_s)
    y = np.ldexp(x.reshape(40, 8, 32).astype(np.float64), 127 - scales.astype(np.int64)[..., None]).reshape(40, 256)
    want_p = _nearest_ties_up(np.abs(y)).astype(np.uint8) | np.where(y < 0, 0x80, 0).astype(np.uint8)
    assert np.array_equal(payload, want_p)


# ---- quantizer v1 -----------------------------------------------------------------------------------
def test_quant_v1_committed_reference_vectors():
    """Outputs of the reference's compiled quantize_host on the committed corpus."""
    h = FIX["quant_h"].view(np.float32)
    p, s, f = O.quant_v1(h)
    assert np.array_equal(f, FIX["quant_faults"])
    assert np.array_equal(p, FIX["quant_payload"]) and np.array_equal(s, FIX["quant_scales"])
    ok = f.ravel() == 0
    assert set(np.unique(s.ravel()[ok])) == set(range(105, 248))           # all 143 scale bytes
    assert len(np.unique(p[ok.nonzero()[0]] & 0x7F)) == 127                # every finite magnitude code
    assert (p[~ok] == 0xA5).all() and (s.ravel()[~ok] == 0xA5).all()      # a faulting block publishes nothing


@needs_ref
def test_quant_v1_live_differential():
    rng = np.random.default_rng(99)
    h = (rng.standard_normal((30000, 32)) * np.exp2(rng.integers(-149, 128, (30000, 1)).astype(np.float64))).astype(np.float32)
    bits = rng.integers(0, 2 ** 32, (5000, 32), dtype=np.uint64).astype(np.uint32).view(np.float32)
    h = np.concatenate([h, bits])
    mine, ref = O.quant_v1(h), O.ref_quant_v1(h)
    assert all(np.array_equal(a, b) for a, b in zip(mine, ref[:3]))


def test_quant_v1_reference_edge_vectors():
    """oracle/tests/test_lattice_quant_v1.py:69,81-90,121-127 of the reference."""
    z = np.zeros(32, np.float32)
    z[3] = -0.0
    p, s, f = O.quant_v1(z)
    assert s.tolist() == [105] and p[3] == 0x80 and (np.delete(p, 3) == 0).all() and f.tolist() == [0]
    assert O.quant_v1(np.full(32, 3e-9, np.float32))[1].tolist() == [105]
    big = np.zeros(32, np.float32)
    big[0] = F32MAX
    p, s, f = O.quant_v1(big)
    assert f.tolist() == [2] and (p == 0xA5).all()  # scale would be 247; reconstruction leaves FP32
    t = np.zeros(32, np.float32)
    t[0], t[1], t[2], t[3] = 448.0, 2.0 ** -10, -(2.0 ** -10), -(2.0 ** -12)
    p, s, f = O.quant_v1(t)
    assert s.tolist() == [127] and p[:4].tolist() == [0x7E, 0x00, 0x80, 0x80]
    for bad in (np.nan, np.inf, -np.inf):
        t[9] = bad
        assert O.quant_v1(t)[2].tolist() == [1]


@pytest.mark.parametrize("a", [1e-4, 1.0, 448.0, 448.0000305, 449.0, 896.0, 0.875, 0.8750001, 3.0e-3, 1.17549435e-38,
                               F32MAX / 2, 2.0 ** 100 * 448, 2.0 ** 100 * 448 * (1 + 2 ** -23)])
def test_quant_v1_scale_is_smallest_power_of_two_that_fits(a):
    h = np.zeros(32, np.float32)
    h[17] = a
    k = int(O.quant_v1(h)[1][0]) - 127
    fa = Fraction(float(np.float32(max(a, 1e-4))))
    assert fa <= 448 * Fraction(2) ** k and not fa <= 448 * Fraction(2) ** (k - 1)


def _rne_e4m3_exact(y: Fraction) -> Fraction:
    """Nearest E4M3FN magnitude to |y| with ties to the even code, over exact rationals."""
    grid = [Fraction(O.e4m3_value(c)) for c in range(0x7F)]
    ay = abs(y)
    best = min(range(0x7F), key=lambda c: (abs(grid[c] - ay), c & 1))
    return grid[best]


def test_quant_v1_exact_rational_referee():
    rng = np.random.default_rng(20260923)
    for _ in range(60):
        h = (rng.standard_normal(32) * 10.0 ** rng.uniform(-12, 12)).astype(np.float32)
        h[rng.integers(0, 32, 3)] *= np.float32(10.0 ** rng.uniform(-8, 0))
        p, s, f = O.quant_v1(h)
        assert f.tolist() == [0]
        k = int(s[0]) - 127
        for x, code in zip(h, p):
            assert Fraction(abs(O.e4m3_value(int(code)))) == _rne_e4m3_exact(Fraction(float(x)) / Fraction(2) ** k)
            assert bool(code & 0x80) == bool(np.signbit(x))


def test_quant_v1_mutants_are_detected():
    """Wrong variants the reference names (kernels/b1/README.md:26-36) must disagree with the codec."""
    rng = np.random.default_rng(3)
    h = (rng.standard_normal((400, 32)) * np.exp2(rng.integers(-20, 20, (400, 1)))).astype(np.float32)
    p, s, _ = O.quant_v1(h)
    k = s.astype(np.int64) - 127
    amax = np.abs(h).max(-1).astype(np.float64)
    nearest = np.rint(np.log2(amax / 448.0)).astype(np.int64)
    assert np.any(nearest != k[:, 0])                                    # nearest-scale mutant
    trunc = np.floor(np.ldexp(np.abs(h).astype(np.float64), 3 - k))      # truncation mutant differs somewhere
    assert np.any(trunc != np.rint(np.ldexp(np.abs(h).astype(np.float64), 3 - k)))
    hb = ((h.view(np.uint32).astype(np.uint64) + 0x7FFF + ((h.view(np.uint32) >> 16) & 1)) & 0xFFFF0000).astype(np.uint32).view(np.float32)
    assert not np.array_equal(O.quant_v1(hb)[0], p)                      # BF16 pre-round mutant


# ---- BF16 ----------------------------------------------------------------------------------------
def test_bf16_rne():
    for v, want in ((1.0 + 1.0 / 256, 0x3F80), (1.0 + 3.0 / 256, 0x3F82), (-(1.0 + 1.0 / 256), 0xBF80), (2.0 ** -127, 0x0040)):
        assert O.LIB.orc_bf16_rne(float(v)) == want
