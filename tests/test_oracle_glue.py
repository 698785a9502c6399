"""Pins of the checker's coordinator-side functions (router selection, the scale half of the wire
quantizer, rank sum, BF16 cast). The reference keeps no vectors for them, so each is held against a
library routine or a closed form chosen to catch a wrong order, a wrong tie rule or a fused operation."""
import numpy as np
from scipy.special import expit

import b1_oracle as O


def test_router_equals_a_stable_sort_of_library_sigmoids():
    rng = np.random.default_rng(5)
    logits = (rng.standard_normal((64, 256)) * 3).astype(np.float32)
    bias = (rng.standard_normal(256) * 0.2).astype(np.float32)
    idx, w = O.router_topk(logits, bias, 8)
    score = expit(logits.astype(np.float64))
    order = np.argsort(-(score + bias.astype(np.float64)), axis=1, kind="stable")[:, :8]
    assert np.array_equal(idx, order)
    chosen = np.take_along_axis(score, order, 1)
    want = chosen / np.cumsum(chosen, axis=1)[:, -1:]
    assert np.max(np.abs(w.astype(np.float64) - want)) <= 2.0 ** -24
    assert np.all(np.abs(w.sum(1, dtype=np.float64) - 1.0) < 1e-6)


def test_router_ties_go_to_the_lower_id_and_bias_only_selects():
    logits = np.zeros((1, 256), np.float32)
    idx, w = O.router_topk(logits, np.zeros(256, np.float32), 8)
    assert idx[0].tolist() == list(range(8)) and np.all(w == np.float32(0.125))
    bias = np.zeros(256, np.float32)
    bias[200:208] = 1.0                       # selection follows score + bias ...
    logits[0, 7] = 2.0                        # ... but the weights use the unbiased scores
    idx, w = O.router_topk(logits, bias, 8)
    assert idx[0].tolist() == list(range(200, 208)) and np.all(w == np.float32(0.125))
    idx, w = O.router_topk(logits, np.zeros(256, np.float32), 2)
    assert idx[0].tolist() == [7, 0]
    s7, s0 = expit(2.0), 0.5
    assert w[0, 0] == np.float32(s7 / (s7 + s0)) and w[0, 1] == np.float32(s0 / (s7 + s0))


def test_q0_scales_closed_form_and_consistency_with_the_full_quantizer():
    e = np.arange(-130, 120)
    x = np.zeros((e.size * 3, 32), np.float32)
    exact = np.ldexp(448.0, e)                # amax = 448 * 2^e exactly -> s = e + 127
    x[0::3, 5] = exact
    x[1::3, 9] = np.nextafter(exact.astype(np.float32), np.float32(np.inf))   # just above -> one more
    x[2::3, 0] = -np.nextafter(exact.astype(np.float32), np.float32(0))       # just below, negative
    s, inv = O.q0_scales(x)
    ok = np.isfinite(exact.astype(np.float32)) & (exact.astype(np.float32) > 0)
    want = np.clip(e + 127, 0, 254)
    assert np.array_equal(s[0::3][ok], want[ok])
    assert np.array_equal(s[1::3][ok & (e < 119)], np.clip(e + 128, 0, 254)[ok & (e < 119)])
    assert np.array_equal(s[2::3][ok], want[ok])
    assert np.array_equal(inv, np.ldexp(1.0, 127 - s.astype(int)).astype(np.float32))
    rng = np.random.default_rng(2)
    y = (rng.standard_normal((16, 4096)) * np.exp2(rng.integers(-20, 20, (16, 1)))).astype(np.float32)
    y[3, 64:96] = 0
    s2, _ = O.q0_scales(y)
    assert np.array_equal(s2.reshape(16, 128), O.q0_quantize(y)[1]) and s2.reshape(16, 128)[3, 2] == 0


def test_rank_sum_is_four_ordered_fp32_additions():
    rng = np.random.default_rng(9)
    p = (rng.standard_normal((4, 50000)) * np.exp2(rng.integers(-12, 12, (4, 50000)))).astype(np.float32)
    bits = (p.view(np.uint32) >> 16).astype(np.uint16)
    vals = (bits.astype(np.uint32) << 16).view(np.float32)
    want = np.float32(0) + vals[0]
    for r in (1, 2, 3):
        want = (want + vals[r]).astype(np.float32)
    got = O.rank_sum_bf16(*bits)
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
    other = ((vals[3] + vals[2]).astype(np.float32) + vals[1]).astype(np.float32) + vals[0]
    assert np.any(other.astype(np.float32) != got)          # the order is observable in this data
    # a case where a fused or wider sum differs: 1 + 2^-24 + 2^-24 + (-1)
    one, tiny = 0x3f80, 0x3380
    assert O.rank_sum_bf16([one], [tiny], [tiny], [0xbf80])[0] == 0.0


def test_bf16_cast_vectors():
    x = np.array([1.0, 1.00390625, 1.01171875, -0.0, np.inf, -np.inf, np.nan, 3.3895314e38, 1e-40], np.float32)
    got = O.bf16_rne_nan(x)
    # 1 + 2^-8 is a midpoint -> even (0x3f80); 1 + 3*2^-8 a midpoint -> even upwards (0x3f82)
    assert got.tolist() == [0x3f80, 0x3f80, 0x3f82, 0x8000, 0x7f80, 0xff80, 0x7fff, 0x7f7f, 0x0001]
