"""GPU parity of the coordinator-side kernels (include/m26c_glue.h) against the CPU checker, through
the C ABI. Bars: routing ids exact and weights within one binary32 ulp (the device's binary64 exp may
differ from the host's in the last place); wire quantizer, frame bytes, rank sum, residual add and
BF16 cast bit-exact. The last test chains them into the FFN: rows quantized on the GPU straight into
a request frame and read in place give the same bits as rows quantized by the checker."""
import numpy as np
import pytest

import b1_oracle as O
from helpers import DeviceLayer
from mimo26f_afd_amd import b1, glue, synth

pytestmark = pytest.mark.gpu
D = b1.DeviceBuffer


def dev(a):
    return D.from_host(np.ascontiguousarray(a))


@pytest.mark.parametrize("rows,n,k", [(1, 256, 8), (257, 256, 8), (33, 64, 1), (5, 1024, 6), (9, 96, 64)])
def test_router_topk(rows, n, k):
    rng = np.random.default_rng(rows * 31 + n)
    logits = (rng.standard_normal((rows, n)) * 3).astype(np.float32)
    logits[0, : n // 2] = 0.25                                   # a long run of exact ties in the first row
    bias = (rng.standard_normal(n) * 0.2).astype(np.float32)
    if rows > 1:
        logits[1] = -40.0                                        # tiny scores: the sum stays the selection-order sum
    dl, db, di, dw = dev(logits), dev(bias), D(rows * k * 4), D(rows * k * 4)
    glue.router_topk(dl.ptr, db.ptr, rows, n, k, di.ptr, dw.ptr)
    idx, w = di.to_host(np.int32).reshape(rows, k), dw.to_host(np.float32).reshape(rows, k)
    ref_idx, ref_w = O.router_topk(logits, bias, k)
    assert np.array_equal(idx, ref_idx)
    assert np.max(np.abs(w.astype(np.float64) - ref_w) / np.spacing(ref_w)) <= 1.0
    assert np.mean(w == ref_w) > 0.999


def test_router_rejects_bad_shapes():
    b = D(4096)
    for n, k in ((0, 1), (100, 4), (2048, 8), (256, 0), (256, 65), (64, 65)):
        with pytest.raises(glue.GlueError) as e:
            glue.router_topk(b.ptr, b.ptr, 1, n, k, b.ptr, b.ptr)
        assert e.value.code == 1
    glue.router_topk(b.ptr, b.ptr, 0, 256, 8, b.ptr, b.ptr)      # no rows: nothing to do, as the reference


def wire_cases():
    rng = np.random.default_rng(77)
    x = synth.bf16_round((rng.standard_normal((96, 4096)) * np.exp2(rng.integers(-30, 30, (96, 1)))).astype(np.float32))
    raw = rng.integers(0, 2 ** 32, (64, 4096), dtype=np.uint64).astype(np.uint32).view(np.float32)   # every exponent, NaNs, infs
    edge = np.zeros((8, 4096), np.float32)
    edge[0, :32] = np.ldexp(1.0, -10) * np.arange(32)            # the subnormal band and its ties
    edge[1, :32] = np.linspace(-480, 480, 32)                    # saturation on both sides
    edge[2, 32:64] = [np.inf] + [1.0] * 31
    edge[3, :32] = [np.nan] + [0.5] * 31                         # a NaN neither sets the scale nor survives
    edge[4, :32] = -0.0
    edge[5, :32] = 1e-45                                         # FP32 subnormals
    edge[6, :32] = np.ldexp(np.arange(32, dtype=np.float32) + 0.5, -3)   # exact half-way points
    edge[7, :32] = 3.0e38
    return np.concatenate([x, raw, edge])


def test_wire_quantizer_bit_exact_two_calls_and_fused_in_frame():
    x = wire_cases()
    rows, cols = x.shape
    with np.errstate(all="ignore"):
        ref_p, ref_s = O.q0_quantize(x)
        _, ref_inv = O.q0_scales(x)
    dx, ds, dinv, dp = dev(x), D(rows * 128), D(rows * 128 * 4), D(rows * cols)
    glue.quant_scales(dx.ptr, rows * 128, ds.ptr, dinv.ptr)
    glue.quantize_hidden_fp8(dx.ptr, dinv.ptr, dp.ptr, rows * cols)
    assert np.array_equal(ds.to_host(np.uint8).reshape(rows, 128), ref_s)
    assert np.array_equal(dinv.to_host(np.uint32), ref_inv.view(np.uint32))
    assert np.array_equal(dp.to_host(np.uint8).reshape(rows, cols), ref_p)
    frame = D(rows * 4224 + 64)                                  # request-frame rows: payload then scales, pitch 4224
    glue.quantize_hidden(dx.ptr, rows, cols, frame.ptr, 4224, frame.ptr + 4096, 4224)
    got = frame.to_host(np.uint8)[: rows * 4224].reshape(rows, 4224)
    assert np.array_equal(got[:, :4096], ref_p) and np.array_equal(got[:, 4096:], ref_s)
    n = 4096 * 3 + 32                                            # a ragged tail for the payload-only entry
    glue.quantize_hidden_fp8(dx.ptr, dinv.ptr, dp.ptr, n)
    assert np.array_equal(dp.to_host(np.uint8)[:n], ref_p.reshape(-1)[:n])


def test_frame_fill_bytes():
    rng = np.random.default_rng(3)
    t, topk, hid, pitch = 37, 8, 4096, 4224
    idx = rng.integers(0, 256, (t, topk)).astype(np.int32)
    w = rng.random((t, topk)).astype(np.float32)
    payload = rng.integers(0, 256, (t, hid), dtype=np.uint8)
    scales = rng.integers(0, 256, (t, hid // 32), dtype=np.uint8)
    src = [dev(a) for a in (idx, w, payload, scales)]            # kept alive across the launch
    want = np.zeros((t * topk, 3), np.uint32)
    want[:, 0] = np.repeat(np.arange(t), topk)
    want[:, 1] = idx.reshape(-1)
    want[:, 2] = w.reshape(-1).view(np.uint32)
    for shift in (0, 8):                                         # a frame's hidden rows start on 8-byte boundaries only
        routes, hidden = D(t * topk * 12 + 16), D(t * pitch + 16)
        glue.frame_fill(*[b.ptr for b in src], t, topk, hid, routes.ptr + shift // 2, hidden.ptr + shift, pitch)
        assert np.array_equal(routes.to_host(np.uint8)[shift // 2:shift // 2 + t * topk * 12].view(np.uint32).reshape(-1, 3), want)
        got = hidden.to_host(np.uint8)[shift:shift + t * pitch].reshape(t, pitch)
        assert np.array_equal(got[:, :hid], payload) and np.array_equal(got[:, hid:hid + hid // 32], scales)
    with pytest.raises(glue.GlueError):                          # rows that would start off an 8-byte boundary are refused
        glue.frame_fill(*[b.ptr for b in src], t, topk, hid, routes.ptr, hidden.ptr + 4, pitch)


def test_rank_sum_residual_and_cast_bit_exact():
    rng = np.random.default_rng(11)
    n = 128 * 4096 + 7
    p = (rng.standard_normal((4, n)) * np.exp2(rng.integers(-12, 12, (4, n)))).astype(np.float32)
    bits = (p.view(np.uint32) >> 16).astype(np.uint16)
    out = D(n * 4)
    planes = [dev(b) for b in bits]
    glue.rank_sum_bf16(*[b.ptr for b in planes], out.ptr, n)
    got = out.to_host(np.float32)
    assert np.array_equal(got.view(np.uint32), O.rank_sum_bf16(*bits).view(np.uint32))
    h = rng.standard_normal(n).astype(np.float32)
    dh = dev(h)
    glue.add_inplace(dh.ptr, out.ptr, n)
    assert np.array_equal(dh.to_host(np.float32).view(np.uint32), (h + got).astype(np.float32).view(np.uint32))
    x = np.concatenate([rng.integers(0, 2 ** 32, 200000, dtype=np.uint64).astype(np.uint32).view(np.float32),
                        np.array([1.0, 1.00390625, 1.01171875, -0.0, np.inf, np.nan, 3.3895314e38], np.float32)])
    y, dx = D(x.size * 2), dev(x)
    glue.f32_to_bf16(dx.ptr, y.ptr, x.size)
    assert np.array_equal(y.to_host(np.uint16), O.bf16_rne_nan(x))


def test_elementwise_kernels_on_unaligned_pointers_and_short_arrays():
    """The 16-byte forms need 16-byte aligned pointers; anything else takes the one-value form. Same bits either
    way, for every length from none to a few groups of eight."""
    rng = np.random.default_rng(12)
    for n in (1, 7, 8, 9, 23, 4099):
        for shift in (0, 1, 2):                                  # in elements: 0 keeps the device buffer's alignment
            p = (rng.standard_normal((4, n + shift)) * 8).astype(np.float32)
            bits = (p.view(np.uint32) >> 16).astype(np.uint16)
            planes, out = [dev(b) for b in bits], D((n + shift) * 4)
            glue.rank_sum_bf16(*[b.ptr + 2 * shift for b in planes], out.ptr + 4 * shift, n)
            got = out.to_host(np.float32)[shift:shift + n]
            assert np.array_equal(got.view(np.uint32), O.rank_sum_bf16(*bits[:, shift:]).view(np.uint32)), (n, shift)
            h = rng.standard_normal(n + shift).astype(np.float32)
            dh = dev(h)
            glue.add_inplace(dh.ptr + 4 * shift, out.ptr + 4 * shift, n)
            back = dh.to_host(np.float32)
            assert np.array_equal(back[shift:].view(np.uint32), (h[shift:] + got).astype(np.float32).view(np.uint32)), (n, shift)
            assert np.array_equal(back[:shift], h[:shift])
            y = D((n + shift) * 2)
            glue.f32_to_bf16(dh.ptr + 4 * shift, y.ptr + 2 * shift, n)
            assert np.array_equal(y.to_host(np.uint16)[shift:shift + n], O.bf16_rne_nan(back[shift:])), (n, shift)


def test_wire_quantizer_on_every_exponent_and_code_boundary():
    """The kernels take the scale and the codes off the bit patterns where a block holds only numbers. Every
    binary32 exponent with the mantissas around the scale rule's 0.875 threshold as a block's amax, and every
    E4M3 value, every midpoint between neighbours and the binary32 numbers either side of it under scale 1
    (a 400.0 leads those blocks), both signs: the same bytes as the CPU rule."""
    rng = np.random.default_rng(14)
    fields = np.arange(0, 255, dtype=np.uint32)
    mants = np.concatenate([np.array([0, 1, 0x3fffff, 0x400000, 0x5fffff, 0x600000, 0x600001, 0x7fffff], np.uint32),
                            rng.integers(0, 1 << 23, 24).astype(np.uint32)])
    amax = ((fields[:, None] << 23) | mants[None, :]).reshape(-1).astype(np.uint32).view(np.float32)
    a = (rng.standard_normal((amax.size, 32)).astype(np.float32) * amax[:, None]).astype(np.float32)
    a[np.abs(a) > amax[:, None]] = 0
    a[:, 5] = amax
    a[::2, 5] *= -1
    codes = np.arange(0, 0x7f, dtype=np.uint32)
    value = np.where(codes < 8, codes * 2.0 ** -9, (1 + (codes & 7) / 8) * 2.0 ** ((codes >> 3).astype(np.int64) - 7)).astype(np.float32)
    mid = ((value[:-1].astype(np.float64) + value[1:]) / 2).astype(np.float32)
    cand = np.concatenate([value, mid, np.nextafter(mid, np.float32(0)), np.nextafter(mid, np.float32(1e9)),
                           rng.uniform(0, 448, 4000).astype(np.float32), np.exp2(rng.uniform(-12, 8.8, 4000)).astype(np.float32)])
    cand = np.resize(cand, (cand.size + 30) // 31 * 31).reshape(-1, 31) * np.where(rng.random(((cand.size + 30) // 31, 31)) < 0.5, -1, 1)
    b = np.concatenate([np.full((cand.shape[0], 1), 400.0, np.float32), cand.astype(np.float32)], axis=1)
    x = np.concatenate([a.reshape(-1), b.reshape(-1)])
    x = np.resize(x, (x.size + 4095) // 4096 * 4096).reshape(-1, 4096).astype(np.float32)
    with np.errstate(all="ignore"):
        ref_p, ref_s = O.q0_quantize(x)
        _, ref_inv = O.q0_scales(x)
    rows = x.shape[0]
    dx, frame, ds, dinv, dp = dev(x), D(rows * 4224 + 64), D(rows * 128), D(rows * 512), D(rows * 4096)
    glue.quantize_hidden(dx.ptr, rows, 4096, frame.ptr, 4224, frame.ptr + 4096, 4224)
    got = frame.to_host(np.uint8)[: rows * 4224].reshape(rows, 4224)
    assert np.array_equal(got[:, 4096:], ref_s) and np.array_equal(got[:, :4096], ref_p)
    glue.quant_scales(dx.ptr, rows * 128, ds.ptr, dinv.ptr)
    glue.quantize_hidden_fp8(dx.ptr, dinv.ptr, dp.ptr, rows * 4096)
    assert np.array_equal(ds.to_host(np.uint8).reshape(rows, 128), ref_s)
    assert np.array_equal(dinv.to_host(np.uint32), ref_inv.view(np.uint32))
    assert np.array_equal(dp.to_host(np.uint8).reshape(rows, 4096), ref_p)


def test_wire_quantizer_row_shapes():
    """Rows shorter than a workgroup's 1024 values, rows that are not a multiple of it, and pitched outputs: the
    same bytes as the CPU rule row by row."""
    rng = np.random.default_rng(13)
    for rows, cols, ppitch, spitch in ((5, 32, 32, 1), (3, 96, 96, 3), (7, 1056, 1056, 33), (4, 1056, 1088, 40), (9, 4096, 4224, 4224),
                                       (1, 4096, 4096, 128), (6, 64, 80, 2)):
        x = synth.bf16_round((rng.standard_normal((rows, cols)) * np.exp2(rng.integers(-20, 20, (rows, 1)))).astype(np.float32))
        ref_p, ref_s = O.q0_quantize(x)
        in_frame = spitch == ppitch and ppitch > cols           # scales behind the payload of the same row
        dp = D(rows * ppitch + 64)
        dsc = dp if in_frame else D(rows * spitch + 64)
        glue.quantize_hidden(dev(x).ptr, rows, cols, dp.ptr, ppitch, dsc.ptr + (cols if in_frame else 0), spitch)
        got_p = dp.to_host(np.uint8)[: rows * ppitch].reshape(rows, ppitch)[:, :cols]
        raw_s = dsc.to_host(np.uint8)
        got_s = (raw_s[cols: cols + rows * spitch] if in_frame else raw_s[: rows * spitch])
        got_s = np.lib.stride_tricks.as_strided(got_s, (rows, cols // 32), (spitch, 1))
        assert np.array_equal(got_p, ref_p) and np.array_equal(got_s, ref_s), (rows, cols, ppitch, spitch)


def test_chain_router_quantizer_frame_ffn():
    """FP32 logits and bf16-valued hidden rows in; the GPU routes, quantizes into a request frame and the
    FFN reads the frame rows in place: the same BF16 bits as the FFN fed with the checker's bytes."""
    wl = synth.make(1, rows=48)
    rng = np.random.default_rng(21)
    logits = (rng.standard_normal((wl.rows, 256)) * 2).astype(np.float32)
    bias = (rng.standard_normal(256) * 0.1).astype(np.float32)
    ref_idx, ref_w = O.router_topk(logits, bias, 8)
    ref_p, ref_s = O.q0_quantize(wl.x)
    pools = synth.Workload("chain", 1, wl.seed, 1, wl.rows, ref_idx, ref_w, wl.x, ref_p, ref_s).pools(np.unique(ref_idx))
    layer = DeviceLayer(pools).layer
    scratch = b1.Scratch()
    di, dw, dl, db = D(wl.rows * 32), D(wl.rows * 32), dev(logits), dev(bias)
    glue.router_topk(dl.ptr, db.ptr, wl.rows, 256, 8, di.ptr, dw.ptr)
    assert np.array_equal(di.to_host(np.int32).reshape(-1, 8), ref_idx)
    frame, dx = D(wl.rows * 4224), dev(wl.x)
    glue.quantize_hidden(dx.ptr, wl.rows, 4096, frame.ptr, 4224, frame.ptr + 4096, 4224)
    out = D(wl.rows * 4096 * 2)
    b1.ffn_dev(layer, scratch, frame.ptr, 4224, frame.ptr + 4096, 4224, di.ptr, dw.ptr, wl.rows, out.ptr)
    got = out.to_host(np.uint16).reshape(wl.rows, 4096)
    gw = dw.to_host(np.float32).reshape(-1, 8)
    rc, _, ref_bf16, _ = O.layer_ffn(pools, ref_p, ref_s, ref_idx, gw)
    assert rc == 0
    a = (got.astype(np.uint32) << 16).view(np.float32).astype(np.float64)
    r = (ref_bf16.astype(np.uint32) << 16).view(np.float32).astype(np.float64)
    assert np.max(np.abs(a - r)) <= 1e-2 * np.max(np.abs(r)) and np.sum(np.abs(a - r)) <= 1e-3 * np.sum(np.abs(r))
    out2, dp, ds = D(wl.rows * 4096 * 2), dev(ref_p), dev(ref_s)  # the same call on the checker's bytes, separate arrays
    b1.ffn_dev(layer, scratch, dp.ptr, 4096, ds.ptr, 128, di.ptr, dw.ptr, wl.rows, out2.ptr)
    assert np.array_equal(out2.to_host(np.uint16).reshape(wl.rows, 4096), got)


def test_roofline_probes_report_plausible_rates():
    """The two measurement aids: a streaming read lands between a third of the HBM peak and the peak,
    the MFMA-only loop between a third of the FP8 peak and a little past it (the nominal 5.0 PFLOP/s is quoted
    at a lower clock than an idle part boosts to: 4.4 to 5.0 have been measured); bad arguments are refused."""
    from mimo26f_afd_amd import probe
    gbs = probe.read_bandwidth_gbps(1 << 30, 3)
    assert 2600 < gbs < 8000, gbs
    tf = probe.mfma_rate_tflops(500, 2)
    assert 1600 < tf < 5000 * 1.1, tf
    with pytest.raises(probe.ProbeError):
        probe.read_bandwidth_gbps(12345, 1)
    with pytest.raises(probe.ProbeError):
        probe.mfma_rate_tflops(0, 1)
    held = probe.mfma_sustained(500, 4)  # the same loop four times back to back, with the clock it ran at
    assert 1600 < held["tflops_first"] < 5500 and 1600 < held["tflops_last"] < 5500, held
    assert 1.0 < held["ghz_first"] < 2.6 and 1.0 < held["ghz_last"] < 2.6, held  # 2.4 GHz is the part's ceiling
    # the matrix pipe's rate follows the clock: 2 x 16 x 16 x 128 flops per MFMA, 32 cycles each, 1024 SIMDs
    assert 0.85 < held["tflops_last"] / (held["ghz_last"] * 1e9 * 1024 * 65536 / 32 / 1e12) <= 1.02, held
    with pytest.raises(probe.ProbeError):
        probe.mfma_sustained(500, 1)
