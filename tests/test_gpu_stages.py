"""GPU parity of the single stages through the C ABI: bucketing, quantizer v1 and combine are
bit-exact against the CPU checker (which the CPU tests pin to the reference)."""
import os

import numpy as np
import pytest

import b1_oracle as O
from helpers import DeviceLayer
from mimo26f_afd_amd import b1, synth

pytestmark = pytest.mark.gpu
FIX = np.load(os.path.join(os.path.dirname(__file__), "golden", "b1_host_units.npz"))


def gpu_plan(ids, w, cap, resident=None):
    ids = np.ascontiguousarray(ids, np.int32).reshape(-1, 8)
    w = np.ascontiguousarray(w, np.float32).reshape(-1, 8)
    rows, n = ids.shape[0], cap * 8
    resident = np.ones(256, np.uint8) if resident is None else resident
    out = O.Plan(cap)  # same poison as the CPU side, so untouched slots compare equal too
    dev = {k: b1.DeviceBuffer.from_host(v) for k, v in dict(ids=ids if rows else np.zeros(8, np.int32),
           w=w if rows else np.zeros(8, np.float32), res=resident, inv=out.inverse, orig=out.original_routes,
           gw=out.grouped_weights, grp=out.groups, cnt=out.group_count, flt=out.fault).items()}
    b1.plan_dev(dev["ids"].ptr, dev["w"].ptr, rows, cap, dev["res"].ptr, dev["inv"].ptr, dev["orig"].ptr, dev["gw"].ptr,
                dev["grp"].ptr, dev["cnt"].ptr, dev["flt"].ptr)
    out.inverse, out.original_routes = dev["inv"].to_host(np.int32), dev["orig"].to_host(np.int32)
    out.grouped_weights, out.groups = dev["gw"].to_host(np.float32), dev["grp"].to_host(O.GROUP_DTYPE)
    out.group_count, out.fault = dev["cnt"].to_host(np.uint32), dev["flt"].to_host(np.uint32)
    assert len(out.groups) == n
    return out


def same_plan(a, b):
    return all(np.array_equal(getattr(a, k), getattr(b, k)) for k in
               ("inverse", "original_routes", "grouped_weights", "groups", "group_count", "fault"))


@pytest.mark.parametrize("rows,cap,kind", [(0, 256, "uniform"), (1, 256, "uniform"), (16, 256, "uniform"), (129, 256, "hot"),
                                            (256, 256, "sparse"), (2048, 2048, "hot"), (3001, 4096, "uniform"),
                                            (8192, 8192, "hot"), (8192, 8192, "zipf")])
def test_bucketing_bit_exact(rows, cap, kind):
    rng = np.random.default_rng(rows * 7 + len(kind))
    resident = None
    if kind == "uniform":
        ids = np.stack([rng.permutation(256)[:8] for _ in range(max(rows, 1))])[:rows]
    elif kind == "hot":  # two experts in every token: many full 16-row groups, long stable runs
        ids = np.stack([np.concatenate([[3, 250], 4 + rng.permutation(240)[:6]])[rng.permutation(8)] for _ in range(rows)])
    elif kind == "sparse":
        chosen = np.array([255, 0, 7, 63, 128, 32, 254, 1])
        ids = np.stack([chosen[rng.permutation(8)] for _ in range(rows)])
        resident = np.zeros(256, np.uint8)
        resident[chosen] = 1
    else:
        from mimo26f_afd_amd import synth
        ids = synth.routes_zipf(11, rows)
    w = rng.random((rows, 8)).astype(np.float32)
    ref = O.plan(cap, ids.reshape(-1, 8), w, resident)
    got = gpu_plan(ids, w, cap, resident)
    assert ref.status == 0 and same_plan(got, ref)


@pytest.mark.parametrize("name", ["a", "b", "c", "d"])
def test_bucketing_reference_vectors(name):
    """Straight against the outputs of the reference's compiled plan_host."""
    ids, w, cap = FIX[f"plan_{name}_ids"], FIX[f"plan_{name}_w"], int(FIX[f"plan_{name}_cap"][0])
    resident = None
    if name == "d":
        resident = np.zeros(256, np.uint8)
        resident[[255, 0, 7, 63, 128, 32, 254, 1]] = 1
    got = gpu_plan(ids, w, cap, resident)
    n, ng = ids.size, int(FIX[f"plan_{name}_count"][0])
    assert got.fault[0] == 0 and got.group_count[0] == ng
    assert np.array_equal(got.inverse[:n], FIX[f"plan_{name}_inverse"]) and np.array_equal(got.original_routes[:n], FIX[f"plan_{name}_original"])
    assert np.array_equal(got.grouped_weights[:n], FIX[f"plan_{name}_gw"])
    assert np.array_equal(got.groups[:ng].view(np.int32).reshape(ng, 19), FIX[f"plan_{name}_groups"])


def test_bucketing_faults_match_and_write_nothing():
    ids = np.stack([np.arange(8) + 8 * t for t in range(20)]).astype(np.int32)
    w = np.full((20, 8), 0.125, np.float32)
    cases = []
    for bad_id in (256, -1, 1 << 20):
        i = ids.copy(); i[7, 3] = bad_id; cases.append((i, w, None))
    i = ids.copy(); i[5, 6] = i[5, 1]; cases.append((i, w, None))
    res = np.ones(256, np.uint8); res[ids[9, 2]] = 0; cases.append((ids, w, res))
    res = np.ones(256, np.uint8); res[200] = 2; cases.append((ids, w, res))
    for bad_w in (np.nan, np.inf, -0.5):
        ww = w.copy(); ww[11, 4] = bad_w; cases.append((ids, ww, None))
    i = ids.copy(); i[3, 2] = i[3, 1]; ww = w.copy(); ww[3, 2] = np.nan; cases.append((i, ww, None))   # weight before duplicate
    i = ids.copy(); i[3, 2] = i[3, 1]; ww = w.copy(); ww[2, 0] = -1.0; cases.append((i, ww, None))     # earlier route wins
    for i, ww, res in cases:
        ref, got = O.plan(256, i, ww, res), gpu_plan(i, ww, 256, res)
        assert ref.status in (7, 8) and same_plan(got, ref)  # untouched poison everywhere but the fault word


def quantize_gpu(h):
    h = np.ascontiguousarray(h, np.float32)
    dh = b1.DeviceBuffer.from_host(h)
    dp = b1.DeviceBuffer.from_host(np.full(h.size, 0xA5, np.uint8))
    ds = b1.DeviceBuffer.from_host(np.full(h.size // 32, 0xA5, np.uint8))
    df = b1.DeviceBuffer.from_host(np.full(h.size // 32, 0x77, np.uint32))
    b1.quantize_dev(dh.ptr, h.size, dp.ptr, ds.ptr, df.ptr)
    return dp.to_host(np.uint8).reshape(h.shape), ds.to_host(np.uint8), df.to_host(np.uint32)


def test_quantizer_byte_exact_on_reference_corpus():
    """The committed corpus with the reference quantize_host's own bytes and fault words."""
    p, s, f = quantize_gpu(FIX["quant_h"].view(np.float32))
    assert np.array_equal(f, FIX["quant_faults"].ravel())
    assert np.array_equal(p, FIX["quant_payload"]) and np.array_equal(s, FIX["quant_scales"].ravel())


def test_quantizer_byte_exact_on_random_and_raw_bit_patterns():
    rng = np.random.default_rng(4)
    h = (rng.standard_normal((200000, 32)) * np.exp2(rng.integers(-149, 128, (200000, 1)).astype(np.float64))).astype(np.float32)
    bits = rng.integers(0, 2 ** 32, (50000, 32), dtype=np.uint64).astype(np.uint32).view(np.float32)
    h = np.concatenate([h, bits])
    ref = O.quant_v1(h)
    p, s, f = quantize_gpu(h)
    assert np.array_equal(f, ref[2].ravel()) and np.array_equal(p, ref[0]) and np.array_equal(s, ref[1].ravel())
    assert (f == 1).sum() > 100 and (f == 2).sum() > 0 and (f == 0).sum() > 200000
    b1.quantize_dev(None, 0, None, None, None)  # empty batches are valid
    with pytest.raises(b1.B1Error):
        b1.quantize_dev(1, 33, 1, 1, 1)


def reduce_gpu(y, w):
    y = np.ascontiguousarray(y, np.float32); w = np.ascontiguousarray(w, np.float32)
    rows = y.shape[0]
    dy, dw = b1.DeviceBuffer.from_host(y), b1.DeviceBuffer.from_host(w)
    dp, db, df = b1.DeviceBuffer(rows * 4096 * 4), b1.DeviceBuffer(rows * 4096 * 2), b1.DeviceBuffer.from_host(np.full(1, 9, np.uint32))
    b1.reduce_dev(dy.ptr, dw.ptr, rows, dp.ptr, db.ptr, df.ptr)
    return int(df.to_host(np.uint32)[0]), dp.to_host(np.float32).reshape(rows, 4096), db.to_host(np.uint16).reshape(rows, 4096)


def test_combine_bit_exact_and_order_exact():
    rng = np.random.default_rng(12)
    y = (rng.standard_normal((37, 8, 4096)) * np.exp2(rng.integers(-40, 40, (37, 8, 1)))).astype(np.float32)
    w = rng.random((37, 8)).astype(np.float32)
    w[0, 0] = 0.0
    # the reference's closed-form traps (crates/mimo26-expert/tests/b1/route.cpp:69-96) in columns 0..5 of row 1
    y[1] = 0; w[1] = 1
    y[1, :4, 0] = [1e8, 1.0, -1e8, 3.0]
    y[1, 0, 1] = -1.0; y[1, 1, 1] = 1.0 + 2.0 ** -23
    y[1, 0, 3] = 1.0 + 1.0 / 256; y[1, 0, 4] = 1.0 + 3.0 / 256; y[1, 0, 5] = -(1.0 + 1.0 / 256)
    y[2] = 0; w[2] = 0.5; y[2, 0, 0] = 2.0 ** -126
    st, part, bf = O.reduce(y, w)
    flt, gp, gb = reduce_gpu(y, w)
    assert st == 0 and flt == 0 and np.array_equal(gp.view(np.uint32), part.view(np.uint32)) and np.array_equal(gb, bf)
    assert gp[1, 0] == 3.0 and gb[1, 3] == 0x3F80 and gb[1, 4] == 0x3F82 and gb[1, 5] == 0xBF80
    assert gp[2, 0] == np.float32(2.0 ** -127) and gb[2, 0] == 0x0040      # subnormal product not flushed
    w2 = w.copy(); w2[1, 1] = 1.0 - 2.0 ** -23
    assert reduce_gpu(y, w2)[1][1, 1] == 0.0                                # multiply and add stay separate


@pytest.mark.parametrize("what", ["nan_w", "neg_w", "inf_w", "nan_y", "bf16_overflow", "product_overflow", "sum_overflow"])
def test_combine_faults(what):
    y = np.ones((2, 8, 4096), np.float32); w = np.full((2, 8), 0.125, np.float32)
    if what == "nan_w": w[1, 2] = np.nan
    if what == "neg_w": w[0, 0] = -1.0
    if what == "inf_w": w[0, 7] = np.inf
    if what == "nan_y": y[1, 3, 77] = np.nan
    if what == "bf16_overflow": y[:] = 0; w[:] = 1; y[0, 0, 5] = 3.4028235e38
    if what == "product_overflow": y[:] = 0; w[:] = 1; w[0, 0] = 2.0; y[0, 0, 5] = 3.4028235e38
    if what == "sum_overflow": y[:] = 0; w[:] = 1; y[0, :2, 5] = 3.4028235e38
    assert O.reduce(y, w)[0] == 8 and reduce_gpu(y, w)[0] != 0


@pytest.mark.parametrize("ranks", [1, 4])
def test_prepared_pool_is_the_forward_map_of_the_canonical_images(ranks):
    """The one-time weight preparation, two-sided like the reference's own test of its permutation
    (crates/mimo26-expert/tests/b1/host.cpp:30-67): the library walks destination cells, the checker
    maps every canonical byte forward; the prepared images must be identical, for one rank's share and
    for four ranks fused, on arbitrary bytes (scale bytes included: the permutation moves bytes, it
    does not read them)."""
    rng = np.random.default_rng(40 + ranks)
    pools = [np.full(synth.EXPERTS * synth.IMAGE_BYTES, 0x22, np.uint8) for _ in range(ranks)]
    experts = (0, 131, 255)
    for pool in pools:
        for e in experts:
            pool[e * synth.IMAGE_BYTES:(e + 1) * synth.IMAGE_BYTES] = rng.integers(0, 256, synth.IMAGE_BYTES, dtype=np.uint8)
    layer = DeviceLayer(pools).layer
    assert layer.intermediate == 512 * ranks and not layer.all_scales_normal()
    ptr, image_bytes, tag = layer.prepared_view()
    assert image_bytes == ranks * synth.IMAGE_BYTES and tag == 0x47393502
    for e in experts + (7,):
        got = np.empty(image_bytes, np.uint8)
        assert b1.load().m26s_b1_copy_to_host(got.ctypes.data, ptr + e * image_bytes, image_bytes) == 0
        want = O.prepared_g950([p[e * synth.IMAGE_BYTES:(e + 1) * synth.IMAGE_BYTES] for p in pools])
        assert np.array_equal(got, want), e
