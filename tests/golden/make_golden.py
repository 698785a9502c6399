#!/usr/bin/env python3
"""Writes tests/golden/b1_host_units.npz: inputs and the outputs of the reference's own B1 host
units (quantize_host, plan_host, reduce_host, m26x_decode_bits) on seeded corpora.

Runs only where oracle/_ref/libb1ref.so was built from the mounted reference tree (make -C oracle);
the fixture it writes is plain data and travels with the repository. ref_mxfp4_golden.json and
ref_e4m3_decode_table.json in this folder are the reference's own golden data files
(oracle/goldens/ there), kept unchanged.
"""
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.join(HERE, "..", "..", "oracle"))
import b1_oracle as O  # noqa: E402


def quant_corpus(rng):
    """Code centres and tie neighbours over every scale, amax transitions, floor neighbours, signed
    zero, FP32 / E4M3 subnormals, extremes, nonfinite values, random exponents."""
    blocks = []
    grid = np.array([O.e4m3_value(c) for c in range(0x7F)], np.float64)
    mids = (grid[:-1] + grid[1:]) / 2
    for k in range(-22, 121):
        for vals in (grid, mids, np.nextafter(mids.astype(np.float32), np.float32(0)), np.nextafter(mids.astype(np.float32), np.float32(1e30))):
            v = np.ldexp(np.asarray(vals, np.float64), k).astype(np.float32)
            v = v[np.isfinite(v)]
            for i in range(0, len(v) - 31, 32):
                b = v[i:i + 32].copy()
                b[0] = np.float32(np.ldexp(448.0, k))  # pins the block scale to k
                b[1::2] *= -1
                blocks.append(b)
    for a in (1e-4, 9.9999e-5, 1.0001e-4, 0.875, 0.8750001, 448.0, 448.00003, 3e-9, 1.17549435e-38, 1e-45, 3.4028235e38, 1.7e38):
        b = np.zeros(32, np.float32)
        b[7] = a
        b[8] = -a / 3
        b[9] = -0.0
        blocks.append(b)
    for bad in (np.nan, np.inf, -np.inf):
        for lane in (0, 13, 31):
            b = rng.standard_normal(32).astype(np.float32)
            b[lane] = bad
            blocks.append(b)
    r = (rng.standard_normal((600, 32)) * np.exp2(rng.integers(-140, 127, (600, 1)).astype(np.float64))).astype(np.float32)
    r[~np.isfinite(r)] = 3.0e38
    blocks.extend(list(r))
    bits = rng.integers(0, 2 ** 32, (300, 32), dtype=np.uint64).astype(np.uint32).view(np.float32)
    blocks.extend(list(bits))
    return np.stack(blocks).astype(np.float32)


def main():
    if O.REF is None:
        sys.exit("oracle/_ref/libb1ref.so is absent: build it where the reference tree is mounted")
    rng = np.random.default_rng(0xB1)
    out = {}
    h = quant_corpus(rng)
    p, s, f, _ = O.ref_quant_v1(h)
    out.update(quant_h=h.view(np.uint32), quant_payload=p, quant_scales=s, quant_faults=f)
    for name, rows, cap, kind in (("a", 1, 256, "uniform"), ("b", 37, 256, "uniform"), ("c", 256, 256, "hot"), ("d", 300, 2048, "sparse")):
        if kind == "uniform":
            ids = np.stack([rng.permutation(256)[:8] for _ in range(rows)])
        elif kind == "hot":
            ids = np.stack([np.concatenate([[3, 250], 4 + rng.permutation(240)[:6]])[rng.permutation(8)] for _ in range(rows)])
        else:
            chosen = np.array([255, 0, 7, 63, 128, 32, 254, 1])
            ids = np.stack([chosen[rng.permutation(8)] for _ in range(rows)])
        ids = ids.astype(np.int32)
        w = rng.random((rows, 8)).astype(np.float32)
        pl = O.ref_plan(cap, ids, w)
        assert pl.status == 0
        ng = int(pl.group_count[0])
        out.update({f"plan_{name}_ids": ids, f"plan_{name}_w": w, f"plan_{name}_cap": np.array([cap]),
                    f"plan_{name}_inverse": pl.inverse[:rows * 8], f"plan_{name}_original": pl.original_routes[:rows * 8],
                    f"plan_{name}_gw": pl.grouped_weights[:rows * 8], f"plan_{name}_groups": pl.groups[:ng].view(np.int32).reshape(ng, 19),
                    f"plan_{name}_count": pl.group_count.copy()})
    y = (rng.standard_normal((2, 8, 4096)) * np.exp2(rng.integers(-20, 20, (2, 8, 1)))).astype(np.float32)
    w = rng.random((2, 8)).astype(np.float32)
    w[0, 0] = 0.0
    st, part, bf = O.ref_reduce(y, w)
    assert st == 0
    cols = np.arange(0, 4096, 13)  # keep the fixture small: every 13th column
    out.update(reduce_y=y[:, :, cols].copy(), reduce_w=w, reduce_partial=part[:, cols].view(np.uint32), reduce_bf16=bf[:, cols])
    out["mxfp4_bits"] = np.array([[O.REF.ref_mxfp4_bits(n, s) for s in range(256)] for n in range(16)], np.uint32)
    path = os.path.join(HERE, "b1_host_units.npz")
    np.savez_compressed(path, **out)
    print("wrote", path, os.path.getsize(path), "bytes;", len(h), "quantizer blocks, faults", np.bincount(f.ravel()))


if __name__ == "__main__":
    main()
