"""Host logic without a GPU: the library loads and exports every symbol include/m26s_b1.h declares,
the host mirror rejects bad extents before reaching the device, the product never touches the
checker, and the workload generator is deterministic and agrees with the checker's wire quantizer."""
import ctypes
import os
import re

import numpy as np
import pytest

import b1_oracle as O
from mimo26f_afd_amd import _lib, b1, build, synth

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_symbols():
    names = set()
    for header in sorted(os.listdir(os.path.join(ROOT, "include"))):
        text = open(os.path.join(ROOT, "include", header)).read()
        text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
        names |= set(re.findall(r"\b(m26s_b1_\w+|m26[cpw]?_\w+)\s*\(", text))
    return sorted(names)


def test_library_exports_every_declared_symbol():
    if not os.path.exists(build.LIB):
        build.build_library()
    if not os.path.exists(build.PROBE_LIB):
        build.build_probe()
    lib, probe = ctypes.CDLL(build.LIB), ctypes.CDLL(build.PROBE_LIB)
    names = declared_symbols()
    assert len(names) >= 36
    for name in names:                      # the measurement aids (m26p_*) live in a library of their own
        home = probe if name.startswith("m26p_") else lib
        assert hasattr(home, name), f"{name} declared in include/*.h but not exported"
        assert name.startswith("m26p_") or not hasattr(probe, name)
    assert not any(hasattr(lib, n) for n in names if n.startswith("m26p_"))
    assert sorted(list(_lib.SIGNATURES) + list(_lib.PROBE_SIGNATURES)) == names  # the Python binding covers the same set


def test_reference_abi_signatures_are_unchanged():
    """The six entry points the reference's Rust side binds (crates/mimo26-spark/src/b1.rs:21-49)."""
    text = open(os.path.join(ROOT, "include", "m26s_b1.h")).read()
    flat = re.sub(r"\s+", " ", text)
    for proto in ("int m26s_b1_layer_new(const uint8_t* canonical_dev, uint64_t canonical_bytes, uint32_t rank, m26s_b1_layer** out, char* err, size_t errlen);",
                  "int m26s_b1_layer_all_normal(const m26s_b1_layer* layer);",
                  "void m26s_b1_layer_free(m26s_b1_layer* layer);",
                  "int m26s_b1_scratch_new(m26s_b1_scratch** out, char* err, size_t errlen);",
                  "void m26s_b1_scratch_free(m26s_b1_scratch* scratch);",
                  "int m26s_b1_ffn(const m26s_b1_layer* layer, m26s_b1_scratch* scratch, const uint8_t* payload, size_t payload_pitch, const uint8_t* scales, size_t scales_pitch, const int32_t* ids, const float* weights, uint32_t rows, uint16_t* bf16_out, float* ms, char* err, size_t errlen);"):
        assert proto in flat, proto


def test_host_mirror_rejects_bad_extents_before_the_device():
    """b1.rs:141-146,165-168,193-195: extent errors are raised on the host side."""
    class Dummy:
        _h = None
    out = np.zeros(16 * 4096, np.uint16)
    with pytest.raises(b1.B1Error, match="extents do not match 16 rows"):
        b1.ffn(Dummy(), Dummy(), np.zeros(15 * 4096, np.uint8), np.zeros(16 * 128, np.uint8), np.zeros(128, np.int32),
               np.zeros(128, np.float32), 16, out)
    with pytest.raises(b1.B1Error, match="extents do not match 0 rows"):
        b1.ffn(Dummy(), Dummy(), np.zeros(0, np.uint8), np.zeros(0, np.uint8), np.zeros(0, np.int32), np.zeros(0, np.float32), 0, out)
    with pytest.raises(b1.B1Error, match="hidden rows do not match"):
        b1.ffn_strided(Dummy(), Dummy(), np.zeros(16 * 4224 - 1, np.uint8), 4224, np.zeros(128, np.int32), np.zeros(128, np.float32), 16, out)
    with pytest.raises(b1.B1Error, match="hidden rows do not match"):
        b1.ffn_strided(Dummy(), Dummy(), np.zeros(16 * 4224, np.uint8), 4100, np.zeros(128, np.int32), np.zeros(128, np.float32), 16, out)


def test_product_never_reaches_the_checker():
    """Nothing under the package, bench-independent, may import or link anything under oracle/."""
    pkg = os.path.join(ROOT, "mimo26f_afd_amd")
    for dirpath, _, files in os.walk(pkg):
        for f in files:
            if f.endswith((".py", ".h", ".hip", ".cpp")):
                text = open(os.path.join(dirpath, f)).read()
                assert "b1_oracle" not in text and "liboracle" not in text and "oracle/" not in text.replace("oracle/lattice", "").replace("oracle/goldens", ""), f


def test_workloads_are_deterministic_and_shaped():
    a, b = synth.make(2), synth.make(2)
    assert np.array_equal(a.ids, b.ids) and np.array_equal(a.payload, b.payload) and np.array_equal(a.weights, b.weights)
    assert a.rows == 128 and a.ranks == 4 and a.intermediate == 2048
    for t in range(128):
        assert len(set(a.ids[t].tolist())) == 8
    for s in range(16):  # tokens of one stream share six experts
        common = set(a.ids[8 * s].tolist())
        for t in range(8 * s, 8 * s + 8):
            common &= set(a.ids[t].tolist())
        assert len(common) >= 6
    assert np.allclose(a.weights.sum(1), 1.0, atol=1e-6) and (a.weights > 0).all()
    assert np.array_equal(synth.expert_image(7, 1, 9), synth.expert_image(7, 1, 9))
    img = synth.expert_image(7, 1, 9)
    for lo, hi in synth.SCALE_REGIONS:
        assert img[lo:hi].min() == 119 and img[lo:hi].max() == 123
    z = synth.make(3, rows=512)
    counts = np.bincount(z.ids.reshape(-1), minlength=256)
    assert counts.max() > 8 * counts[counts > 0].min() and all(len(set(r)) == 8 for r in z.ids.tolist())  # skewed, no repeats
    assert np.abs(z.x).max() == 40.0 and a.algorithmic_bytes() == a.touched().size * 13369344 + 128 * (4224 + 64 + 8192)


def test_generator_wire_quantizer_equals_checker():
    rng = np.random.default_rng(0)
    x = (rng.standard_normal((48, 4096)) * np.exp2(rng.integers(-40, 40, (48, 1)))).astype(np.float32)
    x[0, :32] = 0; x[1, 5] = np.nan; x[2, 7] = -0.0; x[3, :32] = 1e-44; x[4, 3] = 3e38
    for cfg in (1, 3):
        w = synth.make(cfg, rows=64)
        p, s = O.q0_quantize(w.x)
        assert np.array_equal(p, w.payload) and np.array_equal(s, w.scales)
    a, b = synth.q0_quantize(x), O.q0_quantize(x)
    assert np.array_equal(a[0], b[0]) and np.array_equal(a[1], b[1])
