"""MI355X-native routed-expert FFN (B1, E-W4A8-v1) behind the reference's expert-rank ABI.

`b1` mirrors the reference's Rust wrapper (crates/mimo26-spark/src/b1.rs): Layer, Scratch, ffn,
ffn_strided, FfnStats. `synth` generates the seeded benchmark workloads. The compute lives in
csrc/ (HIP, gfx950) and is reached only through the C ABI declared in include/m26s_b1.h.
"""
from . import build  # noqa: F401

__all__ = ["b1", "synth", "build"]
