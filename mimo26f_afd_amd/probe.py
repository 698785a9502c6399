"""What this GPU sustains on the two rooflines the FFN is priced against (include/m26_probe.h)."""
from __future__ import annotations

import ctypes as C

from ._lib import load_probe


class ProbeError(RuntimeError):
    pass


def _run(name: str, *args) -> float:
    value, buf = C.c_double(0.0), C.create_string_buffer(256)
    rc = getattr(load_probe(), name)(*args, C.byref(value), buf, 256)
    if rc != 0:
        raise ProbeError(f"{name}: rc {rc}: {buf.value.decode('utf-8', 'replace')}")
    return value.value


def read_bandwidth_gbps(nbytes: int = 4 << 30, reps: int = 5, stream: int | None = None) -> float:
    """Best of `reps` streaming reads of `nbytes` of device memory, in GB/s."""
    return _run("m26p_read_bandwidth", nbytes, reps, stream)


def mfma_rate_tflops(iters: int = 2000, reps: int = 3, stream: int | None = None) -> float:
    """Best of `reps` runs of nothing but the GEMMs' block-scaled MFMA, in TFLOP/s."""
    return _run("m26p_mfma_rate", iters, reps, stream)


def mfma_sustained(iters: int = 2000, launches: int = 40, stream: int | None = None) -> dict:
    """`launches` runs of the MFMA-only kernel back to back: rate and shader clock of the first and of the last."""
    v = [C.c_double(0.0) for _ in range(4)]
    buf = C.create_string_buffer(256)
    rc = load_probe().m26p_mfma_sustained(iters, launches, stream, *[C.byref(x) for x in v], buf, 256)
    if rc != 0:
        raise ProbeError(f"m26p_mfma_sustained: rc {rc}: {buf.value.decode('utf-8', 'replace')}")
    return dict(tflops_first=v[0].value, tflops_last=v[1].value, ghz_first=v[2].value, ghz_last=v[3].value)
