"""Loads the C-ABI library. There is no fallback: without the HIP library every call raises."""
from __future__ import annotations

import ctypes as C
import os

from . import build

_u8p, _f32p, _i32p, _u32p, _u16p = (C.POINTER(t) for t in (C.c_uint8, C.c_float, C.c_int32, C.c_uint32, C.c_uint16))
_vp, _sz, _cp = C.c_void_p, C.c_size_t, C.c_char_p

# name -> (restype, argtypes); every symbol include/m26s_b1.h, include/m26c_glue.h and include/m26w_frame.h declare
SIGNATURES = {
    "m26w_crc32c_update": (C.c_uint32, [C.c_uint32, _vp, _sz]),
    "m26w_crc32c_update_portable": (C.c_uint32, [C.c_uint32, _vp, _sz]),
    "m26w_request_routes_dev": (C.c_int, [_vp, _vp, C.c_uint32, C.c_uint32, _vp, _vp, _vp, _vp]),
    "m26w_stage_rows_dev": (C.c_int, [_vp, _vp, _sz, _vp]),
    "m26c_router_topk": (C.c_int, [_vp, _vp, C.c_int, C.c_int, C.c_int, _vp, _vp, _vp]),
    "m26c_quant_scales": (C.c_int, [_vp, C.c_long, _vp, _vp, _vp]),
    "m26_quantize_hidden_fp8": (C.c_int, [_vp, _vp, _vp, C.c_int64, _vp]),
    "m26c_quantize_hidden": (C.c_int, [_vp, C.c_long, C.c_int, _vp, _sz, _vp, _sz, _vp]),
    "m26c_frame_fill": (C.c_int, [_vp, _vp, _vp, _vp, C.c_int, C.c_int, C.c_int, _vp, _vp, C.c_int, _vp]),
    "m26c_rank_sum_bf16": (C.c_int, [_vp, _vp, _vp, _vp, _vp, C.c_long, _vp]),
    "m26c_add_inplace": (C.c_int, [_vp, _vp, C.c_long, _vp]),
    "m26c_f32_to_bf16": (C.c_int, [_vp, _vp, C.c_long, _vp]),
    "m26s_b1_layer_new": (C.c_int, [_vp, C.c_uint64, C.c_uint32, C.POINTER(_vp), _cp, _sz]),
    "m26s_b1_layer_all_normal": (C.c_int, [_vp]),
    "m26s_b1_layer_free": (None, [_vp]),
    "m26s_b1_scratch_new": (C.c_int, [C.POINTER(_vp), _cp, _sz]),
    "m26s_b1_scratch_free": (None, [_vp]),
    "m26s_b1_ffn": (C.c_int, [_vp, _vp, _vp, _sz, _vp, _sz, _vp, _vp, C.c_uint32, _vp, _vp, _cp, _sz]),
    "m26s_b1_layer_new_full": (C.c_int, [C.POINTER(_vp), C.c_uint64, C.POINTER(_vp), _cp, _sz]),
    "m26s_b1_layer_intermediate": (C.c_uint32, [_vp]),
    "m26s_b1_layer_view": (C.c_int, [_vp, C.POINTER(_vp), C.POINTER(C.c_uint64), C.POINTER(C.c_uint32)]),
    "m26s_b1_scratch_new_on": (C.c_int, [_vp, C.POINTER(_vp), _cp, _sz]),
    "m26s_b1_ffn_dev": (C.c_int, [_vp, _vp, _vp, _sz, _vp, _sz, _vp, _vp, C.c_uint32, _vp, _vp, _vp, _cp, _sz]),
    "m26s_b1_ffn_enqueue": (C.c_int, [_vp, _vp, _vp, _sz, _vp, _sz, _vp, _vp, C.c_uint32, _vp, _vp, _cp, _sz]),
    "m26s_b1_scratch_sync": (C.c_int, [_vp, _cp, _sz]),
    "m26s_b1_ffn_static": (C.c_int, [_vp, _vp, _sz, _vp, _sz, _vp, _vp, C.c_uint32, _vp, _vp, _vp, _cp, _sz]),
    "m26s_b1_plan_dev": (C.c_int, [_vp, _vp, C.c_uint32, C.c_uint32, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _cp, _sz]),
    "m26s_b1_quantize_dev": (C.c_int, [_vp, C.c_uint64, _vp, _vp, _vp, _cp, _sz]),
    "m26s_b1_reduce_dev": (C.c_int, [_vp, _vp, C.c_uint32, _vp, _vp, _vp, _cp, _sz]),
    "m26s_b1_scratch_set_taps": (None, [_vp, C.c_int]),
    "m26s_b1_scratch_set_option": (C.c_int, [_vp, C.c_int, C.c_int]),
    "m26s_b1_scratch_check_guards": (C.c_int, [_vp, _cp, _sz]),
    "m26s_b1_device_memory": (C.c_int, [C.POINTER(_sz), C.POINTER(_sz)]),
    "m26s_b1_scratch_stream": (_vp, [_vp]),
    "m26s_b1_scratch_view": (C.c_int, [_vp, C.c_int, C.POINTER(_vp), C.POINTER(_sz)]),
    "m26s_b1_copy_to_host": (C.c_int, [_vp, _vp, _sz]),
    "m26s_b1_copy_to_device": (C.c_int, [_vp, _vp, _sz]),
    "m26s_b1_device_alloc": (_vp, [_sz]),
    "m26s_b1_device_free": (None, [_vp]),
}

# the measurement library's symbols (include/m26_probe.h)
PROBE_SIGNATURES = {
    "m26p_read_bandwidth": (C.c_int, [C.c_uint64, C.c_int, _vp, C.POINTER(C.c_double), _cp, _sz]),
    "m26p_mfma_rate": (C.c_int, [C.c_int, C.c_int, _vp, C.POINTER(C.c_double), _cp, _sz]),
    "m26p_mfma_sustained": (C.c_int, [C.c_int, C.c_int, _vp] + [C.POINTER(C.c_double)] * 4 + [_cp, _sz]),
}

_LIB = None
_PROBE = None


def _bind(path: str, signatures: dict) -> C.CDLL:
    lib = C.CDLL(path)
    for name, (res, args) in signatures.items():
        fn = getattr(lib, name)  # AttributeError here = a declared symbol is not exported
        fn.restype = res
        fn.argtypes = args
    return lib


def _on_gpu_box() -> bool:
    return os.path.exists("/dev/kfd")


def load() -> C.CDLL:
    """The built serving library. It is built here only if nothing is there, or, on a machine without a
    GPU (where libraries are built, not run), if a source is newer than it: a GPU run loads what it was
    handed and never compiles."""
    global _LIB
    if _LIB is None:
        path = os.environ.get("M26S_B1_LIB") or build.LIB  # a deployment may point at its own build
        if path == build.LIB and (not os.path.exists(path) or (build.stale() and not _on_gpu_box())):
            build.build_library()
        _LIB = _bind(path, SIGNATURES)
    return _LIB


def load_probe() -> C.CDLL:
    """The measurement library (roofline probes), built on the same terms."""
    global _PROBE
    if _PROBE is None:
        if not os.path.exists(build.PROBE_LIB) or (build.probe_stale() and not _on_gpu_box()):
            build.build_probe()
        _PROBE = _bind(build.PROBE_LIB, PROBE_SIGNATURES)
    return _PROBE
