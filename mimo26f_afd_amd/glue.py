"""Host mirror of include/m26c_glue.h: the coordinator-side kernels around the routed-expert FFN
(routing, wire quantizer, request-frame fill, rank sum, residual add), on device pointers.

Names and argument order follow the reference's bindings (crates/mimo26-coordinator/src/dforward.rs:33-101);
a non-zero return raises GlueError like the reference's `ck(...)`.
"""
from __future__ import annotations

from ._lib import load


class GlueError(RuntimeError):
    def __init__(self, code: int, what: str):
        super().__init__(f"{what}: error {code}")
        self.code = code


def _ck(code: int, what: str) -> None:
    if code != 0:
        raise GlueError(code, what)


def router_topk(logits_dev: int, bias_dev: int, rows: int, n_experts: int, top_k: int, idx_dev: int, w_dev: int,
                stream: int | None = None) -> None:
    _ck(load().m26c_router_topk(logits_dev, bias_dev, rows, n_experts, top_k, idx_dev, w_dev, stream), "router top-k")


def quant_scales(x_dev: int, n_blocks: int, scales_dev: int, scale_inv_dev: int, stream: int | None = None) -> None:
    _ck(load().m26c_quant_scales(x_dev, n_blocks, scales_dev, scale_inv_dev, stream), "quant scales")


def quantize_hidden_fp8(x_dev: int, scale_inv_dev: int, payload_dev: int, n_elem: int, stream: int | None = None) -> None:
    _ck(load().m26_quantize_hidden_fp8(x_dev, scale_inv_dev, payload_dev, n_elem, stream), "quant payload")


def quantize_hidden(x_dev: int, rows: int, cols: int, payload_dev: int, payload_pitch: int, scales_dev: int,
                    scales_pitch: int, stream: int | None = None) -> None:
    _ck(load().m26c_quantize_hidden(x_dev, rows, cols, payload_dev, payload_pitch, scales_dev, scales_pitch, stream),
        "quantize hidden")


def frame_fill(idx_dev: int, wts_dev: int, payload_dev: int, scales_dev: int, t: int, topk: int, hid: int,
               routes_dev: int, hidden_dev: int, pitch: int, stream: int | None = None) -> None:
    _ck(load().m26c_frame_fill(idx_dev, wts_dev, payload_dev, scales_dev, t, topk, hid, routes_dev, hidden_dev, pitch,
                               stream), "frame fill")


def rank_sum_bf16(p0_dev: int, p1_dev: int, p2_dev: int, p3_dev: int, out_dev: int, n: int, stream: int | None = None) -> None:
    _ck(load().m26c_rank_sum_bf16(p0_dev, p1_dev, p2_dev, p3_dev, out_dev, n, stream), "rank sum")


def add_inplace(h_dev: int, a_dev: int, n: int, stream: int | None = None) -> None:
    _ck(load().m26c_add_inplace(h_dev, a_dev, n, stream), "residual add")


def f32_to_bf16(x_dev: int, y_dev: int, n: int, stream: int | None = None) -> None:
    _ck(load().m26c_f32_to_bf16(x_dev, y_dev, n, stream), "bf16 cast")
