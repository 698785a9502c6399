#!/usr/bin/env python3
"""Benchmark of the routed-expert FFN (B1, E-W4A8-v1) on one MI355X.

One step = one pass of the hot path (plan -> FC1 + SwiGLU + requant -> FC2 -> combine) over one
batch of synthetic, device-resident input. Prints ONE JSON line: routed tokens/s per MoE layer for
the 128-token decode/verify layer (256 experts, H 4096, I 2048, top-8), its HBM roofline, the CPU
restatement of the reference timed on the host's cores, and, unless --no-prefill, the same
measurement for the 8192-token prefill chunk against the MFMA peak.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.join(ROOT, "oracle"))

HBM_PEAK_GBS = 8000.0           # MI355X HBM3E, published
MFMA_FP8_PEAK_TFLOPS = 5000.0   # dense FP8 (an FP8 x FP4 block-scaled MFMA issues at the FP8 rate)
NOMINAL_GHZ = 2.4               # the engine clock the published peaks are quoted at
# HBM bytes per launch of the dominant kernels come from the committed counter profile (two rocprofv3 --pmc
# runs of this file, FETCH_SIZE and WRITE_SIZE, each scaled by what the same counter reads for --copy-probe's
# 1 GiB copy): its `traffic_bytes <kernel> <bytes>` rows are read at run time, so the figure printed is the
# one the profile holds, or null when the profile is not there.
TRAFFIC_PROFILE = os.path.join("profiles", "hbm_traffic_decode128_prefill8192.md")
PREFILL_WARMUP, PREFILL_SAMPLES = 10, 31   # the reference's timing protocol (tests/b1_core/bench_connected.cuh:73-81)
PARITY_TOKENS = 64                          # rows checked against the CPU rule on both sides of every timed region
RANK_LAYER_BYTES = 855_638_016              # 256 quarter-slice images: the gate's unique weight and scale bytes
# The reference's gate (crates/mimo26-expert/src/bench.rs:41-48): at least 70 % of the memory peak at M <= 8, STOP below 60 %.
GATE_TARGET, GATE_STOP = 0.70, 0.60


def log(*a):
    print(*a, file=sys.stderr, flush=True)


def profiled_traffic(kernel: str):
    """(HBM bytes per launch of `kernel` from the committed counter profile or None, where it was looked for)."""
    path = os.path.join(ROOT, TRAFFIC_PROFILE)
    try:
        with open(path) as f:
            for line in f:
                tok = line.split()
                if len(tok) == 3 and tok[0] == "traffic_bytes" and tok[1] == kernel:
                    return int(tok[2]), TRAFFIC_PROFILE
    except OSError:
        pass
    return None, TRAFFIC_PROFILE


def spread(samples):
    a = np.asarray(samples, np.float64)
    return dict(median=float(np.median(a)), min=float(a.min()), max=float(a.max()), samples=int(a.size))


def stage(wl, torch, dev):
    """Workload arrays as device tensors."""
    return dict(payload=torch.from_numpy(wl.payload).to(dev), scales=torch.from_numpy(wl.scales).to(dev),
                ids=torch.from_numpy(wl.ids).to(dev), weights=torch.from_numpy(wl.weights).to(dev),
                out=torch.empty((wl.rows, 4096), dtype=torch.int16, device=dev))


def build_layer(wl, torch, dev, b1):
    """Generate the canonical rank pools, upload them, prepare the layer, drop the canonical copies."""
    t0 = time.time()
    pools = wl.pools()
    log(f"[bench] generated {len(pools)} rank pools in {time.time() - t0:.1f}s")
    devs = [torch.from_numpy(p).to(dev) for p in pools]
    torch.cuda.synchronize()
    if len(devs) == 1:
        layer = b1.Layer(devs[0].data_ptr(), devs[0].numel(), 0)
    else:
        layer = b1.Layer.full([d.data_ptr() for d in devs], devs[0].numel())
    del devs
    torch.cuda.empty_cache()
    return layer, pools


def timed_steps(layer, scratch, d, rows, steps, warmup, torch, b1):
    """W untimed steps, then exactly K steps bracketed by synchronisation; returns ms per step."""
    def one():
        b1.ffn_enqueue(layer, scratch, d["payload"].data_ptr(), 4096, d["scales"].data_ptr(), 128, d["ids"].data_ptr(),
                       d["weights"].data_ptr(), rows, d["out"].data_ptr(), None)
    for _ in range(warmup):
        one()
    scratch.sync()
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    e0.record()
    for _ in range(steps):
        one()
    e1.record()
    scratch.sync()
    torch.cuda.synchronize()
    wall_ms = (time.perf_counter() - t0) * 1e3
    return wall_ms / steps, e0.elapsed_time(e1) / steps


def sampled_steps(layer, scratch, d, rows, samples, warmup, torch, b1):
    """`samples` single steps, each between its own pair of events on the launch stream: per-step ms."""
    def one():
        b1.ffn_enqueue(layer, scratch, d["payload"].data_ptr(), 4096, d["scales"].data_ptr(), 128, d["ids"].data_ptr(),
                       d["weights"].data_ptr(), rows, d["out"].data_ptr(), None)
    for _ in range(warmup):
        one()
    scratch.sync()
    pairs = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(samples)]
    for a, b in pairs:
        a.record()
        one()
        b.record()
    scratch.sync()
    torch.cuda.synchronize()
    return [a.elapsed_time(b) for a, b in pairs]


def kernel_phases(layer, scratch, d, rows, reps, b1):
    """Per-kernel durations from the HIP events the library records on its launch stream: the average over
    `reps` calls (what the roofline figures divide by) and the median / min / max of each."""
    rows_ = []
    for _ in range(reps):
        s = b1.ffn_dev(layer, scratch, d["payload"].data_ptr(), 4096, d["scales"].data_ptr(), 128, d["ids"].data_ptr(),
                       d["weights"].data_ptr(), rows, d["out"].data_ptr(), None)
        rows_.append([s.upload_plan_ms, s.phase_ms[0], s.phase_ms[2], s.phase_ms[3], s.gpu_ms])
    a = np.array(rows_)
    acc = a.mean(axis=0)
    return dict(plan_ms=acc[0], fc1_ms=acc[1], fc2_ms=acc[2], reduce_ms=acc[3], gpu_ms=acc[4], reps=reps,
                fc1=spread(a[:, 1]), fc2=spread(a[:, 2]), reduce=spread(a[:, 3]), plan=spread(a[:, 0]))


def bars(got_bits, ref_bits):
    """max-abs / max|ref| and mean relative error of BF16 rows against the CPU checker's BF16 rows."""
    got = (got_bits.astype(np.uint32) << 16).view(np.float32).astype(np.float64)
    ref = (ref_bits.astype(np.uint32) << 16).view(np.float32).astype(np.float64)
    return dict(max_abs_over_max_ref=float(np.max(np.abs(got - ref)) / np.max(np.abs(ref))),
                mean_rel=float(np.sum(np.abs(got - ref)) / np.sum(np.abs(ref))),
                bf16_identical_fraction=float(np.mean(got_bits == ref_bits)))


def sample_parity(wl, pools, before_bits, after_bits, tokens, O):
    """GPU BF16 rows against the CPU checker's BF16 rows on `tokens` (like with like: both sides carry the one
    BF16 rounding of the rank sum), for the output taken before the timed region and the one taken after it
    (the reference's gate validates on both sides of its timing, tests/b1_core/bench_connected.cuh:56-63,85)."""
    ref_rc, _, ref_bits, _ = O.layer_ffn(pools, wl.payload[tokens], wl.scales[tokens], wl.ids[tokens], wl.weights[tokens])
    out = dict(tokens=len(tokens), oracle_rc=ref_rc, **bars(after_bits[tokens], ref_bits))
    out["before_timing"] = bars(before_bits[tokens], ref_bits)
    out["within_bars_before_and_after"] = bool(ref_rc == 0 and all(b["max_abs_over_max_ref"] <= 1e-2 and b["mean_rel"] <= 1e-3
                                                                   for b in (out, out["before_timing"])))
    return out


def cpu_baseline(wl, pools, tokens, O):
    """The CPU restatement of the reference's expert path on bounded samples of the same workload: the W4A8
    lattice (the parity rule: FP64 dots, FP32 boundaries, requantised intermediate) on all host threads,
    which is `value`, the same on one thread, and the reference's E-FP32 twin (FP32 per-MAC accumulation, no
    intermediate requantisation; crates/mimo26-expert/src/grouped.rs:291-336) on all threads and on one."""
    threads = O.hardware_threads()
    few = tokens[:max(1, len(tokens) // 8)]

    def timed(sample, n_threads, efp32):
        t0 = time.perf_counter()
        rc = O.layer_ffn(pools, wl.payload[sample], wl.scales[sample], wl.ids[sample], wl.weights[sample],
                         threads=n_threads, efp32=efp32)[0]
        dt = time.perf_counter() - t0
        return dict(value=len(sample) / dt, unit="routed tok/s per MoE layer", cores=n_threads,
                    sample=f"{len(sample)} tokens ({len(sample) * 8} routes, {np.unique(wl.ids[sample]).size} experts) of the same workload, "
                           f"{dt:.1f}s, rc={rc}")
    full = timed(tokens, threads, False)
    out = dict(value=full["value"], unit=full["unit"], cores=threads, kind="port",
               sample="W4A8 lattice (FP64 dots, FP32 boundaries, requantised intermediate): " + full["sample"])
    out["single_thread"] = timed(few, 1, False)
    out["efp32"] = dict(all_threads=timed(tokens, threads, True), single_thread=timed(few, 1, True),
                        rule="E-FP32 twin: FP32 activations and per-MAC FP32 accumulation in k order, no intermediate requantisation")
    return out


def run_config(cfg, steps, warmup, torch, dev, b1, synth, O, parity_tokens, cpu_tokens, samples=0, variants=()):
    """Correctness before and after the timing, as the reference's bench gate does. `samples` > 0 adds the
    per-step event protocol (that many single steps after `warmup` warm-ups: median / min / max). `variants`:
    scratch options whose step is sampled beside the default (never the headline)."""
    wl = synth.make(cfg)
    log(f"[bench] config {cfg}: {wl.name}")
    layer, pools = build_layer(wl, torch, dev, b1)
    scratch = b1.Scratch(stream=torch.cuda.current_stream().cuda_stream)
    d = stage(wl, torch, dev)
    ph = kernel_phases(layer, scratch, d, wl.rows, 3, b1)  # also the first correctness pass
    before = d["out"].cpu().numpy().view(np.uint16).copy()
    wall_ms, ev_ms = timed_steps(layer, scratch, d, wl.rows, steps, warmup, torch, b1)
    per_step = spread(sampled_steps(layer, scratch, d, wl.rows, samples, warmup, torch, b1)) if samples else None
    ph = kernel_phases(layer, scratch, d, wl.rows, PREFILL_SAMPLES, b1)
    ticks = scratch.view("clock", np.uint64, 4)  # the tile launches of the last call: shader-clock and 100 MHz ticks, FC1 then FC2
    ph["clock_ghz"] = [float(ticks[i]) / float(ticks[i + 1]) * 0.1 if ticks[i + 1] else None for i in (0, 2)]
    after = d["out"].cpu().numpy().view(np.uint16)
    tokens = np.linspace(0, wl.rows - 1, min(parity_tokens, wl.rows)).astype(np.int64)  # spread over the batch
    par = sample_parity(wl, pools, before, after, tokens, O)
    par["bitwise_stable_across_timing"] = bool(np.array_equal(before, after))
    cpu = cpu_baseline(wl, pools, np.arange(min(cpu_tokens, wl.rows)), O) if cpu_tokens else None
    touched = int(wl.touched().size)
    res = dict(wl=wl, ms_per_step=wall_ms, event_ms_per_step=ev_ms, per_step=per_step, phases=ph, parity=par, cpu=cpu, touched=touched)
    res["variants"] = {}
    for name in variants:  # same layer, same inputs, a scratch of its own with the option on
        alt = b1.Scratch(stream=torch.cuda.current_stream().cuda_stream)
        alt.set_option(name, True)
        steps_ms = spread(sampled_steps(layer, alt, d, wl.rows, max(samples, PREFILL_SAMPLES), warmup, torch, b1))
        alt_ph = kernel_phases(layer, alt, d, wl.rows, 11, b1)
        got = d["out"].cpu().numpy().view(np.uint16)
        ref_rc, _, ref_bits, _ = O.layer_ffn(pools, wl.payload[tokens], wl.scales[tokens], wl.ids[tokens], wl.weights[tokens])
        res["variants"][name] = dict(ms_per_step=steps_ms["median"], ms_per_step_spread=steps_ms, fc2_ms=alt_ph["fc2"]["median"],
                                     reduce_ms=alt_ph["reduce"]["median"], same_bits_as_default=bool(np.array_equal(got, after)),
                                     parity_against_the_default_cpu_rule=dict(tokens=len(tokens), oracle_rc=ref_rc, **bars(got[tokens], ref_bits)))
        alt.close()
    del layer, scratch
    return res


def gate_workload(m, synth):
    """The routing of the reference's bandwidth gate (tests/b1_core/bench_connected.cuh:7-12,47-50): 32 * m tokens,
    every run of m tokens shares eight experts, the 32 runs cover all 256 experts exactly once, so every expert gets
    m rows; weights (slot + 1) / 36. Activations: seeded N(0,1) rows through the wire quantizer (the reference
    replays eight captured rows, which this image does not hold)."""
    rows = 32 * m
    perm = np.argsort(synth.uniform(synth.stream_key(synth.BASE_SEED + 60, synth.ROUTES), 256), kind="stable").astype(np.int32)
    ids = perm.reshape(32, 8)[np.arange(rows) // m]
    w = np.tile(np.arange(1, 9, dtype=np.float32) / 36, (rows, 1))
    x = synth._activations(synth.BASE_SEED + 60, rows)
    payload, scales = synth.q0_quantize(x)
    return synth.Workload(f"gate M={m}", 1, synth.BASE_SEED + 1, 1, rows, ids, w, x, payload, scales)


def run_rank_share(torch, dev, b1, synth, O):
    """One TP4 rank's share (I = 512, the reference's deployment shape): configs[0] and configs[1] timed, and the
    reference's own gate: 256 experts of one rank, M = 1..8 rows per expert, 10 warm-ups, 31 event samples,
    median; the gate's timed scope is FC1 + SwiGLU + quantizer + FC2 (plan and combine outside it, reported
    beside), its metric the rank layer's 855,638,016 unique weight and scale bytes over that time."""
    out = {"shape": "256 experts x one TP4 rank's share (I 512), H 4096, top-8", "peak_GBps": HBM_PEAK_GBS}
    wl1 = synth.make(1)
    layer, pools = build_layer(synth.Workload("rank layer", 1, wl1.seed, 1, 0, wl1.ids, wl1.weights, wl1.x, wl1.payload, wl1.scales), torch, dev, b1)
    scratch = b1.Scratch(stream=torch.cuda.current_stream().cuda_stream)

    def timed(wl, parity_rows):
        d = stage(wl, torch, dev)
        kernel_phases(layer, scratch, d, wl.rows, 2, b1)
        before = d["out"].cpu().numpy().view(np.uint16).copy()
        steps = spread(sampled_steps(layer, scratch, d, wl.rows, PREFILL_SAMPLES, PREFILL_WARMUP, torch, b1))
        ph = kernel_phases(layer, scratch, d, wl.rows, PREFILL_SAMPLES, b1)
        after = d["out"].cpu().numpy().view(np.uint16)
        tokens = np.linspace(0, wl.rows - 1, min(parity_rows, wl.rows)).astype(np.int64)
        par = sample_parity(wl, pools, before, after, tokens, O)
        par["bitwise_stable_across_timing"] = bool(np.array_equal(before, after))
        return steps, ph, par

    for cfg in (0, 1):
        wl = synth.make(cfg)
        steps, ph, par = timed(wl, wl.rows)  # every row
        nbytes = wl.algorithmic_bytes()
        gbs = nbytes / (steps["median"] * 1e-3) / 1e9
        out[f"configs[{cfg}]"] = {"workload": wl.name, "experts_touched": int(wl.touched().size), "algorithmic_bytes": nbytes,
                                  "ms_per_step": steps["median"], "ms_per_step_spread": steps, "GBps": gbs, "frac_of_hbm_peak": gbs / HBM_PEAK_GBS,
                                  "tok_per_s": wl.rows / (steps["median"] * 1e-3), "flops": wl.flops(),
                                  "plan_ms": ph["plan"]["median"], "fc1_ms": ph["fc1"]["median"], "fc2_ms": ph["fc2"]["median"],
                                  "reduce_ms": ph["reduce"]["median"], "parity": par}
    gate = []
    scratch.set_option("scope_timing", True)  # FC1 + SwiGLU + quantizer + FC2 between two events, none between the stages
    for m in range(1, 9):
        wl = gate_workload(m, synth)
        steps, ph, par = timed(wl, wl.rows if m in (1, 8) else 32)  # every row at both ends of the sweep, 32 rows between
        scope_ms = ph["fc1"]["median"]
        gbs = RANK_LAYER_BYTES / (scope_ms * 1e-3) / 1e9
        frac = gbs / HBM_PEAK_GBS
        gate.append({"M": m, "rows": wl.rows, "timed_scope_ms": scope_ms, "timed_scope_ms_spread": ph["fc1"],
                     "plan_ms": ph["plan"]["median"], "reduce_ms": ph["reduce"]["median"], "whole_step_ms": steps["median"],
                     "effective_unique_weight_GBps": gbs, "frac_of_hbm_peak": frac,
                     "whole_step_GBps": (RANK_LAYER_BYTES + wl.rows * (4224 + 64 + 8192)) / (steps["median"] * 1e-3) / 1e9,
                     "verdict": "TARGET" if frac >= GATE_TARGET else "STOP" if frac < GATE_STOP else "PIVOT", "parity": par})
    out["gate"] = {"protocol": "reference gate, crates/mimo26-expert/tests/b1_core/bench_connected.cuh:21-88: all 256 experts of one rank, M rows "
                               "per expert, 10 warm-ups, 31 event samples, median; timed scope FC1 + SwiGLU + quantizer + FC2 (per-kernel events of "
                               "the library, each carrying about 3 us of event), plan and combine beside it; metric 855,638,016 B / scope time; "
                               "thresholds of crates/mimo26-expert/src/bench.rs:41-48 against 8 TB/s",
                   "unique_weight_scale_bytes": RANK_LAYER_BYTES, "target_frac": GATE_TARGET, "stop_frac": GATE_STOP, "rows": gate,
                   "reference_published_GB10_GBps": {"first_connected_run_M1..8": [160.65, 160.05, 158.56, 157.13, 155.23, 153.68, 152.50, 152.78],
                                                     "after_tuning_M<=8": 184.0, "GB10_peak": 273.0}}
    scratch.close()
    del layer
    torch.cuda.empty_cache()
    return out


def run_coordinator_kernels(torch, dev):
    """The kernels either side of the path (routing, wire quantizer, frame fill, rank sum, residual add, BF16 cast)
    at the prefill chunk's and the decode batch's row counts: ten launches between two events on torch's stream,
    median of 15 such pairs, the algorithmic bytes of one launch over that time. Each is a pass over a few bytes
    per value, so HBM is the bound; up to about 250 MB a working set also lives in the last-level cache between
    the repeats, and a launch costs about 4 us whatever it moves."""
    from mimo26f_afd_amd import glue
    st = torch.cuda.current_stream().cuda_stream
    H, E, K, PITCH, REPEAT, PAIRS = 4096, 256, 8, 4224, 10, 15

    def timed(fn):
        for _ in range(3):
            fn()
        torch.cuda.synchronize()
        ev = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(PAIRS)]
        for a, b in ev:
            a.record()
            for _ in range(REPEAT):
                fn()
            b.record()
        torch.cuda.synchronize()
        return float(np.median([a.elapsed_time(b) for a, b in ev])) / REPEAT

    out = {"peak_GBps": HBM_PEAK_GBS, "protocol": f"{REPEAT} launches per event pair, median of {PAIRS} pairs; bytes = what one launch must read and write",
           "rows": {}}
    for T in (8192, 128):
        g = torch.Generator(device="cpu").manual_seed(0x26AFD + T)
        x = torch.randn(T, H, generator=g).to(dev)
        a = torch.randn(T, H, generator=g).to(dev)
        logits = torch.randn(T, E, generator=g).to(dev)
        bias = torch.zeros(E, device=dev)
        idx = torch.empty(T, K, dtype=torch.int32, device=dev)
        w = torch.empty(T, K, device=dev)
        frame = torch.empty(T * PITCH + 4096, dtype=torch.uint8, device=dev)
        payload = torch.empty(T, H, dtype=torch.uint8, device=dev)
        scales = torch.empty(T, H // 32, dtype=torch.uint8, device=dev)
        sinv = torch.empty(T * H // 32, device=dev)
        routes = torch.empty(T * K * 12, dtype=torch.uint8, device=dev)
        part = [torch.randn(T, H, generator=g).to(dev).to(torch.bfloat16) for _ in range(4)]
        acc = torch.empty(T, H, device=dev)
        y16 = torch.empty(T, H, dtype=torch.int16, device=dev)
        n = T * H
        glue.router_topk(logits.data_ptr(), bias.data_ptr(), T, E, K, idx.data_ptr(), w.data_ptr(), st)
        glue.quant_scales(x.data_ptr(), n // 32, scales.data_ptr(), sinv.data_ptr(), st)
        cases = {
            "m26c_router_topk": (lambda: glue.router_topk(logits.data_ptr(), bias.data_ptr(), T, E, K, idx.data_ptr(), w.data_ptr(), st),
                                 T * E * 4 + T * K * 8),
            "m26c_quantize_hidden (into frame rows)": (lambda: glue.quantize_hidden(x.data_ptr(), T, H, frame.data_ptr(), PITCH, frame.data_ptr() + H, PITCH, st),
                                                       n * 4 + T * (H + H // 32)),
            "m26c_quant_scales": (lambda: glue.quant_scales(x.data_ptr(), n // 32, scales.data_ptr(), sinv.data_ptr(), st), n * 4 + n // 32 * 5),
            "m26_quantize_hidden_fp8": (lambda: glue.quantize_hidden_fp8(x.data_ptr(), sinv.data_ptr(), payload.data_ptr(), n, st), n * 4 + n // 32 * 4 + n),
            "m26c_frame_fill": (lambda: glue.frame_fill(idx.data_ptr(), w.data_ptr(), payload.data_ptr(), scales.data_ptr(), T, K, H, routes.data_ptr(),
                                                        frame.data_ptr(), PITCH, st), 2 * T * (H + H // 32) + T * K * (8 + 12)),
            "m26c_rank_sum_bf16": (lambda: glue.rank_sum_bf16(*[q.data_ptr() for q in part], acc.data_ptr(), n, st), n * 8 + n * 4),
            "m26c_add_inplace": (lambda: glue.add_inplace(acc.data_ptr(), a.data_ptr(), n, st), n * 12),
            "m26c_f32_to_bf16": (lambda: glue.f32_to_bf16(x.data_ptr(), y16.data_ptr(), n, st), n * 6),
        }
        rows = {}
        for name, (fn, nbytes) in cases.items():
            ms = timed(fn)
            gbs = nbytes / (ms * 1e-3) / 1e9
            rows[name] = {"us": ms * 1e3, "bytes": nbytes, "GBps": gbs, "frac_of_hbm_peak": gbs / HBM_PEAK_GBS}
        out["rows"][str(T)] = rows
    return out


def stack_reference_rows(seed, layer, payload, scales, ids, weights, O, synth):
    """The CPU rule's BF16 rows for a few tokens of one stack layer, its touched experts regenerated on the host."""
    pools = []
    for r in range(4):
        pool = np.full(synth.EXPERTS * synth.IMAGE_BYTES, 0x22, np.uint8)
        for e in np.unique(ids):
            pool[e * synth.IMAGE_BYTES:(e + 1) * synth.IMAGE_BYTES] = synth.expert_image(seed, r, int(e), layer)
        pools.append(pool)
    rc, _, bits, _ = O.layer_ffn(pools, payload, scales, ids, weights)
    return rc, bits


def run_stack(layers, tokens, torch, dev, O):
    """configs[4]: the routed experts of `layers` layers resident in HBM; a prefill in 4096-token
    segments, a 16-token decode step after each. Returns the JSON object of the run."""
    from mimo26f_afd_amd import stack as S, synth
    seg, dec_rows = 4096, 16
    segments = tokens // seg
    t0 = time.time()
    st = S.ResidentStack(layers, torch, dev, log=log)
    log(f"[bench] {layers} layers prepared in {time.time() - t0:.1f}s")
    pre_routes, dec_routes = st.routes(seg, 0), st.routes(dec_rows, 1)
    x_pre = S.activations_dev(torch, dev, st.seed, tokens, 0)
    x_dec = S.activations_dev(torch, dev, st.seed, dec_rows, 1)
    buf_pre, buf_dec = st.buffers(seg), st.buffers(dec_rows)
    ev = lambda: torch.cuda.Event(enable_timing=True)
    check_layers = sorted({0, layers // 2, layers - 1})
    kept = {}

    def sweep(x, routes, buf, timers, keep_as=None):
        for l in range(layers):
            pair = (ev(), ev())
            nxt = st.layer_step(l, x, routes[l][0], routes[l][1], buf, pair)
            timers.append(pair)
            if keep_as is not None and l in check_layers:  # a few rows of this layer's input and output, for the CPU check
                kept[(keep_as, l)] = (buf["frame"][:8].cpu().numpy(), routes[l][0][:8].cpu().numpy(),
                                      routes[l][1][:8].cpu().numpy(), buf["out"][:8].view(torch.int16).cpu().numpy().view(np.uint16))
            x = nxt
        return x

    # warm-up: one segment and one decode step through every layer, kept for the parity sample
    last = sweep(x_pre[:seg], pre_routes, buf_pre, [], "prefill")
    sweep(x_dec, dec_routes, buf_dec, [], "decode")
    st.sync()
    torch.cuda.synchronize()
    pre_t, dec_t = [], []
    e0, e1 = ev(), ev()
    t0 = time.perf_counter()
    e0.record()
    for sgm in range(segments):
        last = sweep(x_pre[sgm * seg:(sgm + 1) * seg], pre_routes, buf_pre, pre_t)
        x_dec = sweep(x_dec, dec_routes, buf_dec, dec_t)
    e1.record()
    st.sync()
    torch.cuda.synchronize()
    wall_ms = (time.perf_counter() - t0) * 1e3
    pre_ms = np.array([a.elapsed_time(b) for a, b in pre_t])
    dec_ms = np.array([a.elapsed_time(b) for a, b in dec_t])
    parity = []
    for (kind, l), (frame, ids, w, got) in sorted(kept.items()):
        rc, ref = stack_reference_rows(st.seed, l, frame[:, :4096].copy(), frame[:, 4096:4224].copy(), ids, w, O, synth)
        g = (got.astype(np.uint32) << 16).view(np.float32).astype(np.float64)
        r = (ref.astype(np.uint32) << 16).view(np.float32).astype(np.float64)
        parity.append(dict(batch=kind, layer=l, tokens=len(ids), oracle_rc=rc, max_abs_over_max_ref=float(np.max(np.abs(g - r)) / np.max(np.abs(r))),
                           mean_rel=float(np.sum(np.abs(g - r)) / np.sum(np.abs(r)))))
    touched = np.mean([np.unique(r[0].cpu().numpy()).size for r in dec_routes])
    dec_bytes = touched * synth.IMAGE_BYTES * 4 + dec_rows * (4224 + 64 + 8192)
    flops = 6 * seg * 8 * 4096 * 2048
    calls = segments * layers
    line = {
        "metric": "routed tok/s per MoE layer; HBM GB/s (decode) and MFMA % of peak (prefill)",
        "value": (seg + dec_rows) * calls / (wall_ms * 1e-3), "unit": "routed tok/s per MoE layer",
        "n_gpus": 1, "steps": segments, "warmup": 1, "ms_per_step": wall_ms / segments,
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "fp8xfp4->f32", "data": "synthetic",
        "config": {"workload": f"configs[4]: {layers} MoE layers' routed experts resident in HBM ({layers * 256 * synth.IMAGE_BYTES * 4 / 1e9:.1f} GB "
                               f"canonical), {tokens}-token prefill in {seg}-token segments, a {dec_rows}-token decode step after each; "
                               "per layer: wire quantizer -> FFN -> residual mix",
                   "whole_schedule_ms": wall_ms, "event_ms": e0.elapsed_time(e1),
                   "hbm_held_GiB": (torch.cuda.mem_get_info()[1] - torch.cuda.mem_get_info()[0]) / 2**30,
                   "final_residual_std": float(last.std())},
        "prefill_ffn": {"ms_per_layer_call": float(np.median(pre_ms)), "min": float(pre_ms.min()), "max": float(pre_ms.max()),
                        "tok_per_s": seg / (float(np.median(pre_ms)) * 1e-3),
                        "tflops": flops / (float(np.median(pre_ms)) * 1e-3) / 1e12,
                        "frac_of_fp8_peak": flops / (float(np.median(pre_ms)) * 1e-3) / 1e12 / MFMA_FP8_PEAK_TFLOPS},
        "decode_ffn": {"ms_per_layer_call": float(np.median(dec_ms)), "min": float(dec_ms.min()), "max": float(dec_ms.max()),
                       "tok_per_s": dec_rows / (float(np.median(dec_ms)) * 1e-3), "experts_touched_mean": float(touched),
                       "GBps": dec_bytes / (float(np.median(dec_ms)) * 1e-3) / 1e9,
                       "frac_of_hbm_peak": dec_bytes / (float(np.median(dec_ms)) * 1e-3) / 1e9 / HBM_PEAK_GBS},
        "parity": parity,
    }
    st.close()
    del st
    torch.cuda.empty_cache()
    return line


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--no-prefill", action="store_true", help="skip the 8192-token prefill measurement")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--copy-probe", action="store_true",
                    help="profiling aid: also run a 1 GiB -> 1 GiB elementwise copy (torch add), the kernel of known "
                         "size that scales the FETCH_SIZE / WRITE_SIZE counters")
    ap.add_argument("--only-prefill", action="store_true",
                    help="profiling aid: run only the prefill measurement and print its object")
    ap.add_argument("--no-stack", action="store_true", help="skip the 48-layer resident stack (configs[4]) object")
    ap.add_argument("--no-rank-share", action="store_true", help="skip the rank-share object (configs[0], configs[1], the reference's gate sweep)")
    ap.add_argument("--no-coordinator-kernels", action="store_true", help="skip the object that times the kernels either side of the path")
    ap.add_argument("--only-coordinator-kernels", action="store_true", help="profiling aid: run only that leg and print its object")
    ap.add_argument("--only-rank-share", action="store_true", help="profiling aid: run only the rank-share leg and print its object")
    ap.add_argument("--no-variants", action="store_true",
                    help="profiling aid: skip the opt-in forms (fused combine, BF16 per-route rows) sampled beside the default, so a kernel "
                         "trace of the run holds the default path's launches only")
    ap.add_argument("--stack", type=int, default=0, metavar="LAYERS",
                    help="run configs[4] instead: this many layers' routed experts resident in HBM (48 = the full model, 164 GB)")
    ap.add_argument("--stack-tokens", type=int, default=65536, help="prefill length of the --stack run (a multiple of 4096)")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build runs on one GPU only (no collectives, no sharding); use --gpus 1")

    import torch
    if not torch.cuda.is_available():
        sys.exit("bench.py: no GPU visible; the HIP path has no CPU fallback")
    from mimo26f_afd_amd import b1, synth
    import b1_oracle as O
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)

    if args.stack:
        print(json.dumps(run_stack(args.stack, args.stack_tokens, torch, dev, O)), flush=True)
        return
    if args.copy_probe:
        src = torch.zeros(1 << 28, dtype=torch.int32, device=dev)
        dst = torch.empty_like(src)
        for _ in range(3):
            torch.add(src, 1, out=dst)
        torch.cuda.synchronize()
        del src, dst
        torch.cuda.empty_cache()
    if args.only_coordinator_kernels:
        print(json.dumps(run_coordinator_kernels(torch, dev)), flush=True)
        return
    if args.only_rank_share:
        print(json.dumps(run_rank_share(torch, dev, b1, synth, O)), flush=True)
        return
    if args.only_prefill:
        pre = run_config(3, args.steps, args.warmup, torch, dev, b1, synth, O, parity_tokens=PARITY_TOKENS, cpu_tokens=0)
        print(json.dumps(dict(ms_per_step=pre["ms_per_step"], phases=pre["phases"], parity=pre["parity"])), flush=True)
        return
    dec = run_config(2, args.steps, args.warmup, torch, dev, b1, synth, O, parity_tokens=PARITY_TOKENS,
                     cpu_tokens=0 if args.no_cpu else 128, samples=PREFILL_SAMPLES, variants=() if args.no_variants else ("fused_combine",))
    wl = dec["wl"]
    inter, U = wl.intermediate, dec["touched"]
    # Algorithmic bytes: unique weight bytes of the touched experts + input rows + ids/weights + BF16 rows;
    # FC1 streams the gate/up two thirds of each image plus the input rows.
    path_bytes = wl.algorithmic_bytes()
    fc1_bytes = U * inter * (4096 + 256) + wl.rows * 4224
    fc1_gbs = fc1_bytes / (dec["phases"]["fc1_ms"] * 1e-3) / 1e9
    path_gbs = path_bytes / (dec["ms_per_step"] * 1e-3) / 1e9
    dec_traffic, traffic_source = profiled_traffic("fc1_kernel<2>")
    line = {
        "metric": "routed tok/s per MoE layer; HBM GB/s (decode) and MFMA % of peak (prefill)",
        "value": wl.rows / (dec["ms_per_step"] * 1e-3),
        "unit": "routed tok/s per MoE layer",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": dec["ms_per_step"],
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "fp8xfp4->f32",
        "data": "synthetic",
        "config": {"workload": "configs[2]: one full MoE layer, decode/verify, 256 experts x I 2048, H 4096, 128 tokens, top-8",
                   "experts_touched": U, "routes": wl.rows * 8, "weights": "MXFP4 e2m1 + e8m0/32, uniform codes, scales 2^-8..2^-4",
                   "activations": "bf16 N(0,1) -> wire quantizer FP8 e4m3 + ue8m0/32"},
        "roofline": {"bound": "hbm", "kernel": "fc1_kernel<2> (gate/up GEMM + SwiGLU + requant)",
                     "achieved": fc1_gbs, "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": fc1_gbs / HBM_PEAK_GBS,
                     "traffic": dec_traffic, "traffic_source": traffic_source, "algorithmic_bytes": fc1_bytes,
                     "kernel_ms": dec["phases"]["fc1_ms"], "kernel_ms_spread": dec["phases"]["fc1"],
                     "path": {"algorithmic_bytes": path_bytes, "achieved": path_gbs, "frac": path_gbs / HBM_PEAK_GBS,
                              "plan_ms": dec["phases"]["plan_ms"], "fc2_ms": dec["phases"]["fc2_ms"],
                              "reduce_ms": dec["phases"]["reduce_ms"], "event_ms_per_step": dec["event_ms_per_step"],
                              "fc2_ms_spread": dec["phases"]["fc2"], "per_step_ms": dec["per_step"]}},
        "cpu_baseline": dec["cpu"],
        "parity": dec["parity"],
        "fused_combine": dec["variants"].get("fused_combine"),   # opt-in form of the combine: same bits, beside the default
    }
    # The same figures against what this box sustains: a streaming read of 4 GiB, and the GEMMs' MFMA alone.
    from mimo26f_afd_amd import probe
    read_gbs = probe.read_bandwidth_gbps()
    line["roofline"]["measured_read_GBps"] = read_gbs
    line["roofline"]["frac_of_measured"] = fc1_gbs / read_gbs
    line["roofline"]["path"]["frac_of_measured"] = path_gbs / read_gbs
    line["value_routes_per_s"] = line["value"] * 8
    if not args.no_prefill:
        # The reference's protocol: at least 10 warm-ups, at least 31 single-step event samples, the median reported.
        p_warm, p_samples = max(PREFILL_WARMUP, args.warmup), max(PREFILL_SAMPLES, args.steps)
        pre = run_config(3, p_samples, p_warm, torch, dev, b1, synth, O, parity_tokens=PARITY_TOKENS, cpu_tokens=0, samples=p_samples,
                         variants=() if args.no_variants else ("bf16_route_rows", "fused_combine"))
        pw = pre["wl"]
        flops = pw.flops()
        step_ms = pre["per_step"]["median"]
        tf = flops / (step_ms * 1e-3) / 1e12
        fc1_flops = 4 * pw.rows * 8 * 4096 * pw.intermediate
        fc1_ms = pre["phases"]["fc1"]["median"]
        fc1_tf = fc1_flops / (fc1_ms * 1e-3) / 1e12
        pre_traffic, _ = profiled_traffic("fc1_tile_kernel")
        line["prefill"] = {
            "workload": "configs[3]: one full MoE layer, prefill chunk, 8192 tokens, Zipf(1.1) routing",
            "value": pw.rows / (step_ms * 1e-3), "unit": "routed tok/s per MoE layer",
            "ms_per_step": step_ms, "ms_per_step_spread": pre["per_step"], "warmup": p_warm,
            "ms_per_step_back_to_back": pre["ms_per_step"], "steps": p_samples,
            "roofline": {"bound": "mfma", "kernel": "fc1_tile_kernel (gate/up GEMM + SwiGLU + requant)", "achieved": fc1_tf, "peak": MFMA_FP8_PEAK_TFLOPS,
                         "unit": "TFLOP/s", "frac": fc1_tf / MFMA_FP8_PEAK_TFLOPS, "traffic": pre_traffic, "traffic_source": traffic_source,
                         "algorithmic_flops": fc1_flops, "kernel_ms": fc1_ms, "kernel_ms_spread": pre["phases"]["fc1"],
                         "path": {"algorithmic_flops": flops, "achieved": tf, "frac": tf / MFMA_FP8_PEAK_TFLOPS,
                                  "plan_ms": pre["phases"]["plan"]["median"], "fc2_ms": pre["phases"]["fc2"]["median"],
                                  "reduce_ms": pre["phases"]["reduce"]["median"], "fc2_ms_spread": pre["phases"]["fc2"]}},
            "parity": pre["parity"],
            # Opt-in forms, never the headline: the reference's MIMO26_B1_Y=bf16 numerical mode (per-route rows kept
            # as BF16: not the default mode's bits) and the combine inside FC2 (the default mode's bits).
            "bf16_route_rows": pre["variants"].get("bf16_route_rows"),
            "fused_combine": pre["variants"].get("fused_combine"),
        }
        for v in ("bf16_route_rows", "fused_combine"):
            if line["prefill"][v]:
                line["prefill"][v]["path_frac_of_fp8_peak"] = flops / (line["prefill"][v]["ms_per_step"] * 1e-3) / 1e12 / MFMA_FP8_PEAK_TFLOPS
        mfma_tf = probe.mfma_rate_tflops()
        line["prefill"]["roofline"]["measured_mfma_TFLOPs"] = mfma_tf
        line["prefill"]["roofline"]["frac_of_measured"] = fc1_tf / mfma_tf
        line["prefill"]["roofline"]["path"]["frac_of_measured"] = tf / mfma_tf
        # The clock the part held: under the tile kernels (one work item in the middle of each launch) and under a
        # loop of nothing but MFMAs that lasts as long as the timed region. `peak` above is the published figure,
        # quoted at the 2.4 GHz the part does not hold under either load; frac_at_clock prices the kernel against
        # the matrix pipe's rate at the clock the kernel itself ran at.
        held = probe.mfma_sustained()
        fc1_ghz, fc2_ghz = pre["phases"]["clock_ghz"]
        line["prefill"]["roofline"]["clock"] = {
            "nominal_ghz": NOMINAL_GHZ, "fc1_tile_kernel_ghz": fc1_ghz, "fc2_tile_kernel_ghz": fc2_ghz,
            "mfma_only_ghz": held["ghz_last"], "mfma_only_TFLOPs_first_launch": held["tflops_first"],
            "mfma_only_TFLOPs_after_40_launches": held["tflops_last"]}
        if fc1_ghz:
            line["prefill"]["roofline"]["frac_at_clock"] = fc1_tf / (MFMA_FP8_PEAK_TFLOPS * fc1_ghz / NOMINAL_GHZ)
    if not args.no_coordinator_kernels:
        try:
            line["coordinator_kernels"] = run_coordinator_kernels(torch, dev)
        except Exception as e:  # a leg beside the headline: reported, never fatal
            line["coordinator_kernels"] = {"error": f"{type(e).__name__}: {e}"}
    if not args.no_rank_share:
        try:
            t0 = time.time()
            line["rank_share"] = run_rank_share(torch, dev, b1, synth, O)
            line["rank_share"]["leg_seconds"] = time.time() - t0
        except Exception as e:  # the headline line must survive a failure of this leg
            line["rank_share"] = {"error": f"{type(e).__name__}: {e}"}
    if not args.no_stack:
        # configs[4] with all 48 layers resident needs about 175 GiB of HBM; without it the object says so.
        free_gib = torch.cuda.mem_get_info()[0] / 2**30
        if free_gib < 200:
            line["stack"] = {"skipped": f"{free_gib:.0f} GiB of HBM free, the 48-layer stack holds 175"}
        else:
            try:
                t0 = time.time()
                st = run_stack(48, 65536, torch, dev, O)
                line["stack"] = {"workload": st["config"]["workload"], "value": st["value"], "unit": st["unit"],
                                 "whole_schedule_ms": st["config"]["whole_schedule_ms"], "hbm_held_GiB": st["config"]["hbm_held_GiB"],
                                 "prefill_ffn": st["prefill_ffn"], "decode_ffn": st["decode_ffn"], "parity": st["parity"],
                                 "leg_seconds": time.time() - t0}
            except Exception as e:  # the headline line must survive a failure of this leg
                line["stack"] = {"error": f"{type(e).__name__}: {e}"}
    print(json.dumps(line), flush=True)


if __name__ == "__main__":
    main()
