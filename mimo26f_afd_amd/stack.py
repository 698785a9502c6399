"""A stack of MoE layers' routed experts resident in HBM, driven segment by segment.

The largest benchmark configuration keeps the routed experts of all 48 layers of a MiMo-shape model
(256 experts x intermediate 2048 per layer, about 164 GB of MXFP4 with scales) on one GPU and pushes
a long prefill through them in 4096-token segments, a 16-token decode step after every segment.
Nothing here is on the reference's expert-rank path itself: it is the harness that feeds that path
layer after layer, so it may use torch for its own arithmetic. Per layer and segment the device does

    residual rows (f32) --row RMS norm, bf16--> hidden rows --wire quantizer--> request-frame rows
        (pitch 4224) --m26s_b1_ffn_enqueue--> BF16 rows --residual mix--> residual rows of the next layer

with the wire quantizer and the FFN going through the library's C ABI. Weights, routes and first
activations come from the same counter-based splitmix64 streams as `synth` (evaluated on the device,
where 164 GB of bytes take seconds); `synth.expert_image(..., layer=l)` regenerates any expert of any
layer on the host, which is how a run is checked against the CPU rule on sampled tokens.
"""
from __future__ import annotations

import math

import numpy as np

from . import b1, glue, synth

_MASK64 = (1 << 64) - 1
FRAME_PITCH = 4224  # payload row then its 128 scale bytes (crates/mimo26-wire/src/layout.rs:55-68)
# Share of the FFN output in the next layer's residual, and the output's standard deviation for
# unit-variance input (CPU rule on this weight distribution): the residual keeps unit variance. The
# FFN's output grows with the square of its input's scale, so a token's rows are normalised before
# every layer, as the model's own pre-norm block does; fed the raw residual, single tokens run away
# within a few dozen layers and the intermediate overflows.
MIX_SHARE, OUTPUT_STD = 0.05, 52.4


def _i64(v: int) -> int:
    v &= _MASK64
    return v - (1 << 64) if v >> 63 else v


def _lsr(z, n: int):
    return (z >> n) & ((1 << (64 - n)) - 1)


def _mix(z):
    z = (z ^ _lsr(z, 30)) * _i64(0xBF58476D1CE4E5B9)
    z = (z ^ _lsr(z, 27)) * _i64(0x94D049BB133111EB)
    return z ^ _lsr(z, 31)


def u64_dev(torch, dev, key: int, count: int):
    """Elements 0..count-1 of stream `key` as int64 bit patterns (synth.u64 on the device)."""
    i = torch.arange(1, count + 1, dtype=torch.int64, device=dev)
    return _mix(i * _i64(0x9E3779B97F4A7C15) + _i64(int(key)))


def uniform_dev(torch, dev, key: int, count: int):
    """Doubles in (0, 1], as synth.uniform."""
    return (_lsr(u64_dev(torch, dev, key, count), 11).to(torch.float64) + 1.0) * 2.0 ** -53


def normal_dev(torch, dev, key: int, count: int):
    u = uniform_dev(torch, dev, key, 2 * count)
    return torch.sqrt(-2.0 * torch.log(u[0::2])) * torch.cos(2.0 * math.pi * u[1::2])


def rank_pool_dev(torch, dev, seed: int, rank: int, layer: int = 0):
    """synth.rank_pool(seed, rank) of `layer` as a uint8 device tensor (855,638,016 bytes)."""
    words = synth.IMAGE_BYTES // 8
    keys = np.array([_i64(int(synth.stream_key(seed, synth.WEIGHTS, rank, layer * synth.EXPERTS + e)))
                     for e in range(synth.EXPERTS)], np.int64)
    i = torch.arange(1, words + 1, dtype=torch.int64, device=dev) * _i64(0x9E3779B97F4A7C15)
    pool = torch.empty((synth.EXPERTS, synth.IMAGE_BYTES), dtype=torch.uint8, device=dev)
    step = 32  # experts per pass: bounds the int64 temporaries to a few hundred MB
    kd = torch.from_numpy(keys).to(dev)
    for e0 in range(0, synth.EXPERTS, step):
        z = _mix(i[None, :] + kd[e0:e0 + step, None])
        pool[e0:e0 + step] = z.view(torch.uint8).view(step, synth.IMAGE_BYTES)
    for lo, hi in synth.SCALE_REGIONS:
        region = pool[:, lo:hi]
        pool[:, lo:hi] = (119 + ((region.to(torch.int32) * 5) >> 8)).to(torch.uint8)
    return pool.view(-1)


def routes_zipf_dev(torch, dev, seed: int, rows: int, layer: int, part: int = 0, s: float = 1.1):
    """Per token 8 distinct experts by exponential-key sampling of a Zipf(s) popularity over a
    permutation of the ids that is the layer's own; (rows, 8) int32 and softmax weights f32."""
    perm_keys = u64_dev(torch, dev, synth.stream_key(seed, synth.ROUTES, 2, layer), synth.EXPERTS)
    # order by the unsigned value: flip the sign bit for a signed sort
    perm = torch.argsort(perm_keys ^ _i64(1 << 63), stable=True)
    p = 1.0 / torch.arange(1, synth.EXPERTS + 1, dtype=torch.float64, device=dev) ** s
    p = p / p.sum()
    u = uniform_dev(torch, dev, synth.stream_key(seed, synth.ROUTES, 3 + part, layer), rows * synth.EXPERTS)
    keys = -torch.log(u).view(rows, synth.EXPERTS) / p
    ranks = torch.topk(keys, synth.TOPK, dim=1, largest=False, sorted=True).indices
    ids = perm[ranks].to(torch.int32).contiguous()
    z = normal_dev(torch, dev, synth.stream_key(seed, synth.LOGITS, part, layer), rows * synth.TOPK).view(rows, synth.TOPK)
    w = torch.softmax(z, dim=1).to(torch.float32).contiguous()
    return ids, w


def activations_dev(torch, dev, seed: int, rows: int, part: int = 0):
    """bf16-valued N(0,1) rows as float32."""
    x = normal_dev(torch, dev, synth.stream_key(seed, synth.ACTIVATIONS, part), rows * synth.HIDDEN)
    return x.to(torch.float32).to(torch.bfloat16).to(torch.float32).view(rows, synth.HIDDEN)


class ResidentStack:
    """`layers` full-intermediate MoE layers prepared once and kept in HBM, one scratch, one stream."""

    def __init__(self, layers: int, torch, dev, seed: int = synth.BASE_SEED + 4, log=None):
        self.torch, self.dev, self.seed, self.count = torch, dev, seed, layers
        self.layers = []
        for l in range(layers):
            pools = [rank_pool_dev(torch, dev, seed, r, l) for r in range(4)]
            torch.cuda.synchronize()
            self.layers.append(b1.Layer.full([p.data_ptr() for p in pools], pools[0].numel()))
            del pools
            if log and (l % 8 == 7 or l == layers - 1):
                log(f"[stack] {l + 1} layers resident, {torch.cuda.memory_allocated() / 2**30:.1f} GiB held by torch "
                    f"(the prepared pools are the library's own)")
        torch.cuda.empty_cache()
        self.stream = torch.cuda.current_stream().cuda_stream
        self.scratch = b1.Scratch(stream=self.stream)
        order = u64_dev(torch, dev, synth.stream_key(seed, synth.SHUFFLE, 1), synth.HIDDEN)
        self.perm = torch.argsort(order ^ _i64(1 << 63), stable=True)
        self.keep, self.gain = math.sqrt(1.0 - MIX_SHARE), math.sqrt(MIX_SHARE) / OUTPUT_STD

    def routes(self, rows: int, part: int):
        """Per layer (ids, weights) for a batch of `rows` tokens; `part` separates the batches."""
        return [routes_zipf_dev(self.torch, self.dev, self.seed, rows, l, part) for l in range(self.count)]

    def buffers(self, rows: int):
        t = self.torch
        return dict(frame=t.empty((rows, FRAME_PITCH), dtype=t.uint8, device=self.dev),
                    out=t.empty((rows, synth.HIDDEN), dtype=t.bfloat16, device=self.dev))

    def layer_step(self, l: int, r, ids, weights, buf, events=None):
        """One layer on residual rows r (f32 [rows, 4096]); returns the next layer's rows. Launches only."""
        t = self.torch
        rows = r.shape[0]
        frame, out = buf["frame"], buf["out"]
        x = (r * t.rsqrt(t.mean(r * r, dim=1, keepdim=True))).to(t.bfloat16).to(t.float32)
        glue.quantize_hidden(x.data_ptr(), rows, synth.HIDDEN, frame.data_ptr(), FRAME_PITCH,
                             frame.data_ptr() + synth.HIDDEN, FRAME_PITCH, self.stream)
        if events is not None:
            events[0].record()
        b1.ffn_enqueue(self.layers[l], self.scratch, frame.data_ptr(), FRAME_PITCH, frame.data_ptr() + synth.HIDDEN,
                       FRAME_PITCH, ids.data_ptr(), weights.data_ptr(), rows, out.data_ptr())
        if events is not None:
            events[1].record()
        return r.index_select(1, self.perm) * self.keep + out.to(t.float32) * self.gain

    def sync(self) -> None:
        """Waits for the launches; raises the first device fault of the batch."""
        self.scratch.sync()

    def close(self) -> None:
        self.scratch.close()
        for layer in self.layers:
            layer.close()
        self.layers = []
