"""The resident-stack harness (the 48-layer configuration, reduced): its device-side generators against
the host ones (CPU tensors here, the GPU in the marked tests) and a short run against the CPU rule."""
import numpy as np
import pytest
import torch

from mimo26f_afd_amd import stack as S
from mimo26f_afd_amd import synth

SEED = synth.BASE_SEED + 4


def test_streams_match_host_generator():
    key = synth.stream_key(SEED, synth.ROUTES, 2, 5)
    got = S.u64_dev(torch, "cpu", key, 1000).numpy().view(np.uint64)
    assert np.array_equal(got, synth.u64(key, 1000))
    assert np.array_equal(S.uniform_dev(torch, "cpu", key, 1000).numpy(), synth.uniform(key, 1000))
    np.testing.assert_allclose(S.normal_dev(torch, "cpu", key, 500).numpy(), synth.normal(key, 500), rtol=0, atol=1e-12)


def test_weight_pool_matches_host_generator():
    pool = S.rank_pool_dev(torch, "cpu", SEED, 2, layer=3).numpy()
    assert pool.size == synth.EXPERTS * synth.IMAGE_BYTES
    for e in (0, 17, 255):
        want = synth.expert_image(SEED, 2, e, layer=3)
        assert np.array_equal(pool[e * synth.IMAGE_BYTES:(e + 1) * synth.IMAGE_BYTES], want), e
    # layer 0 of the stack seed is what the single-layer generator gives
    assert np.array_equal(synth.expert_image(SEED, 1, 9, layer=0), synth.expert_image(SEED, 1, 9))


def test_routes_are_legal_and_skewed():
    ids, w = S.routes_zipf_dev(torch, "cpu", SEED, 2048, layer=7)
    ids, w = ids.numpy(), w.numpy()
    assert ids.shape == (2048, 8) and ids.min() >= 0 and ids.max() < 256
    assert all(len(set(r)) == 8 for r in ids)
    np.testing.assert_allclose(w.sum(axis=1), 1.0, atol=1e-6)
    counts = np.sort(np.bincount(ids.ravel(), minlength=256))[::-1]
    assert counts[0] > 8 * counts[64]  # Zipf(1.1): rank 1 against rank 65
    other, _ = S.routes_zipf_dev(torch, "cpu", SEED, 2048, layer=8)
    assert np.argmax(np.bincount(other.numpy().ravel())) != np.argmax(np.bincount(ids.ravel()))  # own permutation per layer


@pytest.mark.gpu
def test_device_pool_matches_host_generator():
    dev = torch.device("cuda:0")
    pool = S.rank_pool_dev(torch, dev, SEED, 1, layer=40)
    for e in (3, 200):
        got = pool[e * synth.IMAGE_BYTES:(e + 1) * synth.IMAGE_BYTES].cpu().numpy()
        assert np.array_equal(got, synth.expert_image(SEED, 1, e, layer=40)), e


@pytest.mark.gpu
def test_short_stack_against_cpu_rule():
    from helpers import stack_reference_rows
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    layers, seg, segments, dec_rows = 3, 256, 2, 16
    st = S.ResidentStack(layers, torch, dev)
    try:
        pre_routes, dec_routes = st.routes(seg, 0), st.routes(dec_rows, 1)
        x_pre = S.activations_dev(torch, dev, st.seed, seg * segments, 0)
        x_dec = S.activations_dev(torch, dev, st.seed, dec_rows, 1)
        buf_pre, buf_dec = st.buffers(seg), st.buffers(dec_rows)
        checked = 0
        for sgm in range(segments):
            for kind, x, routes, buf in (("prefill", x_pre[sgm * seg:(sgm + 1) * seg], pre_routes, buf_pre),
                                        ("decode", x_dec, dec_routes, buf_dec)):
                for l in range(layers):
                    x = st.layer_step(l, x, routes[l][0], routes[l][1], buf)
                    st.sync()
                    if sgm == segments - 1:  # the last segment's rows went through every earlier layer on the device
                        pick = list(range(4)) + list(range(x.shape[0] - 4, x.shape[0]))  # a two-row sample is at the mercy of one flipped E4M3 code
                        frame = buf["frame"][pick].cpu().numpy()
                        ids, w = routes[l][0][pick].cpu().numpy(), routes[l][1][pick].cpu().numpy()
                        got = buf["out"][pick].view(torch.int16).cpu().numpy().view(np.uint16)
                        rc, ref = stack_reference_rows(st.seed, l, frame[:, :4096].copy(), frame[:, 4096:].copy(), ids, w)
                        assert rc == 0, (kind, l)
                        g = (got.astype(np.uint32) << 16).view(np.float32).astype(np.float64)
                        r = (ref.astype(np.uint32) << 16).view(np.float32).astype(np.float64)
                        assert np.max(np.abs(g - r)) <= 1e-2 * np.max(np.abs(r)), (kind, l)
                        assert np.sum(np.abs(g - r)) <= 1e-3 * np.sum(np.abs(r)), (kind, l)
                        checked += 1
                if kind == "decode":
                    x_dec = x
                assert 0.5 < float(x.std()) < 2.0, (kind, float(x.std()))  # the residual mix holds the scale
        assert checked == 2 * layers
    finally:
        st.close()
