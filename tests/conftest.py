import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
for p in (ROOT, os.path.join(ROOT, "oracle")):
    if p not in sys.path:
        sys.path.insert(0, p)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs an MI355X; runs through the C ABI of the HIP library")
    if _gpu_present():  # before any fixture of any scope makes a buffer or a scratch
        import helpers
        helpers.install_guards()


def _gpu_present() -> bool:
    return os.path.exists("/dev/kfd")


def pytest_collection_modifyitems(config, items):
    if _gpu_present():
        return
    skip = pytest.mark.skip(reason="no GPU in this container")
    for item in items:
        if "gpu" in item.keywords:
            item.add_marker(skip)


@pytest.fixture(autouse=True)
def _red_zones(request):
    """GPU tests run with guarded device buffers and guarded scratches; every guard still alive is read back
    when a test ends."""
    if "gpu" not in request.keywords or not _gpu_present():
        yield
        return
    import helpers
    yield
    helpers.check_all_guards()


@pytest.fixture(scope="session")
def full_layer():
    """The 256 experts of configs[2] / configs[3] at the full intermediate (the two configurations share their
    seeded weights): (the 128-token decode workload, the canonical rank pools on the host, the prepared layer).
    Generated and prepared once per session: 3.4 GB each side."""
    from helpers import DeviceLayer
    from mimo26f_afd_amd import synth
    wl = synth.make(2)
    pools = wl.pools()
    return wl, pools, DeviceLayer(pools).layer


@pytest.fixture(scope="session")
def prefill_chunk_on_gpu(full_layer):
    """configs[3], all 8192 tokens, run once through the device-pointer entry: (workload, BF16 rows, FP32 sums)."""
    from helpers import run_ffn_dev
    from mimo26f_afd_amd import b1, synth
    _, _, layer = full_layer
    wl = synth.make(3)
    scratch = b1.Scratch()
    _, bf, pf = run_ffn_dev(layer, scratch, wl)
    return wl, bf, pf
