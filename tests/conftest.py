import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


@pytest.fixture(scope="session")
def golden():
    import json

    out = {}
    gdir = os.path.join(ROOT, "tests", "golden")
    for name in os.listdir(gdir):
        if name.endswith(".json"):
            with open(os.path.join(gdir, name)) as f:
                out[name[:-5]] = json.load(f)
    return out


@pytest.fixture(scope="session")
def gpu():
    """One Device for the whole GPU session.  Fails loudly without a GPU: there is no fallback."""
    from dynet_amd import Device

    dev = Device(0, mem_mb=(3072, 2048, 1024, 1024))
    # float32 tensors from empty() start as NaN: an output element that a kernel skips fails its comparison
    dev.poison_empty = os.environ.get("DYHIP_TEST_NO_POISON") is None
    yield dev
    dev.close()


@pytest.fixture()
def dev(gpu):
    """Per-test view of the device with the graph pools (FXS, DEDFS, SCS) reset."""
    from dynet_amd import lib

    gpu.sync()
    for which in (lib.POOL_FXS, lib.POOL_DEDFS, lib.POOL_SCS):
        gpu.free_pool(which)
    return gpu
