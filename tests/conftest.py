import os
import sys

import pytest

sys.path.insert(0, os.path.dirname(os.path.dirname(os.path.abspath(__file__))))


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


@pytest.fixture(scope="session")
def device():
    """The one GPU, opened once per test process."""
    from zllm_amd import Device

    d = Device.open(0)
    yield d
    d.deinit()


@pytest.fixture()
def ctx():
    """A kernel-check context on a device of its own, so that object ids and
    failures never leak from one test into the next."""
    from gpucheck import Ctx
    from zllm_amd import Device

    d = Device.open(0)
    c = Ctx(d)
    yield c
    d.deinit()


@pytest.fixture()
def ctx_wide():
    """The same on a device opened with ZHIP_OPTION_WIDE_DECODE: large bf16 / f16 matrices
    take the kernel that reads the weights once for all of a step's tokens."""
    from gpucheck import Ctx
    from zllm_amd import Device

    d = Device.open(0, Device.WIDE_DECODE)
    c = Ctx(d)
    yield c
    d.deinit()
