import os
import sys

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


@pytest.fixture(scope="session")
def oracle():
    """The CPU oracle (test infrastructure), built on demand from oracle/."""
    from oracle import oracle as o
    o.lib()
    return o


@pytest.fixture(scope="session")
def vpq():
    """The product library through its C ABI; fails loudly if it is not built."""
    import vpipe_amd
    vpipe_amd.load()
    return vpipe_amd


@pytest.fixture(scope="session")
def dev():
    import torch
    assert torch.cuda.is_available(), "GPU tests need a GPU"
    return torch.device("cuda:0")


class Dev:
    """numpy <-> torch device tensor helpers for bf16 bit patterns."""

    @staticmethod
    def bf16(bits, dev):
        import torch
        return torch.from_numpy(np.ascontiguousarray(bits).view(np.int16)).to(dev).view(torch.bfloat16)

    @staticmethod
    def u32(words, dev):
        import torch
        return torch.from_numpy(np.ascontiguousarray(words).view(np.int32)).to(dev)

    @staticmethod
    def i16(bits, dev):
        import torch
        return torch.from_numpy(np.ascontiguousarray(bits).view(np.int16)).to(dev)

    @staticmethod
    def bits(t):
        import torch
        if t.dtype == torch.bfloat16:
            t = t.view(torch.int16)
        return t.cpu().numpy().view(np.uint16)

    @staticmethod
    def words(t):
        return t.cpu().numpy().view(np.uint32)


@pytest.fixture(scope="session")
def D():
    return Dev
