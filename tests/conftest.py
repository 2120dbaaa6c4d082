import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


@pytest.fixture(scope="session")
def oracle():
    import oracle as orc

    orc.lib()
    return orc


GUARD_BYTES = 256


@pytest.fixture
def canaries(monkeypatch):
    """Guard bands around every output the host mirror allocates while the fixture is active (the reference's
    metal/test_support.rs:26-77): 256 bytes of 0xA5 before and of 0x5A after each tensor, checked at teardown and on
    demand with ``canaries.check()``.  A kernel that stores a tile past a ragged edge trips them."""
    import torch

    import qwen_llm_amd.binding as binding

    class Guards:
        def __init__(self):
            self.buffers = []

        def empty(self, *size, dtype=torch.float32, device=None, **kw):
            if len(size) == 1 and not isinstance(size[0], int):
                size = tuple(size[0])
            n = 1
            for d in size:
                n *= int(d)
            item = torch.empty((), dtype=dtype).element_size()
            body = (n * item + 255) // 256 * 256
            raw = torch.empty(GUARD_BYTES + body + GUARD_BYTES, dtype=torch.uint8, device=device)
            raw[:GUARD_BYTES] = 0xA5
            raw[GUARD_BYTES + n * item:] = 0x5A
            self.buffers.append((raw, n * item))
            return raw[GUARD_BYTES:GUARD_BYTES + n * item].view(dtype).view(size)

        def check(self):
            torch.cuda.synchronize()
            for raw, nbytes in self.buffers:
                assert bool((raw[:GUARD_BYTES] == 0xA5).all()), "a kernel wrote before its output"
                assert bool((raw[GUARD_BYTES + nbytes:] == 0x5A).all()), "a kernel wrote past its output"
            return len(self.buffers)

    g = Guards()
    monkeypatch.setattr(binding, "_empty", g.empty)
    yield g
    g.check()
