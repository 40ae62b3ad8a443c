import os
import sys

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

TOL_F32 = 1e-4     # max|y-ref|/max|ref| on the fp32 path
TOL_BF16 = 2e-2    # same metric on the bf16 path


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a gfx950 (MI355X) device")


@pytest.fixture(scope="session")
def corc():
    """The C oracle (fp32, shader order)."""
    from oracle import oracle_np
    oracle_np.build()
    return oracle_np.COracle()


@pytest.fixture(scope="session")
def backend():
    """One Compute() for the whole GPU session.  No fallback: if the library or the device is
    missing this raises and the GPU tests fail loudly."""
    import grilly_amd
    b = grilly_amd.Compute()
    yield b
    b.cleanup()


def sweep_rounds():
    """How many times the seeded randomized sweeps repeat with fresh seeds (GRILLY_SWEEP_ROUNDS, default 1: the round
    with the fixed seed that every run shares; more rounds are for longer parity runs on a GPU box)."""
    return max(1, int(os.environ.get("GRILLY_SWEEP_ROUNDS", "1")))


def rng_for(cfg):
    return np.random.default_rng(20260131 + cfg)
