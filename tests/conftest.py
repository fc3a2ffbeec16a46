import os
import sys

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


def make_operand(rng, shape, dtype, dist="uniform"):
    """seeded operand in the oracle's host format (fp16 array, bf16 bit patterns, int8 array)"""
    from oracle import cpu_oracle as co
    if dtype == "int8":
        return rng.integers(-128, 128, size=shape, dtype=np.int64).astype(np.int8)
    x = rng.uniform(-1, 1, size=shape) if dist == "uniform" else rng.standard_normal(size=shape)
    x = x.astype(np.float32)
    if dtype == "float16":
        return x.astype(np.float16)
    return co.float_to_bf16_bits(x)


def to_device(x, dtype):
    """host operand -> torch tensor on cuda:0 with the matching torch dtype"""
    import torch
    if dtype == "bfloat16":
        return torch.from_numpy(x.view(np.int16).copy()).cuda().view(torch.bfloat16)
    return torch.from_numpy(np.ascontiguousarray(x)).cuda()


@pytest.fixture(scope="session")
def gpu():
    import torch
    if not torch.cuda.is_available():
        pytest.fail("a test marked gpu ran without a GPU")
    from amos_amd import _lib
    _lib.load()
    return torch.device("cuda:0")
