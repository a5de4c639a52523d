import os
import sys

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs an MI355X (run with -m gpu on the GPU box)")


def lowdim_data(num, dim=128, latent=12, seed=1, mix_seed=0):
    """Integer-valued (0..255) vectors with low intrinsic dimension: a navigable, tie-rich test distribution."""
    a = np.random.default_rng(mix_seed).standard_normal((latent, dim)).astype(np.float32)
    r = np.random.default_rng(seed)
    z = r.standard_normal((num, latent)).astype(np.float32)
    x = z @ a * 20 + 128 + r.standard_normal((num, dim)).astype(np.float32) * 3
    return np.rint(np.clip(x, 0, 255)).astype(np.float32)


def lowdim_float_data(num, dim=96, latent=10, seed=1, mix_seed=0):
    """Unit-norm float vectors (cosine configuration)."""
    a = np.random.default_rng(mix_seed).standard_normal((latent, dim)).astype(np.float32)
    r = np.random.default_rng(seed)
    z = r.standard_normal((num, latent)).astype(np.float32)
    x = z @ a + r.standard_normal((num, dim)).astype(np.float32) * 0.1
    x /= np.linalg.norm(x, axis=1, keepdims=True)
    return x.astype(np.float32)


@pytest.fixture(scope="session")
def small_index():
    """A complete index built by the CPU oracle on 6000 integer-valued points (3 partitions)."""
    from oracle import oracle as O
    data = lowdim_data(6000, 128, seed=1)
    idx = O.build_index(data, 3, graph_degree=32, knn_degree=32, nnd_iterations=6)
    idx["data"] = data
    idx["queries"] = lowdim_data(300, 128, seed=2)
    return idx
