import os
import sys

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
PKG_PARENT = os.path.join(ROOT, "tensor-product-attention-jax_amd")
for p in (PKG_PARENT, ROOT):
    if p not in sys.path:
        sys.path.insert(0, p)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs an MI355X (run with -m gpu on the GPU box)")


def make_factors(seed, b, lq, lk, h, dk, dv, rq, rk, dist="normal", scale_by_rank=False):
    """Seeded concatenated factors q[b,lq,rq,h+dk], k[b,lk,rk,h+dk], v[b,lk,rk,h+dv] (float32).

    dist="uniform" follows the reference's forward test (uniform [0,1), tpa/tpa_test.py:89-91);
    dist="normal" with scale_by_rank follows the benchmark configurations (N(0,1) / sqrt(R)).
    """
    rng = np.random.Generator(np.random.Philox(seed))

    def draw(shape, r):
        if dist == "uniform":
            x = rng.random(shape, dtype=np.float32)
        else:
            x = rng.standard_normal(shape, dtype=np.float32)
        if scale_by_rank:
            x = x / np.sqrt(np.float32(r))
        return x.astype(np.float32)

    q = draw((b, lq, rq, h + dk), rq)
    k = draw((b, lk, rk, h + dk), rk)
    v = draw((b, lk, rk, h + dv), rk)
    return q, k, v


def segment_ids(length, segment_size, batch):
    """arange(l) // segment_size repeated over the batch (tpa/tpa_test.py:93-99)."""
    return np.repeat((np.arange(length) // segment_size)[None], batch, axis=0).astype(np.int32)


def bf16_round(x):
    """Round float32 to the nearest bfloat16 (ties to even) and return it as float32."""
    import torch

    return torch.from_numpy(np.ascontiguousarray(x)).to(torch.bfloat16).to(torch.float32).numpy()


@pytest.fixture(scope="session")
def gpu():
    import torch

    if not torch.cuda.is_available():
        pytest.fail("this test is marked gpu but no HIP device is visible")
    return torch.device("cuda:0")
