"""Seeded random batches through every entry point against the oracle: widths around every tile count of
the strip kernel (in-memory image of B_g at K = 64 / 128, operand-order blocks otherwise), ragged ends,
tall and short segments, both 16-bit dtypes, with other kernels run in between."""
import numpy as np
import pytest
import torch

from _util import run_all

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("seed", range(6))
def test_random_batches(dev, seed):
    rng = np.random.default_rng(100 + seed)
    nseg = int(rng.integers(3, 40))
    K = rng.choice([64, 128, 64, 128, 32, 72, 8, 200])            # one K per batch or mixed
    Ks = np.where(rng.random(nseg) < 0.7, K, rng.choice([16, 64, 128, 40], nseg)).astype(np.int64)
    N = rng.integers(1, 260, nseg).astype(np.int64)
    N[rng.random(nseg) < 0.2] = rng.choice([16, 32, 64, 96, 128, 160, 256, 33, 2, 1], int((rng.random(nseg) < 0.2).sum()) or 1)[0]
    M = rng.integers(1, 200, nseg).astype(np.int64)
    if seed % 2:
        M[0], N[0] = 700, 37                                       # tall: several strips per wavefront
        N[1] = 300                                                  # one tile-kernel segment in the mix
    H = int(rng.integers(1, 4))
    dtype = torch.float16 if seed % 3 else torch.bfloat16
    scale = float(rng.choice([0.125, 1.0, -0.2]))
    sigma = 0.3 if int(Ks.max()) > 100 else 1.0                     # keeps fp16 scores far from overflow
    run_all(dev, M, N, Ks, H, dtype, scale, seed=seed, sigma=sigma)
    run_all(dev, M, N, Ks, H, dtype, scale, seed=seed + 50, sigma=sigma, summary=False)


@pytest.mark.parametrize("seed", range(3))
def test_random_batches_of_65_to_256_segments(dev, seed):
    # the scheduler build that keeps the main strip list in work buckets; head counts that are not powers of two
    rng = np.random.default_rng(300 + seed)
    nseg = int(rng.integers(65, 257))
    Ks = rng.choice([64, 128, 32, 72, 8], nseg, p=[0.4, 0.3, 0.1, 0.1, 0.1]).astype(np.int64)
    N = rng.integers(1, 260, nseg).astype(np.int64)
    M = rng.integers(1, 150, nseg).astype(np.int64)
    N[:3] = [300, 1, 16]; M[:3] = [40, 5, 3]
    H = int(rng.choice([1, 3, 5, 8, 9]))
    dtype = torch.float16 if seed % 2 else torch.bfloat16
    run_all(dev, M, N, Ks, H, dtype, 0.1, seed=seed, sigma=0.3)
    run_all(dev, M, N, Ks, H, dtype, 0.1, seed=seed + 50, sigma=0.3, summary=False)
