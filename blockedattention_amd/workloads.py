"""Seeded synthetic workloads: the five benchmark configurations.

Sizes come from ``numpy.random.default_rng(seed)`` with the draws in the order
listed; values from ``torch.Generator("cpu").manual_seed(seed)`` in fp32, then
cast to the compute dtype.  Mapping to the operator's names: M = rows of A
(i_b), N = rows of B (k_b), K = reduction length (j_b).
"""
from dataclasses import dataclass

import numpy as np
import torch


@dataclass
class Workload:
    name: str
    M: np.ndarray          # int64 [B]
    N: np.ndarray
    K: np.ndarray
    heads: int
    dtype: torch.dtype     # dtype on the GPU
    scale: float           # softmax scale
    dist: str              # "normal" or "uniform"
    sigma: float = 1.0

    @property
    def nseg(self):
        return int(self.M.shape[0])

    @property
    def Dm1(self):
        return int((self.M * self.K).sum())

    @property
    def Dm2(self):
        return int((self.N * self.K).sum())

    @property
    def Dout(self):
        return int((self.M * self.N).sum())

    @property
    def flops(self):
        return 2 * self.heads * int((self.M * self.N * self.K).sum())

    def pair_bytes(self, elem_bytes=2):
        """A and B read once, probabilities written once."""
        return elem_bytes * self.heads * (self.Dm1 + self.Dm2 + self.Dout)

    def softmax_bytes(self, elem_bytes=2):
        return 2 * elem_bytes * self.heads * self.Dout

    def operands(self, seed=0, dtype=None):
        """(A [H,Dm1], B [H,Dm2]) CPU tensors already cast to ``dtype``."""
        dtype = self.dtype if dtype is None else dtype
        gen = torch.Generator(device="cpu").manual_seed(seed)
        shape_a, shape_b = (self.heads, self.Dm1), (self.heads, self.Dm2)
        if self.dist == "normal":
            a = torch.randn(shape_a, generator=gen, dtype=torch.float32) * self.sigma
            b = torch.randn(shape_b, generator=gen, dtype=torch.float32) * self.sigma
        else:
            a = torch.rand(shape_a, generator=gen, dtype=torch.float32) * 2 - 1
            b = torch.rand(shape_b, generator=gen, dtype=torch.float32) * 2 - 1
        return a.to(dtype), b.to(dtype)


def make(cfg, seed=0, k=None):
    """cfg in 1..5 -> Workload.  k: configuration 5 with another reduction length (the name says which)."""
    rng = np.random.default_rng(seed)
    i64 = np.int64
    if cfg == 1:
        n = rng.integers(8, 33, 64).astype(i64)
        return Workload("cfg1_molecule_64seg_n8-32_k64", n, n.copy(), np.full(64, 64, i64), 1,
                        torch.float16, 64 ** -0.5, "normal")
    if cfg == 2:
        n = rng.integers(32, 129, 256).astype(i64)
        return Workload("cfg2_medium_256seg_x8h_n32-128_k64", n, n.copy(), np.full(256, 64, i64), 8,
                        torch.float16, 64 ** -0.5, "normal")
    if cfg == 3:
        n = np.clip(np.rint(rng.lognormal(3.5, 1.0, 1024)), 2, 512).astype(i64)
        return Workload("cfg3_powerlaw_1024seg_x4h_k128", n, n.copy(), np.full(1024, 128, i64), 4,
                        torch.bfloat16, 128 ** -0.5, "normal")
    if cfg == 4:
        M = rng.integers(16, 257, 512).astype(i64)
        N = rng.integers(16, 257, 512).astype(i64)
        K = rng.choice(np.arange(32, 129, 8), 512).astype(i64)
        return Workload("cfg4_nonsquare_512seg_mn16-256_k32-128", M, N, K, 1, torch.float16, 1.0, "uniform")
    if cfg == 5:
        n = rng.integers(1024, 4097, 16).astype(i64)
        k = 128 if k is None else int(k)
        return Workload(f"cfg5_large_16seg_x16h_n1024-4096_k{k}", n, n.copy(), np.full(16, k, i64), 16,
                        torch.bfloat16, k ** -0.5, "normal", sigma=k ** -0.5)
    raise ValueError("cfg must be 1..5")
