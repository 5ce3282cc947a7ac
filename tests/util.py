"""Helpers shared by the tests: golden-vector loading and seeded workload construction."""
from __future__ import annotations

import json
import os

import numpy as np
import torch

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
DTYPES = {"f32": torch.float32, "bf16": torch.bfloat16, "f16": torch.float16}


def load_golden(name: str):
    with open(os.path.join(GOLDEN, name)) as f:
        return json.load(f)


def bits_to_tensor(bits, dtype: str) -> torch.Tensor:
    """list of binary32 bit patterns (exactly representable in `dtype`) -> 1-D tensor of that dtype"""
    f = torch.from_numpy(np.array(bits, dtype=np.uint32).view(np.float32).copy())
    t = f.to(DTYPES[dtype])
    assert torch.equal(t.float(), f), "golden input is not representable in its dtype"
    return t


def f32_from_bits(bits) -> torch.Tensor:
    return torch.from_numpy(np.array(bits, dtype=np.uint32).view(np.float32).copy())


def outlier_tensor(M: int, K: int, dtype=torch.bfloat16, seed: int = 0, frac: float = 1e-3, scale: float = 50.0):
    """~N(0,1) with a seeded `frac` of the entries multiplied by `scale` (the round-trip workload)."""
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(M, K, generator=g, dtype=torch.float32)
    E = M * K
    g1 = torch.Generator().manual_seed(seed + 1)
    n_out = int(E * frac)
    if n_out:
        pos = torch.randint(0, E, (n_out,), generator=g1)
        x.view(-1)[pos] *= scale
    return x.to(dtype)
