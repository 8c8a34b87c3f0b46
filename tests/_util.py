"""Helpers shared by the tests: torch <-> numpy bit views and seeded synthetic inputs."""
import numpy as np
import torch


def bits16(t: torch.Tensor) -> np.ndarray:
    """bf16 / fp16 torch tensor (any device) -> numpy uint16 bit patterns."""
    return t.detach().cpu().contiguous().view(torch.int16).numpy().view(np.uint16)


def from_bits16(a: np.ndarray, dtype=torch.bfloat16) -> torch.Tensor:
    return torch.from_numpy(np.ascontiguousarray(a).view(np.int16)).view(dtype)


def make_weight(N, K, seed=1234, std=0.02, dtype=torch.bfloat16, special=True):
    """Weights ~N(0, std) from a seed; `special` plants a constant group, a zero row and outliers."""
    g = torch.Generator().manual_seed(seed)
    w = (torch.randn(N, K, generator=g) * std).to(dtype)
    if special and N >= 8 and K >= 64:
        w[3, :32] = 0.0123        # constant group -> scale clamps to eps
        w[5, :] = 0               # all-zero row
        w[1, 7] = 1.5             # outlier
        w[2, 40] = -2.25
    return w


def make_act(M, K, seed=4321, dtype=torch.bfloat16):
    g = torch.Generator().manual_seed(seed)
    return torch.randn(M, K, generator=g).to(dtype)


def rel_l2(a, b):
    a = np.asarray(a, np.float64)
    b = np.asarray(b, np.float64)
    return float(np.linalg.norm(a - b) / max(np.linalg.norm(b), 1e-30))
