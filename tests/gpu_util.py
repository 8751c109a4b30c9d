"""Helpers shared by the GPU parity tests (imported only under -m gpu)."""
import numpy as np
import torch

P = (1 << 64) - (1 << 32) + 1


def rand_field(shape, seed):
    """Uniform canonical field elements as a numpy uint64 array."""
    rng = np.random.default_rng(seed)
    a = rng.integers(0, 1 << 63, size=shape, dtype=np.uint64) * np.uint64(2) \
        + rng.integers(0, 2, size=shape, dtype=np.uint64)
    return a % np.uint64(P)


def to_dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def to_np(t):
    return t.cpu().numpy()


def unhex(v):
    return np.array([int(x, 16) for x in v], dtype=np.uint64)
