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


def rand_field_dev(shape, seed):
    """The same distribution drawn on the device (for shapes too large to draw on the host): 64 random bits,
    the 2^32 - 1 words at or above p taken down by p."""
    g = torch.Generator(device="cuda").manual_seed(seed)
    v = torch.randint(-(1 << 63), (1 << 63) - 1, shape, generator=g, dtype=torch.int64, device="cuda")
    v = torch.where((v < 0) & (v >= -((1 << 32) - 1)), v + ((1 << 32) - 1), v)     # [p, 2^64) as signed words
    return v.view(torch.uint64)


def to_dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def to_np(t):
    return t.cpu().numpy()


def unhex(v):
    return np.array([int(x, 16) for x in v], dtype=np.uint64)
