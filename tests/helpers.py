"""Shared helpers of the test-suite: random TW plans and device plumbing."""
import numpy as np


def random_tiles(rng, K, N, G, k_keep=0.25, n_keep=1.0, empty_every=0, ragged=True):
    """A random tile table over tiles of G original columns."""
    tiles = []
    for t, c0 in enumerate(range(0, N, G)):
        w = min(G, N - c0)
        kt = int(round(K * k_keep))
        if ragged:
            kt = int(np.clip(kt + rng.integers(-kt // 3 - 1, kt // 3 + 2), 0, K))
        nt = int(np.clip(round(w * n_keep), 0, w))
        if empty_every and t % empty_every == empty_every - 1:
            kt = 0
        tiles.append(dict(
            col0=c0, width=w,
            kept_k=np.sort(rng.choice(K, size=kt, replace=False)).astype(np.int32),
            kept_n=np.sort(rng.choice(w, size=nt, replace=False)).astype(np.int32)))
    return tiles


def torch_dtype(dtype):
    import torch
    return torch.float16 if dtype == "f16" else torch.bfloat16


def to_device_bits(bits, shape):
    """uint16 bit patterns -> device int16 tensor (the engine only needs the bytes)."""
    import torch
    return torch.from_numpy(np.ascontiguousarray(bits).view(np.int16).reshape(shape)).cuda()


def from_device_bits(t):
    return t.cpu().numpy().view(np.uint16)
