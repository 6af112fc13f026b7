"""Helpers shared by the GPU parity tests."""
import numpy as np
import torch


def dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def host(t):
    return t.detach().cpu().numpy()


def sc(v):
    """A 1-element device scale tensor."""
    return torch.tensor([float(v)], dtype=torch.float32, device="cuda")


def rand_graph(rng, n, e):
    return rng.integers(0, n, e).astype(np.int64), rng.integers(0, n, e).astype(np.int64)


def powerlaw_graph(rng, n, e, a=1.3):
    """Skewed multigraph: a few hubs with thousands of edges, many leaves."""
    w = 1.0 / np.arange(1, n + 1) ** a
    w /= w.sum()
    return (rng.choice(n, e, p=w).astype(np.int64), rng.choice(n, e, p=w).astype(np.int64))
