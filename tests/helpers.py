"""Shared input builders for the tests: the five BASELINE configurations at
reduced or full size, always from fixed numpy seeds (no torch RNG, so CPU and
GPU boxes build identical tensors)."""
import numpy as np


def logits_uniform(B, V, seed=0):
    """C1: i.i.d. U[0,1) (reference example.py:29)."""
    return np.random.default_rng(seed).random((B, V), dtype=np.float32)


def logits_normal(B, V, sigma, seed=0):
    return (np.random.default_rng(seed).standard_normal((B, V), dtype=np.float32) * np.float32(sigma)).astype(np.float32)


def logits_spiked(B, V, sigma=2.0, n_spikes=16, boost=10.0, seed=0):
    """C3: N(0, sigma) plus +boost on n_spikes random ids per row."""
    rng = np.random.default_rng(seed)
    x = (rng.standard_normal((B, V), dtype=np.float32) * np.float32(sigma)).astype(np.float32)
    for b in range(B):
        ids = rng.choice(V, size=n_spikes, replace=False)
        x[b, ids] += np.float32(boost)
    return x


def penalties_sparse(B, V, frac=0.02, seed=1):
    """C4: 2 % of entries Exp(1), the rest exactly 0."""
    rng = np.random.default_rng(seed)
    p = np.zeros((B, V), dtype=np.float32)
    mask = rng.random((B, V)) < frac
    p[mask] = rng.exponential(1.0, size=int(mask.sum())).astype(np.float32)
    return p


def uniforms(B, seed=2):
    """Injected per-row uniforms in (0, 1]."""
    u = np.random.default_rng(seed).random(B, dtype=np.float32)
    return (np.float32(1.0) - u).astype(np.float32)
