"""Seeded synthetic inputs shared by the parity tests (numpy on the host)."""
import numpy as np

F = np.float32


def counter_case(seed, n_out, n_in, C, g_sigma=0.01, full_range=False, oracle=None):
    """Random packed state, gradient, scale and RMS moment for one counter tensor."""
    rng = np.random.default_rng(seed)
    hi = 64 if full_range else 3 * (2 * C - 1)
    codes = rng.integers(0, hi, (n_out, n_in)).astype(np.uint8)
    G = (rng.standard_normal((n_out, n_in)) * g_sigma).astype(F)
    scale = np.full(n_out, np.sqrt(F(3.0) / (F(2.0) * F(n_in))), dtype=F) * (0.5 + rng.random(n_out)).astype(F)
    v = (rng.random(n_out) * g_sigma ** 2).astype(F)
    state = oracle.pack_codes(codes) if oracle is not None else None
    return codes, state, G, scale, v


def activations(seed, N, n_in, n_out, x_sigma=1.0, dy_sigma=0.01):
    rng = np.random.default_rng(seed)
    x = (rng.standard_normal((N, n_in)) * x_sigma).astype(F)
    dy = (rng.standard_normal((N, n_out)) * dy_sigma).astype(F)
    return x, dy
