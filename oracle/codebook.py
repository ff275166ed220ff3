"""Lloyd-Max scalar codebooks for N(0,1) (oracle; test infrastructure only).

Follows turboquant_utils/codebook.py:18-100 of the reference: 200 Lloyd
iterations started from a uniform split of [-3.5, 3.5], centroids are the
conditional means of the standard normal over each cell, interior boundaries
are midpoints of neighbouring centroids.
"""

from __future__ import annotations

import functools

import numpy as np
import torch


def lloyd_max_gaussian(n_levels: int, n_iters: int = 200):
    """Return (centroids[n_levels], edges[n_levels+1]) as float64 arrays.

    Reference: turboquant_utils/codebook.py:18-68.  The outer edges are the
    +-1e10 stand-ins for infinity used there; a cell whose mass is below 1e-15
    falls back to the midpoint of its clipped extent.
    """
    from scipy.stats import norm

    edges = np.linspace(-3.5, 3.5, n_levels + 1)
    edges[0], edges[-1] = -1e10, 1e10
    cents = np.zeros(n_levels)
    for _ in range(n_iters):
        for i in range(n_levels):
            a, b = edges[i], edges[i + 1]
            mass = norm.cdf(b) - norm.cdf(a)
            if mass > 1e-15:
                cents[i] = (norm.pdf(a) - norm.pdf(b)) / mass
            else:
                cents[i] = 0.5 * (max(a, -3.5) + min(b, 3.5))
        for i in range(1, n_levels):
            edges[i] = 0.5 * (cents[i - 1] + cents[i])
    return cents, edges


@functools.lru_cache(maxsize=None)
def _cached(bit_width: int):
    cents, edges = lloyd_max_gaussian(2 ** bit_width)
    return (torch.tensor(cents, dtype=torch.float32),
            torch.tensor(edges[1:-1], dtype=torch.float32))


def get_codebook(bit_width: int):
    """(centroids fp32 [2^bit], interior boundaries fp32 [2^bit - 1]).

    Reference: turboquant_utils/codebook.py:77-100.
    """
    c, b = _cached(int(bit_width))
    return c.clone(), b.clone()


def uniform_codebook_8bit():
    """Uniform 256-level grid used by the 8-bit WxA8 attention/shared linears.

    Reference: turboquant_utils/quantize.py:398-408: cb[i] = (i-128)*3.5/128,
    boundaries (i-127.5)*3.5/128.
    """
    step = 3.5 / 128.0
    cents = (torch.arange(256, dtype=torch.float32) - 128) * step
    bounds = (torch.arange(255, dtype=torch.float32) - 127.5) * step
    return cents, bounds
