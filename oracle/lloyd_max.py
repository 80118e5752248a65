"""Independent statement of what a Lloyd-Max quantiser of N(0,1) must satisfy (test infrastructure only).

Nothing here generates the product's tables; these functions *check* tables by numerical integration
(scipy.integrate.quad) and hold the textbook values (J. Max, "Quantizing for minimum distortion", IRE Trans.
Inf. Theory 6(1), 1960, Table I) the product's tables are compared against.
"""
import math

import numpy as np
from scipy import integrate

# Positive output levels of the minimum-MSE quantiser of a unit Gaussian (Max 1960, Table I).
TEXTBOOK_LEVELS = {
    1: [0.7980],
    2: [0.4528, 1.510],
    3: [0.2451, 0.7560, 1.344, 2.152],
    4: [0.1284, 0.3881, 0.6568, 0.9424, 1.256, 1.618, 2.069, 2.733],
}
# Mean squared error of those quantisers (same table).
TEXTBOOK_MSE = {1: 0.3634, 2: 0.1175, 3: 0.03454, 4: 0.009497}


def _pdf(x):
    return math.exp(-0.5 * x * x) / math.sqrt(2.0 * math.pi)


def conditional_mean(a, b):
    """E[x | a < x < b] for x ~ N(0,1), by quadrature."""
    num, _ = integrate.quad(lambda x: x * _pdf(x), a, b, epsabs=1e-13, epsrel=1e-13)
    den, _ = integrate.quad(_pdf, a, b, epsabs=1e-13, epsrel=1e-13)
    return num / den


def cell_mass(a, b):
    den, _ = integrate.quad(_pdf, a, b, epsabs=1e-13, epsrel=1e-13)
    return den


def quantiser_mse(bounds, recon):
    """E[(x - Q(x))^2] for thresholds `bounds` and one reconstruction level per cell."""
    edges = [-np.inf] + list(bounds) + [np.inf]
    total = 0.0
    for k, r in enumerate(recon):
        v, _ = integrate.quad(lambda x: (x - r) ** 2 * _pdf(x), edges[k], edges[k + 1], epsabs=1e-13, epsrel=1e-13)
        total += v
    return total


def brute_force_codes(u, levels):
    """Nearest-centroid index per element (ties to the higher index, as `u >= midpoint` does)."""
    u = np.asarray(u, dtype=np.float64)
    levels = np.asarray(levels, dtype=np.float64)
    dist = np.abs(u[..., None] - levels)
    # argmin picks the lowest index on exact ties; flip to prefer the higher one
    rev = np.argmin(dist[..., ::-1], axis=-1)
    return (len(levels) - 1 - rev).astype(np.uint8)
