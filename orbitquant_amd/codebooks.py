"""Lloyd-Max scalar codebooks for one coordinate of a uniform point on S^(d-1).

Host-side constants of the quantized-linear forward: the HIP kernels receive the
`centroids` (2^b fp32) and `boundaries` (2^b - 1 fp32) tables built here.

Behaviour follows the reference's v2 generator
(src/orbitquant/codebooks/lloyd_max.py:385-448): the codebook is the Lloyd-Max
fixed point of the density f(z) ~ (1 - z^2)^((d-3)/2) on [-1, 1], it is solved
on the positive half in fp64 and mirrored, the boundaries are the fp64 midpoints
of neighbouring fp64 centroids, and both tables are cast to fp32 last
(lloyd_max.py:436-446).  `quantize_indices` is `#{j : boundaries[j] < v}` with
ties going to the lower code (lloyd_max.py:40-42).

`get_codebook` follows the reference's numerical recipe step for step (quantile
start by 96 bisections, Lloyd updates over-relaxed by 1.9 while the ordering
survives, stop when a plain update moves less than 1e-13, textbook Lentz
continued fraction with a 3e-14 stopping rule), because the reference stops
~1e-12 short of the true fixed point and an fp32 table is only reproduced bit for
bit by the same fp64 trajectory.  `solve_fixed_point_newton` is an independent
solver (Lloyd warm-up, then Newton on the tridiagonal fixed-point equations) used
to cross-check the tables; the two agree to the last fp32 bit except where an
fp64 value sits within that ~1e-12 of an fp32 rounding midpoint
(`rounding_margin`).
"""

from __future__ import annotations

import math
from dataclasses import dataclass
from functools import lru_cache

import torch

_TINY = 1e-300
_CF_TOL = 3e-14


def _betacf(a: float, b: float, x: float) -> float:
    """Continued fraction of the incomplete beta function (modified Lentz)."""
    front_c = 1.0
    front_d = 1.0 - (a + b) * x / (a + 1.0)
    front_d = 1.0 / (front_d if abs(front_d) > _TINY else _TINY)
    value = front_d
    for m in range(1, 20000):
        two_m = 2.0 * m
        # even step
        num = m * (b - m) * x / ((a + two_m - 1.0) * (a + two_m))
        front_d = 1.0 + num * front_d
        front_c = 1.0 + num / front_c
        front_d = 1.0 / (front_d if abs(front_d) > _TINY else _TINY)
        front_c = front_c if abs(front_c) > _TINY else _TINY
        value *= front_d * front_c
        # odd step
        num = -(a + m) * (a + b + m) * x / ((a + two_m) * (a + two_m + 1.0))
        front_d = 1.0 + num * front_d
        front_c = 1.0 + num / front_c
        front_d = 1.0 / (front_d if abs(front_d) > _TINY else _TINY)
        front_c = front_c if abs(front_c) > _TINY else _TINY
        step = front_d * front_c
        value *= step
        if abs(step - 1.0) < _CF_TOL:
            return value
    raise RuntimeError("incomplete beta continued fraction did not converge")


def _log_beta_prefactor(a: float, b: float, x: float) -> float:
    return (
        math.lgamma(a + b) - math.lgamma(a) - math.lgamma(b)
        + a * math.log(x) + b * math.log1p(-x)
    )


def _ibeta_pair(a: float, b: float, x: float) -> tuple[float, float]:
    """(I_x(a,b), 1 - I_x(a,b)), each computed without cancellation."""
    if x <= 0.0:
        return 0.0, 1.0
    if x >= 1.0:
        return 1.0, 0.0
    pref = math.exp(_log_beta_prefactor(a, b, x))
    if x < (a + 1.0) / (a + b + 2.0):
        lower = pref * _betacf(a, b, x) / a
        return lower, 1.0 - lower
    upper = pref * _betacf(b, a, 1.0 - x) / b
    return 1.0 - upper, upper


class _HalfSphereMarginal:
    """Mass / first moment / density of |z| for z a coordinate on S^(d-1)."""

    def __init__(self, dim: int) -> None:
        if dim < 3:
            raise ValueError("dim must be at least 3 for the Lloyd-Max solver")
        self.dim = dim
        self.b = (dim - 1) / 2.0
        self.log_c = (
            math.lgamma(dim / 2.0) - 0.5 * math.log(math.pi) - math.lgamma(self.b)
        )

    def density(self, z: float) -> float:
        if z >= 1.0:
            return 0.0
        return math.exp(self.log_c + (self.b - 1.0) * math.log1p(-z * z))

    def mass(self, left: float, right: float) -> float:
        """P(left < z < right) for the two-sided density (so half of |z|'s)."""
        lo_cdf, _ = _ibeta_pair(0.5, self.b, left * left)
        if right >= 1.0:
            tail, _ = _ibeta_pair(self.b, 0.5, 1.0 - left * left)
            return 0.5 * tail
        hi_cdf, _ = _ibeta_pair(0.5, self.b, right * right)
        return 0.5 * (hi_cdf - lo_cdf)

    def moment(self, left: float, right: float) -> float:
        """Integral of z f(z) over [left, right] = C [(1-l^2)^b - (1-r^2)^b] / (2b)."""
        log_l = self.b * math.log1p(-left * left) if left < 1.0 else -math.inf
        log_r = self.b * math.log1p(-right * right) if right < 1.0 else -math.inf
        if log_l == -math.inf:
            return 0.0
        diff = math.exp(log_l) * -math.expm1(log_r - log_l)
        return math.exp(self.log_c) * diff / (2.0 * self.b)

    def quantile(self, probability: float) -> float:
        lo, hi = 0.0, 1.0
        for _ in range(96):
            mid = 0.5 * (lo + hi)
            cdf, _ = _ibeta_pair(0.5, self.b, mid * mid)
            if cdf < probability:
                lo = mid
            else:
                hi = mid
        return 0.5 * (lo + hi)


def _edges_of(cents: list[float]) -> list[float]:
    return [0.0] + [0.5 * (cents[i] + cents[i + 1]) for i in range(len(cents) - 1)] + [1.0]


def _solve_tridiagonal(lower, diag, upper, rhs):
    n = len(diag)
    c = [0.0] * n
    d = [0.0] * n
    c[0] = upper[0] / diag[0]
    d[0] = rhs[0] / diag[0]
    for i in range(1, n):
        denom = diag[i] - lower[i] * c[i - 1]
        c[i] = upper[i] / denom if i < n - 1 else 0.0
        d[i] = (rhs[i] - lower[i] * d[i - 1]) / denom
    x = [0.0] * n
    x[-1] = d[-1]
    for i in range(n - 2, -1, -1):
        x[i] = d[i] - c[i] * x[i + 1]
    return x


def solve_positive_centroids(dim: int, bits: int) -> list[float]:
    """fp64 positive-half centroids by the reference's over-relaxed Lloyd iteration
    (src/orbitquant/codebooks/lloyd_max.py:385-434)."""
    if bits <= 0 or bits > 8:
        raise ValueError("bits must be in [1, 8]")
    marginal = _HalfSphereMarginal(dim)
    levels = 1 << bits
    half = levels // 2
    cents = [marginal.quantile((i + 0.5) / half) for i in range(half)]
    for _ in range(max(1024, 6 * levels * levels)):
        edges = _edges_of(cents)
        update = [
            marginal.moment(edges[i], edges[i + 1]) / marginal.mass(edges[i], edges[i + 1])
            for i in range(half)
        ]
        if max(abs(update[i] - cents[i]) for i in range(half)) < 1e-13:
            return update
        relaxed = [cents[i] + 1.9 * (update[i] - cents[i]) for i in range(half)]
        keeps_order = all(
            0.0 < relaxed[i] < (relaxed[i + 1] if i + 1 < half else 1.0) for i in range(half)
        )
        cents = relaxed if keeps_order else update
    raise RuntimeError(f"Lloyd-Max did not converge for dim={dim}, bits={bits}")


def solve_fixed_point_newton(dim: int, bits: int) -> list[float]:
    """fp64 positive-half Lloyd-Max fixed point to the fp64 noise floor."""
    if bits <= 0 or bits > 8:
        raise ValueError("bits must be in [1, 8]")
    marginal = _HalfSphereMarginal(dim)
    half = (1 << bits) // 2
    cents = [marginal.quantile((i + 0.5) / half) for i in range(half)]

    def lloyd_step(current):
        edges = _edges_of(current)
        masses = [marginal.mass(edges[i], edges[i + 1]) for i in range(half)]
        means = [marginal.moment(edges[i], edges[i + 1]) / masses[i] for i in range(half)]
        return edges, masses, means

    for _ in range(24):
        _, _, cents = lloyd_step(cents)

    previous_step = math.inf
    for _ in range(200):
        edges, masses, means = lloyd_step(cents)
        residual = [means[i] - cents[i] for i in range(half)]
        # d mean_i / d edge_i (left edge) and / d edge_{i+1} (right edge)
        lower = [0.0] * half
        diag = [0.0] * half
        upper = [0.0] * half
        for i in range(half):
            left, right = edges[i], edges[i + 1]
            d_left = marginal.density(left) * (means[i] - left) / masses[i] if i > 0 else 0.0
            d_right = (
                marginal.density(right) * (right - means[i]) / masses[i]
                if i < half - 1
                else 0.0
            )
            lower[i] = 0.5 * d_left
            upper[i] = 0.5 * d_right
            diag[i] = 0.5 * d_left + 0.5 * d_right - 1.0
        step = _solve_tridiagonal(lower, diag, upper, [-r for r in residual])
        trial = [cents[i] + step[i] for i in range(half)]
        ordered = all(
            0.0 < trial[i] < (trial[i + 1] if i + 1 < half else 1.0) for i in range(half)
        )
        if not ordered:
            cents = means  # plain Lloyd step keeps the ordering
            continue
        cents = trial
        # Newton converges quadratically: once a step is below 1e-12 the error
        # left after applying it is at the fp64 noise floor.  For many levels
        # the CDF differences that give the interval masses carry ~1e-12 of
        # cancellation noise, so a step that stops shrinking below 1e-10 is the
        # same floor.
        step_size = max(abs(s) for s in step)
        if step_size < 1e-12 or (step_size < 1e-10 and step_size > 0.25 * previous_step):
            break
        previous_step = step_size
    else:
        raise RuntimeError(f"Lloyd-Max Newton solve did not converge (dim={dim}, bits={bits})")
    return cents


@dataclass(frozen=True)
class LloydMaxCodebook:
    dim: int
    bits: int
    centroids: torch.Tensor
    boundaries: torch.Tensor
    algorithm_version: int = 2

    def quantize_indices(self, values: torch.Tensor) -> torch.Tensor:
        bounds = self.boundaries.to(device=values.device, dtype=values.dtype)
        return torch.bucketize(values, bounds).to(torch.uint8)

    def quantize(self, values: torch.Tensor) -> torch.Tensor:
        table = self.centroids.to(device=values.device, dtype=values.dtype)
        return table[self.quantize_indices(values).to(torch.long)]


def _tables_fp64(dim: int, bits: int, solver=None) -> tuple[torch.Tensor, torch.Tensor]:
    positive = (solver or solve_positive_centroids)(dim, bits)
    full = torch.tensor([-v for v in reversed(positive)] + positive, dtype=torch.float64)
    return full, (full[:-1] + full[1:]) / 2


def rounding_margin(dim: int, bits: int) -> float:
    """Smallest fp64 distance of any true-fixed-point entry to an fp32 rounding midpoint."""
    cents, bounds = _tables_fp64(dim, bits, solve_fixed_point_newton)
    worst = math.inf
    for value in torch.cat((cents, bounds)).tolist():
        if value == 0.0:
            continue
        as32 = torch.tensor(value, dtype=torch.float64).to(torch.float32)
        neighbour_up = torch.nextafter(as32, torch.tensor(math.inf, dtype=torch.float32))
        neighbour_dn = torch.nextafter(as32, torch.tensor(-math.inf, dtype=torch.float32))
        for neighbour in (neighbour_up, neighbour_dn):
            midpoint = (float(as32) + float(neighbour)) / 2.0
            worst = min(worst, abs(value - midpoint))
    return worst


@lru_cache(maxsize=256)
def get_codebook(dim: int, bits: int, algorithm_version: int = 2) -> LloydMaxCodebook:
    if algorithm_version != 2:
        raise ValueError("only the exact v2 Lloyd-Max codebook is implemented")
    cents, bounds = _tables_fp64(dim, bits)
    return LloydMaxCodebook(
        dim=dim,
        bits=bits,
        centroids=cents.to(torch.float32),
        boundaries=bounds.to(torch.float32),
        algorithm_version=2,
    )


def clear_codebook_cache() -> None:
    get_codebook.cache_clear()
