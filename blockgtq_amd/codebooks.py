"""Scalar codebooks, Haar rotations and the 256-bin code LUT (host side).

Everything here runs once at calibration time on the CPU and only produces
small arrays (codebooks, rotations, look-up tables) that are uploaded to the
device inside the per-head plan.

Reference behaviour:
  * Lloyd-Max centroids for N(0, 1/d): blockgtq/block_gtq_pipeline.py:24-78
    (identical copy in blockgtq/tq.py:24-83).
  * Haar rotation by QR with positive diag(R):
    blockgtq/block_gtq_pipeline.py:81-92, blockgtq/v_quantize_gpu.py:19-29.
  * Monte-Carlo Lloyd centroids of the V quantizer:
    blockgtq/v_quantize_gpu.py:32-54.
  * 256-bin code LUT: blockgtq/kernels/quant_kernels.py:276-364.
"""
import functools
import math

import numpy as np
import torch

_TWO_BIT_LEVELS = np.array([-1.51, -0.453, 0.453, 1.51])


def lloyd_max_centroids(bit_width: int, d: int, iters: int = 100) -> np.ndarray:
    """Lloyd-Max levels of a N(0, 1/d) coordinate (memoised; see the cached body)."""
    return _lloyd_max_cached(int(bit_width), int(d), int(iters)).copy()


@functools.lru_cache(maxsize=None)
def _lloyd_max_cached(bit_width: int, d: int, iters: int) -> np.ndarray:
    """MSE-optimal scalar levels for a N(0, 1/d) coordinate, float64, sorted.

    ``bit_width == 1`` uses the closed form ``+-sqrt(2/(pi d))`` and
    ``bit_width == 2`` the tabulated ``[+-0.453, +-1.51]/sqrt(d)``; wider
    codebooks run ``iters`` Lloyd iterations on the analytic Gaussian,
    started from the conditional means of the equal-probability cells.
    """
    if bit_width < 1:
        raise ValueError("a codebook needs at least one bit")
    if bit_width == 1:
        c = math.sqrt(2.0 / (math.pi * d))
        return np.array([-c, c])
    if bit_width == 2:
        return _TWO_BIT_LEVELS / math.sqrt(d)

    from scipy.stats import norm

    n = 1 << bit_width
    sigma = 1.0 / math.sqrt(d)

    def cell_means(edges):
        # E[X | lo < X < hi], X ~ N(0, sigma^2), for the n cells cut by `edges`.
        # Evaluated cell by cell exactly like a scalar loop would (first cell
        # through the cdf, last through the survival function), just vectorised.
        lo = np.concatenate([[-np.inf], edges])
        hi = np.concatenate([edges, [np.inf]])
        a, b = lo / sigma, hi / sigma
        mass = norm.cdf(b) - norm.cdf(a)
        mass[0] = norm.cdf(b[0])
        mass[-1] = norm.sf(a[-1])
        with np.errstate(divide='ignore', invalid='ignore'):
            mean = sigma * (norm.pdf(a) - norm.pdf(b)) / mass
        empty = mass < 1e-15
        if empty.any():
            fallback = (lo + hi) / 2.0
            fallback[0] = hi[0] - sigma
            fallback[-1] = lo[-1] + sigma
            mean = np.where(empty, fallback, mean)
        return mean

    edges = norm.ppf(np.linspace(0, 1, n + 1)[1:-1], scale=sigma)
    cents = cell_means(edges)
    for _ in range(iters):
        cents = cell_means((cents[:-1] + cents[1:]) / 2.0)
    cents.sort()
    return cents


def haar_rotation(d: int, seed: int, zero_sign_fix: bool = True) -> np.ndarray:
    """Seeded (d, d) Haar rotation (memoised; see the cached body)."""
    return _haar_cached(int(d), int(seed), bool(zero_sign_fix)).copy()


@functools.lru_cache(maxsize=256)
def _haar_cached(d: int, seed: int, zero_sign_fix: bool) -> np.ndarray:
    """(d, d) float64 proper rotation drawn from ``default_rng(seed)``.

    QR of a standard-normal matrix; columns are flipped so diag(R) is
    positive (which makes the factorisation unique) and the first column is
    negated if the determinant came out negative.  ``zero_sign_fix`` maps a
    zero on diag(R) to +1 as the K-side builder does; the V-side builder
    leaves it at 0 (the two agree whenever diag(R) has no exact zero).
    """
    g = np.random.default_rng(seed).standard_normal((d, d))
    q, r = np.linalg.qr(g)
    sg = np.sign(np.diag(r))
    if zero_sign_fix:
        sg[sg == 0] = 1.0
    q = q * sg[np.newaxis, :]
    if zero_sign_fix:
        neg = np.linalg.slogdet(q)[0] < 0
    else:
        neg = np.linalg.det(q) < 0
    if neg:
        q[:, 0] = -q[:, 0]
    return q


def mc_lloyd_centroids(bit_width: int, d: int) -> np.ndarray:
    """V-side Monte-Carlo Lloyd levels (memoised; see the cached body)."""
    return _mc_lloyd_cached(int(bit_width), int(d)).copy()


@functools.lru_cache(maxsize=None)
def _mc_lloyd_cached(bit_width: int, d: int) -> np.ndarray:
    """V-side codebook: Lloyd on 100k samples of N(0, 1/d), float64, sorted.

    The sample set is redrawn from ``default_rng(0)`` on every iteration, so it
    is the same set each time and the procedure is deterministic.
    """
    n = 1 << bit_width
    if bit_width == 1:
        c = np.sqrt(2.0 / (np.pi * d))
        return np.array([-c, c])
    if bit_width == 2:
        return _TWO_BIT_LEVELS / np.sqrt(d)
    sigma = 1.0 / np.sqrt(d)
    cents = np.linspace(-3 * sigma, 3 * sigma, n)
    for _ in range(100):
        edges = (cents[:-1] + cents[1:]) / 2.0
        samples = np.random.default_rng(0).normal(0, sigma, 100000)
        cell = np.searchsorted(edges, samples)
        new = np.array([samples[cell == i].mean() if (cell == i).any() else cents[i]
                        for i in range(n)])
        if np.allclose(cents, new, atol=1e-8):
            break
        cents = new
    return np.sort(cents)


def build_code_lut(pos_centroids: torch.Tensor, pos_boundaries: torch.Tensor,
                   n_bins: int = 256):
    """256-bin uniform discretisation -> centroid index, one table per codebook.

    Args:
        pos_centroids: (D, max_nc) float32, row j = codebook of dim j (zero padded).
        pos_boundaries: (D, max_nc - 1) float32 midpoints, +inf padded.

    Returns ``(code_lut (n_cb, n_bins) uint8, pos_to_cb (D,) int32,
    offsets (D,) float32, inv_scales (D,) float32)``.  A coordinate ``y`` of
    dim ``j`` is coded as ``code_lut[pos_to_cb[j]][trunc(clamp((y - offsets[j])
    * inv_scales[j], 0, n_bins - 1))]``.  The table covers
    ``[c_min - sp/2, c_max + sp/2]`` with ``sp`` the mean centroid spacing, and
    bin ``i`` maps to the nearest centroid of its centre.
    """
    D = pos_centroids.shape[0]
    dev = pos_centroids.device
    cents_all = pos_centroids.detach().cpu()
    bounds_all = pos_boundaries.detach().cpu()

    offsets = torch.zeros(D, dtype=torch.float32)
    inv_scales = torch.zeros(D, dtype=torch.float32)
    pos_to_cb = torch.zeros(D, dtype=torch.int32)
    reps = []          # (dim, n_centroids) of the first dim using each codebook
    seen = {}

    def lut_range(c):
        lo, hi = c.min().item(), c.max().item()
        half = (hi - lo) / max(c.numel() - 1, 1) * 0.5
        return lo - half, hi + half

    for j in range(D):
        nb = int((bounds_all[j] < 1e30).sum().item())
        nc = max(nb + 1, 2)
        c = cents_all[j, :nc]
        lo, hi = lut_range(c)
        offsets[j] = lo
        # a dim that got 0 bits has an all-zero codebook row: no table, scale 0
        inv_scales[j] = 1.0 / ((hi - lo) / n_bins) if hi > lo else 0.0
        key = (nc, tuple(c.tolist()))
        if key not in seen:
            seen[key] = len(reps)
            reps.append((j, nc))
        pos_to_cb[j] = seen[key]

    code_lut = torch.zeros(len(reps), n_bins, dtype=torch.uint8)
    for cb, (j, nc) in enumerate(reps):
        c = cents_all[j, :nc]
        lo, hi = lut_range(c)
        w = (hi - lo) / n_bins
        centres = torch.linspace(lo + w / 2, hi - w / 2, n_bins, dtype=torch.float32)
        nb = int((bounds_all[j] < 1e30).sum().item())
        if nb > 0:
            idx = torch.searchsorted(bounds_all[j, :nb].contiguous(), centres).clamp(max=nc - 1)
        else:
            idx = (centres > (c[0] + c[1]) / 2.0).long()
        code_lut[cb] = idx.to(torch.uint8)

    return (code_lut.to(dev), pos_to_cb.to(dev), offsets.to(dev), inv_scales.to(dev))
