"""TurboQuant-MSE: seeded Haar rotation + Lloyd-Max scalar codebook, plain torch.

The uniform-width quantizer the unaccelerated path uses for V.  It shares the
analytic Lloyd-Max codebook and the rotation builder with the K-side pipeline
and runs on whatever device its tensors live on; it is not part of the packed
path (that one stores V with ``PolarQuantGPU`` tables through the C ABI).

Reference behaviour: blockgtq/tq.py:104-250.
"""
from typing import Optional

import torch

from .codebooks import haar_rotation, lloyd_max_centroids


class TurboQuantMSE:
    """Round-trip ``x -> ||x|| * R^T renorm(centroids[searchsorted(R x/||x||)])``."""

    def __init__(self, d: int, bit_width: int, seed: int = 42,
                 norm_correction: bool = True,
                 device: Optional[torch.device] = None):
        self.d = d
        self.bit_width = bit_width
        self.n_centroids = 1 << bit_width
        self.norm_correction = norm_correction
        self.device = torch.device(device) if device is not None else torch.device('cpu')
        self.rotation = torch.tensor(haar_rotation(d, seed), dtype=torch.float32,
                                     device=self.device)
        self.rotation_T = self.rotation.T.contiguous()
        self.centroids = torch.tensor(lloyd_max_centroids(bit_width, d),
                                      dtype=torch.float32, device=self.device)
        self.boundaries = (self.centroids[:-1] + self.centroids[1:]) / 2.0

    @torch.no_grad()
    def quantize(self, x: torch.Tensor):
        """(N, d) or (d,) -> (codes int64 of the same shape, raw L2 norms)."""
        single = x.ndim == 1
        x2 = x.unsqueeze(0) if single else x
        norms = torch.norm(x2, dim=1)
        safe = torch.where(norms > 0, norms, torch.ones_like(norms))
        y = (x2 / safe.unsqueeze(1)) @ self.rotation_T
        codes = torch.searchsorted(self.boundaries, y.contiguous())
        return (codes.squeeze(0), norms.squeeze(0)) if single else (codes, norms)

    @torch.no_grad()
    def dequantize(self, codes: torch.Tensor, norms: torch.Tensor) -> torch.Tensor:
        single = codes.ndim == 1
        if single:
            codes, norms = codes.unsqueeze(0), norms.unsqueeze(0)
        y = self.centroids[codes]
        if self.norm_correction:
            n = torch.norm(y, dim=1, keepdim=True)
            y = y / torch.where(n > 1e-10, n, torch.ones_like(n))
        x = (y @ self.rotation) * norms.unsqueeze(1)
        return x.squeeze(0) if single else x

    @torch.no_grad()
    def quantize_dequantize(self, x: torch.Tensor) -> torch.Tensor:
        return self.dequantize(*self.quantize(x))

    compress_decompress = quantize_dequantize


__all__ = ["TurboQuantMSE"]
