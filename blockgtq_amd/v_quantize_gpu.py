"""PolarQuant V quantizer: seeded Haar rotation + scalar codebook (host ctor).

Builds the per-head V tables the device encoder and the decode kernel read
(rotation, boundaries, centroids, fp16 LUT) and offers the plain-torch
quantize/dequantize pair for inspection.  The production encode path is
``bgtq_encode_v`` in the C ABI, not these torch methods.

Reference behaviour: blockgtq/v_quantize_gpu.py:19-166.
"""
import numpy as np
import torch

from .codebooks import haar_rotation, mc_lloyd_centroids


class PolarQuantGPU:
    """Seed-deterministic V quantizer; no calibration data needed."""

    def __init__(self, d: int, bit_width: int, seed: int = 42,
                 norm_correction: bool = True, device=None):
        self.d = d
        self.bit_width = bit_width
        self.n_centroids = 1 << bit_width
        self.norm_correction = norm_correction
        self.device = torch.device(device) if device is not None else torch.device('cpu')
        rot = haar_rotation(d, seed, zero_sign_fix=False)
        self.rotation = torch.from_numpy(rot.astype(np.float32)).to(self.device)
        cents = mc_lloyd_centroids(bit_width, d)
        self.centroids = torch.from_numpy(cents.astype(np.float32)).to(self.device)
        self.boundaries = torch.from_numpy(
            ((cents[:-1] + cents[1:]) / 2.0).astype(np.float32)).to(self.device)

    @torch.no_grad()
    def quantize(self, v: torch.Tensor):
        """(N, D) -> codes (N, D) uint8, raw L2 norms (N,) fp16."""
        single = v.dim() == 1
        x = (v.unsqueeze(0) if single else v).float()
        norms = x.norm(dim=1)
        y = (self.rotation @ (x / norms.clamp(min=1e-8).unsqueeze(1)).T).T
        codes = torch.searchsorted(self.boundaries, y.contiguous()).to(torch.uint8)
        norms = norms.to(torch.float16)
        return (codes.squeeze(0), norms.squeeze(0)) if single else (codes, norms)

    @torch.no_grad()
    def quantize_packed(self, v: torch.Tensor):
        from .v_packing import pack_v_codes
        codes, norms = self.quantize(v)
        return pack_v_codes(codes, self.bit_width), norms

    @torch.no_grad()
    def dequantize(self, codes: torch.Tensor, norms: torch.Tensor) -> torch.Tensor:
        single = codes.dim() == 1
        if single:
            codes, norms = codes.unsqueeze(0), norms.unsqueeze(0)
        y = self.centroids[codes.long()].float()
        if self.norm_correction:
            y = y / y.norm(dim=1, keepdim=True).clamp(min=1e-10)
        x = (self.rotation.T @ y.T).T * norms.float().unsqueeze(1)
        x = x.to(torch.float16)
        return x.squeeze(0) if single else x

    @property
    def v_lut(self) -> torch.Tensor:
        """Centroids as fp16, the table the attention kernel dequantises with."""
        return self.centroids.to(torch.float16)
