"""Per-head K quantisation plan: allocation -> permutation, groups, rotation, codebooks.

Host-side only.  ``BlockGTQPipeline`` turns calibration activations of one KV
head into the static tensors every kernel of the packed path consumes:

  * ``bit_allocation`` (n_blocks,) int64 - bits per RoPE block,
  * ``_head_perm`` (D,) - coordinates ordered by ascending bit width, the two
    coordinates of a block adjacent,
  * one group per distinct bit width (contiguous in ``_head_perm`` order) with
    its own rotation (identity below ``rotation_threshold``, Haar above) and
    Lloyd-Max codebook for N(0, 1/group_dim),
  * ``_block_rot_T`` (D, D) block-diagonal rotation, transposed,
  * ``_pos_centroids`` / ``_pos_boundaries`` per-coordinate codebooks.

Blocks that received 0 bits (possible only when ``min_bits == 0``) sit at the
front of ``_head_perm``; they belong to no group (``_group_of == -1``), occupy
no bytes in the packed record, own no norm and reconstruct to zero.  The
reference cannot represent them (its codebook builder indexes an empty array).

Reference behaviour: blockgtq/block_gtq_pipeline.py:95-246.
"""
from typing import Optional

import torch

from .allocator import greedy_bit_allocation
from .codebooks import haar_rotation, lloyd_max_centroids
from .freq_analysis import compute_freq_importance_energy
from .rope_utils import decompose_freq_blocks, get_rope_frequencies


class BlockGTQPipeline:
    """Calibrated K-side plan of one KV head (no device kernels in here)."""

    def __init__(self, head_dim: int, avg_bits: float = 3.0,
                 rotation_threshold: int = 3,
                 min_bits: int = 1, max_bits: int = 8,
                 rope_base: float = 1e6,
                 device: Optional[torch.device] = None,
                 verbose: bool = False):
        self.head_dim = head_dim
        self.n_freqs = head_dim // 2
        self.avg_bits = avg_bits
        self.rotation_threshold = rotation_threshold
        self.min_bits = min_bits
        self.max_bits = max_bits
        self.rope_base = rope_base
        self.device = torch.device(device) if device is not None else torch.device('cpu')
        self.verbose = verbose
        self._calibrated = False
        self._perm_baked = False
        self.bit_allocation = None
        self.freqs = get_rope_frequencies(head_dim, rope_base)

    # ------------------------------------------------------------------
    def calibrate(self, q_data: torch.Tensor, k_data: torch.Tensor):
        """q_data: (Nq, D), k_data: (Nk, D) activations of this KV head."""
        scores = compute_freq_importance_energy(
            decompose_freq_blocks(q_data, self.head_dim),
            decompose_freq_blocks(k_data, self.head_dim))
        budget = int(self.n_freqs * self.avg_bits)
        self._calib_scores = scores
        self.set_allocation(greedy_bit_allocation(
            scores, budget, self.min_bits, self.max_bits))

    def set_allocation(self, bit_allocation: torch.Tensor):
        """Install a bit allocation directly and rebuild every derived tensor."""
        self.bit_allocation = bit_allocation.detach().cpu().long()
        self._post_allocation_setup()

    # ------------------------------------------------------------------
    def _post_allocation_setup(self, summary: str = "BlockGTQ"):
        L, hd, rt = self.n_freqs, self.head_dim, self.rotation_threshold
        dev = self.device
        bits = self.bit_allocation

        # torch's default (unstable) argsort decides the order of equal-width
        # blocks, exactly as in the reference.
        order = bits.argsort()
        bits_sorted = bits[order]

        head_perm = torch.empty(hd, dtype=torch.long)
        head_perm[0::2] = order
        head_perm[1::2] = order + L
        inv_perm = torch.empty_like(head_perm)
        inv_perm[head_perm] = torch.arange(hd)
        self._head_perm = head_perm.to(dev)
        self._head_perm_inv = inv_perm.to(dev)

        widths = sorted(int(b) for b in bits_sorted.unique().tolist() if int(b) > 0)
        n_zero = int((bits_sorted == 0).sum().item()) * 2
        self._n_zero_dims = n_zero

        block_rot = torch.zeros(hd, hd, dtype=torch.float32)
        slices, off = [], n_zero
        for bw in widths:
            d_bw = int((bits_sorted == bw).sum().item()) * 2
            s, e = off, off + d_bw
            slices.append((s, e))
            if bw < rt:
                block_rot[s:e, s:e] = torch.eye(d_bw)
            else:
                block_rot[s:e, s:e] = torch.tensor(
                    haar_rotation(d_bw, 42 + bw), dtype=torch.float32)
            off = e
        self._group_slices = slices
        self._group_bits = widths
        self._n_groups = len(slices)
        self._single_group = (self._n_groups == 1 and n_zero == 0)

        self._block_rot_T = block_rot.T.contiguous().to(dev)
        self._block_rot_unperm = block_rot[:, inv_perm].contiguous().to(dev)

        max_nc = max([1 << bw for bw in widths] + [2])
        pos_b = torch.full((hd, max_nc - 1), float('inf'), dtype=torch.float32)
        pos_c = torch.zeros((hd, max_nc), dtype=torch.float32)
        group_of = torch.full((hd,), -1, dtype=torch.long)
        group_mask = torch.zeros(hd, max(self._n_groups, 1), dtype=torch.float32)
        for gi, ((s, e), bw) in enumerate(zip(slices, widths)):
            c = torch.tensor(lloyd_max_centroids(bw, e - s), dtype=torch.float32)
            b = (c[:-1] + c[1:]) / 2.0
            pos_b[s:e, :b.numel()] = b
            pos_c[s:e, :c.numel()] = c
            group_of[s:e] = gi
            group_mask[s:e, gi] = 1.0
        self._pos_boundaries = pos_b.to(dev)
        self._pos_centroids = pos_c.to(dev)
        self._group_of = group_of.to(dev)
        self._group_mask = group_mask.to(dev)
        self._row_idx = torch.arange(hd, device=dev).unsqueeze(1)
        self._calibrated = True

        if self.verbose:
            from collections import Counter
            dist = dict(sorted(Counter(bits.tolist()).items()))
            print(f"  {summary}: eff={self.effective_bits_per_dim:.2f}b/d, "
                  f"grps={self._n_groups}, dist={dist}")

    @property
    def effective_bits_per_dim(self):
        if self.bit_allocation is None:
            return self.avg_bits
        return self.bit_allocation.float().sum().item() / self.n_freqs

    @torch.no_grad()
    def bake_permutation_into_kproj(self, k_proj_weight: torch.Tensor,
                                    kv_head_idx: int, n_kv_heads: int,
                                    k_proj_bias: Optional[torch.Tensor] = None) -> None:
        """Reorder the rows of this head's ``k_proj`` slice into ``_head_perm``
        order in place (blockgtq/block_gtq_pipeline.py:255-306)."""
        assert self._calibrated, "calibrate() must be called before baking"
        assert kv_head_idx < n_kv_heads
        hd = self.head_dim
        assert k_proj_weight.shape[0] == n_kv_heads * hd
        perm = self._head_perm.detach().cpu()
        lo, hi = kv_head_idx * hd, (kv_head_idx + 1) * hd
        k_proj_weight[lo:hi] = k_proj_weight[lo:hi].clone()[perm]
        if k_proj_bias is not None:
            k_proj_bias[lo:hi] = k_proj_bias[lo:hi].clone()[perm]
        self._perm_baked = True

    @torch.no_grad()
    def compress_decompress(self, k: torch.Tensor) -> torch.Tensor:
        """Quantise-then-reconstruct ``k`` (..., D) in plain torch on ``k``'s
        plan device: permute, per-group norm, rotate, nearest centroid,
        renormalise the reconstruction per group, undo rotation and permutation
        (blockgtq/block_gtq_pipeline.py:309-357).  Coordinates of 0-bit blocks
        come back as 0, and so does a group whose input norm is 0 (as in the
        packed record, which stores that norm; the reference's multi-group
        branch rescales such a group by 1 instead)."""
        assert self._calibrated
        hd = self.head_dim
        x = k.reshape(-1, hd).float()
        if not self._perm_baked:
            x = x[:, self._head_perm]
        live = (self._group_of >= 0)
        gidx = self._group_of.clamp(min=0)
        norms_g = torch.sqrt((x * x) @ self._group_mask)
        safe_g = torch.where(norms_g > 0, norms_g, torch.ones_like(norms_g))
        per_pos = safe_g[:, gidx]
        y = (x / per_pos) @ self._block_rot_T
        idx_t = torch.searchsorted(self._pos_boundaries, y.T.contiguous())
        idx_t = idx_t.clamp(max=self._pos_centroids.shape[1] - 1)
        y_hat = self._pos_centroids[self._row_idx, idx_t].T.contiguous()
        yh_g = torch.sqrt((y_hat * y_hat) @ self._group_mask)
        yh_safe = torch.where(yh_g > 1e-10, yh_g, torch.ones_like(yh_g))
        y_hat = y_hat / yh_safe[:, gidx] * norms_g[:, gidx] * live
        return (y_hat @ self._block_rot_unperm).reshape(*k.shape[:-1], hd)
