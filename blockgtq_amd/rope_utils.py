"""RoPE helpers for the split-half layout (host side).

Block ``i`` of a ``head_dim``-wide vector is the coordinate pair
``(i, i + head_dim // 2)``.  Reference behaviour: blockgtq/rope_utils.py:10-101.
"""
import torch


def get_rope_frequencies(head_dim: int, rope_base: float = 10000.0) -> torch.Tensor:
    """theta_i = base ** (-2 i / head_dim), i = 0 .. head_dim/2 - 1."""
    idx = torch.arange(0, head_dim, 2, dtype=torch.float32)
    return 1.0 / (rope_base ** (idx / head_dim))


def decompose_freq_blocks(x: torch.Tensor, head_dim: int) -> torch.Tensor:
    """(..., head_dim) -> (..., head_dim/2, 2) with block i = (x[i], x[i+L])."""
    half = head_dim // 2
    return torch.stack([x[..., :half], x[..., half:]], dim=-1)


def compose_freq_blocks(blocks: torch.Tensor) -> torch.Tensor:
    """Inverse of :func:`decompose_freq_blocks`."""
    return torch.cat([blocks[..., 0], blocks[..., 1]], dim=-1)


def apply_rope_to_blocks(blocks: torch.Tensor, freqs: torch.Tensor,
                         positions: torch.Tensor) -> torch.Tensor:
    """Rotate every 2-D block by ``position * theta_i``."""
    ang = positions.unsqueeze(-1).float() * freqs.to(positions.device)
    c, s = torch.cos(ang), torch.sin(ang)
    a, b = blocks[..., 0], blocks[..., 1]
    return torch.stack([a * c - b * s, a * s + b * c], dim=-1)


def undo_rope_from_blocks(blocks_rot: torch.Tensor, freqs: torch.Tensor,
                          positions: torch.Tensor) -> torch.Tensor:
    return apply_rope_to_blocks(blocks_rot, freqs, -positions)


def compute_rope_kernel(q_blocks: torch.Tensor, k_blocks: torch.Tensor,
                        freqs: torch.Tensor, delta: torch.Tensor) -> torch.Tensor:
    """q^T R_delta k summed over all blocks."""
    return (q_blocks * apply_rope_to_blocks(k_blocks, freqs, delta)).sum(dim=(-2, -1))


def select_freq_dims(selected_indices: torch.Tensor, head_dim: int) -> torch.Tensor:
    """Coordinate indices (sorted) covered by the given block indices."""
    half = head_dim // 2
    return torch.sort(torch.cat([selected_indices, selected_indices + half]))[0]


def apply_rope(x: torch.Tensor, positions: torch.Tensor,
               rope_base: float) -> torch.Tensor:
    """Split-half RoPE on (..., T, head_dim) at integer ``positions`` (T,)."""
    hd = x.shape[-1]
    blocks = decompose_freq_blocks(x.float(), hd)
    pos = positions.to(x.device)
    pos = pos.reshape((1,) * (blocks.dim() - 3) + (-1,)).expand(blocks.shape[:-2])
    rot = apply_rope_to_blocks(blocks, get_rope_frequencies(hd, rope_base), pos)
    return compose_freq_blocks(rot)
