"""Seeded synthetic K/V/Q tensors of the benchmark configurations.

Keys are N(0,1) (or Student-t) draws whose RoPE blocks are scaled by per-(head,
block) energies drawn log-uniformly, so the greedy allocator produces a
non-uniform bit allocation; RoPE is applied afterwards at the token positions.
Everything is generated on the CPU from ``torch.Generator().manual_seed(seed)``
and is therefore identical on every machine.
"""
import math

import torch

from .rope_utils import apply_rope


def block_energies(n_heads: int, n_blocks: int, gen: torch.Generator,
                   lo: float = 0.05, hi: float = 20.0) -> torch.Tensor:
    """(n_heads, n_blocks) energies, log-uniform in [lo, hi]."""
    u = torch.rand(n_heads, n_blocks, generator=gen)
    return torch.exp(math.log(lo) + u * (math.log(hi) - math.log(lo)))


def _draw(shape, gen, student_t_nu=None):
    z = torch.randn(shape, generator=gen)
    if student_t_nu is None:
        return z
    # t_nu = z / sqrt(chi2_nu / nu), chi2 as a sum of nu squared normals
    chi2 = torch.randn(shape + (int(student_t_nu),), generator=gen).square().sum(-1)
    return z / torch.sqrt(chi2 / student_t_nu)


def make_keys(n_heads: int, T: int, head_dim: int, energies: torch.Tensor,
              rope_theta: float, gen: torch.Generator, pos0: int = 0,
              student_t_nu=None) -> torch.Tensor:
    """(n_heads, T, head_dim) float32 post-RoPE keys with per-block energy scaling."""
    half = head_dim // 2
    k = _draw((n_heads, T, head_dim), gen, student_t_nu)
    amp = energies.sqrt()                                  # (n_heads, n_blocks)
    k = k * torch.cat([amp, amp], dim=-1).unsqueeze(1)
    assert amp.shape[-1] == half
    return apply_rope(k, torch.arange(pos0, pos0 + T), rope_theta)


def make_values(n_heads: int, T: int, head_dim: int, gen: torch.Generator,
                student_t_nu=None) -> torch.Tensor:
    return _draw((n_heads, T, head_dim), gen, student_t_nu)


def make_queries(n_heads: int, head_dim: int, rope_theta: float, position: int,
                 gen: torch.Generator) -> torch.Tensor:
    """(n_heads, head_dim) float32 queries with RoPE at ``position``."""
    q = torch.randn(n_heads, 1, head_dim, generator=gen)
    return apply_rope(q, torch.tensor([position]), rope_theta)[:, 0]


def energy_scores(energies_k: torch.Tensor, q_energy: float = 1.0) -> torch.Tensor:
    """Closed-form allocator scores of the synthetic distribution: every K block
    has E||k_i||^2 = 2 e_i, every Q block E||q_i||^2 = 2 q_energy."""
    return (2.0 * q_energy + 2.0 * energies_k) / 2.0
