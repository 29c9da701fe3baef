"""Per-RoPE-block importance scores (host side).

``s_i = (E||q_i||^2 + E||k_i||^2) / 2`` with the expectation taken over
calibration samples; every query head of a GQA group counts as its own
sample.  Reference behaviour: blockgtq/freq_analysis.py:18-35.
"""
import torch


def compute_freq_importance_energy(q_blocks: torch.Tensor,
                                   k_blocks: torch.Tensor) -> torch.Tensor:
    """q_blocks: (Nq, n_blocks, 2), k_blocks: (Nk, n_blocks, 2) -> (n_blocks,)."""
    eq = q_blocks.square().sum(dim=-1).mean(dim=0)
    ek = k_blocks.square().sum(dim=-1).mean(dim=0)
    return (eq + ek) / 2
