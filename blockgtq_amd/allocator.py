"""Greedy integer bit allocation over RoPE 2-D blocks (host side).

Minimises ``sum_i s_i * 4**(-b_i)`` subject to ``sum_i b_i == budget`` and
``min_bits <= b_i <= max_bits`` by handing out one bit at a time to the block
with the largest current term.  The objective is separable and convex in each
``b_i`` so the greedy schedule is the exact optimum; ties go to the lowest
block index.

Reference behaviour: blockgtq/allocator.py:20-55 (float64 priorities computed
from float32 scores, ``np.argmax`` tie-break, early stop when the best
priority is not positive).
"""
import numpy as np
import torch


def greedy_bit_allocation(scores: torch.Tensor, total_budget: int,
                          min_bits: int = 1, max_bits: int = 8) -> torch.Tensor:
    """Return an int64 tensor of per-block bit widths.

    ``scores`` is a 1-D tensor of non-negative importances.  If the budget
    cannot be spent (every block saturated at ``max_bits`` or every remaining
    score non-positive) the allocation simply stops early.
    """
    s = scores.detach().cpu().float().numpy().astype(np.float64)
    n = s.shape[0]
    bits = np.full(n, int(min_bits), dtype=np.int64)
    left = int(total_budget) - int(bits.sum())
    if left <= 0:
        return torch.from_numpy(bits)

    # 4**(-b) is a power of two, so s * 4**(-b) is exact in float64 and the
    # incremental update below reproduces a full recomputation bit for bit.
    prio = s * np.power(4.0, -bits.astype(np.float64))
    prio[bits >= max_bits] = -1.0
    while left > 0:
        i = int(np.argmax(prio))
        if prio[i] <= 0:
            break
        bits[i] += 1
        left -= 1
        prio[i] = -1.0 if bits[i] >= max_bits else s[i] * 4.0 ** (-float(bits[i]))
    return torch.from_numpy(bits)
