"""Shared builders for the test-suite: seeded heads, plans and synthetic caches."""
import numpy as np
import torch

from blockgtq_amd import BlockGTQQuantizer, greedy_bit_allocation
from blockgtq_amd import synthetic as syn


def make_quantizer(seed=0, budget=192, min_bits=1, max_bits=5, v_bits=3, head=0,
                   device='cpu', rotation_threshold=2, alloc=None):
    """One calibrated head.  The allocation comes from the greedy allocator on
    log-uniform block energies unless given explicitly."""
    gen = torch.Generator().manual_seed(seed)
    energies = syn.block_energies(1, 64, gen)
    if alloc is None:
        alloc = greedy_bit_allocation(2.0 * energies[0], budget, min_bits, max_bits)
    q = BlockGTQQuantizer(128, rotation_threshold=rotation_threshold, device=device)
    q.calibrate_from_allocation(torch.as_tensor(alloc, dtype=torch.long))
    q.init_v_quantizer(v_bits, seed=42 + head)
    return q, energies


def make_kv(energies, T, seed=1, rope_theta=5e5, student_t_nu=None, n_q=4):
    """fp16 numpy K (T,128), V (T,128), Q (n_q,128) for one head."""
    gen = torch.Generator().manual_seed(seed)
    k = syn.make_keys(1, T, 128, energies, rope_theta, gen, student_t_nu=student_t_nu)[0]
    v = syn.make_values(1, T, 128, gen, student_t_nu=student_t_nu)[0]
    q = syn.make_queries(n_q, 128, rope_theta, T, gen)
    return (k.half().numpy(), v.half().numpy(), q.half().numpy())


def stream_pack(codes, bw):
    """Independent LSB-first bit-stream writer: (N, L) codes -> (N, ceil(L*bw/8)) bytes."""
    codes = np.asarray(codes, dtype=np.uint64)
    N, L = codes.shape
    nbytes = (L * bw + 7) // 8
    out = np.zeros((N, nbytes), dtype=np.uint8)
    for r in range(N):
        acc = 0
        for i in range(L):
            acc |= (int(codes[r, i]) & ((1 << bw) - 1)) << (i * bw)
        out[r] = np.frombuffer(acc.to_bytes(nbytes, 'little'), dtype=np.uint8)
    return out
