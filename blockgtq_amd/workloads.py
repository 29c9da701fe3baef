"""Synthetic benchmark workloads: geometry, per-head calibration, cache filling.

A workload is a model geometry (layers, query/KV heads, RoPE base), a batch of
context lengths and a K/V bit budget.  ``build_manager`` calibrates one
quantizer per (layer, KV head) from seeded block energies and returns a
``BlockGTQKVManager``; ``fill_cache`` draws fp16 K/V on the device layer by
layer and pushes them through the quantise-and-pack kernels.
"""
from dataclasses import dataclass, field
from typing import List, Optional

import torch

from . import synthetic as syn
from .allocator import greedy_bit_allocation
from .packed_kv_manager import BlockGTQKVManager
from .quantizer import BlockGTQQuantizer
from .rope_utils import apply_rope


@dataclass
class Workload:
    name: str
    n_layers: int
    n_q: int
    n_kv: int
    batch: int
    context: int                      # tokens already in the cache (max over rows)
    rope_theta: float
    k_bits: float = 3.0
    v_bits: int = 3
    min_bits: int = 1
    max_bits: int = 8
    seq_lens: Optional[List[int]] = None
    student_t_nu: Optional[int] = None
    seed: int = 1234
    head_dim: int = 128
    n_sink: int = 0                   # with-buffer setting: fp16 sink tokens ...
    window: int = 0                   # ... and fp16 recent window next to the packed cache
    extra: dict = field(default_factory=dict)


WORKLOADS = {
    # Llama-3.1-8B head geometry, one layer, CPU-runnable
    "llama8b_4k_k3v3": Workload("llama8b_4k_k3v3", 1, 32, 8, 1, 4096, 5e5,
                                min_bits=1, max_bits=5, seed=1234),
    # Qwen2.5-3B geometry, the configuration the headline metric is quoted on
    "qwen3b_b8_32k_k3v3": Workload("qwen3b_b8_32k_k3v3", 36, 16, 2, 8, 32768, 1e6, seed=1235),
    # long-context split stress, K2V2 with 0-bit blocks, heavy tails
    "llama8b_128k_k2v2": Workload("llama8b_128k_k2v2", 1, 32, 8, 1, 131072, 5e5,
                                  k_bits=2.0, v_bits=2, min_bits=0, max_bits=4,
                                  student_t_nu=4, seed=1236),
}


def _ragged_lens(batch: int, lo: int, hi: int, seed: int) -> List[int]:
    gen = torch.Generator().manual_seed(seed)
    return [int(x) for x in torch.randint(lo, hi + 1, (batch,), generator=gen)]


# Qwen3-8B geometry, ragged batch in the with-buffer setting: K3V3 packed cache plus 4 fp16
# sink tokens and a 128-token fp16 recent window, one append per sequence per step
WORKLOADS["qwen3_8b_b32_ragged_buffered"] = Workload(
    "qwen3_8b_b32_ragged_buffered", 36, 32, 8, 32, 16384, 1e6, seed=1237,
    seq_lens=_ragged_lens(32, 1024, 16384, 1237), n_sink=4, window=128)


def calibrate_layer(w: Workload, layer: int, device):
    """Quantizers of one layer.  Scores are the closed-form block energies of the
    synthetic distribution (Q and K share the per-block scaling), so the
    allocation equals what calibration tensors drawn from it converge to."""
    gen = torch.Generator().manual_seed(w.seed * 1000 + layer)
    energies = syn.block_energies(w.n_kv, w.head_dim // 2, gen)
    budget = int((w.head_dim // 2) * w.k_bits)
    qs = []
    for h in range(w.n_kv):
        alloc = greedy_bit_allocation(2.0 * energies[h], budget, w.min_bits, w.max_bits)
        q8 = BlockGTQQuantizer(w.head_dim, avg_bits=w.k_bits, min_bits=w.min_bits,
                               max_bits=w.max_bits, device=device)
        q8.calibrate_from_allocation(alloc)
        q8.init_v_quantizer(w.v_bits, seed=42 + h)
        qs.append(q8)
    return qs, energies


def build_manager(w: Workload, device, max_T: Optional[int] = None, n_layers: Optional[int] = None):
    """Calibrated manager plus the per-layer block energies used to draw keys."""
    L = n_layers or w.n_layers
    mgr = BlockGTQKVManager(L, w.n_q, w.n_kv, w.head_dim, max_T or (w.context + 16),
                            batch_size=w.batch, k_avg_bits=w.k_bits, v_bits=w.v_bits,
                            device=device, min_bits=w.min_bits, max_bits=w.max_bits,
                            n_sink=w.n_sink, recent_window=w.window)
    energies = []
    for li in range(L):
        qs, e = calibrate_layer(w, li, device)
        mgr.set_quantizers(li, qs)
        energies.append(e)
    return mgr, energies


def draw_kv(w: Workload, energies: torch.Tensor, T: int, layer: int, device, pos0: int = 0):
    """fp16 K, V (B, n_kv, T, D) drawn on ``device`` (seeded per layer)."""
    dev = torch.device(device)
    gen = torch.Generator(device=dev).manual_seed(w.seed * 7919 + layer)
    shape = (w.batch, w.n_kv, T, w.head_dim)

    def draw():
        z = torch.randn(shape, generator=gen, device=dev)
        if w.student_t_nu:
            chi2 = torch.zeros(shape, device=dev)
            for _ in range(int(w.student_t_nu)):
                chi2 += torch.randn(shape, generator=gen, device=dev).square()
            z = z / torch.sqrt(chi2 / w.student_t_nu)
        return z

    amp = energies.sqrt().to(dev)
    k = draw() * torch.cat([amp, amp], dim=-1).view(1, w.n_kv, 1, w.head_dim)
    k = apply_rope(k, torch.arange(pos0, pos0 + T), w.rope_theta)
    v = draw()
    return k.half(), v.half()


def draw_q(w: Workload, layer: int, device, position: int):
    """fp16 queries (B, n_q, 1, D) with RoPE at ``position``."""
    dev = torch.device(device)
    gen = torch.Generator(device=dev).manual_seed(w.seed * 104729 + layer)
    q = torch.randn((w.batch, w.n_q, 1, w.head_dim), generator=gen, device=dev)
    return apply_rope(q, torch.tensor([position]), w.rope_theta).half()


def fill_cache(mgr: BlockGTQKVManager, w: Workload, energies, device, chunk: int = 8192):
    """Encode ``w.context`` synthetic tokens per row into every layer of ``mgr``."""
    if mgr.buffered:
        lens = w.seq_lens or [w.context] * w.batch
        for li in range(mgr.n_layers):
            k, v = draw_kv(w, energies[li], max(lens), li * 4096, device)
            mgr.fill_buffered(li, k, v, lens)
            del k, v
        mgr.set_seq_lens(lens)
        return
    for li in range(mgr.n_layers):
        for lo in range(0, w.context, chunk):
            n = min(chunk, w.context - lo)
            k, v = draw_kv(w, energies[li], n, li * 4096 + lo // chunk, device, pos0=lo)
            mgr._encode_kv(li, k, v, lo)
    if w.seq_lens is not None:
        mgr.set_seq_lens(w.seq_lens)
    else:
        mgr.seq_len = w.context


def algorithmic_bytes_per_layer(mgr: BlockGTQKVManager, layer: int, seq_lens, nibble: bool = False) -> int:
    """Bytes one decode-attention launch must read/write by construction: every
    visible token's own K record, its fp16 group norms, V record and V norm,
    plus the queries in and the outputs out.  ``nibble``: the records of the
    production cache's default layout (K as nibbles + raw bytes, V as nibbles)."""
    total = 0
    vb = mgr.hd // 2 if nibble else mgr._vpb
    plans = mgr._batched_args[layer]['plans_np']
    for T_b in seq_lens:
        fp16_rows = min(T_b, mgr.n_sink + mgr.window) if mgr.buffered else 0
        for hi, q8 in enumerate(mgr.quantizers[layer]):
            kb = int(plans[hi]['k_mixed_bytes']) if nibble else q8._total_packed_bytes
            total += (T_b - fp16_rows) * (kb + 2 * q8._n_groups + vb + 2)
            total += fp16_rows * mgr.hd * 2 * 2            # fp16 K and V rows of the buffer
    total += len(seq_lens) * mgr.n_q * mgr.hd * 2 * 2
    return total
