"""V-side packing format helpers (host side, pure torch, any device).

Format of one V record (same per-width rules as a K segment): the codes of all
``D`` dims form one LSB-first stream of ``bits``-bit fields; for 3 bits that is
8 codes per 3-byte group.  Reference behaviour: blockgtq/v_packing.py:17-175.
"""
import torch


def packed_v_bytes(D: int, bits: int) -> int:
    """Bytes per token of a V record with ``bits`` per code."""
    if bits == 1:
        return (D + 7) // 8
    if bits == 2:
        return (D + 3) // 4
    if bits == 3:
        return ((D + 7) // 8) * 3
    if bits == 4:
        return (D + 1) // 2
    raise ValueError(f"V packing supports 1-4 bits, got {bits}")


def pack_v_codes(codes: torch.Tensor, bits: int) -> torch.Tensor:
    """(..., D) uint8 codes -> (..., packed_v_bytes) uint8 records.

    Written as a bit-matrix scatter: code ``d`` contributes bit ``k`` to stream
    bit ``d*bits + k``; stream bit ``s`` lands in byte ``s // 8`` at ``s % 8``.
    """
    shape = codes.shape
    D = shape[-1]
    nb = packed_v_bytes(D, bits)
    flat = codes.reshape(-1, D).to(torch.int64)
    dev = codes.device
    k = torch.arange(bits, device=dev)
    bitvals = (flat.unsqueeze(-1) >> k) & 1                      # (N, D, bits)
    stream = bitvals.reshape(flat.shape[0], D * bits)
    pad = nb * 8 - D * bits
    if pad:
        stream = torch.cat([stream, stream.new_zeros(flat.shape[0], pad)], dim=1)
    weights = (1 << torch.arange(8, device=dev)).to(torch.int64)
    out = (stream.reshape(flat.shape[0], nb, 8) * weights).sum(dim=-1)
    return out.to(torch.uint8).reshape(*shape[:-1], nb)


def unpack_v_codes(packed: torch.Tensor, bits: int, D: int) -> torch.Tensor:
    """Inverse of :func:`pack_v_codes` via the per-dim two-byte window rule."""
    lo_b, hi_b, sh_lo, sh_hi, mask = build_v_unpack_tables(bits, D, device=packed.device)
    p = packed.to(torch.int32)
    lo = p[..., lo_b.long()]
    hi = p[..., hi_b.long()]
    return (((lo >> sh_lo) | (hi << sh_hi)) & mask).to(torch.uint8)


def build_v_unpack_tables(bits: int, D: int, device=None):
    """Per-dim tables such that
    ``code[d] = ((rec[byte_lo[d]] >> shift_lo[d]) | (rec[byte_hi[d]] << shift_hi[d])) & mask[d]``.

    A code that does not straddle a byte has ``byte_hi == byte_lo`` and
    ``shift_hi == 8`` so the high byte contributes nothing under the mask.
    """
    d = torch.arange(D, dtype=torch.int32)
    start = d * bits
    byte_lo = start // 8
    sh_lo = start % 8
    crosses = (sh_lo + bits) > 8
    byte_hi = torch.where(crosses, byte_lo + 1, byte_lo)
    sh_hi = torch.where(crosses, 8 - sh_lo, torch.full_like(sh_lo, 8))
    mask = torch.full((D,), (1 << bits) - 1, dtype=torch.int32)
    out = (byte_lo, byte_hi, sh_lo, sh_hi, mask)
    if device is not None:
        out = tuple(t.to(device) for t in out)
    return out
