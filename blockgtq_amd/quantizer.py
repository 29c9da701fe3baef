"""Per-head Block-GTQ quantizer: host plan + device encode entry points.

``BlockGTQQuantizer`` keeps the public surface of the reference class
(blockgtq/quantizer.py:1000-1591): calibrate on the host, then quantise K/V on
the device.  All device work goes through the C ABI (include/bgtq.h); the
per-head static tables travel as one ``bgtq_head_plan``.

Module-level helpers mirror blockgtq/quantizer.py:34-102 (``build_pack_meta``)
and :1598-2172 (the batched multi-head encoders).
"""
from typing import Optional

import torch

from . import _capi, plan as _plan
from .codebooks import build_code_lut
from .pipeline import BlockGTQPipeline
from .v_packing import packed_v_bytes


# ===========================================================================
# Packing metadata
# ===========================================================================

def build_pack_meta(bit_allocation: torch.Tensor, head_perm: torch.Tensor) -> dict:
    """Segment table of the bit-packed K record.

    Returns a dict keyed by bit width (1..8) with ``start`` (first packed dim),
    ``length``, ``pack_offset`` (byte offset) and ``packed_bytes``, plus
    ``total_packed_bytes``, ``nopack_start`` / ``nopack_len`` / ``nopack_off``
    (the run of dims stored as raw bytes, bw >= 5; ``nopack_start`` is the head
    width when there is none) and the identity ``pack_perm`` /
    ``inv_pack_perm`` (``head_perm`` already sorts dims by bit width, so no
    second permutation exists).  Dims with 0 bits take no bytes.
    """
    HD = head_perm.shape[0]
    per_dim = torch.cat([bit_allocation, bit_allocation]).cpu()[head_perm.cpu()]
    if (per_dim[1:] < per_dim[:-1]).any():
        raise ValueError("head_perm does not order dims by ascending bit width")
    meta, off = {}, 0
    for bw in range(1, 9):
        idx = (per_dim == bw).nonzero(as_tuple=True)[0]
        if idx.numel() == 0:
            continue
        start, length = int(idx[0]), int(idx.numel())
        nbytes = _plan.segment_bytes(bw, length)
        meta[bw] = {'start': start, 'length': length,
                    'pack_offset': off, 'packed_bytes': nbytes}
        off += nbytes
    raw = [bw for bw in range(5, 9) if bw in meta]
    meta['nopack_start'] = meta[raw[0]]['start'] if raw else HD
    meta['nopack_off'] = meta[raw[0]]['pack_offset'] if raw else 0
    meta['nopack_len'] = sum(meta[bw]['length'] for bw in raw)
    meta['total_packed_bytes'] = off
    meta['pack_perm'] = torch.arange(HD)
    meta['inv_pack_perm'] = torch.arange(HD)
    return meta


# ===========================================================================
# Quantizer
# ===========================================================================

class BlockGTQQuantizer:
    """Calibrated quantizer of one (layer, KV head).

    Bit widths 1-4 are bit-packed, 5-8 stored as raw bytes.  ``device`` is
    where the encode/rotate entry points run; calibration itself is host work.
    """

    def __init__(self, head_dim: int, avg_bits: float = 3.0,
                 rotation_threshold: int = 2,
                 min_bits: int = 1, max_bits: int = 8,
                 rope_base: float = 1e6, n_bins: int = 256,
                 device: Optional[torch.device] = None, verbose: bool = False):
        self.head_dim = head_dim
        self.avg_bits = avg_bits
        self.rotation_threshold = rotation_threshold
        self.min_bits = min_bits
        self.max_bits = max_bits
        self.rope_base = rope_base
        self.n_bins = n_bins
        self.device = torch.device(device) if device is not None else torch.device('cuda:0')
        self.verbose = verbose
        self.bit_allocation = None
        self._calibrated = False
        self._plan_np = None
        self._plan_dev = None

    # ------------------------------------------------------------------ host
    def _pipeline(self) -> BlockGTQPipeline:
        return BlockGTQPipeline(
            head_dim=self.head_dim, avg_bits=self.avg_bits,
            rotation_threshold=self.rotation_threshold,
            min_bits=self.min_bits, max_bits=self.max_bits,
            rope_base=self.rope_base, device='cpu', verbose=self.verbose)

    def calibrate(self, q_data: torch.Tensor, k_data: torch.Tensor):
        """Allocate bits from (N, D) calibration activations and build all tables."""
        ref = self._pipeline()
        ref.calibrate(q_data.detach().float().cpu(), k_data.detach().float().cpu())
        self._adopt(ref)

    def calibrate_from_allocation(self, bit_allocation: torch.Tensor):
        """Build all tables from a given per-block bit allocation."""
        ref = self._pipeline()
        ref.set_allocation(bit_allocation)
        self._adopt(ref)

    def _adopt(self, ref: BlockGTQPipeline):
        dev = self.device
        self.bit_allocation = ref.bit_allocation
        self._n_groups = ref._n_groups
        self._n_zero_dims = ref._n_zero_dims
        self._single_group = ref._single_group
        self._group_bits = list(ref._group_bits)
        self._group_of_full = ref._group_of                        # -1 on 0-bit dims
        self._group_of = None if ref._single_group else ref._group_of.to(dev)
        self._head_perm = ref._head_perm.contiguous().to(dev)
        self._block_rot_T = ref._block_rot_T.contiguous().to(dev)
        self._rot_unperm = ref._block_rot_unperm.contiguous().to(dev)
        self._pos_centroids = ref._pos_centroids.contiguous().to(dev)
        self._pos_boundaries = ref._pos_boundaries.contiguous().to(dev)

        lut, p2cb, offs, invs = build_code_lut(ref._pos_centroids, ref._pos_boundaries,
                                               n_bins=self.n_bins)
        self._code_lut = lut.contiguous().to(dev)
        self._pos_to_cb = p2cb.contiguous().to(dev)
        self._lut_offsets = offs.contiguous().to(dev)
        self._lut_inv_scales = invs.contiguous().to(dev)
        self._n_codebooks = lut.shape[0]

        self._pack_meta = build_pack_meta(self.bit_allocation, ref._head_perm)
        self._pack_perm = self._pack_meta['pack_perm'].to(dev)
        self._inv_pack_perm = self._pack_meta['inv_pack_perm'].to(dev)
        self._total_packed_bytes = self._pack_meta['total_packed_bytes']
        self._total_bits = int(self.bit_allocation.sum().item()) * 2
        self._calibrated = True
        self._q_perm_baked = False
        self._plan_np = self._plan_dev = None
        if self.verbose:
            pm = self._pack_meta
            segs = ', '.join(f"{bw}b:{pm[bw]['length']}d->{pm[bw]['packed_bytes']}B"
                             for bw in range(1, 9) if bw in pm)
            print(f"  BlockGTQ: HD={self.head_dim}, n_groups={self._n_groups}, "
                  f"pack=[{segs}], total={self._total_packed_bytes}B")

    @property
    def effective_bits_per_dim(self):
        if self.bit_allocation is None:
            return self.avg_bits
        return self.bit_allocation.float().sum().item() / (self.head_dim // 2)

    @property
    def pack_meta(self):
        return self._pack_meta

    @property
    def composite_q_perm(self) -> torch.Tensor:
        """Original coordinate of every packed dim (``q[..., perm]`` lines Q up with K)."""
        assert self._calibrated
        return self._head_perm[self._pack_perm]

    def build_kernel_args(self) -> dict:
        """Arguments of ``fused_blockgtq_decode_attention`` for this head:
        ``codebook_flat`` (fp16 centroids of the segments, concatenated),
        ``lut_offset`` / ``norm_group`` per packed dim, ``segments_b`` =
        ``[(bw, start, length, pack_off, lut_off, norm_idx)]`` and
        ``total_packed_bytes`` (blockgtq/quantizer.py:1093-1148).  ``plan``
        carries the quantizer itself so the fused wrapper can reach the device
        plan without a second lookup."""
        assert self._calibrated
        hd, pm, dev = self.head_dim, self._pack_meta, self.device
        parts, segments = [], []
        lut_offset = torch.zeros(hd, dtype=torch.int32)
        norm_group = torch.zeros(hd, dtype=torch.int32)
        lut_off = 0
        for si, bw in enumerate(b for b in range(1, 9) if b in pm):
            s, ln = pm[bw]['start'], pm[bw]['length']
            parts.append(self._pos_centroids[s, :1 << bw].to(torch.float16).cpu())
            lut_offset[s:s + ln] = lut_off
            norm_group[s:s + ln] = si
            segments.append((bw, s, ln, pm[bw]['pack_offset'], lut_off, si))
            lut_off += 1 << bw
        flat = torch.cat(parts) if parts else torch.zeros(0, dtype=torch.float16)
        from .kernels import register_kernel_args
        return register_kernel_args({
            'codebook_flat': flat.to(dev),
            'lut_offset': lut_offset.to(dev),
            'norm_group': norm_group.to(dev),
            'segments_b': segments,
            'total_packed_bytes': pm['total_packed_bytes'],
            'quantizer': self,
        })

    # -------------------------------------------------------------- plan
    def plan(self):
        """This head's ``bgtq_head_plan`` as a (1,) structured numpy array."""
        assert self._calibrated and hasattr(self, '_v_bits'), \
            "calibrate() and init_v_quantizer() first"
        if self._plan_np is None:
            self._plan_np = _plan.build_head_plan(self)
        return self._plan_np

    def device_plan(self) -> torch.Tensor:
        if self._plan_dev is None:
            self._plan_dev = _plan.upload_plans(self.plan(), self.device)
        return self._plan_dev

    # -------------------------------------------------------------- Q side
    @torch.no_grad()
    def rotate_q_for_packed_kernel(self, q: torch.Tensor) -> torch.Tensor:
        """(..., D) queries -> permuted + rotated into the packed K space, same dtype
        (computed in fp32, rounded to fp16; blockgtq/quantizer.py:1160-1187)."""
        assert self._calibrated
        _capi.require_cuda(q, "q")
        shape = q.shape
        q2 = q.reshape(-1, 1, self.head_dim).to(torch.float16).contiguous()
        out = torch.empty_like(q2)
        L = _capi.lib()
        _capi.check(L.bgtq_rotate_q(
            _capi.ptr(self.device_plan()), _capi.ptr(q2), q2.stride(0), q2.stride(1),
            _capi.ptr(out), out.stride(0), out.stride(1),
            q2.shape[0], 1, 1, _capi.stream_ptr(q.device)), "bgtq_rotate_q")
        return out.to(q.dtype).reshape(shape)

    @torch.no_grad()
    def bake_permutation_into_qproj(self, q_proj_weight: torch.Tensor,
                                    kv_head_idx: int, n_kv_heads: int, n_q_heads: int,
                                    q_proj_bias: Optional[torch.Tensor] = None) -> None:
        """Fold permutation + rotation into the ``q_proj`` rows of this KV head's
        query group, in place, so that the projection's output equals
        ``rotate_q_for_packed_kernel`` of the original projection's output.

        The kernels and ``rotate_q_for_packed_kernel`` compute
        ``q' = q[head_perm] @ block_rot_T`` (blockgtq/quantizer.py:1180-1187), i.e.
        ``q' = block_rot_T^T (W x + b)[head_perm]``, hence
        ``W' = block_rot_T^T W[head_perm]`` and ``b' = block_rot_T^T b[head_perm]``.
        The reference's own baking routine multiplies by ``block_rot_T`` without the
        transpose (blockgtq/quantizer.py:1232), which disagrees with its query rotation
        for every non-symmetric rotation block; this implementation follows the query
        rotation, the one the attention kernel's results are defined by."""
        assert self._calibrated, "calibrate() must be called before baking"
        assert kv_head_idx < n_kv_heads
        hd = self.head_dim
        gqa = n_q_heads // n_kv_heads
        assert q_proj_weight.shape[0] == n_q_heads * hd
        hp = self._head_perm.cpu()
        rot = self._block_rot_T.cpu().float().t().contiguous()
        for g in range(gqa):
            lo = (kv_head_idx * gqa + g) * hd
            w = q_proj_weight[lo:lo + hd].detach().clone().cpu()[hp].float()
            q_proj_weight[lo:lo + hd] = (rot @ w).to(q_proj_weight.dtype).to(q_proj_weight.device)
            if q_proj_bias is not None:
                bvec = q_proj_bias[lo:lo + hd].detach().clone().cpu()[hp].float()
                q_proj_bias[lo:lo + hd] = (rot @ bvec).to(q_proj_bias.dtype).to(q_proj_bias.device)
        self._q_perm_baked = True

    # -------------------------------------------------------------- K side
    @torch.no_grad()
    def compress(self, k: torch.Tensor, block_n: int = 32, *, corrected: bool = False,
                 quant_mode: int = _plan.QUANT_LUT256):
        """(..., D) fp16 -> codes (..., D) uint8 in packed order, norms (..., n_groups) fp32."""
        assert self._calibrated
        _capi.require_cuda(k, "k")
        hd = self.head_dim
        x = k.reshape(-1, hd).to(torch.float16).contiguous()
        N = x.shape[0]
        ng = max(self._n_groups, 1)
        codes = torch.empty(N, hd, dtype=torch.uint8, device=k.device)
        norms = torch.zeros(N, ng, dtype=torch.float32, device=k.device)
        L = _capi.lib()
        _capi.check(L.bgtq_compress_k_codes(
            _capi.ptr(self.device_plan()), _capi.ptr(x), N, _capi.ptr(codes), _capi.ptr(norms),
            ng, int(corrected), quant_mode, _capi.stream_ptr(k.device)), "bgtq_compress_k_codes")
        return codes.reshape(*k.shape[:-1], hd), norms.reshape(*k.shape[:-1], ng)

    @torch.no_grad()
    def correct_norms(self, k: torch.Tensor, raw_norms: torch.Tensor,
                      block_n: int = 32) -> torch.Tensor:
        """Group norms divided by ``||centroids[codes]||`` of the same group."""
        _, corr = self.compress(k, corrected=True)
        return corr.reshape(raw_norms.shape)

    @torch.no_grad()
    def compress_packed(self, k: torch.Tensor, block_n: int = 32,
                        norm_correct: bool = False):
        """(..., D) fp16 -> bit-packed records (..., total_packed_bytes) uint8,
        group norms (..., n_groups) fp32, information bits per vector."""
        assert self._calibrated
        _capi.require_cuda(k, "k")
        hd = self.head_dim
        x = k.reshape(1, 1, -1, hd).to(torch.float16).contiguous()
        N = x.shape[2]
        tpb, ng = self._total_packed_bytes, max(self._n_groups, 1)
        packed = torch.empty(1, 1, N, max(tpb, 1), dtype=torch.uint8, device=k.device)
        norms16 = torch.empty(1, 1, N, ng, dtype=torch.float16, device=k.device)
        encode_k_into(self.device_plan(), x, packed, norms16, 0, tpb, ng, _plan.K_BITPACKED)
        if norm_correct:
            norms = self.compress(k, corrected=True)[1]
        else:
            norms = self.compress(k)[1]
        return (packed[0, 0, :, :tpb].reshape(*k.shape[:-1], tpb),
                norms.reshape(*k.shape[:-1], ng), self._total_bits)

    @torch.no_grad()
    def compress_decompress(self, k: torch.Tensor, block_n: int = 32) -> torch.Tensor:
        """Quantise on the device, reconstruct with torch ops: centroid gather,
        per-group norm correction, inverse rotation and un-permutation."""
        codes, norms = self.compress(k, corrected=True)
        hd = self.head_dim
        c = codes.reshape(-1, hd).long()
        cents = self._pos_centroids.to(k.device)
        y = cents[torch.arange(hd, device=k.device).unsqueeze(0), c]
        grp = self._group_of_full.to(k.device)
        scale = norms.reshape(-1, norms.shape[-1])[:, grp.clamp(min=0)] * (grp >= 0)
        out = (y * scale) @ self._rot_unperm.to(k.device)
        return out.reshape(k.shape)

    # -------------------------------------------------------------- V side
    def init_v_quantizer(self, v_bits: int = 3, seed: int = 42):
        """Seed-deterministic V rotation + codebook; needs no calibration data."""
        from .v_quantize_gpu import PolarQuantGPU
        self._v_quantizer = PolarQuantGPU(d=self.head_dim, bit_width=v_bits, seed=seed,
                                          device=self.device)
        self._v_bits = v_bits
        self._v_seed = seed
        self._v_rot_T = self._v_quantizer.rotation.T.contiguous()
        self._v_rot = self._v_quantizer.rotation.contiguous()
        self._v_boundaries = self._v_quantizer.boundaries.contiguous()
        self._v_centroids_f32 = self._v_quantizer.centroids.contiguous()
        self._plan_np = self._plan_dev = None

    @property
    def v_bits(self) -> int:
        return getattr(self, '_v_bits', 0)

    @property
    def v_lut(self) -> torch.Tensor:
        assert hasattr(self, '_v_quantizer'), "call init_v_quantizer() first"
        return self._v_quantizer.v_lut

    @torch.no_grad()
    def compress_v(self, v: torch.Tensor):
        """(..., D) fp16 -> codes (..., D) uint8, corrected norms (...,) fp16."""
        assert hasattr(self, '_v_quantizer'), "call init_v_quantizer() first"
        _capi.require_cuda(v, "v")
        hd = self.head_dim
        x = v.reshape(-1, hd).to(torch.float16).contiguous()
        N = x.shape[0]
        codes = torch.empty(N, hd, dtype=torch.uint8, device=v.device)
        norms = torch.empty(N, dtype=torch.float16, device=v.device)
        L = _capi.lib()
        _capi.check(L.bgtq_compress_v_codes(
            _capi.ptr(self.device_plan()), _capi.ptr(x), N, _capi.ptr(codes), _capi.ptr(norms),
            _capi.stream_ptr(v.device)), "bgtq_compress_v_codes")
        return codes.reshape(*v.shape[:-1], hd), norms.reshape(v.shape[:-1])

    @torch.no_grad()
    def compress_v_packed(self, v: torch.Tensor, block_n: int = 32):
        """(..., D) fp16 -> packed records (..., packed_v_bytes) uint8, norms (...,) fp16."""
        assert hasattr(self, '_v_quantizer'), "call init_v_quantizer() first"
        _capi.require_cuda(v, "v")
        hd = self.head_dim
        x = v.reshape(1, 1, -1, hd).to(torch.float16).contiguous()
        N = x.shape[2]
        pb = packed_v_bytes(hd, self._v_bits)
        packed = torch.empty(1, 1, N, pb, dtype=torch.uint8, device=v.device)
        norms = torch.empty(1, 1, N, dtype=torch.float16, device=v.device)
        encode_v_into(self.device_plan(), x, packed, norms, 0, pb, _plan.V_BITPACKED)
        return packed.reshape(*v.shape[:-1], pb), norms.reshape(v.shape[:-1])


# ===========================================================================
# Direct-to-cache encoders (thin wrappers of the C ABI)
# ===========================================================================

def _t_pos_args(t_pos):
    if isinstance(t_pos, torch.Tensor):
        assert t_pos.dtype == torch.int32 and t_pos.is_cuda
        return _capi.ptr(t_pos), 0
    return None, int(t_pos)


def _cache_capacity(t_pos, S: int, *cache_tensors) -> int:
    """Token capacity of the cache views an append writes to (their common size along the
    token axis).  A host position that would run past it raises here, before any launch, as the
    reference's slice assignment would; device positions are bounded by the kernels, which drop
    records outside the capacity."""
    max_T = min(int(t.shape[2]) for t in cache_tensors)
    if not isinstance(t_pos, torch.Tensor) and int(t_pos) + int(S) > max_T:
        raise ValueError(f"append of {S} token(s) at position {int(t_pos)} exceeds the cache capacity {max_T}")
    return max_T


def encode_k_into(plans: torch.Tensor, k: torch.Tensor, k_packed: torch.Tensor,
                  k_norms: torch.Tensor, t_pos, row_width: int, norm_width: int,
                  k_layout: int, quant_mode: int = _plan.QUANT_LUT256):
    """Encode ``k`` (B, n_kv, S, D) fp16 into cache views ``k_packed``
    (B, n_kv, T, >=row_width) uint8 and ``k_norms`` (B, n_kv, T, >=norm_width)
    fp16 at token ``t_pos`` (int, or int32 device tensor of per-row positions)."""
    _capi.require_cuda(k, "k")
    assert k.dtype == torch.float16 and k.stride(-1) == 1
    assert k_packed.dtype == torch.uint8 and k_packed.stride(-1) == 1
    assert k_norms.dtype == torch.float16 and k_norms.stride(-1) == 1
    B, H, S, _ = k.shape
    tp, ts = _t_pos_args(t_pos)
    max_T = _cache_capacity(t_pos, S, k_packed, k_norms)
    L = _capi.lib()
    _capi.check(L.bgtq_encode_k(
        _capi.ptr(plans), _capi.ptr(k), k.stride(0), k.stride(1), k.stride(2), B, H, S,
        _capi.ptr(k_packed), k_packed.stride(0), k_packed.stride(1), k_packed.stride(2), row_width,
        _capi.ptr(k_norms), k_norms.stride(0), k_norms.stride(1), k_norms.stride(2), norm_width,
        tp, ts, max_T, k_layout, quant_mode, _capi.stream_ptr(k.device)), "bgtq_encode_k")


def encode_v_into(plans: torch.Tensor, v: torch.Tensor, v_packed: torch.Tensor,
                  v_norms: torch.Tensor, t_pos, row_width: int, v_layout: int):
    """Encode ``v`` (B, n_kv, S, D) fp16 into ``v_packed`` (B, n_kv, T, >=row_width)
    uint8 and ``v_norms`` (B, n_kv, T) fp16 at token ``t_pos``."""
    _capi.require_cuda(v, "v")
    assert v.dtype == torch.float16 and v.stride(-1) == 1
    assert v_packed.dtype == torch.uint8 and v_packed.stride(-1) == 1
    assert v_norms.dtype == torch.float16
    B, H, S, _ = v.shape
    tp, ts = _t_pos_args(t_pos)
    max_T = _cache_capacity(t_pos, S, v_packed, v_norms)
    L = _capi.lib()
    _capi.check(L.bgtq_encode_v(
        _capi.ptr(plans), _capi.ptr(v), v.stride(0), v.stride(1), v.stride(2), B, H, S,
        _capi.ptr(v_packed), v_packed.stride(0), v_packed.stride(1), v_packed.stride(2), row_width,
        _capi.ptr(v_norms), v_norms.stride(0), v_norms.stride(1), v_norms.stride(2),
        tp, ts, max_T, v_layout, _capi.stream_ptr(v.device)), "bgtq_encode_v")


# ===========================================================================
# Batched (all KV heads of a layer) helpers with the reference's signatures
# ===========================================================================

def build_batched_encode_args(quantizers: list, device='cuda') -> dict:
    """Stack the per-head plans of one layer (blockgtq/quantizer.py:1598-1747).

    The returned dict keeps the size fields callers read (``max_tpb``,
    ``max_n_groups``, ``max_mixed_bytes``, ``v_packed_bytes``,
    ``v_nibble_bytes`` ...) and adds ``plans``: the uploaded
    ``bgtq_head_plan[n_kv]`` every device entry point takes.
    """
    q0 = quantizers[0]
    hd, v_bits = q0.head_dim, q0._v_bits
    plans_np = _plan.stack_plans(quantizers)
    ns = [q._pack_meta['nopack_start'] for q in quantizers]
    nl = [q._pack_meta['nopack_len'] for q in quantizers]
    return {
        'plans_np': plans_np,
        'plans': _plan.upload_plans(plans_np, device),
        'n_kv': len(quantizers), 'hd': hd, 'n_bins': q0.n_bins,
        'v_bits': v_bits, 'v_n_cents': 1 << v_bits,
        'v_packed_bytes': packed_v_bytes(hd, v_bits), 'v_nibble_bytes': hd // 2,
        'max_n_groups': max(max(q._n_groups for q in quantizers), 1),
        'max_n_codebooks': max(q._n_codebooks for q in quantizers),
        'max_tpb': max(q._total_packed_bytes for q in quantizers),
        'max_mixed_bytes': int(plans_np['k_mixed_bytes'].max()),
        'mixed_nopack_starts': ns, 'mixed_nopack_lens': nl,
    }


def _batched_k(k_flat, args, layout, width):
    n_kv, N, hd = k_flat.shape
    ng = args['max_n_groups']
    packed = torch.empty(1, n_kv, N, max(width, 1), dtype=torch.uint8, device=k_flat.device)
    norms = torch.empty(1, n_kv, N, ng, dtype=torch.float16, device=k_flat.device)
    encode_k_into(args['plans'], k_flat.to(torch.float16).unsqueeze(0), packed, norms,
                  0, width, ng, layout)
    return packed[0, :, :, :width], norms[0].float()


@torch.no_grad()
def compress_k_packed_batched(k_flat: torch.Tensor, args: dict, block_n: int = 32):
    """(n_kv, N, D) fp16 -> bit-packed (n_kv, N, max_tpb) uint8 and raw group
    norms (n_kv, N, max_n_groups) fp32 holding fp16-rounded values (what the
    cache stores)."""
    return _batched_k(k_flat, args, _plan.K_BITPACKED, args['max_tpb'])


@torch.no_grad()
def compress_k_mixed_batched(k_flat: torch.Tensor, args: dict, block_n: int = 32,
                             norm_correct: bool = True):
    """(n_kv, N, D) fp16 -> mixed nibble/byte records (n_kv, N, max_mixed_bytes)
    and corrected group norms (fp16-rounded values in fp32)."""
    if not norm_correct:
        raise NotImplementedError("the mixed layout always stores corrected norms")
    return _batched_k(k_flat, args, _plan.K_MIXED, args['max_mixed_bytes'])


@torch.no_grad()
def compress_k_nibble4_batched(k_flat: torch.Tensor, args: dict, block_n: int = 32):
    """(n_kv, N, D) fp16 -> every code of a vector as a nibble, two per byte in
    packed order (even position in the low nibble; codes wider than 4 bits keep
    their low 4), (n_kv, N, D/2) uint8, and raw group norms (n_kv, N,
    max_n_groups) fp32.  Reference: blockgtq/quantizer.py:1751-1841."""
    _capi.require_cuda(k_flat, "k_flat")
    n_kv, N, hd = k_flat.shape
    ng = args['max_n_groups']
    x = k_flat.to(torch.float16).contiguous()
    codes = torch.empty(n_kv, N, hd, dtype=torch.uint8, device=k_flat.device)
    norms = torch.zeros(n_kv, N, ng, dtype=torch.float32, device=k_flat.device)
    L, st = _capi.lib(), _capi.stream_ptr(k_flat.device)
    for h in range(n_kv):
        _capi.check(L.bgtq_compress_k_codes(
            _capi.ptr(args['plans'][h * _plan.PLAN_DTYPE.itemsize:]), _capi.ptr(x[h]), N, _capi.ptr(codes[h]), _capi.ptr(norms[h]),
            ng, 0, _plan.QUANT_LUT256, st), "bgtq_compress_k_codes")
    return ((codes[..., 0::2] & 0xF) | ((codes[..., 1::2] & 0xF) << 4)).contiguous(), norms


def _batched_v(v_flat, args, layout, width):
    n_kv, N, hd = v_flat.shape
    packed = torch.empty(1, n_kv, N, width, dtype=torch.uint8, device=v_flat.device)
    norms = torch.empty(1, n_kv, N, dtype=torch.float16, device=v_flat.device)
    encode_v_into(args['plans'], v_flat.to(torch.float16).unsqueeze(0), packed, norms,
                  0, width, layout)
    return packed[0], norms[0]


@torch.no_grad()
def compress_v_packed_batched(v_flat: torch.Tensor, args: dict, block_n: int = 32):
    """(n_kv, N, D) fp16 -> (n_kv, N, vpb) uint8, corrected norms (n_kv, N) fp16."""
    return _batched_v(v_flat, args, _plan.V_BITPACKED, args['v_packed_bytes'])


@torch.no_grad()
def compress_v_nibble4_batched(v_flat: torch.Tensor, args: dict, block_n: int = 32):
    """(n_kv, N, D) fp16 -> (n_kv, N, D/2) uint8 nibble records, norms (n_kv, N) fp16."""
    return _batched_v(v_flat, args, _plan.V_NIBBLE, args['v_nibble_bytes'])
