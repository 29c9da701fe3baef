"""Attention over the packed cache, reference-compatible entries.

``fused_blockgtq_decode_attention`` keeps the argument list of
blockgtq/kernels/fused_packed_attention.py:1541-1570 so existing call sites
(per-KV-head slices of the cache plus that head's ``build_kernel_args`` dict)
keep working; underneath it is one ``bgtq_decode_attn`` + one
``bgtq_lse_reduce`` launch.  The cache classes of this package do not go
through here: they launch all KV heads at once via :mod:`blockgtq_amd.ops`.
"""
import math
import weakref

import numpy as np
import torch

from .. import ops, plan as _plan

# id(codebook_flat tensor object) -> (weak reference to that tensor, weak reference to the quantizer
# that produced it via build_kernel_args()).  The tensor OBJECT is the key, not its address: memory
# of a freed codebook can be handed to another tensor, an id is only trusted while its object lives.
_QUANTIZER_OF_CODEBOOK = {}


def register_kernel_args(kernel_args: dict):
    """Remember which quantizer a ``build_kernel_args`` dict came from, so the
    fused entry can find that head's device plan from ``codebook_flat`` alone."""
    q = kernel_args.get('quantizer')
    t = kernel_args['codebook_flat']
    if q is not None and t.numel():
        key = id(t)

        def forget(ref, key=key):
            if _QUANTIZER_OF_CODEBOOK.get(key, (None,))[0] is ref:
                del _QUANTIZER_OF_CODEBOOK[key]

        _QUANTIZER_OF_CODEBOOK[key] = (weakref.ref(t, forget), weakref.ref(q))
    return kernel_args


def _quantizer_of(codebook_flat):
    """The quantizer registered for exactly this tensor object, if it is still alive."""
    entry = _QUANTIZER_OF_CODEBOOK.get(id(codebook_flat))
    if entry is None or entry[0]() is not codebook_flat:
        return None
    return entry[1]()


def _plan_from_args(codebook_flat, segments, v_lut, v_rotation, v_bits, device):
    """Decode-only plan assembled from the loose arguments of the fused entry
    (used when the codebook was not produced by this package's quantizer)."""
    p = np.zeros((), dtype=_plan.PLAN_DTYPE)
    segs = [s for s in segments if s[2] > 0]
    p['n_seg'] = len(segs)
    cb = codebook_flat.detach().cpu().to(torch.float16).numpy().view(np.uint16)
    first = min([s[1] for s in segs], default=0)
    p['n_zero_dims'] = first
    p['group_of'][...] = -1
    p['nopack_start'], nopack_len = _plan.HEAD_DIM, 0
    tot = 0
    for g, (bw, start, length, pack_off, lut_off, _norm_idx) in enumerate(segs):
        p['seg_bw'][g], p['seg_start'][g], p['seg_len'][g] = bw, start, length
        p['seg_pack_off'][g] = pack_off
        p['group_of'][start:start + length] = g
        p['k_codebook_f16'][g, :1 << bw] = cb[lut_off:lut_off + (1 << bw)]
        tot = max(tot, pack_off + _plan.segment_bytes(bw, length))
        if bw >= 5:
            p['nopack_start'] = min(int(p['nopack_start']), start)
            nopack_len += length
    p['nopack_len'] = nopack_len
    nib = (int(p['nopack_start']) - first) // 2
    for g, (bw, start, length, *_r) in enumerate(segs):
        p['seg_mixed_off'][g] = ((start - first) // 2 if bw <= 4
                                 else nib + (start - int(p['nopack_start'])))
    p['k_row_bytes'] = tot
    p['k_mixed_bytes'] = nib + nopack_len
    p['v_bits'] = v_bits
    lut = v_lut.detach().cpu().to(torch.float16).numpy().view(np.uint16)
    p['v_lut_f16'][:lut.size] = lut
    if v_rotation is not None:
        p['v_rot'] = v_rotation.detach().cpu().float().numpy().reshape(-1)
    _plan.fill_decode_steps(p)
    return _plan.upload_plans(p.reshape(1), device)


@torch.no_grad()
def fused_blockgtq_decode_attention(
    q, k_packed, k_norms, codebook_flat, lut_offset, norm_group, segments,
    v_codes, v_norms, v_lut,
    scale=None, block_t=64, block_m=16, t_splits=32,
    v_skip_thresh=0.0, v_norm_scale=None, onebit_fast='auto', q_pack_perm=None,
    v_bits=0, v_rotation=None, k_nibble=False, v_nibble=False,
    v_paired_2b=False, k_paired_2b=False, k_paired_4b=False,
    k_paired_8b=False, k_paired_1b=False, return_lse=False,
):
    """Decode attention of one KV head's query group over its packed cache slice.

    q (B, gqa, 1, D) fp16, already permuted + rotated
    (``rotate_q_for_packed_kernel``); k_packed (B, 1, T, Kb) uint8; k_norms
    (B, 1, T, G) fp16; v_codes (B, 1, T, Vb) uint8 packed at ``v_bits`` (or as
    nibbles when ``v_nibble``); v_norms (B, 1, T) fp16.  Returns
    (B, gqa, 1, D) fp16 and, with ``return_lse``, the total log-sum-exp (B, gqa).

    ``block_t``, ``block_m``, ``onebit_fast`` and the ``*_paired_*`` switches
    selected speed variants of the reference kernel with identical results;
    they are accepted and ignored.  Layout features no caller of the reference
    uses (raw uint8 V codes, int4 V norms, ``v_skip_thresh``) are rejected.
    """
    assert q.dim() == 4 and q.shape[2] == 1
    assert len(segments) <= 8
    if v_skip_thresh:
        raise NotImplementedError("v_skip_thresh changes results; not built")
    if v_norms.dtype != torch.float16:
        raise NotImplementedError("only fp16 V norms are supported")
    if not v_nibble and not (1 <= int(v_bits) <= 4):
        raise NotImplementedError("V must be bit-packed (v_bits 1..4) or nibble-packed")
    B, n_q, _, D = q.shape
    n_kv = k_packed.shape[1]
    if n_kv != 1:
        raise NotImplementedError("pass one KV head per call (each head owns its plan)")
    T = k_packed.shape[2]
    if q_pack_perm is not None:
        q = q[:, :, :, q_pack_perm]
    quant = _quantizer_of(codebook_flat)
    if quant is not None:
        plans = quant.device_plan()
    else:
        plans = _plan_from_args(codebook_flat, segments, v_lut, v_rotation,
                                int(v_bits) if not v_nibble else max(int(v_bits), 1), q.device)
    if v_norms.dim() == 4:
        v_norms = v_norms[..., 0]
    q3 = q.reshape(B, n_q, D).to(torch.float16).contiguous()
    res = ops.decode_attention(
        plans, q3, k_packed, k_norms, v_codes, v_norms, T,
        n_splits=max(1, min(int(t_splits), 512)),
        k_layout=_plan.K_MIXED if k_nibble else _plan.K_BITPACKED,
        v_layout=_plan.V_NIBBLE if v_nibble else _plan.V_BITPACKED,
        scale=(1.0 / math.sqrt(D)) if scale is None else scale,
        unrotate=v_rotation is not None, return_lse=return_lse)
    if return_lse:
        return res[0].unsqueeze(2), res[1]
    return res.unsqueeze(2)


@torch.no_grad()
def fused_blockgtq_prefill_attention(
    q, k_packed, k_norms, codebook_flat, lut_offset, norm_group, segments,
    v_codes, v_norms, v_lut,
    scale=None, block_q=64, block_t=64, v_skip_thresh=0.0, v_norm_scale=None,
    v_bits=0, v_rotation=None, is_causal=True, q_pos_offset=0,
    k_nibble=False, v_nibble=False, min_seg_for_dot=16,
):
    """Prompt-phase attention of one KV head's query group over its packed cache
    slice (argument list of blockgtq/kernels/fused_packed_attention.py:2597-2620).

    q (B, gqa, S_q, D) fp16 already permuted + rotated; cache slices as for the
    decode entry.  Query token s sees records ``t <= q_pos_offset + s`` when
    ``is_causal``.  Returns (B, gqa, S_q, D) fp16.  ``bgtq_prefill_attn`` attends
    straight over the records; record tensors whose rows it cannot walk are first
    copied into rows it can.
    ``block_q``, ``block_t`` and ``min_seg_for_dot`` tuned the reference kernel and
    are ignored."""
    assert q.dim() == 4
    assert len(segments) <= 8
    if v_skip_thresh:
        raise NotImplementedError("v_skip_thresh changes results; not built")
    if v_norms.dtype != torch.float16:
        raise NotImplementedError("only fp16 V norms are supported")
    if not v_nibble and not (1 <= int(v_bits) <= 4):
        raise NotImplementedError("V must be bit-packed (v_bits 1..4) or nibble-packed")
    if k_packed.shape[1] != 1:
        raise NotImplementedError("pass one KV head per call (each head owns its plan)")
    T = k_packed.shape[2]
    quant = _quantizer_of(codebook_flat)
    if quant is not None:
        plans = quant.device_plan()
    else:
        plans = _plan_from_args(codebook_flat, segments, v_lut, v_rotation,
                                int(v_bits) if not v_nibble else max(int(v_bits), 1), q.device)
    if v_norms.dim() == 4:
        v_norms = v_norms[..., 0]
    kl = _plan.K_MIXED if k_nibble else _plan.K_BITPACKED
    vl = _plan.V_NIBBLE if v_nibble else _plan.V_BITPACKED
    return ops.prefill_attention_records(
        plans, q.to(torch.float16), k_packed, k_norms, v_codes, v_norms, T, k_layout=kl, v_layout=vl,
        scale=scale, is_causal=is_causal, q_pos_offset=q_pos_offset, unrotate=v_rotation is not None)


def build_segments_from_pack_meta(pack_meta, codebook_flat=None, pos_centroids=None):
    """``[(bw, dim_start, dim_len, pack_off, lut_off, norm_idx)]`` in ascending
    bit width (blockgtq/kernels/fused_packed_attention.py:2763-2787)."""
    out, lut_off = [], 0
    for idx, bw in enumerate(b for b in range(1, 9) if b in pack_meta):
        m = pack_meta[bw]
        out.append((bw, m['start'], m['length'], m['pack_offset'], lut_off, idx))
        lut_off += 1 << bw
    return out


__all__ = ["fused_blockgtq_decode_attention", "fused_blockgtq_prefill_attention",
           "build_segments_from_pack_meta",
           "register_kernel_args"]
