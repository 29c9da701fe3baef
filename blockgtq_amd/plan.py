"""Host mirror of ``bgtq_head_plan`` (include/bgtq.h) and its builder.

One plan per (layer, KV head) gathers every static table the device kernels
read: the K segment table, permutation, 256-bin code LUT, codebooks in fp32
and fp16, the block-diagonal K rotation, and the V rotation/boundaries/LUT.
Plans of the KV heads of one layer are concatenated and uploaded once.
"""
import numpy as np
import torch

HEAD_DIM = 128
MAX_SEGMENTS = 8
MAX_CENTROIDS = 256
LUT_BINS = 256
MAX_STEPS = 12

K_BITPACKED, K_MIXED = 0, 1
V_BITPACKED, V_NIBBLE = 0, 1
QUANT_LUT256, QUANT_EXACT = 0, 1

_S, _D, _C = MAX_SEGMENTS, HEAD_DIM, MAX_CENTROIDS

PLAN_DTYPE = np.dtype([
    ('n_seg', '<i4'), ('n_zero_dims', '<i4'), ('k_row_bytes', '<i4'),
    ('k_mixed_bytes', '<i4'), ('nopack_start', '<i4'), ('nopack_len', '<i4'),
    ('v_bits', '<i4'), ('reserved0', '<i4'),
    ('seg_bw', '<i4', (_S,)), ('seg_start', '<i4', (_S,)), ('seg_len', '<i4', (_S,)),
    ('seg_pack_off', '<i4', (_S,)), ('seg_mixed_off', '<i4', (_S,)),
    ('seg_identity', '<i4', (_S,)),
    ('head_perm', '<i4', (_D,)), ('group_of', '<i4', (_D,)),
    ('lut_offset', '<f4', (_D,)), ('lut_inv_scale', '<f4', (_D,)),
    ('code_lut', 'u1', (_S, LUT_BINS)),
    ('k_centroids', '<f4', (_S, _C)), ('k_boundaries', '<f4', (_S, _C)),
    ('k_codebook_f16', '<u2', (_S, _C)),
    ('k_rot_T', '<f4', (_D * _D,)),
    ('v_centroids', '<f4', (16,)), ('v_boundaries', '<f4', (16,)),
    ('v_lut_f16', '<u2', (16,)),
    ('v_rot_T', '<f4', (_D * _D,)), ('v_rot', '<f4', (_D * _D,)),
    ('n_steps', '<i4'), ('reserved1', '<i4', (3,)), ('step', '<i4', (MAX_STEPS, 8)),
    ('n_packed_steps', '<i4'), ('reserved2', '<i4', (3,)),
    ('steptab', '<u4', (MAX_STEPS, 4, 8)), ('qunit_dim', '<i4', (32,)), ('qunit_len', '<i4', (32,)),
    ('lut_image', '<u4', (29184 // 4,)),
    ('n_steps_mixed', '<i4'), ('n_packed_steps_mixed', '<i4'), ('reserved3', '<i4', (2,)),
    ('steptab_mixed', '<u4', (MAX_STEPS, 4, 8)), ('qunit_dim_mixed', '<i4', (32,)),
    ('qunit_len_mixed', '<i4', (32,)), ('lut_image_mixed', '<u4', (43008 // 4,)),
    ('n_steps_dense', '<i4'), ('n_packed_steps_dense', '<i4'),
    ('n_steps_dense_mixed', '<i4'), ('n_packed_steps_dense_mixed', '<i4'),
    ('steptab_dense', '<u4', (MAX_STEPS, 2, 4, 8)), ('steptab_dense_mixed', '<u4', (MAX_STEPS, 2, 4, 8)),
], align=True)

# byte offsets inside lut_image (BGTQ_LUT_* of include/bgtq.h)
LUT_K = {1: 0, 2: 512, 3: 2560, 4: 10752}
LUT_KRAW, LUT_V, LUT_IMAGE_BYTES = 18944, 20992, 29184
LUTM_KRAW, LUTM_V, LUTM_IMAGE_BYTES = 32768, 34816, 43008      # BGTQ_LUTM_*


def segment_bytes(bw: int, length: int) -> int:
    """Bytes a K segment of ``length`` codes takes in the bit-packed record."""
    if bw == 1:
        return (length + 7) // 8
    if bw == 2:
        return (length + 3) // 4
    if bw == 3:
        return ((length + 7) // 8) * 3
    if bw == 4:
        return (length + 1) // 2
    return length


def _pair_table(cb16: np.ndarray, bw: int) -> np.ndarray:
    """Bank-replicated pair table of one code width: entry (c0 | c1 << bw)."""
    e = np.arange(1 << (2 * bw))
    pairs = cb16[e & ((1 << bw) - 1)].astype(np.uint32) | (cb16[e >> bw].astype(np.uint32) << 16)
    return np.repeat(pairs, 8 if bw == 4 else 32)


def fill_decode_steps(p) -> None:
    """Derive the MFMA step schedule of the bit-packed K record, its LDS-ready
    form and the pair tables from the segment table, codebooks and V LUT
    already stored in plan ``p`` (a 0-d structured array)."""
    m, n_packed, unit = 0, 0, 1
    p['step'][...] = 0
    p['steptab'][...] = 0
    p['qunit_dim'][...] = 0
    p['qunit_len'][...] = 0
    for s in range(int(p['n_seg'])):
        bw, ln = int(p['seg_bw'][s]), int(p['seg_len'][s])
        start, end = int(p['seg_start'][s]), int(p['seg_start'][s]) + ln
        n_units = (ln + 7) // 8
        unit_bytes = bw if bw <= 4 else 8
        for u0 in range(0, n_units, 4):
            if m >= MAX_STEPS:
                raise ValueError("segment table needs more MFMA steps than the plan holds")
            nu = min(4, n_units - u0)
            off0 = int(p['seg_pack_off'][s]) + u0 * unit_bytes
            p['step'][m] = (off0, unit_bytes, 2 * bw if bw <= 4 else 0, bw, s,
                            int(u0 + 4 >= n_units), nu, start + u0 * 8)
            for g in range(4):
                gg = min(g, nu - 1)
                table = LUT_K[bw] if bw <= 4 else LUT_KRAW + (bw - 5) * 512
                mask = 7 * 4 if bw == 4 else (31 * 4 if bw <= 3 else 0)
                q_off = 0
                if g < nu:
                    d0 = start + (u0 + g) * 8
                    p['qunit_dim'][unit], p['qunit_len'][unit] = d0, min(8, end - d0)
                    q_off = 16 * unit
                    unit += 1
                p['steptab'][m, g] = (off0 + gg * unit_bytes, 0, table, mask,
                                      2 * bw if bw <= 4 else 0, 5 if bw == 4 else 7, s * 128, q_off)
            n_packed += bw <= 4
            m += 1
    p['n_steps'] = m
    p['n_packed_steps'] = n_packed

    img = np.zeros(LUT_IMAGE_BYTES // 4, dtype=np.uint32)
    for s in range(int(p['n_seg'])):
        bw = int(p['seg_bw'][s])
        cb = p['k_codebook_f16'][s]
        if bw <= 4:
            t = _pair_table(cb, bw)
            img[LUT_K[bw] // 4:LUT_K[bw] // 4 + t.size] = t
        else:
            raw = np.zeros(256, dtype=np.uint16)
            raw[:1 << bw] = cb[:1 << bw]
            o = (LUT_KRAW + (bw - 5) * 512) // 4
            img[o:o + 128] = raw.view(np.uint32)
    vb = int(p['v_bits'])
    if 1 <= vb <= 4:
        t = _pair_table(p['v_lut_f16'], vb)
        img[LUT_V // 4:LUT_V // 4 + t.size] = t
    p['lut_image'] = img
    _fill_dense(p, '')
    _fill_mixed_tables(p)


def _fill_dense(p, suffix: str) -> None:
    """Two-segment schedule for query groups of at most 8 heads, derived from the
    one-segment schedule ``steptab<suffix>``: the packed units keep their order and
    their table entries, but a step takes the next four of them as long as they
    belong to at most two segments; the first segment of a step owns column half
    0, the second half 1.  Raw-byte steps follow unchanged (half 1 all zero)."""
    tab = p['steptab' + suffix]
    n_steps, n_packed = int(p['n_steps' + suffix]), int(p['n_packed_steps' + suffix])
    units = []                                   # table rows of the real packed units, in order
    for m in range(n_packed):
        for g in range(4):
            row = tab[m, g]
            if int(row[7]) != 0:
                units.append(row.copy())
    dense = p['steptab_dense' + suffix]
    dense[...] = 0
    m = i = 0
    while i < len(units):
        step, segs = [], []
        while i < len(units) and len(step) < 4:
            seg = int(units[i][6])
            if seg not in segs:
                if len(segs) == 2:
                    break
                segs.append(seg)
            step.append(units[i])
            i += 1
        for half in range(2):
            own = segs[min(half, len(segs) - 1)]
            for g in range(4):
                row = step[min(g, len(step) - 1)].copy()
                mine = g < len(step) and int(row[6]) == own and (half == 0 or len(segs) == 2)
                row[7] = row[7] if mine else 0
                row[6] = own
                dense[m, half, g] = row
        m += 1
    n_dense_packed = m
    for r in range(n_packed, n_steps):           # raw-byte steps: half 0 as it is, half 1 silent
        if m >= MAX_STEPS:
            raise ValueError("segment table needs more MFMA steps than the plan holds")
        dense[m, 0] = tab[r]
        dense[m, 1] = tab[r]
        dense[m, 1, :, 7] = 0
        m += 1
    p['n_steps_dense' + suffix] = m
    p['n_packed_steps_dense' + suffix] = n_dense_packed


def _byte_pair_table(cb16: np.ndarray, bw: int) -> np.ndarray:
    """Pair table indexed by a byte that holds two codes as nibbles (low nibble first)."""
    b = np.arange(256)
    lo, hi = b & 15, b >> 4
    ok = (lo < (1 << bw)) & (hi < (1 << bw))
    pairs = cb16[np.where(ok, lo, 0)].astype(np.uint32) | (cb16[np.where(ok, hi, 0)].astype(np.uint32) << 16)
    return np.repeat(np.where(ok, pairs, 0).astype(np.uint32), 8)


def _fill_mixed_tables(p) -> None:
    """Step schedule, query units and table image of the mixed K / nibble V layouts."""
    m, n_packed, unit, n_ptab = 0, 0, 1, 0
    p['steptab_mixed'][...] = 0
    p['qunit_dim_mixed'][...] = 0
    p['qunit_len_mixed'][...] = 0
    img = np.zeros(LUTM_IMAGE_BYTES // 4, dtype=np.uint32)
    for s in range(int(p['n_seg'])):
        bw, ln = int(p['seg_bw'][s]), int(p['seg_len'][s])
        start, end = int(p['seg_start'][s]), int(p['seg_start'][s]) + ln
        n_units = (ln + 7) // 8
        unit_bytes = 4 if bw <= 4 else 8
        cb = p['k_codebook_f16'][s]
        if bw <= 4:
            table = n_ptab * 8192                 # at most 4 distinct widths <= 4 bits
            img[table // 4:table // 4 + 2048] = _byte_pair_table(cb, bw)
            n_ptab += 1
        else:
            table = LUTM_KRAW + (bw - 5) * 512
            raw = np.zeros(256, dtype=np.uint16)
            raw[:1 << bw] = cb[:1 << bw]
            img[table // 4:table // 4 + 128] = raw.view(np.uint32)
        for u0 in range(0, n_units, 4):
            if m >= MAX_STEPS:
                raise ValueError("segment table needs more MFMA steps than the plan holds")
            nu = min(4, n_units - u0)
            off0 = int(p['seg_mixed_off'][s]) + u0 * unit_bytes
            for g in range(4):
                gg = min(g, nu - 1)
                q_off = 0
                if g < nu:
                    d0 = start + (u0 + g) * 8
                    p['qunit_dim_mixed'][unit], p['qunit_len_mixed'][unit] = d0, min(8, end - d0)
                    q_off = 16 * unit
                    unit += 1
                p['steptab_mixed'][m, g] = (off0 + gg * unit_bytes, 0, table, 7 * 4 if bw <= 4 else 0,
                                            8 if bw <= 4 else 0, 5, s * 128, q_off)
            n_packed += bw <= 4
            m += 1
    p['n_steps_mixed'] = m
    p['n_packed_steps_mixed'] = n_packed
    vb = int(p['v_bits'])
    if 1 <= vb <= 4:
        img[LUTM_V // 4:LUTM_V // 4 + 2048] = _byte_pair_table(p['v_lut_f16'], vb)
    p['lut_image_mixed'] = img
    _fill_dense(p, '_mixed')


def build_head_plan(quantizer) -> np.ndarray:
    """Fill one ``bgtq_head_plan`` from a calibrated ``BlockGTQQuantizer``
    whose V quantizer has been initialised."""
    q = quantizer
    hd = q.head_dim
    if hd != HEAD_DIM:
        raise ValueError(f"kernels are built for head_dim {HEAD_DIM}, got {hd}")
    pm = q._pack_meta
    widths = [bw for bw in range(1, 9) if bw in pm]
    if len(widths) > MAX_SEGMENTS:
        raise ValueError("more than 8 distinct bit widths")
    p = np.zeros((), dtype=PLAN_DTYPE)
    p['n_seg'] = len(widths)
    p['n_zero_dims'] = q._n_zero_dims
    p['k_row_bytes'] = pm['total_packed_bytes']
    p['nopack_start'] = pm['nopack_start']
    p['nopack_len'] = pm['nopack_len']
    nib_bytes = (pm['nopack_start'] - q._n_zero_dims) // 2
    p['k_mixed_bytes'] = nib_bytes + pm['nopack_len']
    p['v_bits'] = q._v_bits
    p['k_boundaries'][...] = np.inf
    p['v_boundaries'][...] = np.inf

    cents = q._pos_centroids.detach().cpu().numpy()
    bounds = q._pos_boundaries.detach().cpu().numpy()
    code_lut = q._code_lut.detach().cpu().numpy()
    pos_to_cb = q._pos_to_cb.detach().cpu().numpy()
    group_of = (q._group_of_full.detach().cpu().numpy())
    rot_T = q._block_rot_T.detach().cpu().numpy().astype(np.float32)
    for g, bw in enumerate(widths):
        s, ln = pm[bw]['start'], pm[bw]['length']
        nc = 1 << bw
        p['seg_bw'][g] = bw
        p['seg_start'][g] = s
        p['seg_len'][g] = ln
        p['seg_pack_off'][g] = pm[bw]['pack_offset']
        p['seg_mixed_off'][g] = ((s - q._n_zero_dims) // 2 if bw <= 4
                                 else nib_bytes + (s - pm['nopack_start']))
        blk = rot_T[s:s + ln, s:s + ln]
        p['seg_identity'][g] = int(np.array_equal(blk, np.eye(ln, dtype=np.float32)))
        if not (group_of[s:s + ln] == g).all():
            raise ValueError("segments and norm groups disagree")
        cb = int(pos_to_cb[s])
        if not (pos_to_cb[s:s + ln] == cb).all():
            raise ValueError("a segment uses more than one codebook")
        p['code_lut'][g] = code_lut[cb]
        p['k_centroids'][g, :nc] = cents[s, :nc]
        p['k_boundaries'][g, :nc - 1] = bounds[s, :nc - 1]
        p['k_codebook_f16'][g, :nc] = cents[s, :nc].astype(np.float16).view(np.uint16)
    p['head_perm'] = q._head_perm.detach().cpu().numpy().astype(np.int32)
    p['group_of'] = group_of.astype(np.int32)
    p['lut_offset'] = q._lut_offsets.detach().cpu().numpy()
    p['lut_inv_scale'] = q._lut_inv_scales.detach().cpu().numpy()
    p['k_rot_T'] = rot_T.reshape(-1)

    nv = 1 << q._v_bits
    vc = q._v_centroids_f32.detach().cpu().numpy()
    p['v_centroids'][:nv] = vc
    p['v_boundaries'][:nv - 1] = q._v_boundaries.detach().cpu().numpy()
    p['v_lut_f16'][:nv] = vc.astype(np.float16).view(np.uint16)
    p['v_rot_T'] = q._v_rot_T.detach().cpu().numpy().astype(np.float32).reshape(-1)
    p['v_rot'] = q._v_rot.detach().cpu().numpy().astype(np.float32).reshape(-1)
    fill_decode_steps(p)
    return p.reshape(1)


def stack_plans(quantizers) -> np.ndarray:
    """Plans of all KV heads of one layer as one (n_kv,) structured array."""
    return np.concatenate([build_head_plan(q) for q in quantizers])


def upload_plans(plans: np.ndarray, device) -> torch.Tensor:
    """Copy a structured plan array to ``device`` as a flat uint8 tensor."""
    raw = torch.from_numpy(np.ascontiguousarray(plans).view(np.uint8).copy())
    return raw.to(device)


def cache_row_bytes(record_bytes: int) -> int:
    """Row width of a packed K or V cache for records of ``record_bytes``: a multiple
    of 4 (rows start on a dword) that is not a multiple of 32.  The decode kernel
    keeps a tile of rows in LDS at this stride and 16 lanes read the same column
    of 16 consecutive rows; with a stride of 32, 64, 96 or 128 bytes those reads
    fall on a quarter of the 64 LDS banks and serialise four-fold.  A 128-byte
    record keeps its width: rows wider than that are beyond what the encoders
    and the fast decode kernel take."""
    row = max(4, (int(record_bytes) + 3) // 4 * 4)
    return row + 4 if row % 32 == 0 and row < HEAD_DIM else row

