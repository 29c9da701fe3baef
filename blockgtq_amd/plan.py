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
MAX_UNITS = 24
MAX_WALK = 12
ROT_COL = 48

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
    ('k_rot_cols', '<f4', (_D, ROT_COL)), ('rot_compact', '<i4', (4,)),
    ('enc_dim', '<i4', (_D, 4)), ('enc_byte', '<u4', (2, _D, 2)),
    ('v_centroids', '<f4', (16,)), ('v_boundaries', '<f4', (16,)),
    ('v_lut_f16', '<u2', (16,)),
    ('v_rot_T', '<f4', (_D * _D,)), ('v_rot', '<f4', (_D * _D,)),
    ('v_rot_T4', '<f4', (_D // 4, _D, 4)), ('enc_vbyte', '<u4', (2, _D // 2, 2)),
    ('n_units', '<i4', (2,)), ('n_pair_units', '<i4', (2,)),
    ('kend', '<u4', (2,)), ('kfirst', '<u4', (2, 2)), ('reserved1', '<u4', (2,)),
    ('kprog', '<u4', (2, MAX_UNITS, 8)), ('kunit', '<u4', (2, MAX_UNITS)),
    ('swalk', '<u4', (2, MAX_WALK, 4)), ('n_walk', '<u4', (4,)), ('sunit', '<u4', (2, MAX_UNITS)),
    ('lut_image', '<u4', (2, 20480 // 4)), ('vlut_image', '<u4', (2, 8192 // 4)),
], align=True)

# byte offsets inside lut_image[K_BITPACKED] / lut_image[K_MIXED] (BGTQ_LUT_* / BGTQ_LUTM_* of include/bgtq.h)
LUT_K = {3: 0, 2: 8192, 4: 10240, 1: 11264}    # each on a multiple of its size once VLUT_BYTES is added
LUT_KRAW, LUT_K5P, LUT_IMAGE_BYTES = 11776, 13824, 20480
LUT_KQ = {1: 17920, 2: 18432}                  # four codes per 8-byte entry (decode kernel, bit-packed image)
LUTM_KRAW = 4096
VLUT_BYTES = 8192          # the kernel's table area starts with the V table; the K image follows it


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


def _replicas(bw: int) -> int:
    """Copies of every pair-table entry: 32 (one per lane of a half-wave) for tables of at most
    64 entries, none for the 256-entry table."""
    return 32 if bw <= 3 else 1


def _pair_table(cb16: np.ndarray, bw: int) -> np.ndarray:
    """Pair table of one code width, entry (c0 | c1 << bw), bank-replicated for bw <= 3."""
    e = np.arange(1 << (2 * bw))
    pairs = cb16[e & ((1 << bw) - 1)].astype(np.uint32) | (cb16[e >> bw].astype(np.uint32) << 16)
    return np.repeat(pairs, _replicas(bw))


def _byte_pair_table(cb16: np.ndarray, bw: int) -> np.ndarray:
    """256-entry pair table indexed by a byte that holds two codes as nibbles (low nibble first)."""
    b = np.arange(256)
    lo, hi = b & 15, b >> 4
    ok = (lo < (1 << bw)) & (hi < (1 << bw))
    pairs = cb16[np.where(ok, lo, 0)].astype(np.uint32) | (cb16[np.where(ok, hi, 0)].astype(np.uint32) << 16)
    return np.where(ok, pairs, 0).astype(np.uint32)


def _quad_table(cb16: np.ndarray, bw: int) -> np.ndarray:
    """Entry i = c0 | c1 << bw | c2 << 2 bw | c3 << 3 bw -> two words: (cb[c0] | cb[c1] << 16, cb[c2] | cb[c3] << 16)."""
    i = np.arange(1 << (4 * bw))
    m = (1 << bw) - 1
    c = [cb16[(i >> (k * bw)) & m].astype(np.uint32) for k in range(4)]
    return np.stack([c[0] | (c[1] << 16), c[2] | (c[3] << 16)], axis=1).reshape(-1)


def _raw_table(cb16: np.ndarray, bw: int) -> np.ndarray:
    raw = np.zeros(256, dtype=np.uint16)
    raw[:1 << bw] = cb16[:1 << bw]
    return raw.view(np.uint32)




PATH_B1, PATH_B2, PATH_B3, PATH_BYTE, PATH_RAW = 1, 2, 3, 4, 5
STEP_RAW, STEP_RAW5 = 32, 40


def fill_segment_walk(p) -> None:
    """The K record as the decode attention kernel walks it: per layout a list of steps (runs of
    up to 8 units of one segment: kind, table address, byte offset, norm column, first unit) and
    the unit -> dims map."""
    p['swalk'][...] = 0
    p['n_walk'][...] = 0
    p['sunit'][...] = 0
    for layout in (K_BITPACKED, K_MIXED):
        units, steps, n_ptab = [], [], 0
        for s in range(int(p['n_seg'])):
            bw, ln, start = int(p['seg_bw'][s]), int(p['seg_len'][s]), int(p['seg_start'][s])
            if layout == K_BITPACKED:
                off = int(p['seg_pack_off'][s])
                w = bw if bw <= 4 else 0
                table = LUT_K[bw] if bw <= 4 else LUT_K5P if bw == 5 else LUT_KRAW + (bw - 5) * 512
            else:
                off = int(p['seg_mixed_off'][s])
                w = 4 if bw <= 4 else 0
                table = n_ptab * 1024 if bw <= 4 else LUT_K5P if bw == 5 else LUTM_KRAW + (bw - 5) * 512
                n_ptab += bw <= 4
            if bw == 5:
                p['n_walk'][2 + layout] = 1
            n_u = (ln + 7) // 8
            unit_bytes = w if w else 8
            for u0 in range(0, n_u, 8):
                run = min(8, n_u - u0)
                at = off + u0 * unit_bytes
                kind = (w - 1) * 8 + run - 1 if w else (STEP_RAW5 if bw == 5 else STEP_RAW) + run - 1
                steps.append([(at & 3) | (kind << 2), VLUT_BYTES + table,
                              (at & ~3) | (2 * s << 8) | (16 * (len(units) + u0) << 16), 0])
            units += [(start + 8 * u) | (min(8, ln - 8 * u) << 8) for u in range(n_u)]
        if len(units) > MAX_UNITS or len(steps) > MAX_WALK:
            raise ValueError("segment table needs more units or steps than the plan holds")
        p['swalk'][layout, :len(steps)] = steps
        p['n_walk'][layout] = len(steps)
        p['sunit'][layout, :len(units)] = units


def _seg_bytes(bw: int, ln: int) -> int:
    return {1: (ln + 7) // 8, 2: (ln + 3) // 4, 3: (ln + 7) // 8 * 3, 4: (ln + 1) // 2}.get(bw, ln)


def fill_encoder_tables(p) -> None:
    """Per packed dim and per record byte what the K encoder's threads would otherwise derive from
    the segment table: the dim's segment range, source dim and rotation flag, and the codes a
    record byte is made of (both K layouts)."""
    n_seg, D = int(p['n_seg']), HEAD_DIM
    for j in range(D):
        g = int(p['group_of'][j])
        gs = int(p['seg_start'][g]) if g >= 0 else 0
        ge = gs + int(p['seg_len'][g]) if g >= 0 else 0
        ident = int(p['seg_identity'][g]) if g >= 0 else 0
        p['enc_dim'][j] = [g, gs, ge, ident | (int(p['head_perm'][j]) << 8)]
    p['enc_byte'][...] = 0
    z, nps, npl = int(p['n_zero_dims']), int(p['nopack_start']), int(p['nopack_len'])
    for j in range(D):
        for layout in (K_BITPACKED, K_MIXED):
            mode = bw = c0 = clen = idx = 0
            if layout == K_MIXED:
                nib = (nps - z) >> 1
                if j < nib:
                    mode, bw, c0, clen, idx = 1, 4, z, nps - z, j
                elif j < nib + npl:
                    mode, c0 = 2, nps + (j - nib)
            else:
                for s in range(n_seg):
                    off, sb, sl = int(p['seg_pack_off'][s]), int(p['seg_bw'][s]), int(p['seg_len'][s])
                    if off <= j < off + _seg_bytes(sb, sl):
                        if sb >= 5:
                            mode, c0 = 2, int(p['seg_start'][s]) + (j - off)
                        else:
                            mode, bw, c0, clen, idx = 1, sb, int(p['seg_start'][s]), sl, j - off
            if mode == 1:
                bit0 = idx * 8
                first = bit0 // bw
                skip = bit0 - first * bw
                last = min((bit0 + 7) // bw, clen - 1)
                n = max(last - first + 1, 0)
                p['enc_byte'][layout, j] = [1 | (bw << 2) | (skip << 6) | (n << 8), c0 + first]
            elif mode == 2:
                p['enc_byte'][layout, j] = [2, c0]


def fill_decode_steps(p) -> None:
    """Derive the unit programs of both K record layouts and the table images from the
    segment table, codebooks and V LUT already stored in plan ``p`` (a 0-d structured array)."""
    for f in ('kprog', 'kunit', 'n_units', 'n_pair_units', 'kend', 'kfirst'):
        p[f][...] = 0
    for layout in (K_BITPACKED, K_MIXED):
        img = np.zeros(LUT_IMAGE_BYTES // 4, dtype=np.uint32)
        units, progs, offs = [], [], []     # per unit: dims, parameter row (without the next unit's offset), byte offset
        n_ptab = n_pair = kend = 0
        for s in range(int(p['n_seg'])):
            bw, ln = int(p['seg_bw'][s]), int(p['seg_len'][s])
            start = int(p['seg_start'][s])
            cb = p['k_codebook_f16'][s]
            seg_off = int(p['seg_pack_off' if layout == K_BITPACKED else 'seg_mixed_off'][s])
            n_u = (ln + 7) // 8
            if bw <= 4:
                if n_pair != len(units):
                    raise ValueError("a pair-table segment follows a raw-byte segment")
                if layout == K_BITPACKED:
                    table, unit_bytes, pw = LUT_K[bw], bw, 2 * bw
                    t = _pair_table(cb, bw)
                    tsh, rep_mask = (7, 31 * 4) if bw <= 3 else (2, 0)
                else:
                    table, unit_bytes, pw, tsh, rep_mask = n_ptab * 1024, 4, 8, 2, 0
                    t = _byte_pair_table(cb, bw)
                    n_ptab += 1
                img[table // 4:table // 4 + t.size] = t
                if layout == K_BITPACKED and bw in LUT_KQ:
                    q = _quad_table(cb, bw)
                    img[LUT_KQ[bw] // 4:LUT_KQ[bw] // 4 + q.size] = q
                row = [(pw * i - tsh) % 32 for i in range(4)] + [((1 << pw) - 1) << tsh, VLUT_BYTES + table, rep_mask]
                n_pair += n_u
            else:
                table = (LUT_KRAW if layout == K_BITPACKED else LUTM_KRAW) + (bw - 5) * 512
                img[table // 4:table // 4 + 128] = _raw_table(cb, bw)
                if bw == 5:
                    e = np.arange(1024)
                    img[LUT_K5P // 4:LUT_K5P // 4 + 1024] = cb[e & 31].astype(np.uint32) | (cb[e >> 5].astype(np.uint32) << 16)
                unit_bytes = 8
                row = [0, 0, 0, 0, 0, VLUT_BYTES + table, 0]
            if bw > 4 and len(units) % 2:
                # the kernel takes pair-table units two at a time: an empty unit evens them out
                units.append(0)
                progs.append([0] * 7)
                offs.append(0)
                n_pair += 1
            for u in range(n_u):
                d0 = start + 8 * u
                units.append(d0 | (min(8, start + ln - d0) << 8))
                progs.append(row)
                offs.append(seg_off + u * unit_bytes)
            kend |= 1 << (len(units) - 1)
        if n_pair == len(units) and n_pair % 2:
            units.append(0)
            progs.append([0] * 7)
            offs.append(0)
            n_pair += 1
        if len(units) > MAX_UNITS:
            raise ValueError("segment table needs more units than the plan holds")
        for u, row in enumerate(progs):
            p['kprog'][layout, u] = row + [offs[u + 2] if u + 2 < len(units) else 0]
        p['kunit'][layout, :len(units)] = units
        p['n_units'][layout] = len(units)
        p['n_pair_units'][layout] = n_pair
        p['kend'][layout] = kend
        p['kfirst'][layout] = (offs + [0, 0])[:2]
        p['lut_image'][layout] = img
    vb = int(p['v_bits'])
    p['vlut_image'][...] = 0
    if 1 <= vb <= 4:
        t = _pair_table(p['v_lut_f16'], vb)
        p['vlut_image'][V_BITPACKED, :t.size] = t
        p['vlut_image'][V_NIBBLE, :256] = _byte_pair_table(p['v_lut_f16'], vb)
    fill_segment_walk(p)
    fill_encoder_tables(p)


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
    # the rotation by columns, each cut down to its own diagonal block (read by the single-row append)
    p['k_rot_cols'][...] = 0
    compact = True
    for g in range(len(widths)):
        s0, ln = int(p['seg_start'][g]), int(p['seg_len'][g])
        if int(p['seg_identity'][g]):
            continue
        if ln > ROT_COL:
            compact = False
            continue
        p['k_rot_cols'][s0:s0 + ln, :ln] = rot_T[s0:s0 + ln, s0:s0 + ln].T
    p['rot_compact'][...] = 0
    p['rot_compact'][0] = int(compact)

    nv = 1 << q._v_bits
    vc = q._v_centroids_f32.detach().cpu().numpy()
    p['v_centroids'][:nv] = vc
    p['v_boundaries'][:nv - 1] = q._v_boundaries.detach().cpu().numpy()
    p['v_lut_f16'][:nv] = vc.astype(np.float16).view(np.uint16)
    p['v_rot_T'] = q._v_rot_T.detach().cpu().numpy().astype(np.float32).reshape(-1)
    p['v_rot'] = q._v_rot.detach().cpu().numpy().astype(np.float32).reshape(-1)
    p['v_rot_T4'] = p['v_rot_T'].reshape(HEAD_DIM // 4, 4, HEAD_DIM).transpose(0, 2, 1)
    p['enc_vbyte'][...] = 0
    for layout, bw in ((V_BITPACKED, int(q._v_bits)), (V_NIBBLE, 4)):
        for j in range(HEAD_DIM * bw // 8):
            first = j * 8 // bw
            skip = j * 8 - first * bw
            n = min((j * 8 + 7) // bw, HEAD_DIM - 1) - first + 1
            p['enc_vbyte'][layout, j] = [1 | (bw << 2) | (skip << 6) | (n << 8), first]
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

