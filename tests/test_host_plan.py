"""Host-side plan builders against closed forms, invariants and brute force."""
import ctypes
import itertools
import math
import re
import os

import numpy as np
import pytest
import torch

from blockgtq_amd import BlockGTQPipeline, BlockGTQQuantizer, greedy_bit_allocation
from blockgtq_amd import codebooks, plan as P, v_packing
from blockgtq_amd.quantizer import build_pack_meta
from helpers import make_kv, make_quantizer, stream_pack

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


# ---------------------------------------------------------------- allocator
def _objective(s, b):
    return float((np.asarray(s, dtype=np.float64) * 4.0 ** (-np.asarray(b, dtype=np.float64))).sum())


@pytest.mark.parametrize("seed", range(6))
def test_allocator_is_the_exact_optimum_on_small_problems(seed):
    rng = np.random.default_rng(seed)
    n = int(rng.integers(2, 6))
    lo, hi = int(rng.integers(0, 2)), int(rng.integers(3, 5))
    budget = int(rng.integers(n * lo, n * hi + 1))
    s = torch.tensor(rng.uniform(0.01, 50.0, n), dtype=torch.float32)
    got = greedy_bit_allocation(s, budget, lo, hi).numpy()
    assert got.sum() == budget and got.min() >= lo and got.max() <= hi
    best = min(_objective(s.numpy(), b)
               for b in itertools.product(range(lo, hi + 1), repeat=n) if sum(b) == budget)
    assert _objective(s.numpy(), got) == pytest.approx(best, rel=1e-12)


def test_allocator_invariants_and_ties():
    s = torch.ones(8)
    # equal scores: bits go to the lowest indices first
    assert greedy_bit_allocation(s, 8 + 3, 1, 4).tolist() == [2, 2, 2, 1, 1, 1, 1, 1]
    # monotone in the score
    s = torch.tensor([0.1, 1.0, 10.0, 100.0])
    a = greedy_bit_allocation(s, 12, 1, 8).tolist()
    assert a == sorted(a) and sum(a) == 12
    # budget below the floor: everything stays at min_bits
    assert greedy_bit_allocation(s, 2, 1, 8).tolist() == [1, 1, 1, 1]
    # budget above the ceiling: saturates at max_bits
    assert greedy_bit_allocation(s, 99, 1, 3).tolist() == [3, 3, 3, 3]
    # zero scores never receive bits beyond the floor
    assert greedy_bit_allocation(torch.tensor([0.0, 1.0]), 6, 0, 8).tolist() == [0, 6]


# ---------------------------------------------------------------- codebooks
def test_centroid_closed_forms():
    d = 36
    c1 = codebooks.lloyd_max_centroids(1, d)
    assert np.allclose(c1, [-math.sqrt(2 / (math.pi * d)), math.sqrt(2 / (math.pi * d))], rtol=0, atol=1e-15)
    c2 = codebooks.lloyd_max_centroids(2, d)
    assert np.allclose(c2 * math.sqrt(d), [-1.51, -0.453, 0.453, 1.51], atol=1e-12)
    # textbook Lloyd-Max levels of the unit Gaussian, 8 and 16 levels
    c3 = codebooks.lloyd_max_centroids(3, d) * math.sqrt(d)
    assert np.allclose(c3[4:], [0.2451, 0.7560, 1.3439, 2.1520], atol=2e-4)
    assert np.allclose(c3, -c3[::-1], atol=1e-9)
    # 16 levels: 100 Lloyd iterations stop a little short of the textbook optimum
    c4 = codebooks.lloyd_max_centroids(4, d) * math.sqrt(d)
    assert np.allclose(c4[8:], [0.1284, 0.3881, 0.6568, 0.9424, 1.2562, 1.6181, 2.0690, 2.7326], atol=2e-2)
    assert np.allclose(c4, -c4[::-1], atol=1e-9)


def _cell_means_by_quadrature(edges, sig):
    from scipy.stats import norm
    from scipy import integrate
    ext = np.concatenate([[-14 * sig], edges, [14 * sig]])
    out = []
    for lo, hi in zip(ext[:-1], ext[1:]):
        num = integrate.quad(lambda x: x * norm.pdf(x, scale=sig), lo, hi, epsabs=0, epsrel=1e-12)[0]
        den = integrate.quad(lambda x: norm.pdf(x, scale=sig), lo, hi, epsabs=0, epsrel=1e-12)[0]
        out.append(num / den)
    return np.array(out)


def test_three_bit_centroids_are_a_lloyd_fixed_point():
    d = 128
    c = codebooks.lloyd_max_centroids(3, d)
    again = _cell_means_by_quadrature((c[:-1] + c[1:]) / 2, 1 / math.sqrt(d))
    assert np.allclose(c, again, rtol=1e-7, atol=1e-10)


def test_lloyd_schedule_against_numerical_integration():
    """100 Lloyd iterations from the equal-mass cells, cell means by quadrature
    instead of the pdf/cdf closed form."""
    from scipy.stats import norm
    bw, d = 4, 20
    sig = 1 / math.sqrt(d)
    n = 1 << bw
    c = _cell_means_by_quadrature(norm.ppf(np.linspace(0, 1, n + 1)[1:-1], scale=sig), sig)
    for _ in range(100):
        c = _cell_means_by_quadrature((c[:-1] + c[1:]) / 2, sig)
    assert np.allclose(codebooks.lloyd_max_centroids(bw, d), np.sort(c), rtol=1e-7, atol=1e-10)


@pytest.mark.parametrize("fix", [True, False])
def test_rotation_is_proper_and_deterministic(fix):
    r = codebooks.haar_rotation(48, 45, zero_sign_fix=fix)
    assert np.allclose(r.T @ r, np.eye(48), atol=1e-12)
    assert np.linalg.det(r) == pytest.approx(1.0, abs=1e-10)
    assert np.array_equal(r, codebooks.haar_rotation(48, 45, zero_sign_fix=fix))
    assert not np.allclose(r, codebooks.haar_rotation(48, 46, zero_sign_fix=fix))
    # uniqueness of QR with positive diag(R): Q^T G must be upper triangular, diag > 0
    g = np.random.default_rng(45).standard_normal((48, 48))
    rr = r.T @ g
    rr[:, 0] *= 1.0  # no-op, keeps the intent readable
    lower = np.tril(rr, -1)
    if np.linalg.det(np.linalg.qr(g)[0] * np.sign(np.diag(np.linalg.qr(g)[1]))) > 0:
        assert np.allclose(lower, 0, atol=1e-10) and (np.diag(rr) > 0).all()


def test_mc_lloyd_centroids_properties():
    c = codebooks.mc_lloyd_centroids(3, 128)
    assert c.shape == (8,) and (np.diff(c) > 0).all()
    # fixed point on its own sample set
    sig = 1 / np.sqrt(128)
    x = np.random.default_rng(0).normal(0, sig, 100000)
    cell = np.searchsorted((c[:-1] + c[1:]) / 2, x)
    means = np.array([x[cell == i].mean() for i in range(8)])
    assert np.allclose(c, means, atol=2e-8)
    # and close to the analytic Lloyd-Max levels (sampling noise of 100k draws)
    assert np.allclose(c, codebooks.lloyd_max_centroids(3, 128), atol=1.5e-3)


def test_code_lut_is_nearest_centroid_of_bin_centres():
    q, _ = make_quantizer(seed=3, max_bits=6)
    lut = q._code_lut.numpy()
    for g, bw in enumerate(q._group_bits):
        s = q._pack_meta[bw]['start']
        c = q._pos_centroids[s, :1 << bw].double().numpy()
        off, inv = float(q._lut_offsets[s]), float(q._lut_inv_scales[s])
        centres = off + (np.arange(256) + 0.5) / inv
        nearest = np.abs(centres[:, None] - c[None, :]).argmin(1)
        row = lut[int(q._pos_to_cb[s])]
        assert (np.diff(row.astype(int)) >= 0).all()
        assert row[0] == 0 and row[-1] == (1 << bw) - 1
        # bins whose centre sits within fp32 noise of a boundary may go either way
        b = (c[:-1] + c[1:]) / 2
        near = np.abs(centres[:, None] - b[None, :]).min(1) < 1e-6
        assert (row[~near] == nearest[~near]).all()
        # table spans [c_min - sp/2, c_max + sp/2]
        sp = (c[-1] - c[0]) / (len(c) - 1)
        assert off == pytest.approx(c[0] - sp / 2, rel=1e-6)
        assert 256 / inv == pytest.approx(c[-1] - c[0] + sp, rel=1e-6)


# ---------------------------------------------------------------- pipeline
def test_pipeline_layout_invariants():
    q, _ = make_quantizer(seed=5, min_bits=0, max_bits=6, budget=160)
    bits = q.bit_allocation
    hp = q._head_perm
    per_dim = torch.cat([bits, bits])[hp]
    assert sorted(hp.tolist()) == list(range(128))
    assert (per_dim[1:] >= per_dim[:-1]).all()
    assert ((hp[1::2] - hp[0::2]) == 64).all()            # a block's two dims stay adjacent
    rot = q._block_rot_T.T
    assert torch.allclose(rot @ rot.T, torch.diag((per_dim > 0).float()), atol=1e-5)
    for g, bw in enumerate(q._group_bits):
        m = q._pack_meta[bw]
        s, e = m['start'], m['start'] + m['length']
        blk = rot[s:e, s:e]
        assert rot[s:e, :s].abs().sum() == 0 and rot[s:e, e:].abs().sum() == 0
        if bw < q.rotation_threshold:
            assert torch.equal(blk, torch.eye(e - s))
        else:
            assert not torch.equal(blk, torch.eye(e - s))
        assert (q._group_of_full[s:e] == g).all()
    assert (q._group_of_full[:q._n_zero_dims] == -1).all()


def test_pack_meta_sizes_match_the_documented_example():
    # 1b x 10 blocks, 2b x 12, 3b x 18, 4b x 16, 5b x 8 -> bytes 3+6+15+16+16 = 56
    alloc = torch.tensor([1] * 10 + [2] * 12 + [3] * 18 + [4] * 16 + [5] * 8)
    pipe = BlockGTQPipeline(128, device='cpu')
    pipe.set_allocation(alloc)
    pm = build_pack_meta(alloc, pipe._head_perm)
    assert [pm[b]['length'] for b in (1, 2, 3, 4, 5)] == [20, 24, 36, 32, 16]
    assert [pm[b]['packed_bytes'] for b in (1, 2, 3, 4, 5)] == [3, 6, 15, 16, 16]
    assert [pm[b]['pack_offset'] for b in (1, 2, 3, 4, 5)] == [0, 3, 9, 24, 40]
    assert pm['total_packed_bytes'] == 56
    assert (pm['nopack_start'], pm['nopack_len'], pm['nopack_off']) == (112, 16, 40)
    # widths <= 4 only: the raw-byte run starts past the end of the vector
    pm = build_pack_meta(torch.full((64,), 3), BlockGTQPipeline(128, device='cpu')._head_perm
                         if False else torch.arange(128).view(2, 64).T.reshape(-1))
    assert pm['nopack_start'] == 128 and pm['nopack_len'] == 0 and pm['total_packed_bytes'] == 48


def test_plan_struct_mirrors_the_quantizer():
    q, _ = make_quantizer(seed=9, max_bits=7, budget=200)
    p = q.plan()[0]
    n = int(p['n_seg'])
    assert n == q._n_groups
    assert int(p['k_row_bytes']) == q._total_packed_bytes
    assert int(p['k_mixed_bytes']) == q._pack_meta['nopack_start'] // 2 + q._pack_meta['nopack_len']
    assert sum(int(x) for x in p['seg_len'][:n]) == 128
    for g in range(n):
        bw = int(p['seg_bw'][g])
        nc = 1 << bw
        assert np.isinf(p['k_boundaries'][g][nc - 1:]).all()
        c = p['k_centroids'][g][:nc]
        assert np.allclose(p['k_boundaries'][g][:nc - 1], (c[:-1] + c[1:]) / 2, atol=1e-7)
        assert np.array_equal(p['k_codebook_f16'][g][:nc].view(np.float16), c.astype(np.float16))
    assert np.array_equal(p['v_rot'].reshape(128, 128), p['v_rot_T'].reshape(128, 128).T)     # (the V append reads columns of one as rows of the other)


def _unit_fields(row):
    """Fields of a unit's parameter row (include/bgtq.h, bgtq_head_plan.kprog); next_off is the byte
    offset of the unit after the next."""
    return dict(rot=[int(x) for x in row[0:4]], mask=int(row[4]), table=int(row[5]), rep_mask=int(row[6]),
                next_off=int(row[7]))


@pytest.mark.parametrize("seed,min_bits,max_bits,budget", [(9, 1, 7, 200), (4, 0, 4, 128), (5, 1, 5, 192)])
def test_decode_schedule_and_tables_cover_the_record(seed, min_bits, max_bits, budget):
    """The unit programs and the table images in the plan, checked against what they stand for:
    every packed dim of every segment is read exactly once through a query range, unit byte offsets
    walk each segment's stream (every row names the offset of the unit two on), the last unit of
    every segment is flagged, pair-table units come before raw-byte units and are an even number, the rotations bring every
    code pair of a unit to the entry-index position of its table, and a pair-table entry
    (c0 | c1 << bw) holds the two fp16 centroids, in every bank replica."""
    from blockgtq_amd import plan as P
    q, _ = make_quantizer(seed=seed, min_bits=min_bits, max_bits=max_bits, budget=budget)
    p = q.plan()[0]
    n_seg = int(p['n_seg'])
    for layout in (P.K_BITPACKED, P.K_MIXED):
        n_units = int(p['n_units'][layout])
        assert 1 <= n_units <= P.MAX_UNITS
        assert not p['kunit'][layout, n_units:].any() and not p['kprog'][layout, n_units:].any()
        seen = np.zeros(128, dtype=int)
        u, n_ptab, n_pair, kend = 0, 0, 0, 0
        offs = [int(x) for x in p['kfirst'][layout]]          # byte offsets of the units, as the rows chain them
        for s in range(n_seg):
            bw = int(p['seg_bw'][s])
            start, length = int(p['seg_start'][s]), int(p['seg_len'][s])
            seg_off = int(p['seg_mixed_off' if layout else 'seg_pack_off'][s])
            unit_bytes = 8 if bw > 4 else (bw if layout == P.K_BITPACKED else 4)
            if bw > 4 and u % 2 and n_pair == u:
                # the empty unit that makes the number of pair-table units even
                assert int(p['kunit'][layout, u]) == 0 and not p['kprog'][layout, u, :7].any()
                offs.append(int(p['kprog'][layout, u, 7]))
                u += 1
                n_pair += 1
            for i in range((length + 7) // 8):
                f = _unit_fields(p['kprog'][layout, u])
                d0, ln = int(p['kunit'][layout, u]) & 0xFF, int(p['kunit'][layout, u]) >> 8
                assert d0 == start + 8 * i and ln == min(8, start + length - d0) and ln >= 1
                assert offs[u] == seg_off + i * unit_bytes
                offs.append(f['next_off'])
                seen[d0:d0 + ln] += 1
                if bw > 4:
                    assert f['rep_mask'] == 0 and f['mask'] == 0
                    assert f['table'] == P.VLUT_BYTES + (P.LUTM_KRAW if layout else P.LUT_KRAW) + (bw - 5) * 512
                else:
                    assert n_pair == u                    # no raw-byte unit so far
                    n_pair += 1
                    if layout == P.K_BITPACKED:
                        pw, tsh = 2 * bw, (7 if bw <= 3 else 2)
                        assert f['table'] == P.VLUT_BYTES + P.LUT_K[bw]
                        assert f['rep_mask'] == (124 if bw <= 3 else 0)
                    else:
                        pw, tsh = 8, 2
                        assert f['table'] == P.VLUT_BYTES + 1024 * n_ptab and f['rep_mask'] == 0
                    assert f['mask'] == ((1 << pw) - 1) << tsh
                    unit = 0x9E3779B9 & ((1 << (4 * pw)) - 1)            # any bit pattern of the unit's width
                    for k in range(4):
                        rot = ((unit >> f['rot'][k]) | (unit << (32 - f['rot'][k]))) & 0xFFFFFFFF
                        assert (rot & f['mask']) >> tsh == (unit >> (pw * k)) & ((1 << pw) - 1)
                u += 1
            if bw <= 4 and layout == P.K_MIXED:
                n_ptab += 1
            kend |= 1 << (u - 1)
        if n_pair == u and u % 2:                             # all units are pair-table units, an odd number
            assert int(p['kunit'][layout, u]) == 0 and not p['kprog'][layout, u].any()
            offs.append(0)
            u += 1
            n_pair += 1
        assert u == n_units and offs[n_units:] == [0, 0]
        assert int(p['n_pair_units'][layout]) == n_pair and n_pair % 2 == 0 and int(p['kend'][layout]) == kend
        z = int(p['n_zero_dims'])
        assert (seen[z:] == 1).all() and (seen[:z] == 0).all()
    img = p['lut_image'][P.K_BITPACKED]
    imgm = p['lut_image'][P.K_MIXED]
    i_ptab = 0
    for s in range(n_seg):
        bw = int(p['seg_bw'][s])
        cb = p['k_codebook_f16'][s]
        if bw <= 4:
            rep = 1 if bw == 4 else 32
            t = img[P.LUT_K[bw] // 4:][:(1 << 2 * bw) * rep].reshape(-1, rep)
            assert (t == t[:, :1]).all()
            tm = imgm[256 * i_ptab:256 * (i_ptab + 1)]
            i_ptab += 1
            for c0 in range(1 << bw):
                for c1 in range(1 << bw):
                    assert int(t[c0 | (c1 << bw), 0]) == int(cb[c0]) | (int(cb[c1]) << 16)
                    assert int(tm[c0 | (c1 << 4)]) == int(cb[c0]) | (int(cb[c1]) << 16)
            if bw in P.LUT_KQ:        # four codes an entry: the halves of its two words in code order
                tq = img[P.LUT_KQ[bw] // 4:][:2 << (4 * bw)].view(np.uint16).reshape(-1, 4)
                for i in range(1 << (4 * bw)):
                    assert [int(x) for x in tq[i]] == [int(cb[(i >> (k * bw)) & ((1 << bw) - 1)]) for k in range(4)]
        else:
            for im, base in ((img, P.LUT_KRAW), (imgm, P.LUTM_KRAW)):
                raw = im[(base + (bw - 5) * 512) // 4:][:128].view(np.uint16)
                assert np.array_equal(raw[:1 << bw], cb[:1 << bw]) and not raw[1 << bw:].any()
    vb = int(p['v_bits'])
    rep = 1 if vb == 4 else 32
    tv = p['vlut_image'][P.V_BITPACKED][:(1 << 2 * vb) * rep].reshape(-1, rep)
    tn = p['vlut_image'][P.V_NIBBLE][:256]
    vl = p['v_lut_f16']
    for c0 in range(1 << vb):
        for c1 in range(1 << vb):
            assert (tv[c0 | (c1 << vb)] == (int(vl[c0]) | (int(vl[c1]) << 16))).all()
            assert int(tn[c0 | (c1 << 4)]) == int(vl[c0]) | (int(vl[c1]) << 16)


@pytest.mark.parametrize("alloc", [None, [3] * 64, [1, 2, 3] + [4] * 5 + [5] + [8] * 55, [5] * 40 + [2] * 24])
def test_record_walk_covers_every_unit_once(alloc):
    """The decode kernel's walk over a K record: steps of at most 8 units, each inside one segment,
    in record order; a step's byte offset, first unit, norm column, kind and table follow from the
    segment table; units tile the segments' dims; 5-bit codes come with their pair table."""
    from blockgtq_amd import plan as P
    q, _ = make_quantizer(seed=17, min_bits=1, max_bits=8, budget=200, alloc=alloc)
    p = q.plan()[0]
    n_seg = int(p['n_seg'])
    for layout in (P.K_BITPACKED, P.K_MIXED):
        n_walk = int(p['n_walk'][layout])
        assert 1 <= n_walk <= P.MAX_WALK and not p['swalk'][layout, n_walk:].any()
        steps = [[int(x) for x in row] for row in p['swalk'][layout, :n_walk]]
        units = [int(x) for x in p['sunit'][layout]]
        i = u = n_ptab = 0
        for s in range(n_seg):
            bw, ln, start = int(p['seg_bw'][s]), int(p['seg_len'][s]), int(p['seg_start'][s])
            off = int(p['seg_pack_off' if layout == P.K_BITPACKED else 'seg_mixed_off'][s])
            w = (bw if layout == P.K_BITPACKED else 4) if bw <= 4 else 0
            n_u = (ln + 7) // 8
            for k in range(n_u):                                   # the unit map: 8 dims a unit, the last one shorter
                assert units[u + k] == (start + 8 * k) | (min(8, ln - 8 * k) << 8)
            done = 0
            while done < n_u:
                w0, tab, w2, w3 = steps[i]
                run = min(8, n_u - done)
                at = off + done * (w if w else 8)
                kind = (w - 1) * 8 + run - 1 if w else (P.STEP_RAW5 if bw == 5 else P.STEP_RAW) + run - 1
                assert w0 == (at & 3) | (kind << 2) and w3 == 0
                assert w2 == (at & ~3) | (2 * s << 8) | (16 * (u + done) << 16)
                if w and layout == P.K_BITPACKED:
                    assert tab == P.VLUT_BYTES + P.LUT_K[bw]
                elif w:
                    assert tab == P.VLUT_BYTES + 1024 * n_ptab
                elif bw == 5:
                    assert tab == P.VLUT_BYTES + P.LUT_K5P
                else:
                    assert tab == P.VLUT_BYTES + (P.LUT_KRAW if layout == P.K_BITPACKED else P.LUTM_KRAW) + (bw - 5) * 512
                done += run
                i += 1
            u += n_u
            n_ptab += bw <= 4 and layout == P.K_MIXED
        assert i == n_walk and not any(units[u:])
        has5 = 5 in [int(b) for b in p['seg_bw'][:n_seg]]
        assert int(p['n_walk'][2 + layout]) == int(has5)
        if has5:
            cb = p['k_codebook_f16'][[int(b) for b in p['seg_bw'][:n_seg]].index(5)]
            t = p['lut_image'][layout][P.LUT_K5P // 4:][:1024]
            for c0, c1 in ((0, 0), (31, 0), (0, 31), (7, 19), (31, 31)):
                assert int(t[c0 | (c1 << 5)]) == int(cb[c0]) | (int(cb[c1]) << 16)


@pytest.mark.parametrize("alloc,mn,mx", [(None, 1, 7), (None, 0, 4), ([3] * 64, 1, 8), ([1, 2, 3] + [4] * 5 + [5] + [8] * 55, 1, 8)])
def test_encoder_tables_write_the_record_an_independent_packer_writes(alloc, mn, mx):
    """The K encoder's ready-made tables: `enc_dim` repeats the segment table per dim; a record
    assembled byte by byte from `enc_byte` (mode, width, skip, count, first code) equals, segment by
    segment, the independent LSB-first bit-stream writer (whole 8-code groups for 3-bit codes), the
    nibble stream and the raw bytes; `k_rot_cols` holds every rotated dim's column of its block."""
    from blockgtq_amd import plan as P
    q, _ = make_quantizer(seed=23, min_bits=mn, max_bits=mx, budget=190, alloc=alloc)
    p = q.plan()[0]
    n_seg = int(p['n_seg'])
    segs = [(int(p['seg_bw'][s]), int(p['seg_start'][s]), int(p['seg_len'][s])) for s in range(n_seg)]
    for j in range(128):
        g, gs, ge, w = (int(x) for x in p['enc_dim'][j])
        assert g == int(p['group_of'][j]) and (w >> 8) == int(p['head_perm'][j])
        if g >= 0:
            assert (gs, ge) == (segs[g][1], segs[g][1] + segs[g][2]) and (w & 255) == int(p['seg_identity'][g])
        else:
            assert (gs, ge, w & 255) == (0, 0, 0)
    rng = np.random.default_rng(5)
    codes = np.zeros(128, dtype=np.int64)
    for bw, s0, ln in segs:
        codes[s0:s0 + ln] = rng.integers(0, 1 << bw, ln)

    def assemble(layout, n_bytes):
        out = np.zeros(n_bytes, dtype=np.uint8)
        for j in range(n_bytes):
            w0, first = (int(x) for x in p['enc_byte'][layout, j])
            mode, bw, skip, n = w0 & 3, (w0 >> 2) & 15, (w0 >> 6) & 3, w0 >> 8
            if mode == 1:
                acc = 0
                for i in range(n):
                    acc |= int(codes[first + i]) << (i * bw)
                out[j] = (acc >> skip) & 255
            elif mode == 2:
                out[j] = codes[first]
        return out

    want = np.zeros(int(p['k_row_bytes']), dtype=np.uint8)
    for s, (bw, s0, ln) in enumerate(segs):
        off = int(p['seg_pack_off'][s])
        if bw >= 5:
            want[off:off + ln] = codes[s0:s0 + ln]
        else:
            padded = np.zeros((ln + 7) // 8 * 8 if bw == 3 else ln, dtype=np.int64)
            padded[:ln] = codes[s0:s0 + ln]
            b = stream_pack(padded[None], bw)[0]
            want[off:off + len(b)] = b
    assert np.array_equal(assemble(P.K_BITPACKED, len(want)), want)
    z, nps, npl = int(p['n_zero_dims']), int(p['nopack_start']), int(p['nopack_len'])
    wantm = np.concatenate([stream_pack(codes[None, z:nps], 4)[0], codes[nps:nps + npl].astype(np.uint8)])
    assert len(wantm) == int(p['k_mixed_bytes']) and np.array_equal(assemble(P.K_MIXED, len(wantm)), wantm)
    assert not p['enc_byte'][P.K_BITPACKED, len(want):].any() and not p['enc_byte'][P.K_MIXED, len(wantm):].any()

    rot = p['k_rot_T'].reshape(128, 128)
    short = all(ln <= P.ROT_COL or int(p['seg_identity'][s]) for s, (_, _, ln) in enumerate(segs))
    assert int(p['rot_compact'][0]) == int(short)
    for s, (bw, s0, ln) in enumerate(segs):
        if int(p['seg_identity'][s]) or ln > P.ROT_COL:
            continue
        for j in range(s0, s0 + ln):
            assert np.array_equal(p['k_rot_cols'][j][:ln], rot[s0:s0 + ln, j]) and not p['k_rot_cols'][j][ln:].any()


# ---------------------------------------------------------------- V packing
@pytest.mark.parametrize("bits", [1, 2, 3, 4])
def test_v_packing_matches_a_plain_bit_stream(bits):
    rng = np.random.default_rng(bits)
    codes = rng.integers(0, 1 << bits, size=(17, 128)).astype(np.uint8)
    packed = v_packing.pack_v_codes(torch.tensor(codes), bits).numpy()
    assert packed.shape[1] == v_packing.packed_v_bytes(128, bits) == {1: 16, 2: 32, 3: 48, 4: 64}[bits]
    assert np.array_equal(packed, stream_pack(codes, bits))
    back = v_packing.unpack_v_codes(torch.tensor(packed), bits, 128).numpy()
    assert np.array_equal(back, codes)
    if bits == 3:       # the 8-codes-in-3-bytes formulas
        c = codes[:, :8].astype(int)
        assert np.array_equal(packed[:, 0], (c[:, 0] | c[:, 1] << 3 | c[:, 2] << 6) & 0xFF)
        assert np.array_equal(packed[:, 1], (c[:, 2] >> 2 | c[:, 3] << 1 | c[:, 4] << 4 | c[:, 5] << 7) & 0xFF)
        assert np.array_equal(packed[:, 2], (c[:, 5] >> 1 | c[:, 6] << 2 | c[:, 7] << 5) & 0xFF)


# ---------------------------------------------------------------- library surface
def _emulate_steps(p, rec, norms, qrot, layout):
    """Scores of one token record computed the way the MFMA kernel walks the plan: unit after unit,
    8 codes through the unit's pair table (rotate, mask, read) or raw-byte table times the unit's
    query range, summed over a segment (up to the unit flagged as its last), times the segment's norm."""
    from blockgtq_amd import plan as P
    img = p['lut_image'][layout].view(np.uint8)
    out = np.zeros(qrot.shape[0])
    recp = np.concatenate([rec, np.zeros(16, np.uint8)])
    seg_sum = np.zeros(qrot.shape[0])
    offs, s = [int(x) for x in p['kfirst'][layout]], 0
    for u in range(int(p['n_units'][layout])):
        off = offs[u]
        f = _unit_fields(p['kprog'][layout, u])
        table = f['table'] - P.VLUT_BYTES
        d0, ln = int(p['kunit'][layout, u]) & 0xFF, int(p['kunit'][layout, u]) >> 8
        if u < int(p['n_pair_units'][layout]):
            raw = int.from_bytes(recp[off:off + 4].tobytes(), 'little')
            vals = []
            for k in range(4):
                rot = ((raw >> f['rot'][k]) | (raw << (32 - f['rot'][k]))) & 0xFFFFFFFF
                a = table + (rot & f['mask'])
                vals += list(img[a:a + 4].view(np.float16))
        else:
            vals = [img[table + 2 * int(recp[off + k]):][:2].view(np.float16)[0] for k in range(8)]
        seg_sum += qrot[:, d0:d0 + ln].astype(np.float64) @ np.array(vals[:ln], np.float64)
        offs.append(f['next_off'])
        if (int(p['kend'][layout]) >> u) & 1:
            out += seg_sum * float(norms[s])
            seg_sum[:] = 0
            s += 1
    assert s == int(p['n_seg'])
    return out


@pytest.mark.parametrize("seed,min_bits,max_bits,budget", [(9, 1, 7, 200), (4, 0, 4, 128), (5, 1, 5, 192), (2, 2, 2, 128)])
def test_step_tables_reproduce_the_checker_scores(oracle_lib, seed, min_bits, max_bits, budget):
    """The step schedules of both record layouts, walked on the CPU, give q . dequant(k) of the
    checker exactly."""
    q, en = make_quantizer(seed=seed, min_bits=min_bits, max_bits=max_bits, budget=budget)
    k, _, qq = make_kv(en, 4, seed=seed)
    plan = q.plan()
    p = plan[0]
    ng = int(p['n_seg'])
    codes, raw, corr = oracle_lib.encode_k(plan, k)
    qr = oracle_lib.rotate_q(plan, qq).astype(np.float32)
    for mixed in (False, True):
        kp = oracle_lib.pack_k(plan, codes, int(mixed))
        nr = (corr if mixed else raw)[:, :max(ng, 1)]
        kn = oracle_lib.f2h(nr).view(np.float16).astype(np.float32)
        for t in range(k.shape[0]):
            ref = qr.astype(np.float64) @ oracle_lib.dequant_k(plan, codes[t:t + 1], oracle_lib.f2h(nr[t:t + 1]))[0].astype(np.float64)
            got = _emulate_steps(p, kp[t], kn[t], qr, int(mixed))
            assert np.abs(got - ref).max() < 1e-9


def test_cache_rows_avoid_strides_that_collide_in_lds():
    from blockgtq_amd.plan import cache_row_bytes
    for n in range(1, 129):
        row = cache_row_bytes(n)
        assert row >= n and row % 4 == 0 and row - n < 8 and row <= 128
        if row < 128:
            # 16 consecutive rows must start in 16 different groups of 4 banks (64 banks of 4 bytes)
            assert len({(r * row // 4) % 64 // 4 for r in range(16)}) == 16 or row % 32 != 0
            assert row % 32 != 0
    assert cache_row_bytes(57) == 60 and cache_row_bytes(61) == 68 and cache_row_bytes(128) == 128


def test_library_loads_and_exports_every_declared_symbol():
    from blockgtq_amd import _capi
    lib = _capi.lib()
    text = open(os.path.join(ROOT, "include", "bgtq.h")).read()
    declared = set(re.findall(r"\b(bgtq_[a-z_0-9]+)\s*\(", text))
    declared -= {"bgtq_head_plan"}
    assert declared, "no declarations parsed"
    missing = [name for name in sorted(declared) if not hasattr(lib, name)]
    assert not missing, f"library lacks {missing}"
    assert lib.bgtq_plan_sizeof() == P.PLAN_DTYPE.itemsize
    assert lib.bgtq_abi_version() >= 1
    assert lib.bgtq_workspace_bytes(2, 16, 8) == 2 * 16 * 8 * 129 * 4
    assert lib.bgtq_strerror(-1).decode() == "invalid argument"
    # argument validation happens on the host before any launch
    assert lib.bgtq_encode_k(None, None, 0, 0, 0, 1, 1, 1, None, 0, 0, 0, 8,
                             None, 0, 0, 0, 1, None, 0, 4, 0, 0, None) == -1
    # an empty call is legal and launches nothing
    assert lib.bgtq_encode_k(None, None, 0, 0, 0, 1, 1, 0, None, 0, 0, 0, 8,
                             None, 0, 0, 0, 1, None, 0, 4, 0, 0, None) == 0
    # an append that would run past the cache capacity is refused before any launch
    one = ctypes.c_void_p(16)          # non-null placeholders: the capacity check comes before any use
    assert lib.bgtq_encode_k(one, one, 0, 0, 0, 1, 1, 2, one, 0, 0, 0, 8,
                             one, 0, 0, 0, 1, None, 3, 4, 0, 0, None) == -3


def test_device_paths_refuse_cpu_tensors():
    from blockgtq_amd import _capi
    q, _ = make_quantizer(seed=1)
    with pytest.raises(_capi.BgtqError):
        q.compress(torch.zeros(4, 128, dtype=torch.float16))


def test_saved_calibration_rebuilds_identical_plans(tmp_path):
    from blockgtq_amd import calibration
    quantizers = [[make_quantizer(seed=10 * li + hi, head=hi, budget=192 - 32 * li,
                                  min_bits=li, max_bits=5 - li)[0] for hi in range(2)]
                  for li in range(2)]
    path = tmp_path / "calib.npz"
    calibration.save_calibration(path, quantizers)
    assert path.stat().st_size < 16384                 # allocations, not activations
    loaded, batched_args, kernel_args = calibration.load_calibration(path, device='cpu')
    assert len(loaded) == 2 and len(loaded[0]) == 2 and len(batched_args) == 2
    for li in range(2):
        for hi in range(2):
            a, b = quantizers[li][hi], loaded[li][hi]
            assert torch.equal(a.bit_allocation, b.bit_allocation)
            assert a.plan().tobytes() == b.plan().tobytes()
            assert kernel_args[li][hi]['segments_b'] == a.build_kernel_args()['segments_b']
        stacked = P.stack_plans(quantizers[li])
        assert batched_args[li]['plans'].numpy().tobytes() == stacked.tobytes()
    # a file of another format version is refused, not misread
    with np.load(path) as f:
        fields = {k: f[k] for k in f.files}
    fields['format'] = np.int64(99)
    np.savez(tmp_path / "other.npz", **fields)
    with pytest.raises(ValueError):
        calibration.load_calibration(tmp_path / "other.npz", device='cpu')


# ---------------------------------------------------------------- q_proj baking
@pytest.mark.parametrize("seed,with_bias", [(3, True), (11, False)])
def test_baked_q_proj_equals_rotation_of_the_projection(oracle_lib, seed, with_bias):
    """A q_proj with permutation + rotation folded in must produce what the checker's query
    rotation makes of the original projection's output, to fp32 rounding.  The head has rotated
    (non-identity, non-symmetric) groups; a transposed rotation misses by O(1)."""
    n_kv, gqa, hid = 2, 3, 40
    heads = [make_quantizer(seed=seed + h, head=h)[0] for h in range(n_kv)]
    assert any(int(q.plan()['seg_identity'][0][g]) == 0 for q in heads for g in range(int(q.plan()['n_seg'][0])))
    gen = torch.Generator().manual_seed(seed)
    W = torch.randn(n_kv * gqa * 128, hid, generator=gen)
    b = torch.randn(n_kv * gqa * 128, generator=gen) if with_bias else None
    x = torch.randn(5, hid, generator=gen)
    y = x @ W.T + (b if with_bias else 0.0)                    # original projection, (5, n_q * 128)
    Wb, bb = W.clone(), (b.clone() if with_bias else None)
    for h, q in enumerate(heads):
        q.bake_permutation_into_qproj(Wb, h, n_kv, n_kv * gqa, q_proj_bias=bb)
        assert q._q_perm_baked
    yb = x @ Wb.T + (bb if with_bias else 0.0)
    for h, q in enumerate(heads):
        rot = q._block_rot_T.double().numpy()
        hp = q._head_perm.numpy()
        for g in range(gqa):
            lo = (h * gqa + g) * 128
            want = y[:, lo:lo + 128].double().numpy()[:, hp] @ rot       # q[head_perm] @ block_rot_T
            got = yb[:, lo:lo + 128].double().numpy()
            assert np.abs(got - want).max() < 2e-4 * max(1.0, np.abs(want).max())
            # and the checker's rotation of the fp16-rounded projection agrees with both
            y16 = y[:, lo:lo + 128].half().numpy()
            ref = oracle_lib.rotate_q(q.plan(), y16).astype(np.float64)
            assert np.abs(got - ref).max() < 2e-2 * max(1.0, np.abs(want).max())     # fp16 in and out


def test_bench_allocations_follow_calibration_on_drawn_tensors():
    """The headline workload takes its per-head bit allocations from the closed-form block
    energies of the synthetic distribution.  Calibrating on 2048 drawn tokens of that
    distribution (queries and keys share the per-block scaling; every query head of the group
    is a sample) through ``BlockGTQQuantizer.calibrate`` reproduces them up to the sampling
    noise of the block energies: the same bit budget, most heads identical, and where a head
    differs it is one bit moved between two blocks whose scores are nearly tied."""
    from blockgtq_amd import synthetic as syn, workloads as wl
    w = wl.WORKLOADS["qwen3b_b8_32k_k3v3"]
    gqa = w.n_q // w.n_kv
    identical = total = 0
    for layer in (0, 1, 9, 18, 27, 35):
        qs, energies = wl.calibrate_layer(w, layer, 'cpu')
        for h in range(w.n_kv):
            gen = torch.Generator().manual_seed(w.seed * 31 + layer * 7 + h)
            k = syn.make_keys(1, 2048, 128, energies[h:h + 1], w.rope_theta, gen)[0]
            q = syn.make_keys(1, 2048 * gqa, 128, energies[h:h + 1], w.rope_theta, gen)[0]
            drawn = BlockGTQQuantizer(128, avg_bits=w.k_bits, min_bits=w.min_bits, max_bits=w.max_bits, device='cpu')
            drawn.calibrate(q, k)
            diff = drawn.bit_allocation - qs[h].bit_allocation
            assert int(diff.sum()) == 0 and int(diff.abs().max()) <= 1 and int((diff != 0).sum()) <= 4, (layer, h, diff)
            identical += int((diff == 0).all())
            total += 1
    assert identical >= total * 2 // 3, (identical, total)


@pytest.mark.parametrize('v_bits', [2, 3, 4])
def test_v_encoder_tables(v_bits):
    """`enc_vbyte` assembles, byte by byte, the V record that the independent LSB-first bit-stream writer
    writes (both layouts); `v_rot_T4` is `v_rot_T` with four rows interleaved."""
    from blockgtq_amd import plan as P
    q, _ = make_quantizer(seed=29, v_bits=v_bits)
    p = q.plan()[0]
    codes = np.random.default_rng(v_bits).integers(0, 1 << v_bits, 128)
    for layout, bw in ((P.V_BITPACKED, v_bits), (P.V_NIBBLE, 4)):
        n_bytes = 16 * bw
        out = np.zeros(n_bytes, dtype=np.uint8)
        for j in range(n_bytes):
            w0, first = (int(x) for x in p['enc_vbyte'][layout, j])
            mode, w, skip, n = w0 & 3, (w0 >> 2) & 15, (w0 >> 6) & 3, w0 >> 8
            assert (mode, w) == (1, bw)
            acc = 0
            for i in range(n):
                acc |= int(codes[first + i]) << (i * bw)
            out[j] = (acc >> skip) & 255
        assert np.array_equal(out, stream_pack(codes[None], bw)[0])
        assert not p['enc_vbyte'][layout, n_bytes:].any()
    vt = p['v_rot_T'].reshape(128, 128)
    for r in (0, 1, 5, 66, 127):
        assert np.array_equal(p['v_rot_T4'][r // 4, :, r % 4], vt[r])
