"""Pins for the CPU checker (oracle/): every function is checked against
something that does not share its formula - an independent bit-stream writer,
numpy/torch library routines, closed forms and invariants."""
import numpy as np
import pytest
import torch
import torch.nn.functional as F

from blockgtq_amd import v_packing
from helpers import make_kv, make_quantizer, stream_pack


@pytest.fixture(scope="module")
def head(oracle_lib):
    q, en = make_quantizer(seed=11, max_bits=6, budget=192)
    k, v, qq = make_kv(en, 300, n_q=4)
    return oracle_lib, q, q.plan(), k, v, qq


# ------------------------------------------------------------ fp16 conversion
def test_half_conversions_match_numpy(oracle_lib):
    allh = np.arange(65536, dtype=np.uint16)
    f = oracle_lib.h2f(allh)
    ref = allh.view(np.float16).astype(np.float32)
    assert np.array_equal(f.view(np.uint32)[~np.isnan(ref)], ref.view(np.uint32)[~np.isnan(ref)])
    rng = np.random.default_rng(0)
    x = np.concatenate([
        rng.standard_normal(200000).astype(np.float32) * np.float32(10.0) ** rng.integers(-9, 6, 200000).astype(np.float32),
        np.array([0.0, -0.0, 65504.0, 65519.9, 65520.0, 1e9, -1e9, 2.0 ** -24, 2.0 ** -25,
                  np.nextafter(np.float32(2.0 ** -25), np.float32(1)), 6.1e-5, 6.0975e-5], dtype=np.float32)])
    # every tie between two halves must go to the even one
    ties = (allh[:-1].view(np.float16).astype(np.float64) + allh[1:].view(np.float16).astype(np.float64)) / 2
    ties = ties[np.isfinite(ties)].astype(np.float32)
    x = np.concatenate([x, ties])
    with np.errstate(over='ignore'):
        ref16 = x.astype(np.float16).view(np.uint16)
    assert np.array_equal(oracle_lib.f2h(x), ref16)


# ------------------------------------------------------------ packers
def test_k_bit_packed_record_is_a_per_segment_bit_stream(head):
    orc, q, plan, k, v, qq = head
    codes, _, _ = orc.encode_k(plan, k)
    rec = orc.pack_k(plan, codes, 0)
    p = plan[0]
    assert rec.shape[1] == int(p['k_row_bytes'])
    for g in range(int(p['n_seg'])):
        bw, s, ln, off = (int(p[f][g]) for f in ('seg_bw', 'seg_start', 'seg_len', 'seg_pack_off'))
        seg = codes[:, s:s + ln]
        assert seg.max() < (1 << bw)
        if bw >= 5:
            assert np.array_equal(rec[:, off:off + ln], seg)
        else:
            want = stream_pack(seg, bw)
            nbytes = {1: (ln + 7) // 8, 2: (ln + 3) // 4, 3: ((ln + 7) // 8) * 3, 4: (ln + 1) // 2}[bw]
            got = rec[:, off:off + nbytes]
            assert np.array_equal(got[:, :want.shape[1]], want)
            assert (got[:, want.shape[1]:] == 0).all()          # tail of the last 3-byte group
    assert np.array_equal(orc.unpack_k(plan, rec, 0), codes)


@pytest.mark.parametrize("with_zero_bit_blocks", [False, True])
def test_k_mixed_record_layout(head, with_zero_bit_blocks):
    """Nibbles of the <= 4-bit dims (two per byte, low nibble first), then one byte per wider code;
    dims of 0-bit blocks come first in packed order and take no room in the record."""
    orc, q, plan, k, v, qq = head
    if with_zero_bit_blocks:
        q, en = make_quantizer(seed=1, min_bits=0, max_bits=8, budget=160)
        plan = q.plan()
        k, _, _ = make_kv(en, 200)
    codes, _, _ = orc.encode_k(plan, k)
    rec = orc.pack_k(plan, codes, 1)
    z = int(plan[0]['n_zero_dims'])
    ns, nl = int(plan[0]['nopack_start']), int(plan[0]['nopack_len'])
    assert (z > 0) == with_zero_bit_blocks and z % 2 == 0 and nl > 0
    nib = (ns - z) // 2
    assert rec.shape[1] == nib + nl == int(plan[0]['k_mixed_bytes'])
    assert np.array_equal(rec[:, :nib], (codes[:, z:ns:2] & 15) | ((codes[:, z + 1:ns:2] & 15) << 4))
    assert np.array_equal(rec[:, nib:], codes[:, ns:ns + nl])
    back = orc.unpack_k(plan, rec, 1)
    assert np.array_equal(back[:, z:], codes[:, z:]) and not back[:, :z].any()


@pytest.mark.parametrize("bits,nibble", [(1, False), (2, False), (3, False), (4, False), (2, True), (3, True)])
def test_v_record_against_stream_writer_and_table_rule(oracle_lib, bits, nibble):
    rng = np.random.default_rng(bits)
    codes = rng.integers(0, 1 << bits, size=(33, 128)).astype(np.uint8)
    rec = oracle_lib.pack_v(codes, bits, nibble)
    eff = 4 if nibble else bits
    assert np.array_equal(rec, stream_pack(codes, eff))
    # the per-dim two-byte-window rule the reference's decode kernel unpacks with
    lo_b, hi_b, sh_lo, sh_hi, mask = (t.numpy() for t in v_packing.build_v_unpack_tables(eff, 128))
    r = rec.astype(np.int32)
    got = ((r[:, lo_b] >> sh_lo) | (r[:, hi_b] << sh_hi)) & mask
    assert np.array_equal(got.astype(np.uint8), codes)
    assert np.array_equal(oracle_lib.unpack_v(rec, bits, nibble), codes)


# ------------------------------------------------------------ V encode
def test_v_codes_are_searchsorted_of_the_rotated_unit_vector(head):
    orc, q, plan, k, v, qq = head
    codes, norms = orc.encode_v(plan, v)
    x = v.astype(np.float64)
    n = np.sqrt((x * x).sum(1))
    y = (x / n[:, None]) @ plan[0]['v_rot_T'].reshape(128, 128).astype(np.float64)
    b = plan[0]['v_boundaries'][:7].astype(np.float64)
    want = np.searchsorted(b, y)                     # count of boundaries strictly below y
    near = np.abs(y[..., None] - b).min(-1) < 1e-6   # fp32 rounding may flip these
    assert (codes[~near] == want[~near]).all() and near.mean() < 1e-3
    # stored norm: ||v|| / ||centroids[codes]||, fp16
    cn = np.sqrt((plan[0]['v_centroids'][codes].astype(np.float64) ** 2).sum(1))
    ref = (n / cn).astype(np.float32)
    assert np.abs(orc.h2f(norms) - ref).max() <= np.abs(ref).max() * 2.0 ** -11
    # dequantised vector has the norm of the input (that is what the correction is for)
    vhat = orc.dequant_v(plan, codes, norms)
    assert np.allclose(np.sqrt((vhat.astype(np.float64) ** 2).sum(1)), n, rtol=2e-3)


# ------------------------------------------------------------ K encode
def test_k_codes_reduce_to_plain_scalar_quantisation_without_rotation(oracle_lib):
    # every block 1 bit, threshold 2 -> one identity-rotation group: code = sign of x
    q, en = make_quantizer(seed=2, alloc=[1] * 64)
    plan = q.plan()
    assert int(plan[0]['n_seg']) == 1 and int(plan[0]['seg_identity'][0]) == 1
    k, _, _ = make_kv(en, 200)
    codes, raw, corr = oracle_lib.encode_k(plan, k)
    x = k.astype(np.float64)[:, plan[0]['head_perm']]
    clear = np.abs(x) / np.sqrt((x * x).sum(1, keepdims=True)) > 1e-3
    assert (codes[clear] == (x > 0)[clear]).all()
    assert np.allclose(raw[:, 0], np.sqrt((x * x).sum(1)), rtol=1e-6)
    # all centroids have magnitude c: ||centroids[codes]|| = c * sqrt(128)
    c = np.sqrt(2 / (np.pi * 128))
    assert np.allclose(corr[:, 0], raw[:, 0] / (c * np.sqrt(128)), rtol=1e-5)
    # both quantisation rules agree away from the boundary
    codes_exact, _, _ = oracle_lib.encode_k(plan, k, quant_mode=1)
    assert (codes_exact[clear] == codes[clear]).all()


def test_k_codes_follow_the_rotated_coordinates(head):
    orc, q, plan, k, v, qq = head
    p = plan[0]
    codes_lut, raw, corr = orc.encode_k(plan, k, 0)
    codes_exact, raw2, _ = orc.encode_k(plan, k, 1)
    assert np.array_equal(raw, raw2)
    x = k.astype(np.float64)[:, p['head_perm']]
    rot_T = p['k_rot_T'].reshape(128, 128).astype(np.float64)
    for g in range(int(p['n_seg'])):
        bw, s, ln = int(p['seg_bw'][g]), int(p['seg_start'][g]), int(p['seg_len'][g])
        xs = x[:, s:s + ln]
        n = np.sqrt((xs * xs).sum(1))
        assert np.allclose(raw[:, g], n, rtol=1e-6)
        y = (xs / n[:, None]) @ rot_T[s:s + ln, s:s + ln]
        b = p['k_boundaries'][g][:(1 << bw) - 1].astype(np.float64)
        want = np.searchsorted(b, y)
        near = np.abs(y[..., None] - b).min(-1) < 1e-6
        got = codes_exact[:, s:s + ln]
        assert (got[~near] == want[~near]).all()
        # the 256-bin table differs from the exact rule only by one level, and rarely
        lut = codes_lut[:, s:s + ln].astype(int)
        assert np.abs(lut - want).max() <= 1 and (lut != want).mean() < 0.05
        # norm correction: ||centroids[codes]|| * corrected == ||x||
        cn = np.sqrt((p['k_centroids'][g][codes_lut[:, s:s + ln]].astype(np.float64) ** 2).sum(1))
        assert np.allclose(corr[:, g] * cn, n, rtol=1e-5)
    assert (raw[:, int(p['n_seg']):] == 0).all()


def test_q_rotation_is_permute_then_matmul(head):
    orc, q, plan, k, v, qq = head
    got = orc.rotate_q(plan, qq).astype(np.float32)
    want = qq.astype(np.float64)[:, plan[0]['head_perm']] @ plan[0]['k_rot_T'].reshape(128, 128).astype(np.float64)
    assert np.abs(got - want).max() < 4e-3          # fp16 rounding of O(1) values
    # orthogonality: rotated q . rotated k == q . k
    kk = orc.rotate_q(plan, k[:4]).astype(np.float64)
    assert np.allclose((got.astype(np.float64) * kk).sum(1),
                       (qq.astype(np.float64) * k[:4].astype(np.float64)).sum(1), atol=0.08)


# ------------------------------------------------------------ attention
def _cache(orc, plan, k, v, k_layout=0, v_layout=0):
    codes, raw, corr = orc.encode_k(plan, k)
    ng = int(plan[0]['n_seg'])
    kn = orc.f2h((corr if k_layout else raw)[:, :ng])
    kp = orc.pack_k(plan, codes, k_layout)
    vc, vn = orc.encode_v(plan, v)
    vp = orc.pack_v(vc, int(plan[0]['v_bits']), bool(v_layout))
    return codes, kn, kp, vc, vn, vp


@pytest.mark.parametrize("k_layout,v_layout", [(0, 0), (1, 1), (0, 1)])
def test_attention_equals_library_sdpa_on_dequantised_tensors(head, k_layout, v_layout):
    orc, q, plan, k, v, qq = head
    codes, kn, kp, vc, vn, vp = _cache(orc, plan, k, v, k_layout, v_layout)
    qr = orc.rotate_q(plan, qq)
    out, lse = orc.decode_attn(plan, qr, kp, kn, vp, vn, k_layout=k_layout, v_layout=v_layout)
    khat = torch.tensor(orc.dequant_k(plan, codes, kn)).double()
    vhat = torch.tensor(orc.dequant_v(plan, vc, vn)).double()
    qt = torch.tensor(qr.astype(np.float32)).double()
    ref = F.scaled_dot_product_attention(qt[None], khat[None], vhat[None])[0]
    ref = ref @ torch.tensor(plan[0]['v_rot'].reshape(128, 128)).double()
    assert np.abs(out - ref.numpy()).max() < 1e-6
    logits = (qt @ khat.T) / np.sqrt(128)
    assert np.abs(lse - torch.logsumexp(logits, -1).numpy()).max() < 1e-5


def test_attention_is_invariant_to_the_partition_count(head):
    orc, q, plan, k, v, qq = head
    codes, kn, kp, vc, vn, vp = _cache(orc, plan, k, v)
    qr = orc.rotate_q(plan, qq)
    base, lse0 = orc.decode_attn(plan, qr, kp, kn, vp, vn, n_splits=1)
    for ns in (2, 7, 299, 300, 512):           # 512 > T: empty partitions are skipped
        out, lse = orc.decode_attn(plan, qr, kp, kn, vp, vn, n_splits=ns)
        assert np.abs(out - base).max() < 1e-6 and np.abs(lse - lse0).max() < 1e-5
    # unrotate is linear: merging then rotating == the flag
    rot, _ = orc.decode_attn(plan, qr, kp, kn, vp, vn, unrotate=False)
    assert np.abs(rot @ plan[0]['v_rot'].reshape(128, 128) - base).max() < 1e-5


def test_quantised_attention_tracks_exact_attention(head):
    """End to end: packed attention approximates fp attention on the raw K/V
    (K3V3 quantisation noise, not a bug-sized error)."""
    orc, q, plan, k, v, qq = head
    codes, kn, kp, vc, vn, vp = _cache(orc, plan, k, v, 1, 0)
    out, _ = orc.decode_attn(plan, orc.rotate_q(plan, qq), kp, kn, vp, vn, k_layout=1)
    kt, vt, qt = (torch.tensor(a.astype(np.float32)) for a in (k, v, qq))
    ref = F.scaled_dot_product_attention(qt[None], kt[None], vt[None])[0].numpy()
    rel = np.linalg.norm(out - ref) / np.linalg.norm(ref)
    assert rel < 0.6


def test_empty_context_gives_zero_and_minus_infinity(head):
    orc, q, plan, k, v, qq = head
    codes, kn, kp, vc, vn, vp = _cache(orc, plan, k[:4], v[:4])
    out, lse = orc.decode_attn(plan, orc.rotate_q(plan, qq), kp, kn, vp, vn, T=0)
    assert (out == 0).all() and np.isneginf(lse).all()
