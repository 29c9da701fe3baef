"""GPU parity: quantise-and-pack kernels and query rotation, bit-exact against
the CPU checker on the same seeded inputs (called through the C ABI)."""
import numpy as np
import pytest
import torch

from blockgtq_amd import plan as P
from helpers import make_kv, make_quantizer

pytestmark = pytest.mark.gpu
DEV = "cuda:0"

HEADS = [  # budget, min, max, v_bits, rotation_threshold
    (192, 1, 5, 3, 2),     # K3V3, Llama-style 1..5 bits
    (192, 1, 8, 3, 2),     # default bit range
    (128, 0, 4, 2, 2),     # K2V2 with 0-bit blocks
    (300, 2, 8, 4, 1),     # wide codes stored as raw bytes, every group rotated
    (64, 1, 1, 1, 2),      # single 1-bit group, identity rotation
    (192, 3, 3, 3, 9),     # uniform 3 bits, nothing rotated
]


def _encode_on_gpu(q, k, v, k_layout, v_layout, t_pos=3, pad=5, quant_mode=0):
    from blockgtq_amd.quantizer import encode_k_into, encode_v_into
    pl = q.plan()[0]
    T = k.shape[0]
    own = int(pl['k_mixed_bytes'] if k_layout else pl['k_row_bytes'])
    kw = max(4, (own + 3) // 4 * 4)
    ng = max(int(pl['n_seg']), 1) + 1                   # one spare norm column
    vw = {1: 16, 2: 32, 3: 48, 4: 64}[4 if v_layout else int(pl['v_bits'])]
    kt = torch.tensor(k).view(1, 1, T, 128).to(DEV)
    vt = torch.tensor(v).view(1, 1, T, 128).to(DEV)
    kp = torch.full((1, 1, T + pad + t_pos, kw + 4), 0xAB, dtype=torch.uint8, device=DEV)
    kn = torch.full((1, 1, T + pad + t_pos, ng), 7.0, dtype=torch.float16, device=DEV)
    vp = torch.full((1, 1, T + pad + t_pos, vw), 0xCD, dtype=torch.uint8, device=DEV)
    vn = torch.full((1, 1, T + pad + t_pos), 7.0, dtype=torch.float16, device=DEV)
    plans = q.device_plan()
    encode_k_into(plans, kt, kp, kn, t_pos, kw, ng, k_layout, quant_mode)
    encode_v_into(plans, vt, vp, vn, t_pos, vw, v_layout)
    torch.cuda.synchronize()
    return kp.cpu().numpy()[0, 0], kn.cpu().numpy()[0, 0], vp.cpu().numpy()[0, 0], vn.cpu().numpy()[0, 0], kw, ng, vw


@pytest.mark.parametrize("cfg", HEADS)
@pytest.mark.parametrize("k_layout,v_layout", [(0, 0), (1, 1)])
def test_packed_records_are_bit_exact(oracle_lib, cfg, k_layout, v_layout):
    budget, mn, mx, vb, rt = cfg
    q, en = make_quantizer(seed=budget + mx, budget=budget, min_bits=mn, max_bits=mx, v_bits=vb,
                           device=DEV, rotation_threshold=rt)
    pl = q.plan()
    T = 333                                            # not a multiple of any tile
    k, v, _ = make_kv(en, T, seed=budget)
    kp, kn, vp, vn, kw, ng, vw = _encode_on_gpu(q, k, v, k_layout, v_layout)
    codes, raw, corr = oracle_lib.encode_k(pl, k)
    want_k = oracle_lib.pack_k(pl, codes, k_layout, kw)
    want_kn = oracle_lib.f2h((corr if k_layout else raw)[:, :ng])
    vc, want_vn = oracle_lib.encode_v(pl, v)
    want_v = oracle_lib.pack_v(vc, vb, bool(v_layout))
    t0 = 3
    assert np.array_equal(kp[t0:t0 + T, :kw], want_k)
    assert np.array_equal(kn[t0:t0 + T].view(np.uint16), want_kn)
    assert np.array_equal(vp[t0:t0 + T], want_v)
    assert np.array_equal(vn[t0:t0 + T].view(np.uint16), want_vn)
    # nothing outside the addressed slots or beyond the record width is touched
    assert (kp[:t0] == 0xAB).all() and (kp[t0 + T:] == 0xAB).all() and (kp[:, kw:] == 0xAB).all()
    assert (vp[:t0] == 0xCD).all() and (vp[t0 + T:] == 0xCD).all()
    assert (kn[:t0] == 7).all() and (kn[t0 + T:] == 7).all() and (vn[:t0] == 7).all() and (vn[t0 + T:] == 7).all()
    # the spare norm column and the bytes past the head's own record are zeroed
    assert (kn[t0:t0 + T, int(pl['n_seg'][0]):] == 0).all()
    own = int(pl['k_mixed_bytes'][0] if k_layout else pl['k_row_bytes'][0])
    assert (kp[t0:t0 + T, own:kw] == 0).all()


def test_exact_boundary_rule_and_unpacked_codes(oracle_lib):
    q, en = make_quantizer(seed=21, max_bits=6, device=DEV)
    pl = q.plan()
    k, v, _ = make_kv(en, 257)
    kt, vt = torch.tensor(k).to(DEV), torch.tensor(v).to(DEV)
    for mode in (P.QUANT_LUT256, P.QUANT_EXACT):
        codes, norms = q.compress(kt, quant_mode=mode)
        want, raw, corr = oracle_lib.encode_k(pl, k, mode)
        assert np.array_equal(codes.cpu().numpy(), want)
        assert np.array_equal(norms.cpu().numpy(), raw[:, :q._n_groups])
        _, cn = q.compress(kt, corrected=True, quant_mode=mode)
        assert np.array_equal(cn.cpu().numpy(), corr[:, :q._n_groups])
    vc, vn = q.compress_v(vt)
    wc, wn = oracle_lib.encode_v(pl, v)
    assert np.array_equal(vc.cpu().numpy(), wc)
    assert np.array_equal(vn.cpu().numpy().view(np.uint16), wn)
    packed, norms, bits = q.compress_packed(kt)
    assert bits == int(q.bit_allocation.sum()) * 2
    assert np.array_equal(packed.cpu().numpy(), oracle_lib.pack_k(pl, oracle_lib.encode_k(pl, k)[0], 0))
    vpk, _ = q.compress_v_packed(vt)
    assert np.array_equal(vpk.cpu().numpy(), oracle_lib.pack_v(wc, 3))


def test_edge_inputs(oracle_lib):
    """Zero rows, huge and tiny magnitudes, a single row, an empty call."""
    q, en = make_quantizer(seed=4, device=DEV)
    pl = q.plan()
    k, v, _ = make_kv(en, 8)
    k[0] = 0; v[0] = 0
    k[1] *= np.float16(200.0); v[1] *= np.float16(200.0)
    k[2] = (k[2].astype(np.float32) * 1e-4).astype(np.float16)
    v[2] = (v[2].astype(np.float32) * 1e-4).astype(np.float16)
    k[3, 1:] = 0; v[3, 1:] = 0                    # one-hot rows
    for rows in (slice(0, 8), slice(5, 6)):
        kp, kn, vp, vn, kw, ng, vw = _encode_on_gpu(q, k[rows], v[rows], 0, 0)
        n = k[rows].shape[0]
        codes, raw, _ = oracle_lib.encode_k(pl, k[rows])
        vc, wvn = oracle_lib.encode_v(pl, v[rows])
        assert np.array_equal(kp[3:3 + n, :kw], oracle_lib.pack_k(pl, codes, 0, kw))
        assert np.array_equal(kn[3:3 + n].view(np.uint16), oracle_lib.f2h(raw[:, :ng]))
        assert np.array_equal(vp[3:3 + n], oracle_lib.pack_v(vc, 3))
        assert np.array_equal(vn[3:3 + n].view(np.uint16), wvn)
    from blockgtq_amd.quantizer import encode_k_into
    empty = torch.zeros(1, 1, 0, 128, dtype=torch.float16, device=DEV)
    encode_k_into(q.device_plan(), empty, torch.zeros(1, 1, 4, 64, dtype=torch.uint8, device=DEV),
                  torch.zeros(1, 1, 4, 8, dtype=torch.float16, device=DEV), 0, 64, 8, 0)


def test_batched_heads_ragged_positions_and_strided_input(oracle_lib):
    """All KV heads of a layer in one launch, per-row write positions, and
    inputs that are views of a (B, S, H, D) projection output."""
    from blockgtq_amd.quantizer import build_batched_encode_args, encode_k_into, encode_v_into
    qs, ens = zip(*[make_quantizer(seed=30 + h, head=h, device=DEV, max_bits=5 + h) for h in range(3)])
    args = build_batched_encode_args(list(qs), device=DEV)
    B, S, H = 2, 5, 3
    gen = torch.Generator().manual_seed(9)
    proj_k = torch.randn(B, S, H, 128, generator=gen).half().to(DEV)
    proj_v = torch.randn(B, S, H, 128, generator=gen).half().to(DEV)
    k, v = proj_k.transpose(1, 2), proj_v.transpose(1, 2)        # (B, H, S, D), non-contiguous
    kw = (args['max_tpb'] + 3) // 4 * 4
    ng = args['max_n_groups']
    kp = torch.zeros(B, H, 40, kw, dtype=torch.uint8, device=DEV)
    kn = torch.zeros(B, H, 40, ng, dtype=torch.float16, device=DEV)
    vp = torch.zeros(B, H, 40, 48, dtype=torch.uint8, device=DEV)
    vn = torch.zeros(B, H, 40, dtype=torch.float16, device=DEV)
    pos = torch.tensor([7, 31], dtype=torch.int32, device=DEV)
    encode_k_into(args['plans'], k, kp, kn, pos, kw, ng, 0)
    encode_v_into(args['plans'], v, vp, vn, pos, 48, 0)
    torch.cuda.synchronize()
    for b in range(B):
        for h in range(H):
            pl = args['plans_np'][h:h + 1]
            kk = k[b, h].cpu().numpy()
            codes, raw, _ = oracle_lib.encode_k(pl, kk)
            t0 = int(pos[b])
            assert np.array_equal(kp[b, h, t0:t0 + S].cpu().numpy(), oracle_lib.pack_k(pl, codes, 0, kw))
            assert np.array_equal(kn[b, h, t0:t0 + S].cpu().numpy().view(np.uint16), oracle_lib.f2h(raw[:, :ng]))
            vc, wn = oracle_lib.encode_v(pl, v[b, h].cpu().numpy())
            assert np.array_equal(vp[b, h, t0:t0 + S].cpu().numpy(), oracle_lib.pack_v(vc, 3))
            assert np.array_equal(vn[b, h, t0:t0 + S].cpu().numpy().view(np.uint16), wn)
            assert (kp[b, h, :t0] == 0).all() and (kp[b, h, t0 + S:] == 0).all()


def test_large_prefill_shape_round_trips(oracle_lib):
    """Prefill-sized call (16-row tiles): bit-exact on a sample of rows, and every
    record unpacks to codes that re-pack to the same bytes."""
    q, en = make_quantizer(seed=8, device=DEV)
    pl = q.plan()
    T = 8192 + 13
    k, v, _ = make_kv(en, T)
    kp, kn, vp, vn, kw, ng, vw = _encode_on_gpu(q, k, v, 0, 0, t_pos=0, pad=0)
    rows = np.r_[0:40, T - 40:T, 4000:4040]
    codes, raw, _ = oracle_lib.encode_k(pl, k[rows])
    assert np.array_equal(kp[rows, :kw], oracle_lib.pack_k(pl, codes, 0, kw))
    own = int(pl['k_row_bytes'][0])
    allc = oracle_lib.unpack_k(pl, kp[:, :own], 0)
    assert np.array_equal(oracle_lib.pack_k(pl, allc, 0), kp[:, :own])
    vc = oracle_lib.unpack_v(vp, 3)
    assert np.array_equal(oracle_lib.pack_v(vc, 3), vp)


def test_query_rotation_is_bit_exact(oracle_lib):
    from blockgtq_amd import ops
    from blockgtq_amd.quantizer import build_batched_encode_args
    qs = [make_quantizer(seed=50 + h, head=h, device=DEV, min_bits=0, max_bits=6, budget=150)[0] for h in range(2)]
    args = build_batched_encode_args(qs, device=DEV)
    gen = torch.Generator().manual_seed(3)
    q = torch.randn(3, 8, 128, generator=gen).half().to(DEV)     # 2 KV heads x gqa 4
    got = ops.rotate_q(args['plans'], q, 2).cpu().numpy()
    for h in range(2):
        want = oracle_lib.rotate_q(args['plans_np'][h:h + 1], q[:, 4 * h:4 * h + 4].reshape(-1, 128).cpu().numpy())
        assert np.array_equal(got[:, 4 * h:4 * h + 4].reshape(-1, 128).view(np.uint16), want.view(np.uint16))
    single = qs[1].rotate_q_for_packed_kernel(q[:, 4:8])
    assert np.array_equal(single.cpu().numpy(), got[:, 4:8])


@pytest.mark.parametrize("S", [1, 3, 40])
def test_fused_prepare_equals_the_three_separate_calls(S):
    """``bgtq_decode_prepare`` (append-encode K, V and rotate Q in one launch) writes the
    same bytes as ``bgtq_encode_k`` + ``bgtq_encode_v`` + ``bgtq_rotate_q``; S = 40 with
    B = 2 takes its prefill-sized route."""
    from blockgtq_amd import ops
    from blockgtq_amd.quantizer import build_batched_encode_args, encode_k_into, encode_v_into
    qs = [make_quantizer(seed=70 + h, head=h, device=DEV, max_bits=5)[0] for h in range(2)]
    args = build_batched_encode_args(qs, device=DEV)
    B, H, gqa = 2, 2, 4
    gen = torch.Generator().manual_seed(11 + S)
    k = torch.randn(B, H, S, 128, generator=gen).half().to(DEV)
    v = torch.randn(B, H, S, 128, generator=gen).half().to(DEV)
    q = torch.randn(B, H * gqa, 128, generator=gen).half().to(DEV)
    kw = (args['max_tpb'] + 3) // 4 * 4
    ng = args['max_n_groups']
    pos = torch.tensor([3, 17], dtype=torch.int32, device=DEV)

    def buffers():
        return (torch.zeros(B, H, 64, kw, dtype=torch.uint8, device=DEV),
                torch.zeros(B, H, 64, ng, dtype=torch.float16, device=DEV),
                torch.zeros(B, H, 64, 48, dtype=torch.uint8, device=DEV),
                torch.zeros(B, H, 64, dtype=torch.float16, device=DEV))

    kp0, kn0, vp0, vn0 = buffers()
    encode_k_into(args['plans'], k, kp0, kn0, pos, kw, ng, 0)
    encode_v_into(args['plans'], v, vp0, vn0, pos, 48, 0)
    q0 = ops.rotate_q(args['plans'], q, H)
    kp1, kn1, vp1, vn1 = buffers()
    q1 = ops.decode_prepare(args['plans'], k, v, q, kp1, kn1, vp1, vn1, pos, kw, ng, 48, H, 0, 0)
    torch.cuda.synchronize()
    assert kp0.any() and vp0.any()
    for a, b in ((kp0, kp1), (vp0, vp1), (q0, q1)):
        assert torch.equal(a, b)
    assert torch.equal(kn0.view(torch.int16), kn1.view(torch.int16))
    assert torch.equal(vn0.view(torch.int16), vn1.view(torch.int16))


def test_appends_past_the_cache_capacity_write_nothing(oracle_lib):
    """A host position beyond the capacity raises before any launch; device positions beyond it
    are dropped by the kernels (both append sizes: the 2-row decode tiles and the 16-row tiles,
    and the fused prepare launch), and rows inside the capacity are still written correctly.
    The cache tensors are views into a larger buffer so that a stray write would be seen."""
    from blockgtq_amd import ops
    from blockgtq_amd.quantizer import build_batched_encode_args, encode_k_into, encode_v_into
    qs, ens = zip(*[make_quantizer(seed=50 + h, head=h, device=DEV) for h in range(2)])
    args = build_batched_encode_args(list(qs), device=DEV)
    kw, ng, H, cap = (args['max_tpb'] + 3) // 4 * 4, args['max_n_groups'], 2, 12
    for B, S in ((3, 1), (3, 30)):                       # decode-sized and prefill-sized launches
        big_k = torch.full((B, H, cap + 40, kw), 0xEE, dtype=torch.uint8, device=DEV)
        big_n = torch.full((B, H, cap + 40, ng), 5.0, dtype=torch.float16, device=DEV)
        big_v = torch.full((B, H, cap + 40, 48), 0xEE, dtype=torch.uint8, device=DEV)
        big_vn = torch.full((B, H, cap + 40), 5.0, dtype=torch.float16, device=DEV)
        kp, kn, vp, vn = big_k[:, :, :cap], big_n[:, :, :cap], big_v[:, :, :cap], big_vn[:, :, :cap]
        gen = torch.Generator().manual_seed(S)
        k = torch.randn(B, H, S, 128, generator=gen).half().to(DEV)
        v = torch.randn(B, H, S, 128, generator=gen).half().to(DEV)
        q = torch.randn(B, H * 4, 128, generator=gen).half().to(DEV)
        with pytest.raises(ValueError):
            encode_k_into(args['plans'], k, kp, kn, cap - S + 1, kw, ng, 0)
        with pytest.raises(ValueError):
            ops.decode_prepare(args['plans'], k, v, q, kp, kn, vp, vn, cap, kw, ng, 48, H, 0, 0)
        pos = torch.tensor([cap - S - 1 if S < cap else 0, cap - 1, cap + 5], dtype=torch.int32, device=DEV)
        for fused in (False, True):
            big_k.fill_(0xEE); big_n.fill_(5.0); big_v.fill_(0xEE); big_vn.fill_(5.0)
            if fused:
                ops.decode_prepare(args['plans'], k, v, q, kp, kn, vp, vn, pos, kw, ng, 48, H, 0, 0)
            else:
                encode_k_into(args['plans'], k, kp, kn, pos, kw, ng, 0)
                encode_v_into(args['plans'], v, vp, vn, pos, 48, 0)
            torch.cuda.synchronize()
            assert (big_k[:, :, cap:] == 0xEE).all() and (big_v[:, :, cap:] == 0xEE).all()
            assert (big_n[:, :, cap:] == 5.0).all() and (big_vn[:, :, cap:] == 5.0).all()
            for b in range(B):
                t0 = int(pos[b])
                n_in = max(0, min(S, cap - t0))           # rows of this batch row that fit
                for h in range(H):
                    pl = args['plans_np'][h:h + 1]
                    codes, raw, _ = oracle_lib.encode_k(pl, k[b, h].cpu().numpy())
                    want = oracle_lib.pack_k(pl, codes, 0, kw)
                    assert np.array_equal(kp[b, h, t0:t0 + n_in].cpu().numpy(), want[:n_in])
                    vc, wn = oracle_lib.encode_v(pl, v[b, h].cpu().numpy())
                    assert np.array_equal(vp[b, h, t0:t0 + n_in].cpu().numpy(), oracle_lib.pack_v(vc, 3)[:n_in])
                    assert (kp[b, h, :min(t0, cap)] == 0xEE).all()


def test_every_code_as_a_nibble_for_all_heads(oracle_lib):
    """``compress_k_nibble4_batched``: byte j of a record holds the codes at packed positions 2j
    (low nibble) and 2j+1 of the checker's code vector, codes wider than four bits cut to their low
    four; the norms are the checker's raw group norms."""
    from blockgtq_amd.quantizer import build_batched_encode_args, compress_k_nibble4_batched
    made = [make_quantizer(seed=70 + h, head=h, device=DEV, min_bits=0, max_bits=6, budget=170) for h in range(3)]
    qs = [m[0] for m in made]
    args = build_batched_encode_args(qs, device=DEV)
    N = 77
    k = np.stack([make_kv(made[h][1], N, seed=90 + h)[0] for h in range(3)])
    nib, norms = compress_k_nibble4_batched(torch.tensor(k).to(DEV), args)
    assert nib.shape == (3, N, 64) and nib.dtype == torch.uint8
    assert norms.shape == (3, N, args['max_n_groups']) and norms.dtype == torch.float32
    nib, norms = nib.cpu().numpy(), norms.cpu().numpy()
    wide = False
    for h in range(3):
        codes, raw, _ = oracle_lib.encode_k(args['plans_np'][h:h + 1], k[h])
        wide |= bool((codes > 15).any())
        assert np.array_equal(nib[h], (codes[:, 0::2] & 15) | ((codes[:, 1::2] & 15) << 4))
        ng = raw.shape[1]
        assert np.array_equal(norms[h][:, :min(ng, norms.shape[2])], raw[:, :norms.shape[2]])
    assert wide
