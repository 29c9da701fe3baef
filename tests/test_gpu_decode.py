"""GPU parity: fused packed decode attention + partition merge against the CPU
checker, within 2e-3 max-abs (fp32 accumulate, fp16 output), through the C ABI
and through the cache classes."""
import numpy as np
import pytest
import torch

from blockgtq_amd import ops, plan as P
from blockgtq_amd import workloads as wl
from helpers import make_kv, make_quantizer

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
TOL = 2e-3
LSE_TOL = 1e-3


@pytest.fixture(params=["auto", "generic"], autouse=True)
def decode_path(request):
    """Every test runs twice: with the automatic kernel choice (MFMA kernel where
    the layout allows it) and with the layout-agnostic kernel forced."""
    from blockgtq_amd import _capi
    lib = _capi.lib()
    assert lib.bgtq_set_decode_path(0 if request.param == "auto" else 1) == 0
    yield request.param
    lib.bgtq_set_decode_path(0)


def _reference(orc, mgr_plans, quantizers, kp, kn, vp, vn, q_rot, lens, gqa, k_layout=0, v_layout=0, v_bits=3):
    B, H = kp.shape[:2]
    out = np.zeros((B, H * gqa, 128), np.float32)
    lse = np.zeros((B, H * gqa), np.float32)
    for b in range(B):
        for h in range(H):
            pl = mgr_plans[h:h + 1]
            own = int(pl['k_mixed_bytes'][0] if k_layout else pl['k_row_bytes'][0])
            ng = max(int(pl['n_seg'][0]), 1)
            T = lens[b]
            o, l = orc.decode_attn(pl, q_rot[b, h * gqa:(h + 1) * gqa], kp[b, h, :T, :max(own, 1)],
                                   kn[b, h, :T, :ng], vp[b, h, :T], vn[b, h, :T],
                                   k_layout=k_layout, v_layout=v_layout)
            out[b, h * gqa:(h + 1) * gqa] = o
            lse[b, h * gqa:(h + 1) * gqa] = l
    return out, lse


def _build(budget, mn, mx, vb, n_kv, gqa, B, T, seed, k_layout=0, v_layout=0, student=None):
    from blockgtq_amd.quantizer import build_batched_encode_args, encode_k_into, encode_v_into
    qs, ens = zip(*[make_quantizer(seed=seed + h, head=h, budget=budget, min_bits=mn, max_bits=mx,
                                   v_bits=vb, device=DEV) for h in range(n_kv)])
    args = build_batched_encode_args(list(qs), device=DEV)
    own = args['max_mixed_bytes'] if k_layout else args['max_tpb']
    kw = max(4, (own + 3) // 4 * 4)
    ng = args['max_n_groups']
    vw = 64 if v_layout else args['v_packed_bytes']
    ks, vs, qq = [], [], []
    for h in range(n_kv):
        kb, vb_, qb = [], [], []
        for b in range(B):
            k, v, q = make_kv(ens[h], T, seed=seed * 31 + h * 7 + b, n_q=gqa, student_t_nu=student)
            kb.append(k); vb_.append(v); qb.append(q)
        ks.append(np.stack(kb)); vs.append(np.stack(vb_)); qq.append(np.stack(qb))
    k = torch.tensor(np.stack(ks, 1)).to(DEV)             # (B, H, T, D)
    v = torch.tensor(np.stack(vs, 1)).to(DEV)
    q = torch.tensor(np.concatenate(qq, 1)).to(DEV)        # (B, H*gqa, D)
    kp = torch.zeros(B, n_kv, T + 2, kw, dtype=torch.uint8, device=DEV)
    kn = torch.zeros(B, n_kv, T + 2, ng, dtype=torch.float16, device=DEV)
    vp = torch.zeros(B, n_kv, T + 2, vw, dtype=torch.uint8, device=DEV)
    vn = torch.zeros(B, n_kv, T + 2, dtype=torch.float16, device=DEV)
    encode_k_into(args['plans'], k, kp, kn, 0, kw, ng, k_layout)
    encode_v_into(args['plans'], v, vp, vn, 0, vw, v_layout)
    q_rot = ops.rotate_q(args['plans'], q, n_kv)
    return args, list(qs), q_rot, kp, kn, vp, vn


CASES = [  # budget mn mx vb n_kv gqa B T k_layout v_layout
    (192, 1, 5, 3, 2, 4, 1, 1000, 0, 0),
    (192, 1, 8, 3, 2, 8, 2, 777, 0, 0),
    (192, 1, 8, 3, 2, 8, 2, 777, 1, 1),
    (128, 0, 4, 2, 2, 4, 1, 1500, 0, 0),
    (128, 0, 4, 2, 2, 4, 1, 700, 1, 1),        # 0-bit blocks in the nibble record
    (160, 0, 8, 3, 2, 8, 2, 300, 1, 0),        # 0-bit blocks, nibbles and raw bytes
    (300, 2, 8, 4, 1, 16, 1, 300, 0, 0),
    (300, 2, 8, 4, 1, 16, 1, 300, 1, 0),
    (64, 1, 1, 1, 1, 1, 3, 64, 0, 1),
    (192, 3, 3, 3, 3, 2, 1, 513, 0, 0),
    (192, 1, 5, 3, 2, 7, 1, 400, 0, 0),       # odd head groups on either side of the 8-head schedule
    (192, 1, 5, 3, 1, 12, 2, 333, 0, 0),      # 9..16 heads: two launches of the matrix-core kernel
    (192, 1, 5, 3, 2, 9, 1, 333, 1, 0),
    (160, 1, 6, 4, 2, 3, 2, 200, 1, 1),
    (192, 1, 5, 3, 2, 8, 2, 1022, 0, 0),      # T + 2 rows: every (row, head) slice of the cache starts on a 16-byte boundary
    (192, 1, 8, 3, 2, 4, 2, 510, 1, 1),
]


@pytest.mark.parametrize("case", CASES)
def test_decode_matches_checker(oracle_lib, case, decode_path):
    budget, mn, mx, vb, n_kv, gqa, B, T, kl, vl = case
    args, qs, q_rot, kp, kn, vp, vn = _build(budget, mn, mx, vb, n_kv, gqa, B, T, seed=budget + T, k_layout=kl, v_layout=vl)
    ref, ref_lse = _reference(oracle_lib, args['plans_np'], qs, kp.cpu().numpy(), kn.cpu().numpy(),
                              vp.cpu().numpy(), vn.cpu().numpy(), q_rot.cpu().numpy(), [T] * B, gqa, kl, vl, vb)
    for ns in (1, 3, 16, 0):
        out, lse = ops.decode_attention(args['plans'], q_rot, kp, kn, vp, vn, T, n_splits=ns,
                                        k_layout=kl, v_layout=vl, return_lse=True)
        torch.cuda.synchronize()
        assert np.abs(out.float().cpu().numpy() - ref).max() < TOL
        assert np.abs(lse.cpu().numpy() - ref_lse).max() < LSE_TOL
        assert ops.last_decode_path() == (ops.MFMA_PATH if decode_path == "auto" else ops.GENERIC_PATH)


def test_tiny_contexts_and_empty_partitions(oracle_lib):
    args, qs, q_rot, kp, kn, vp, vn = _build(192, 1, 5, 3, 2, 4, 2, 70, seed=5)
    kpn, knn, vpn, vnn, qn = (t.cpu().numpy() for t in (kp, kn, vp, vn, q_rot))
    for T in (1, 2, 63, 64, 65, 70):
        ref, ref_lse = _reference(oracle_lib, args['plans_np'], qs, kpn, knn, vpn, vnn, qn, [T, T], 4)
        for ns in (1, 8, 64, 512):                  # more partitions than tokens
            out, lse = ops.decode_attention(args['plans'], q_rot, kp, kn, vp, vn, T, n_splits=ns, return_lse=True)
            assert np.abs(out.float().cpu().numpy() - ref).max() < TOL, (T, ns)
            assert np.abs(lse.cpu().numpy() - ref_lse).max() < LSE_TOL
    out, lse = ops.decode_attention(args['plans'], q_rot, kp, kn, vp, vn, 0, n_splits=4, return_lse=True)
    assert (out == 0).all() and torch.isinf(lse).all()


def test_ragged_batch(oracle_lib):
    args, qs, q_rot, kp, kn, vp, vn = _build(192, 1, 6, 3, 2, 4, 4, 600, seed=9)
    lens = [600, 1, 257, 64]
    lens_dev = torch.tensor(lens, dtype=torch.int32, device=DEV)
    ref, ref_lse = _reference(oracle_lib, args['plans_np'], qs, kp.cpu().numpy(), kn.cpu().numpy(),
                              vp.cpu().numpy(), vn.cpu().numpy(), q_rot.cpu().numpy(), lens, 4)
    for ns in (1, 5, 32):
        out, lse = ops.decode_attention(args['plans'], q_rot, kp, kn, vp, vn, 600, seq_lens=lens_dev,
                                        n_splits=ns, return_lse=True)
        assert np.abs(out.float().cpu().numpy() - ref).max() < TOL
        assert np.abs(lse.cpu().numpy() - ref_lse).max() < LSE_TOL


def test_heavy_tailed_long_context_split_stress(oracle_lib):
    """K2V2 with 0-bit blocks, Student-t(4) coordinates, many partitions."""
    args, qs, q_rot, kp, kn, vp, vn = _build(128, 0, 4, 2, 1, 4, 1, 20000, seed=77, student=4)
    ref, ref_lse = _reference(oracle_lib, args['plans_np'], qs, kp.cpu().numpy(), kn.cpu().numpy(),
                              vp.cpu().numpy(), vn.cpu().numpy(), q_rot.cpu().numpy(), [20000], 4, v_bits=2)
    # Student-t values push outputs to |x| ~ 4-5 where fp16 itself is spaced 3.9e-3 apart,
    # so the 2e-3 bound is applied relative to max(1, |reference|).
    bound = TOL * np.maximum(1.0, np.abs(ref))
    for ns in (1, 64, 500):
        out, lse = ops.decode_attention(args['plans'], q_rot, kp, kn, vp, vn, 20000, n_splits=ns, return_lse=True)
        assert (np.abs(out.float().cpu().numpy() - ref) < bound).all()
        assert np.abs(lse.cpu().numpy() - ref_lse).max() < LSE_TOL


def test_manager_append_and_attend_matches_checker(oracle_lib):
    """Config-1 geometry (32 query / 8 KV heads) at a reduced context through the
    manager API: append one token, attend, compare, repeat."""
    w = wl.Workload("t", 2, 32, 8, 2, 500, 5e5, min_bits=1, max_bits=5, seed=4321)
    mgr, energies = wl.build_manager(w, DEV)
    wl.fill_cache(mgr, w, energies, DEV)
    for step in range(2):
        for li in range(2):
            T = mgr.seq_len
            q = wl.draw_q(w, li + 10 * step, DEV, T)
            k1, v1 = wl.draw_kv(w, energies[li], 1, 555 + li + 10 * step, DEV, pos0=T)
            out = mgr.append_and_attend(li, q, k1, v1)
            assert out.shape == (2, 32, 1, 128) and out.dtype == torch.float16
            plans = mgr._batched_args[li]['plans_np']
            q_rot = ops.rotate_q(mgr._batched_args[li]['plans'], q[:, :, 0].contiguous(), 8)
            ref, _ = _reference(oracle_lib, plans, mgr.quantizers[li],
                                mgr._k_packed[li].cpu().numpy(), mgr._k_norms[li].cpu().numpy(),
                                mgr._v_packed[li].cpu().numpy(), mgr._v_norms[li].cpu().numpy(),
                                q_rot.cpu().numpy(), [T + 1] * 2, 4)
            assert np.abs(out[:, :, 0].float().cpu().numpy() - ref).max() < TOL
        mgr.increment_seq_len()
    assert mgr.seq_len == 502
    assert mgr.cache_memory_bytes() < mgr.fp16_cache_bytes() / 3


def test_production_cache_and_fused_entry(oracle_lib):
    """Nibble layouts through BlockGTQProductionCache, and the reference-style
    per-head fused entry on slices of its cache."""
    from blockgtq_amd import BlockGTQProductionCache
    from blockgtq_amd.calibration import build_quantizers
    from blockgtq_amd.kernels import fused_blockgtq_decode_attention
    gen = torch.Generator().manual_seed(5)
    n_layers, nkv, nq, T = 1, 2, 8, 400
    en = wl.syn.block_energies(nkv, 64, gen)
    amp = torch.cat([en.sqrt(), en.sqrt()], -1).unsqueeze(1)
    layer_data = {0: {'q': torch.randn(nkv, 1024, 128, generator=gen) * amp,
                      'k': torch.randn(nkv, 256, 128, generator=gen) * amp}}
    quantizers, ba, ka = build_quantizers(layer_data, n_layers, nkv, 128, device=DEV)
    cache = BlockGTQProductionCache(quantizers, ba, ka, n_layers, nkv, nq, 128, T + 8, device=DEV)
    k = (torch.randn(1, nkv, T, 128, generator=gen) * amp).half().to(DEV)
    v = torch.randn(1, nkv, T, 128, generator=gen).half().to(DEV)
    cache._encode_batched(0, k, v, 0)
    cache.seq_len = T
    q = torch.randn(1, nq, 1, 128, generator=gen).half().to(DEV)
    k1 = (torch.randn(1, nkv, 1, 128, generator=gen) * amp).half().to(DEV)
    v1 = torch.randn(1, nkv, 1, 128, generator=gen).half().to(DEV)
    out = cache.encode_and_attend(0, q, k1, v1)
    q_rot = ops.rotate_q(ba[0]['plans'], q[:, :, 0].contiguous(), nkv)
    ref, ref_lse = _reference(oracle_lib, ba[0]['plans_np'], quantizers[0], cache.k_packed[0].cpu().numpy(),
                              cache.k_norms[0].cpu().numpy(), cache.v_packed[0].cpu().numpy(),
                              cache.v_norms[0].cpu().numpy(), q_rot.cpu().numpy(), [T + 1], 4, 1, 1)
    assert np.abs(out[:, :, 0].float().cpu().numpy() - ref).max() < TOL
    # the appended record equals the checker's bytes
    pl = ba[0]['plans_np'][1:2]
    codes, _, corr = oracle_lib.encode_k(pl, k1[0, 1].cpu().numpy())
    own = int(pl['k_mixed_bytes'][0])
    assert np.array_equal(cache.k_packed[0, 0, 1, T, :own].cpu().numpy(), oracle_lib.pack_k(pl, codes, 1)[0])
    # per-head fused entry with the reference's argument list
    Tn = T + 1
    for hi in range(nkv):
        q8, a = quantizers[0][hi], ka[0][hi]
        q_h = q8.rotate_q_for_packed_kernel(q[:, hi * 4:(hi + 1) * 4])
        o, lse = fused_blockgtq_decode_attention(
            q_h, cache.k_packed[0, :, hi:hi + 1, :Tn], cache.k_norms[0, :, hi:hi + 1, :Tn],
            a['codebook_flat'], a['lut_offset'], a['norm_group'], a['segments_b'],
            cache.v_packed[0, :, hi:hi + 1, :Tn], cache.v_norms[0, :, hi:hi + 1, :Tn], q8.v_lut,
            scale=cache.scale, t_splits=8, v_bits=3, v_rotation=q8._v_rot,
            k_nibble=True, v_nibble=True, return_lse=True)
        assert o.shape == (1, 4, 1, 128)
        assert np.abs(o[0, :, 0].float().cpu().numpy() - ref[0, hi * 4:(hi + 1) * 4]).max() < TOL
        assert np.abs(lse[0].cpu().numpy() - ref_lse[0, hi * 4:(hi + 1) * 4]).max() < LSE_TOL
        # the same call with tensors this package has never seen (copies of the codebook, the V table
        # and the V rotation): the entry must assemble the head's plan from its arguments alone
        o2, lse2 = fused_blockgtq_decode_attention(
            q_h, cache.k_packed[0, :, hi:hi + 1, :Tn], cache.k_norms[0, :, hi:hi + 1, :Tn],
            a['codebook_flat'].clone(), a['lut_offset'], a['norm_group'], list(a['segments_b']),
            cache.v_packed[0, :, hi:hi + 1, :Tn], cache.v_norms[0, :, hi:hi + 1, :Tn], q8.v_lut.clone(),
            scale=cache.scale, t_splits=8, v_bits=3, v_rotation=q8._v_rot.clone(),
            k_nibble=True, v_nibble=True, return_lse=True)
        assert np.abs(o2[0, :, 0].float().cpu().numpy() - ref[0, hi * 4:(hi + 1) * 4]).max() < TOL
        assert np.abs(lse2[0].cpu().numpy() - ref_lse[0, hi * 4:(hi + 1) * 4]).max() < LSE_TOL


def test_full_size_properties_config1():
    """Llama-3.1-8B head geometry at the full 4096-token context: invariance to
    the partition count and to the order of the context (softmax over a set)."""
    w = wl.WORKLOADS["llama8b_4k_k3v3"]
    mgr, energies = wl.build_manager(w, DEV)
    wl.fill_cache(mgr, w, energies, DEV)
    T = mgr.seq_len
    q = wl.draw_q(w, 0, DEV, T)[:, :, 0].contiguous()
    plans = mgr._batched_args[0]['plans']
    q_rot = ops.rotate_q(plans, q, w.n_kv)
    args = (mgr._k_packed[0], mgr._k_norms[0], mgr._v_packed[0], mgr._v_norms[0])
    base = ops.decode_attention(plans, q_rot, *args, T, n_splits=1, k_row_width=mgr._k_rows[0], v_row_width=mgr._vpb).float()
    for ns in (7, 64, 512):
        o = ops.decode_attention(plans, q_rot, *args, T, n_splits=ns, k_row_width=mgr._k_rows[0], v_row_width=mgr._vpb).float()
        assert (o - base).abs().max() < 1e-3
    perm = torch.randperm(T, generator=torch.Generator().manual_seed(1)).to(DEV)
    shuffled = tuple(t[:, :, :T][:, :, perm].contiguous() for t in args)
    o = ops.decode_attention(plans, q_rot, *shuffled, T, n_splits=16, k_row_width=mgr._k_rows[0], v_row_width=mgr._vpb).float()
    assert (o - base).abs().max() < 1e-3
    # doubling the context by repeating it leaves the output unchanged
    doubled = tuple(torch.cat([t[:, :, :T], t[:, :, :T]], dim=2).contiguous() for t in args)
    o = ops.decode_attention(plans, q_rot, *doubled, 2 * T, n_splits=32, k_row_width=mgr._k_rows[0], v_row_width=mgr._vpb).float()
    assert (o - base).abs().max() < 1e-3


@pytest.mark.parametrize("name", ["qwen3b_b8_32k_k3v3", "llama8b_128k_k2v2"])
def test_full_size_properties_long_contexts(name):
    """The 32k-token batch-8 workload and the 131072-token K2V2 workload (0-bit blocks,
    heavy-tailed data), one layer at full size: invariance to the partition count and to
    the order of the context, equality of the two decode kernels, and the LSE of a context
    repeated twice (+ln 2)."""
    from blockgtq_amd import _capi
    lib = _capi.lib()
    w = wl.WORKLOADS[name]
    mgr, energies = wl.build_manager(w, DEV, n_layers=1)
    wl.fill_cache(mgr, w, energies, DEV)
    T = mgr.seq_len
    assert T == w.context
    q = wl.draw_q(w, 0, DEV, T)[:, :, 0].contiguous()
    plans = mgr._batched_args[0]['plans']
    q_rot = ops.rotate_q(plans, q, w.n_kv)
    args = (mgr._k_packed[0], mgr._k_norms[0], mgr._v_packed[0], mgr._v_norms[0])
    kw = dict(k_row_width=mgr._k_rows[0], v_row_width=mgr._vpb, return_lse=True)
    base, base_lse = ops.decode_attention(plans, q_rot, *args, T, n_splits=0, **kw)
    base = base.float()
    assert torch.isfinite(base).all() and torch.isfinite(base_lse).all()
    tol = 2e-3 * max(1.0, float(base.abs().max()))
    for ns in (1, 37, 512):
        o, l = ops.decode_attention(plans, q_rot, *args, T, n_splits=ns, **kw)
        assert (o.float() - base).abs().max() < tol and (l - base_lse).abs().max() < LSE_TOL
    perm = torch.randperm(T, generator=torch.Generator().manual_seed(3)).to(DEV)
    shuffled = tuple(t[:, :, :T][:, :, perm].contiguous() for t in args)
    o, l = ops.decode_attention(plans, q_rot, *shuffled, T, n_splits=64, **kw)
    assert (o.float() - base).abs().max() < tol and (l - base_lse).abs().max() < LSE_TOL
    del shuffled
    if w.batch * T <= 1 << 18:                    # the layout-agnostic kernel is slow: long single rows only
        assert lib.bgtq_set_decode_path(1) == 0
        try:
            o, l = ops.decode_attention(plans, q_rot, *args, T, n_splits=128, **kw)
        finally:
            lib.bgtq_set_decode_path(0)
        assert (o.float() - base).abs().max() < tol and (l - base_lse).abs().max() < LSE_TOL
    half = T // 2                                  # first half repeated twice: same output, LSE + ln 2
    o1, l1 = ops.decode_attention(plans, q_rot, *args, half, n_splits=0, **kw)
    twice = tuple(torch.cat([t[:, :, :half], t[:, :, :half]], dim=2).contiguous() for t in args)
    o2, l2 = ops.decode_attention(plans, q_rot, *twice, 2 * half, n_splits=0, **kw)
    assert (o2.float() - o1.float()).abs().max() < tol
    assert (l2 - l1 - float(np.log(2.0))).abs().max() < LSE_TOL


def test_window_partial_merges_like_one_softmax(oracle_lib):
    """Closed form: softmax over [window ++ packed] == lse-merge of the two partials."""
    from blockgtq_amd import _capi
    args, qs, q_rot, kp, kn, vp, vn = _build(192, 1, 5, 3, 2, 4, 2, 300, seed=13)
    gen = torch.Generator().manual_seed(2)
    W = 37
    q = torch.randn(2, 8, 128, generator=gen).half().to(DEV)
    q_rot = ops.rotate_q(args['plans'], q, 2)
    kb = torch.randn(2, 2, W, 128, generator=gen).half().to(DEV)
    vb = torch.randn(2, 2, W, 128, generator=gen).half().to(DEV)
    lens = torch.tensor([W, 5], dtype=torch.int32, device=DEV)
    po = torch.empty(2, 8, 128, device=DEV); pl = torch.empty(2, 8, device=DEV)
    L = _capi.lib()
    _capi.check(L.bgtq_window_attn(_capi.ptr(q), q.stride(0), q.stride(1), _capi.ptr(kb), _capi.ptr(vb),
                                   kb.stride(0), kb.stride(1), kb.stride(2), _capi.ptr(lens), W, 2, 2, 4,
                                   128 ** -0.5, _capi.ptr(po), _capi.ptr(pl), _capi.stream_ptr()), "window")
    out, lse = ops.decode_attention(args['plans'], q_rot, kp, kn, vp, vn, 300, n_splits=4, return_lse=True,
                                    extra_out=po, extra_lse=pl)
    ref_p, lse_p = _reference(oracle_lib, args['plans_np'], qs, kp.cpu().numpy(), kn.cpu().numpy(),
                              vp.cpu().numpy(), vn.cpu().numpy(), q_rot.cpu().numpy(), [300, 300], 4)
    for b in range(2):
        n = int(lens[b])
        for hq in range(8):
            h = hq // 4
            lw = (q[b, hq].double() @ kb[b, h, :n].double().T).cpu() / np.sqrt(128)
            w_lse = torch.logsumexp(lw, 0)
            w_out = torch.softmax(lw, 0) @ vb[b, h, :n].double().cpu()
            a = torch.tensor([float(lse_p[b, hq]), float(w_lse)], dtype=torch.float64)
            wgt = torch.softmax(a, 0)
            want = wgt[0] * torch.tensor(ref_p[b, hq]).double() + wgt[1] * w_out
            assert (out[b, hq].double().cpu() - want).abs().max() < TOL
            assert abs(float(lse[b, hq]) - float(torch.logsumexp(a, 0))) < LSE_TOL


def test_with_buffer_manager_keeps_sink_and_window_in_fp16(oracle_lib):
    """Ragged batch with 4 fp16 sink tokens and a 16-token fp16 recent window: after a few
    appends the output equals one softmax over [sink | dequantised middle | recent], where the
    middle tokens went through the packers exactly once, when they left the window."""
    from blockgtq_amd.packed_kv_manager import BlockGTQKVManager
    ns, win, B, H, gqa, L = 4, 16, 3, 2, 4, 1
    lens0 = [40, 21, 33]                         # row 1 starts with one packed token, others more
    steps = 5
    qs, ens = zip(*[make_quantizer(seed=90 + h, head=h, device=DEV, max_bits=5) for h in range(H)])
    mgr = BlockGTQKVManager(L, H * gqa, H, 128, 128, batch_size=B, device=DEV, n_sink=ns, recent_window=win)
    mgr.set_quantizers(0, list(qs))
    Tmax = max(lens0) + steps
    hist_k = np.zeros((B, H, Tmax, 128), np.float16)
    hist_v = np.zeros((B, H, Tmax, 128), np.float16)
    for b in range(B):
        for h in range(H):
            k, v, _ = make_kv(ens[h], Tmax, seed=500 + 10 * b + h)
            hist_k[b, h], hist_v[b, h] = k, v
    k0 = torch.tensor(hist_k[:, :, :max(lens0)]).to(DEV)
    v0 = torch.tensor(hist_v[:, :, :max(lens0)]).to(DEV)
    # rows shorter than the padded prefix: their tail positions come from their own history
    # later, so hand every row its own first lens0[b] tokens and let the padding be ignored
    mgr.fill_buffered(0, k0, v0, lens0)
    mgr.set_seq_lens(lens0)
    lens = list(lens0)
    plans_np = mgr._batched_args[0]['plans_np']
    gen = torch.Generator().manual_seed(77)
    for step in range(steps):
        q = torch.randn(B, H * gqa, 1, 128, generator=gen).half().to(DEV)
        k1 = torch.tensor(np.stack([hist_k[b, :, lens[b]] for b in range(B)])[:, :, None]).to(DEV)
        v1 = torch.tensor(np.stack([hist_v[b, :, lens[b]] for b in range(B)])[:, :, None]).to(DEV)
        out = mgr.append_and_attend(0, q, k1, v1)[:, :, 0].float().cpu().numpy()
        mgr.increment_seq_len()
        lens = [t + 1 for t in lens]
        qn = q[:, :, 0].cpu().numpy()
        for b in range(B):
            T = lens[b]
            for h in range(H):
                pl = plans_np[h:h + 1]
                mid = slice(ns, T - win)
                codes, raw, _ = oracle_lib.encode_k(pl, hist_k[b, h, mid])
                kd = oracle_lib.dequant_k(pl, codes, oracle_lib.f2h(raw[:, :max(int(pl['n_seg'][0]), 1)]))
                vc, vn = oracle_lib.encode_v(pl, hist_v[b, h, mid])
                vd = oracle_lib.dequant_v(pl, vc, vn).astype(np.float64) @ pl['v_rot'][0].reshape(128, 128).astype(np.float64)
                fp = np.r_[0:ns, T - win:T]
                qh = qn[b, h * gqa:(h + 1) * gqa]
                q_rot = oracle_lib.rotate_q(pl, qh).astype(np.float64)
                logits = np.concatenate([q_rot @ kd.astype(np.float64).T,
                                         qh.astype(np.float64) @ hist_k[b, h, fp].astype(np.float64).T], 1) / np.sqrt(128)
                p = np.exp(logits - logits.max(1, keepdims=True))
                p /= p.sum(1, keepdims=True)
                ref = p @ np.concatenate([vd, hist_v[b, h, fp].astype(np.float64)], 0)
                got = out[b, h * gqa:(h + 1) * gqa]
                assert np.abs(got - ref).max() < TOL, (step, b, h, np.abs(got - ref).max())


def test_with_buffer_manager_at_the_full_ragged_shape(oracle_lib, decode_path):
    """The ragged with-buffer workload at its stated shape, one layer: 32 sequences of 1024..16384
    tokens, 32 query / 8 KV heads, 4 fp16 sink tokens, 128-token fp16 window, two appends through
    the manager.  Three (row, head) pairs are checked against one fp64 softmax over
    [sink | dequantised middle | window] built from the checker's records; all rows and heads
    must agree between two managers that partition the context differently."""
    if decode_path == "generic":
        pytest.skip("the layout-agnostic kernel is covered at this shape's reduced size above")
    w = wl.WORKLOADS["qwen3_8b_b32_ragged_buffered"]
    lens = list(w.seq_lens)
    Tmax, steps, ns, win, gqa = max(lens), 2, w.n_sink, w.window, w.n_q // w.n_kv
    assert w.batch == 32 and w.n_kv == 8 and min(lens) >= 1024 and Tmax <= 16384 and (ns, win) == (4, 128)
    mgrs = []
    for n_splits in (0, 5):
        mgr, energies = wl.build_manager(w, DEV, max_T=Tmax + steps + 8, n_layers=1)
        mgr.n_splits = n_splits
        mgrs.append(mgr)
    hist_k, hist_v = wl.draw_kv(w, energies[0], Tmax + steps, 0, DEV)
    for mgr in mgrs:
        mgr.fill_buffered(0, hist_k[:, :, :Tmax], hist_v[:, :, :Tmax], lens)
        mgr.set_seq_lens(lens)
    plans_np = mgrs[0]._batched_args[0]['plans_np']
    rows = [int(np.argmin(lens)), int(np.argmax(lens)), 7]
    pairs = list(zip(rows, (0, 7, 3)))
    ar = torch.arange(w.batch, device=DEV)
    gen = torch.Generator().manual_seed(31)
    for step in range(steps):
        q = torch.randn(w.batch, w.n_q, 1, 128, generator=gen).half().to(DEV)
        at = torch.tensor(lens, device=DEV)
        k1 = hist_k[ar, :, at].unsqueeze(2).contiguous()
        v1 = hist_v[ar, :, at].unsqueeze(2).contiguous()
        outs = [mgr.append_and_attend(0, q, k1, v1)[:, :, 0].float() for mgr in mgrs]
        for mgr in mgrs:
            mgr.increment_seq_len()
        lens = [t + 1 for t in lens]
        assert torch.isfinite(outs[0]).all()
        assert (outs[0] - outs[1]).abs().max() < 1e-3
        got_all = outs[0].cpu().numpy()
        for b, h in pairs:
            T = lens[b]
            hk = hist_k[b, h, :T].cpu().numpy()
            hv = hist_v[b, h, :T].cpu().numpy()
            pl = plans_np[h:h + 1]
            mid = slice(ns, T - win)
            codes, raw, _ = oracle_lib.encode_k(pl, hk[mid])
            kd = oracle_lib.dequant_k(pl, codes, oracle_lib.f2h(raw[:, :max(int(pl['n_seg'][0]), 1)]))
            vc, vn = oracle_lib.encode_v(pl, hv[mid])
            vd = oracle_lib.dequant_v(pl, vc, vn).astype(np.float64) @ pl['v_rot'][0].reshape(128, 128).astype(np.float64)
            fp = np.r_[0:ns, T - win:T]
            qh = q[b, h * gqa:(h + 1) * gqa, 0].cpu().numpy()
            q_rot = oracle_lib.rotate_q(pl, qh).astype(np.float64)
            logits = np.concatenate([q_rot @ kd.astype(np.float64).T,
                                     qh.astype(np.float64) @ hk[fp].astype(np.float64).T], 1) / np.sqrt(128)
            p = np.exp(logits - logits.max(1, keepdims=True))
            p /= p.sum(1, keepdims=True)
            ref = p @ np.concatenate([vd, hv[fp].astype(np.float64)], 0)
            got = got_all[b, h * gqa:(h + 1) * gqa]
            assert np.abs(got - ref).max() < TOL, (step, b, h, np.abs(got - ref).max())


@pytest.mark.parametrize("k_layout,v_layout,vb", [(0, 0, 3), (1, 1, 3), (1, 0, 4), (0, 1, 2), (1, 1, 4)])
def test_mfma_kernel_takes_every_record_layout(oracle_lib, k_layout, v_layout, vb):
    """With the layout-agnostic kernel switched off, the MFMA kernel must accept bit-packed
    and mixed K records and bit-packed and nibble V records in any combination."""
    from blockgtq_amd import _capi
    lib = _capi.lib()
    args, qs, q_rot, kp, kn, vp, vn = _build(192, 1, 6, vb, 2, 4, 2, 333, seed=7 + 3 * k_layout + v_layout,
                                             k_layout=k_layout, v_layout=v_layout)
    ref, ref_lse = _reference(oracle_lib, args['plans_np'], qs, kp.cpu().numpy(), kn.cpu().numpy(),
                              vp.cpu().numpy(), vn.cpu().numpy(), q_rot.cpu().numpy(), [333] * 2, 4,
                              k_layout, v_layout, vb)
    # the same records in rows 4 bytes wider, as the cache classes store 32- and 64-byte records
    vw = vp.shape[-1]
    vp_wide = torch.full((*vp.shape[:-1], P.cache_row_bytes(vw)), 0xA5, dtype=torch.uint8, device=DEV)[..., :vw]
    vp_wide.copy_(vp)
    assert lib.bgtq_set_decode_path(2) == 0
    try:
        for ns in (1, 4):
            for vrec in (vp, vp_wide):
                out, lse = ops.decode_attention(args['plans'], q_rot, kp, kn, vrec, vn, 333, n_splits=ns,
                                                k_layout=k_layout, v_layout=v_layout, return_lse=True)
                assert np.abs(out.float().cpu().numpy() - ref).max() < TOL
                assert np.abs(lse.cpu().numpy() - ref_lse).max() < LSE_TOL
    finally:
        lib.bgtq_set_decode_path(0)


def test_production_cache_tracks_the_unpacked_torch_path():
    """No checker involved: the cache's output against softmax attention in fp64
    over K round-tripped by the plain-torch pipeline and V round-tripped by the
    torch V quantizer (same tables, different arithmetic and no byte format)."""
    from blockgtq_amd import BlockGTQPipeline, BlockGTQProductionCache
    from blockgtq_amd.calibration import build_quantizers
    gen = torch.Generator().manual_seed(8)
    nkv, nq, T = 2, 8, 700
    en = wl.syn.block_energies(nkv, 64, gen)
    amp = torch.cat([en.sqrt(), en.sqrt()], -1).unsqueeze(1)
    layer_data = {0: {'q': torch.randn(nkv, 1024, 128, generator=gen) * amp,
                      'k': torch.randn(nkv, 256, 128, generator=gen) * amp}}
    quantizers, ba, ka = build_quantizers(layer_data, 1, nkv, 128, device=DEV)
    cache = BlockGTQProductionCache(quantizers, ba, ka, 1, nkv, nq, 128, T + 8, device=DEV)
    cache.quant_mode = P.QUANT_EXACT       # the 256-bin table moves codes near cell edges (1e-2 here)
    k = (torch.randn(1, nkv, T + 1, 128, generator=gen) * amp).half().to(DEV)
    v = torch.randn(1, nkv, T + 1, 128, generator=gen).half().to(DEV)
    q = (torch.randn(1, nq, 1, 128, generator=gen) * amp.repeat_interleave(4, 0).unsqueeze(0) * 0.3).half().to(DEV)
    cache._encode_batched(0, k[:, :, :T], v[:, :, :T], 0)
    cache.seq_len = T
    out = cache.encode_and_attend(0, q, k[:, :, T:], v[:, :, T:])[0, :, 0].double().cpu()
    for hi in range(nkv):
        q8 = quantizers[0][hi]
        pipe = BlockGTQPipeline(128, rotation_threshold=q8.rotation_threshold, device=DEV)
        pipe.set_allocation(q8.bit_allocation)
        k_hat = pipe.compress_decompress(k[0, hi].float()).double().cpu()
        v_hat = q8._v_quantizer.dequantize(*q8._v_quantizer.quantize(v[0, hi].float())).double().cpu()
        qh = q[0, hi * 4:(hi + 1) * 4, 0].double().cpu()
        ref = torch.softmax(qh @ k_hat.T / 128 ** 0.5, -1) @ v_hat
        assert (out[hi * 4:(hi + 1) * 4] - ref).abs().max() < TOL


@pytest.mark.parametrize("k_layout,v_layout,vb", [(0, 0, 3), (1, 1, 3), (0, 0, 2), (1, 0, 4)])
def test_dequantised_records_equal_the_checker_bit_for_bit(oracle_lib, k_layout, v_layout, vb):
    mn = 0 if vb == 2 else 1
    args, qs, q_rot, kp, kn, vp, vn = _build(160, mn, 6, vb, 2, 4, 2, 211, seed=40 + vb + k_layout,
                                             k_layout=k_layout, v_layout=v_layout)
    T = 209                                   # not a multiple of the kernel's token tile
    k_hat, v_hat = ops.dequant_kv(args['plans'], kp, kn, vp, vn, T, k_layout=k_layout, v_layout=v_layout)
    assert k_hat.shape == (2, 2, T, 128) and v_hat.dtype == torch.float16
    for b in range(2):
        for h in range(2):
            pl = args['plans_np'][h:h + 1]
            ng = int(pl[0]['n_seg'])
            codes = oracle_lib.unpack_k(pl, kp[b, h, :T].cpu().numpy(), k_layout)
            ref_k = oracle_lib.dequant_k(pl, codes, kn[b, h, :T, :max(ng, 1)].cpu().numpy())
            vcodes = oracle_lib.unpack_v(vp[b, h, :T].cpu().numpy(), vb if not v_layout else 4, bool(v_layout))
            ref_v = oracle_lib.dequant_v(pl, vcodes, vn[b, h, :T].cpu().numpy())
            # centroid (fp16) x norm (fp16) is exact in fp32, so one rounding on either side
            assert np.array_equal(k_hat[b, h].cpu().numpy().view(np.uint16), ref_k.astype(np.float16).view(np.uint16))
            assert np.array_equal(v_hat[b, h].cpu().numpy().view(np.uint16), ref_v.astype(np.float16).view(np.uint16))


def _causal_reference(orc, pl, q_rot, kp, kn, vp, vn, k_layout, v_layout, vb, offset, scale=128 ** -0.5):
    """fp64 attention of q_rot (gqa, S, 128) over one head's records, row s seeing t <= offset + s."""
    T = kp.shape[0]
    ng = int(pl[0]['n_seg'])
    k_hat = orc.dequant_k(pl, orc.unpack_k(pl, kp, k_layout), kn[:, :max(ng, 1)]).astype(np.float64)
    v_hat = orc.dequant_v(pl, orc.unpack_v(vp, vb if not v_layout else 4, bool(v_layout)), vn).astype(np.float64)
    logits = q_rot.astype(np.float64) @ k_hat.T * scale
    S = q_rot.shape[1]
    mask = np.arange(T)[None, :] <= (offset + np.arange(S))[:, None]
    logits = np.where(mask[None], logits, -np.inf)
    p = np.exp(logits - logits.max(-1, keepdims=True))
    p /= p.sum(-1, keepdims=True)
    return (p @ v_hat) @ pl[0]['v_rot'].reshape(128, 128).astype(np.float64)


@pytest.mark.parametrize("k_layout,v_layout", [(0, 0), (1, 1)])
def test_prompt_attention_over_the_packed_cache(oracle_lib, k_layout, v_layout):
    """Reference-style per-head entry: whole prompt (S = T), and a later chunk of
    queries against a longer cache (q_pos_offset)."""
    from blockgtq_amd.kernels import fused_blockgtq_prefill_attention
    from helpers import make_kv
    vb, T, gqa = 3, 150, 4
    args, qs, _, kp, kn, vp, vn = _build(192, 1, 6, vb, 2, gqa, 1, T, seed=61 + k_layout,
                                         k_layout=k_layout, v_layout=v_layout)
    gen = torch.Generator().manual_seed(5)
    for hi in range(2):
        q8 = qs[hi]
        a = q8.build_kernel_args()
        q = (torch.randn(1, gqa, T, 128, generator=gen) * 0.7).half().to(DEV)
        q_rot = q8.rotate_q_for_packed_kernel(q)
        pl = args['plans_np'][hi:hi + 1]
        sl = lambda x: x[:, hi:hi + 1, :T]
        for S, off in ((T, 0), (37, T - 37)):
            out = fused_blockgtq_prefill_attention(
                q_rot[:, :, T - S:], sl(kp), sl(kn), a['codebook_flat'], a['lut_offset'], a['norm_group'],
                a['segments_b'], sl(vp), sl(vn), q8.v_lut, v_bits=vb, v_rotation=q8._v_rot,
                is_causal=True, q_pos_offset=off, k_nibble=bool(k_layout), v_nibble=bool(v_layout))
            assert out.shape == (1, gqa, S, 128) and out.dtype == torch.float16
            ref = _causal_reference(oracle_lib, pl, q_rot[0, :, T - S:].cpu().numpy(), kp[0, hi, :T].cpu().numpy(),
                                    kn[0, hi, :T].cpu().numpy(), vp[0, hi, :T].cpu().numpy(),
                                    vn[0, hi, :T].cpu().numpy(), k_layout, v_layout, vb, off)
            assert np.abs(out[0].double().cpu().numpy() - ref).max() < TOL


def test_prompt_attention_rows_equal_decode_steps():
    """Size-independent property through the cache class: row s of the prompt-phase
    attention is the decode attention of that query over the first s + 1 records."""
    from blockgtq_amd import BlockGTQProductionCache
    from blockgtq_amd.calibration import build_quantizers
    from blockgtq_amd.prefill import packed_prefill_attention
    gen = torch.Generator().manual_seed(12)
    nkv, nq, T = 2, 8, 300
    en = wl.syn.block_energies(nkv, 64, gen)
    amp = torch.cat([en.sqrt(), en.sqrt()], -1).unsqueeze(1)
    layer_data = {0: {'q': torch.randn(nkv, 1024, 128, generator=gen) * amp,
                      'k': torch.randn(nkv, 256, 128, generator=gen) * amp}}
    quantizers, ba, ka = build_quantizers(layer_data, 1, nkv, 128, device=DEV)
    cache = BlockGTQProductionCache(quantizers, ba, ka, 1, nkv, nq, 128, T + 8, device=DEV, batch_size=2)
    k = (torch.randn(2, nkv, T, 128, generator=gen) * amp).half().to(DEV)
    v = torch.randn(2, nkv, T, 128, generator=gen).half().to(DEV)
    q = (torch.randn(2, nq, T, 128, generator=gen) * 0.5).half().to(DEV)
    cache._encode_batched(0, k, v, 0)
    full = packed_prefill_attention(cache, 0, q, T)
    assert full.shape == (2, nq, T, 128)
    plans = ba[0]['plans']
    for s in (0, 63, 64, 299):
        q_rot = ops.rotate_q(plans, q[:, :, s].contiguous(), nkv)
        dec = ops.decode_attention(plans, q_rot, cache.k_packed[0], cache.k_norms[0], cache.v_packed[0],
                                   cache.v_norms[0], s + 1, k_layout=cache._k_layout, v_layout=cache._v_layout,
                                   k_row_width=cache.k_bytes_per_tok, v_row_width=cache.vpb)
        assert (full[:, :, s].float() - dec.float()).abs().max() < TOL


@pytest.mark.parametrize("gqa,n_kv,B,T,S,kl,vl,vb,mn,mx,causal", [
    (8, 2, 2, 333, 333, 0, 0, 3, 1, 6, True),      # whole prompt, two tiles and a tail per late block
    (4, 2, 1, 500, 77, 1, 1, 3, 1, 8, True),       # a later chunk of queries, nibble records, raw-byte units
    (1, 3, 1, 200, 200, 0, 0, 2, 0, 4, True),      # one query head per KV head, 0-bit blocks, 2-bit V
    (3, 1, 2, 190, 190, 0, 1, 4, 1, 5, True),      # query groups that do not divide the 128 rows of a work-group
    (16, 1, 1, 130, 130, 1, 0, 4, 2, 8, True),
    (8, 1, 1, 150, 40, 0, 0, 3, 1, 5, False),      # no mask: every query sees all records
])
def test_prompt_kernel_all_heads_in_one_launch(oracle_lib, decode_path, gqa, n_kv, B, T, S, kl, vl, vb, mn, mx, causal):
    """``bgtq_prefill_attn`` (every KV head and batch row in one launch) against fp64 attention over the
    checker's dequantised records, row s seeing records t <= T - S + s."""
    if decode_path == "generic":
        pytest.skip("one kernel serves this entry point")
    args, qs, _, kp, kn, vp, vn = _build(192 if mx > 4 else 128, mn, mx, vb, n_kv, gqa, B, T, seed=70 + gqa + kl,
                                         k_layout=kl, v_layout=vl)
    gen = torch.Generator().manual_seed(gqa)
    q = (torch.randn(B, n_kv * gqa, S, 128, generator=gen) * 0.6).half().to(DEV)
    q_rot = torch.stack([ops.rotate_q(args['plans'], q[:, :, s].contiguous(), n_kv) for s in range(S)], 2)
    off = T - S
    out = ops.prefill_attention_packed(args['plans'], q_rot.contiguous(), kp, kn, vp, vn, T, k_layout=kl, v_layout=vl,
                                       is_causal=causal, q_pos_offset=off)
    assert out is not None, "the kernel refused a layout it is meant to take"
    assert out.shape == (B, n_kv * gqa, S, 128) and out.dtype == torch.float16
    got = out.float().cpu().numpy()
    for b in range(B):
        for h in range(n_kv):
            ref = _causal_reference(oracle_lib, args['plans_np'][h:h + 1], q_rot[b, h * gqa:(h + 1) * gqa].cpu().numpy(),
                                    kp[b, h, :T].cpu().numpy(), kn[b, h, :T].cpu().numpy(), vp[b, h, :T].cpu().numpy(),
                                    vn[b, h, :T].cpu().numpy(), kl, vl, vb, off if causal else T)
            assert np.abs(got[b, h * gqa:(h + 1) * gqa] - ref).max() < TOL
    # without the un-rotation the kernel's output times the V rotation is the same thing
    raw = ops.prefill_attention_packed(args['plans'], q_rot.contiguous(), kp, kn, vp, vn, T, k_layout=kl, v_layout=vl,
                                       is_causal=causal, q_pos_offset=off, unrotate=False)
    v_rot = torch.stack([q8._v_rot.float() for q8 in qs]).to(DEV)
    back = (raw.float().reshape(B, n_kv, gqa * S, 128) @ v_rot.unsqueeze(0)).reshape(B, n_kv * gqa, S, 128)
    assert (back - out.float()).abs().max() < TOL


def test_prompt_kernel_refuses_layouts_it_cannot_take():
    """Strided K records come back as 'unsupported' from the entry point (None here) with nothing
    launched; the host wrapper copies such records into rows the kernel walks and gives the very
    result of the conforming call, so no other attention stands behind the kernel.  An empty batch
    is no error."""
    from blockgtq_amd import _capi
    args, qs, q_rot1, kp, kn, vp, vn = _build(192, 1, 5, 3, 1, 4, 1, 100, seed=5)
    g = torch.Generator(device=DEV).manual_seed(6)
    q = torch.randn(1, 4, 8, 128, generator=g, device=DEV).half()
    wide = torch.zeros(1, 1, 102, kp.shape[-1] + 4, dtype=torch.uint8, device=DEV)
    wide[..., :kp.shape[-1]] = kp
    strided = wide[..., :kp.shape[-1]]
    assert ops.prefill_attention_packed(args['plans'], q, strided, kn, vp, vn, 100) is None
    want = ops.prefill_attention_packed(args['plans'], q, kp, kn, vp, vn, 100, q_pos_offset=92)
    assert want is not None
    got = ops.prefill_attention_records(args['plans'], q, strided, kn, vp, vn, 100, q_pos_offset=92)
    assert torch.equal(got, want)
    odd_q = torch.zeros(1, 4, 8, 132, dtype=torch.float16, device=DEV)[..., 2:130]
    odd_q.copy_(q)
    assert torch.equal(ops.prefill_attention_records(args['plans'], odd_q, kp, kn, vp, vn, 100, q_pos_offset=92), want)
    assert ops.prefill_attention_records(args['plans'], q[:0], kp[:0], kn[:0], vp[:0], vn[:0], 100).shape == (0, 4, 8, 128)
    code = _capi.lib().bgtq_prefill_attn(
        _capi.ptr(args['plans']), _capi.ptr(q), q.stride(0), q.stride(1), q.stride(2),
        _capi.ptr(kp), kp.stride(0), kp.stride(1), kp.stride(2), kp.shape[-1],
        _capi.ptr(kn), kn.stride(0), kn.stride(1), kn.stride(2),
        _capi.ptr(vp), vp.stride(0), vp.stride(1), vp.stride(2), vp.shape[-1],
        _capi.ptr(vn), vn.stride(0), vn.stride(1), vn.stride(2),
        0, 1, 4, 8, 100, 92, 1, 0, 0, 0.088, 1,
        _capi.ptr(want), want.stride(0), want.stride(1), want.stride(2), _capi.stream_ptr(torch.device(DEV)))
    assert code == 0


def test_merge_entry_point_refuses_what_its_kernel_cannot_take():
    """Misaligned partial vectors and more partitions than the kernel's table holds come back
    as error codes from the C-ABI, before anything is launched."""
    from blockgtq_amd import _capi
    L = _capi.lib()
    q, _ = make_quantizer(seed=3, device=DEV)
    plans = q.device_plan()
    part = torch.zeros(4 * 128 + 4, dtype=torch.float32, device=DEV)
    lse = torch.zeros(4, dtype=torch.float32, device=DEV)
    out = torch.zeros(1, 1, 128, dtype=torch.float16, device=DEV)
    st = _capi.stream_ptr(torch.device(DEV))

    def call(part_ptr, n_splits):
        return L.bgtq_lse_reduce(_capi.ptr(plans), part_ptr, _capi.ptr(lse), n_splits, None, None, 0,
                                 1, 1, 1, 1, _capi.ptr(out), out.stride(0), out.stride(1), None, st)

    assert call(_capi.ptr(part), 4) == 0
    assert call(_capi.ptr(part[1:]), 4) != 0                   # 4 bytes off a 16-byte boundary
    assert call(_capi.ptr(part), 513) != 0                     # BGTQ_MAX_SPLITS is 512
    torch.cuda.synchronize()
    with pytest.raises(_capi.BgtqError):
        _capi.check(call(_capi.ptr(part[1:]), 4), "bgtq_lse_reduce")


def test_window_swap_equals_indexed_copies():
    """The one-launch ring update of the with-buffer append against the tensor operations it
    replaces, bit for bit, on strided buffers (a layer slice of a larger tensor)."""
    g = torch.Generator(device=DEV).manual_seed(5)
    B, n_kv, W = 5, 3, 12
    big_k = torch.randn(2, B, n_kv, W, 128, generator=g, device=DEV).half()
    big_v = torch.randn(2, B, n_kv, W, 128, generator=g, device=DEV).half()
    kb, vb = big_k[1], big_v[1]
    new = torch.randn(2, B, n_kv, 3, 128, generator=g, device=DEV).half()
    nk, nv = new[0][:, :, 1], new[1][:, :, 1]                 # (B, n_kv, D) views with gaps
    slot = torch.tensor([0, 11, 4, 4, 7], dtype=torch.int32, device=DEV)
    ar = torch.arange(B, device=DEV)
    ref_k, ref_v = kb.clone(), vb.clone()
    want_old_k = ref_k[ar, :, slot.long()].unsqueeze(2).clone()
    want_old_v = ref_v[ar, :, slot.long()].unsqueeze(2).clone()
    ref_k[ar, :, slot.long()] = nk
    ref_v[ar, :, slot.long()] = nv
    old_k, old_v = ops.window_swap(kb, vb, nk, nv, slot)
    assert torch.equal(old_k, want_old_k) and torch.equal(old_v, want_old_v)
    assert torch.equal(kb, ref_k) and torch.equal(vb, ref_v)
    assert torch.equal(big_k[0], big_k[0]) and not torch.isnan(big_k[0].float()).any()
    # a slot outside the ring moves nothing for that row
    before = kb.clone()
    slot2 = torch.tensor([-1, 12, 3, 3, 3], dtype=torch.int32, device=DEV)
    old_k2, _ = ops.window_swap(kb, vb, nk, nv, slot2)
    assert torch.equal(kb[:2], before[:2]) and not old_k2[:2].any()
    assert torch.equal(kb[2:, :, 3], nk[2:])


@pytest.mark.parametrize("B,n_kv,gqa,W,lens,offset", [
    (3, 2, 4, 132, [132, 77, 0], 0),        # four heads per pass, an empty row
    (2, 1, 7, 40, [40, 1], 0),              # two passes, the second with three heads
    (2, 2, 1, 200, [200, 129], 0),          # one head per KV head
    (1, 1, 2, 4000, [3999], 0),             # window too long for four score rows in LDS
    (2, 2, 4, 50, [50, 13], 1),             # rows off the 16-byte boundaries: the general kernel
])
def test_window_attention_every_path(B, n_kv, gqa, W, lens, offset):
    """fp16 window partial against a float64 softmax: out within 1e-3, lse within 1e-3."""
    g = torch.Generator(device=DEV).manual_seed(W + gqa)
    n_q = n_kv * gqa

    def buf(*shape):                         # optionally shifted by `offset` halves inside a larger block
        flat = torch.randn(int(np.prod(shape)) + 8, generator=g, device=DEV).half()
        return flat[offset:offset + int(np.prod(shape))].view(*shape)

    q, kb, vb = buf(B, n_q, 128), buf(B, n_kv, W, 128), buf(B, n_kv, W, 128)
    lens_t = torch.tensor(lens, dtype=torch.int32, device=DEV)
    po, pl = ops.window_attention(q, kb, vb, lens_t, n_kv)
    for b in range(B):
        n = lens[b]
        for hq in range(n_q):
            if n == 0:
                assert float(pl[b, hq]) == float("-inf") and not po[b, hq].any()
                continue
            h = hq // gqa
            lw = (q[b, hq].double() @ kb[b, h, :n].double().T) / np.sqrt(128)
            want = torch.softmax(lw, 0) @ vb[b, h, :n].double()
            assert (po[b, hq].double() - want).abs().max() < 1e-3
            assert abs(float(pl[b, hq]) - float(torch.logsumexp(lw, 0))) < 1e-3


def test_manager_with_rotated_queries_equals_manager_that_rotates_them():
    """Queries that arrive rotated (rotation folded into q_proj) take the K/V-only append; cache
    bytes and outputs equal those of the manager that rotates the queries itself."""
    w = wl.Workload("t", 2, 16, 2, 2, 300, 1e6, min_bits=1, max_bits=5, seed=99)
    a, energies = wl.build_manager(w, DEV)
    b, _ = wl.build_manager(w, DEV)
    wl.fill_cache(a, w, energies, DEV)
    wl.fill_cache(b, w, energies, DEV)
    for li in range(2):
        for qz in b.quantizers[li]:
            qz._q_perm_baked = True                      # b's caller hands over rotated queries
    for step in range(2):
        for li in range(2):
            T = a.seq_len
            q = wl.draw_q(w, li + 7 * step, DEV, T)
            k1, v1 = wl.draw_kv(w, energies[li], 1, 31 + li + 7 * step, DEV, pos0=T)
            out_a = a.append_and_attend(li, q, k1, v1)
            q_rot = ops.rotate_q(a._batched_args[li]['plans'], q[:, :, 0].contiguous(), w.n_kv)
            out_b = b.append_and_attend(li, q_rot.unsqueeze(2), k1, v1)
            assert torch.equal(out_a, out_b)
            assert torch.equal(a._k_packed[li], b._k_packed[li]) and torch.equal(a._v_packed[li], b._v_packed[li])
            assert torch.equal(a._k_norms[li], b._k_norms[li]) and torch.equal(a._v_norms[li], b._v_norms[li])
        a.increment_seq_len(); b.increment_seq_len()


def test_manager_with_baked_q_proj_equals_manager_that_rotates_queries():
    """bake_q_permutations folds permutation + rotation into q_proj.  A manager whose model went
    through it, fed the baked projection's output, must fill a byte-identical cache and return the
    same attention (within 2e-3) as the plain manager fed the original projection's output."""
    import copy
    import types
    w = wl.Workload("t", 2, 16, 2, 2, 300, 1e6, min_bits=1, max_bits=5, seed=101)
    a, energies = wl.build_manager(w, DEV)
    b, _ = wl.build_manager(w, DEV)
    wl.fill_cache(a, w, energies, DEV)
    wl.fill_cache(b, w, energies, DEV)
    hid = 96
    torch.manual_seed(5)

    def fake_model():
        layers = [types.SimpleNamespace(self_attn=types.SimpleNamespace(
            q_proj=torch.nn.Linear(hid, w.n_q * 128, bias=(li == 0)).to(DEV))) for li in range(2)]
        return types.SimpleNamespace(model=types.SimpleNamespace(layers=layers))

    plain = fake_model()
    baked = copy.deepcopy(plain)
    b.bake_q_permutations(baked, w.n_kv, w.n_q)
    assert all(qz._q_perm_baked for li in range(2) for qz in b.quantizers[li])
    assert not any(qz._q_perm_baked for li in range(2) for qz in a.quantizers[li])
    g = torch.Generator(device=DEV).manual_seed(17)
    with torch.no_grad():
        for step in range(2):
            for li in range(2):
                T = a.seq_len
                x = torch.randn(w.batch, hid, generator=g, device=DEV)
                k1, v1 = wl.draw_kv(w, energies[li], 1, 41 + li + 7 * step, DEV, pos0=T)
                qa = plain.model.layers[li].self_attn.q_proj(x).view(w.batch, w.n_q, 1, 128).half()
                qb = baked.model.layers[li].self_attn.q_proj(x).view(w.batch, w.n_q, 1, 128).half()
                out_a = a.append_and_attend(li, qa, k1, v1)
                out_b = b.append_and_attend(li, qb, k1, v1)
                assert (out_a.float() - out_b.float()).abs().max() < TOL
                assert torch.equal(a._k_packed[li], b._k_packed[li]) and torch.equal(a._v_packed[li], b._v_packed[li])
                assert torch.equal(a._k_norms[li], b._k_norms[li]) and torch.equal(a._v_norms[li], b._v_norms[li])
            a.increment_seq_len(); b.increment_seq_len()


def test_plan_with_many_units_and_every_code_width(oracle_lib):
    """Six segments (1..5 and 8 bits) of lengths 2, 2, 2, 10, 2, 110: 20 units, most of them in the last
    segment (a loop, where the usual segments are straight-line code), 8 query heads per KV head,
    bit-packed and mixed records."""
    from blockgtq_amd.quantizer import build_batched_encode_args, encode_k_into, encode_v_into
    alloc = [1, 2, 3] + [4] * 5 + [5] + [8] * 55
    T, gqa = 300, 8
    for kl in (0, 1):
        q, en = make_quantizer(seed=3, alloc=alloc, device=DEV)
        args = build_batched_encode_args([q], device=DEV)
        assert int(args['plans_np']['n_seg'][0]) == 6
        own = args['max_mixed_bytes'] if kl else args['max_tpb']
        kw = P.cache_row_bytes(own)
        k, v, qq = make_kv(en, T, seed=77, n_q=gqa)
        kp = torch.zeros(1, 1, T + 2, kw, dtype=torch.uint8, device=DEV)
        kn = torch.zeros(1, 1, T + 2, args['max_n_groups'], dtype=torch.float16, device=DEV)
        vp = torch.zeros(1, 1, T + 2, args['v_packed_bytes'], dtype=torch.uint8, device=DEV)
        vn = torch.zeros(1, 1, T + 2, dtype=torch.float16, device=DEV)
        encode_k_into(args['plans'], torch.tensor(k[None, None]).to(DEV), kp, kn, 0, kw, args['max_n_groups'], kl)
        encode_v_into(args['plans'], torch.tensor(v[None, None]).to(DEV), vp, vn, 0, args['v_packed_bytes'], 0)
        q_rot = ops.rotate_q(args['plans'], torch.tensor(qq[None]).to(DEV), 1)
        ref, ref_lse = _reference(oracle_lib, args['plans_np'], [q], kp.cpu().numpy(), kn.cpu().numpy(),
                                  vp.cpu().numpy(), vn.cpu().numpy(), q_rot.cpu().numpy(), [T], gqa, kl, 0, 3)
        for ns in (1, 3):
            out, lse = ops.decode_attention(args['plans'], q_rot, kp, kn, vp, vn, T, n_splits=ns, k_layout=kl,
                                            return_lse=True)
            assert np.abs(out.float().cpu().numpy() - ref).max() < TOL, (kl, ns)
            assert np.abs(lse.cpu().numpy() - ref_lse).max() < LSE_TOL


def test_a_length_beyond_the_stated_capacity_is_clamped(oracle_lib):
    """``T`` is the capacity bound of a ragged call: a row whose device-side length exceeds it
    attends to ``T`` records, as if its length were ``T``."""
    args, qs, q_rot, kp, kn, vp, vn = _build(192, 1, 5, 3, 2, 4, 2, 200, seed=41)
    good = torch.tensor([200, 57], dtype=torch.int32, device=DEV)
    bad = torch.tensor([100000, 57], dtype=torch.int32, device=DEV)
    o0 = ops.decode_attention(args['plans'], q_rot, kp, kn, vp, vn, 200, seq_lens=good, n_splits=4)
    o1 = ops.decode_attention(args['plans'], q_rot, kp, kn, vp, vn, 200, seq_lens=bad, n_splits=4)
    assert torch.equal(o0, o1)


def test_mfma_kernel_refuses_strides_its_addressing_cannot_hold():
    """The fast kernel forms addresses from 32-bit factors; strides or slices of 4 GB and more are
    refused before anything is launched (forced fast path: the refusal is reported, not papered over)."""
    from blockgtq_amd import _capi
    lib = _capi.lib()
    args, qs, q_rot, kp, kn, vp, vn = _build(192, 1, 5, 3, 1, 4, 1, 70, seed=43)
    part = torch.empty(4 * 129, dtype=torch.float32, device=DEV)

    def call(kp_sb, kp_st, T):
        return lib.bgtq_decode_attn(
            _capi.ptr(args['plans']), _capi.ptr(q_rot), q_rot.stride(0), q_rot.stride(1),
            _capi.ptr(kp), kp_sb, kp.stride(1), kp_st, kp.shape[-1],
            _capi.ptr(kn), kn.stride(0), kn.stride(1), kn.stride(2),
            _capi.ptr(vp), vp.stride(0), vp.stride(1), vp.stride(2), vp.shape[-1],
            _capi.ptr(vn), vn.stride(0), vn.stride(1), vn.stride(2),
            None, T, 1, 1, 4, 1, _capi.ptr(part), _capi.ptr(part[4 * 128:]), 0, 0, 1.0 / 128 ** 0.5,
            _capi.stream_ptr(q_rot.device))

    assert lib.bgtq_set_decode_path(2) == 0
    try:
        assert call(kp.stride(0), kp.stride(2), 70) == 0
        assert lib.bgtq_last_decode_path() == 2
        assert call(1 << 32, kp.stride(2), 70) == -2            # batch stride
        assert call(kp.stride(0), 1 << 26, 1) == -2             # (T + 64) * token stride >= 4 GB
    finally:
        lib.bgtq_set_decode_path(0)
    torch.cuda.synchronize()


def test_prompt_kernel_at_the_end_to_end_layer_shape(oracle_lib, decode_path):
    """``bgtq_prefill_attn`` at the layer shape of the end-to-end workload (4 rows, 16 query / 2 KV heads,
    8192-token prompt, K3V3): sampled query rows (first, last, work-group and tile edges, random ones)
    against fp64 attention over the checker's dequantised records, then a chunk of 512 queries at
    position 7680 of the same cache."""
    if decode_path == "generic":
        pytest.skip("one kernel serves this entry point")
    B, n_kv, gqa, T = 4, 2, 8, 8192
    args, qs, _, kp, kn, vp, vn = _build(192, 1, 8, 3, n_kv, gqa, B, T, seed=501)
    gen = torch.Generator().manual_seed(502)
    q = (torch.randn(B, n_kv * gqa, T, 128, generator=gen) * 0.6).half().to(DEV)

    def rot(x):                                        # (B, n_q, S, D) -> rotated, one launch
        Bq, nq, S, D = x.shape
        flat = x.permute(0, 2, 1, 3).reshape(Bq * S, nq, D).contiguous()
        return ops.rotate_q(args['plans'], flat, n_kv).reshape(Bq, S, nq, D).permute(0, 2, 1, 3).contiguous()

    q_rot = rot(q)
    out = ops.prefill_attention_packed(args['plans'], q_rot, kp, kn, vp, vn, T, is_causal=True)
    assert out is not None and out.shape == (B, n_kv * gqa, T, 128)
    chunk = ops.prefill_attention_packed(args['plans'], q_rot[:, :, 7680:].contiguous(), kp, kn, vp, vn, T,
                                         is_causal=True, q_pos_offset=7680)
    assert chunk is not None and chunk.shape == (B, n_kv * gqa, 512, 128)
    rng = np.random.default_rng(503)
    edges = [0, 1, 31, 32, 63, 64, 65, 127, 128, 255, 256, 257, 511, 512, 1023, 1024, 4095, 4096, 4097,
             7679, 7680, 7681, 8127, 8128, 8190, 8191]
    got, got_c, qr = out.float().cpu().numpy(), chunk.float().cpu().numpy(), q_rot.cpu().numpy()
    for b in range(B):
        for h in range(n_kv):
            pl = args['plans_np'][h:h + 1]
            ng = int(pl[0]['n_seg'])
            k_hat = oracle_lib.dequant_k(pl, oracle_lib.unpack_k(pl, kp[b, h, :T].cpu().numpy(), 0),
                                         kn[b, h, :T, :max(ng, 1)].cpu().numpy()).astype(np.float64)
            v_hat = oracle_lib.dequant_v(pl, oracle_lib.unpack_v(vp[b, h, :T].cpu().numpy(), 3, False),
                                         vn[b, h, :T].cpu().numpy()).astype(np.float64)
            R = pl[0]['v_rot'].reshape(128, 128).astype(np.float64)
            rows = sorted(set(edges) | set(int(x) for x in rng.integers(0, T, 38)))
            for sidx in rows:
                qv = qr[b, h * gqa:(h + 1) * gqa, sidx].astype(np.float64)          # (gqa, 128)
                lg = qv @ k_hat[:sidx + 1].T * 128 ** -0.5
                pr = np.exp(lg - lg.max(-1, keepdims=True))
                pr /= pr.sum(-1, keepdims=True)
                ref = (pr @ v_hat[:sidx + 1]) @ R
                assert np.abs(got[b, h * gqa:(h + 1) * gqa, sidx] - ref).max() < TOL, (b, h, sidx)
                if sidx >= 7680:
                    assert np.abs(got_c[b, h * gqa:(h + 1) * gqa, sidx - 7680] - ref).max() < TOL, (b, h, sidx)
