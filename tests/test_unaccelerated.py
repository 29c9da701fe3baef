"""The unpacked (plain torch) quantise-reconstruct path, checked against the
packed path's CPU checker and against what the mathematics fixes."""
import numpy as np
import pytest
import torch

from blockgtq_amd import BlockGTQPipeline
from blockgtq_amd.tq import TurboQuantMSE
from blockgtq_amd import unaccelerated as ua
from helpers import make_kv, make_quantizer


@pytest.mark.parametrize("seed,mn,mx,budget", [(11, 1, 6, 192), (4, 0, 4, 128), (7, 3, 3, 192)])
def test_k_round_trip_equals_packed_record_dequantised(oracle_lib, seed, mn, mx, budget):
    """Matrix-form round trip == checker's exact-mode codes + corrected norms,
    un-rotated and un-permuted (the norms pass through fp16 in the record)."""
    q, en = make_quantizer(seed=seed, min_bits=mn, max_bits=mx, budget=budget)
    k, _, _ = make_kv(en, 256, seed=seed + 1)
    plan = q.plan()
    pipe = BlockGTQPipeline(128, rotation_threshold=q.rotation_threshold, min_bits=mn, max_bits=mx)
    pipe.set_allocation(q.bit_allocation)
    got = pipe.compress_decompress(torch.tensor(k.astype(np.float32))).double().numpy()

    codes, raw, corr = oracle_lib.encode_k(plan, k, quant_mode=1)
    ng = int(plan[0]['n_seg'])
    khat = oracle_lib.dequant_k(plan, codes, oracle_lib.f2h(corr[:, :max(ng, 1)])).astype(np.float64)
    rot = pipe._block_rot_T.T.double().numpy()                 # y = x @ rot.T  =>  x = y @ rot
    ref = np.zeros_like(khat)
    ref[:, pipe._head_perm.numpy()] = khat @ rot
    scale = np.abs(k.astype(np.float64)).max()
    bad = np.abs(got - ref) > 2e-3 * scale
    # a coordinate within float rounding of a cell edge may fall either side
    assert bad.any(axis=1).mean() < 0.02, bad.any(axis=1).mean()
    if mn == 0:
        zero_dims = pipe._head_perm[:pipe._n_zero_dims].numpy()
        assert pipe._n_zero_dims > 0 and np.all(got[:, zero_dims] == 0)


def test_k_round_trip_keeps_group_norms_and_shapes():
    q, en = make_quantizer(seed=3)
    pipe = BlockGTQPipeline(128, rotation_threshold=2)
    pipe.set_allocation(q.bit_allocation)
    x = torch.randn(2, 5, 128)
    y = pipe.compress_decompress(x)
    assert y.shape == x.shape
    xp, yp = x.reshape(-1, 128)[:, pipe._head_perm], y.reshape(-1, 128)[:, pipe._head_perm]
    for s, e in pipe._group_slices:
        assert torch.allclose(xp[:, s:e].norm(dim=1), yp[:, s:e].norm(dim=1), rtol=1e-4)
    assert torch.equal(pipe.compress_decompress(torch.zeros(3, 128)), torch.zeros(3, 128))


@pytest.mark.parametrize("bits,nmse", [(2, 0.1175), (3, 0.03454), (4, 0.009497)])
def test_turboquant_round_trip(bits, nmse):
    """Norm is kept exactly (renormalised reconstruction); the error of a b-bit
    Lloyd-Max quantiser of a Gaussian coordinate is the textbook distortion."""
    tq = TurboQuantMSE(128, bits, seed=1003)
    r = tq.rotation.double()
    assert torch.allclose(r @ r.T, torch.eye(128, dtype=torch.float64), atol=1e-6)
    x = torch.randn(4096, 128, generator=torch.Generator().manual_seed(0)) * 3.0
    y = tq.compress_decompress(x)
    assert torch.allclose(y.norm(dim=1), x.norm(dim=1), rtol=1e-4)
    codes, norms = tq.quantize(x)
    assert int(codes.max()) == (1 << bits) - 1 and int(codes.min()) == 0
    assert torch.equal(tq.dequantize(codes, norms), y)
    assert torch.allclose(tq.compress_decompress(x[0]), y[0], atol=1e-6)
    rel = ((y - x) ** 2).sum() / (x ** 2).sum()
    assert abs(float(rel) / nmse - 1) < 0.1, float(rel)


def _quantizers(n_layers, nkv):
    gen = torch.Generator().manual_seed(2)
    data = {li: {'q': torch.randn(nkv, 512, 128, generator=gen) * torch.linspace(0.2, 3, 128),
                 'k': torch.randn(nkv, 128, 128, generator=gen) * torch.linspace(0.2, 3, 128)}
            for li in range(n_layers)}
    return ua.build_unaccelerated_quantizers(data, n_layers, nkv, 128, device='cpu')


def test_round_trip_heads_is_the_per_head_reconstruction():
    kq, vq = _quantizers(2, 2)
    assert kq[0][0].rotation_threshold == 1 and vq[1][1].bit_width == 3
    g = torch.Generator().manual_seed(5)
    k = (torch.randn(3, 2, 7, 128, generator=g) * torch.linspace(0.2, 3, 128)).half()
    v = torch.randn(3, 2, 7, 128, generator=g).half()
    k_hat, v_hat = ua.round_trip_heads(kq[1], vq[1], k, v)
    assert k_hat.shape == k.shape and k_hat.dtype == torch.float32 and v_hat.dtype == torch.float32
    for h in range(2):
        for b in range(3):
            assert torch.allclose(k_hat[b, h], kq[1][h].compress_decompress(k[b, h].float()), atol=1e-6)
            assert torch.allclose(v_hat[b, h], vq[1][h].compress_decompress(v[b, h].float()), atol=1e-6)
    cos = torch.nn.functional.cosine_similarity(k_hat.flatten(), k.float().flatten(), dim=0)
    assert 0.9 < float(cos) < 1.0
    # heads use their own quantizers: swapping them changes the result
    swapped, _ = ua.round_trip_heads(kq[1][::-1], vq[1], k, v)
    assert not torch.allclose(swapped, k_hat)


def test_quantizers_from_allocations_reproduce_calibrated_ones():
    kq, vq = _quantizers(1, 2)
    k2, v2 = ua.quantizers_from_allocations([q.bit_allocation for q in kq[0]], 128, 3,
                                            [1000, 1001], rotation_threshold=1)
    x = torch.randn(33, 128, generator=torch.Generator().manual_seed(8)) * torch.linspace(0.2, 3, 128)
    for h in range(2):
        assert torch.equal(k2[h].compress_decompress(x), kq[0][h].compress_decompress(x))
        assert torch.equal(v2[h].compress_decompress(x), vq[0][h].compress_decompress(x))


def test_decode_attention_expands_kv_heads_for_their_query_groups():
    g = torch.Generator().manual_seed(9)
    B, n_q, nkv, T = 2, 8, 2, 37
    q = torch.randn(B, n_q, 128, generator=g).half()
    k = torch.randn(B, nkv, T, 128, generator=g)
    v = torch.randn(B, nkv, T, 128, generator=g)
    out = ua.decode_attention(q, k, v)
    assert out.shape == (B, n_q, 128) and out.dtype == torch.float32
    assert torch.equal(out, ua.decode_attention(q.unsqueeze(2), k, v))
    for b in range(B):
        for hq in range(n_q):
            h = hq // (n_q // nkv)
            s = (q[b, hq].double() @ k[b, h].double().T) / 128 ** 0.5
            ref = torch.softmax(s, -1) @ v[b, h].double()
            assert torch.allclose(out[b, hq].double(), ref, atol=1e-5)
    half_scale = ua.decode_attention(q, k, v, scale=0.5 / 128 ** 0.5)
    assert not torch.allclose(half_scale, out)


@pytest.mark.parametrize("k_layout,v_layout", [(0, 0), (1, 1)])
def test_checker_attention_tracks_the_unpacked_path(oracle_lib, k_layout, v_layout):
    """Whole chain of the checker (exact cell search, records, packed attention,
    V un-rotation) against fp64 softmax attention over the torch round trips.
    Bit-packed records carry raw group norms, so there K is compared without
    the renormalisation of the reconstruction."""
    q8, en = make_quantizer(seed=21, max_bits=6, budget=192)
    k, v, qq = make_kv(en, 500, seed=22)
    plan = q8.plan()
    pipe = BlockGTQPipeline(128, rotation_threshold=q8.rotation_threshold, max_bits=6)
    pipe.set_allocation(q8.bit_allocation)
    kt = torch.tensor(k.astype(np.float32))
    if k_layout:
        k_hat = pipe.compress_decompress(kt).double()
    else:                                   # centroids * raw norm, no renormalisation
        x = kt[:, pipe._head_perm]
        n = torch.sqrt((x * x) @ pipe._group_mask)[:, pipe._group_of]
        y = (x / n) @ pipe._block_rot_T
        idx = torch.searchsorted(pipe._pos_boundaries, y.T.contiguous())
        y_hat = pipe._pos_centroids[pipe._row_idx, idx].T
        k_hat = ((y_hat * n) @ pipe._block_rot_unperm).double()
    vq = q8._v_quantizer
    v_hat = vq.dequantize(*vq.quantize(torch.tensor(v.astype(np.float32)))).double()
    qt = torch.tensor(qq.astype(np.float32)).double()
    ref = torch.softmax(qt @ k_hat.T / 128 ** 0.5, -1) @ v_hat

    codes, raw, corr = oracle_lib.encode_k(plan, k, quant_mode=1)
    ng = int(plan[0]['n_seg'])
    kn = oracle_lib.f2h((corr if k_layout else raw)[:, :ng])
    kp = oracle_lib.pack_k(plan, codes, k_layout)
    vc, vn = oracle_lib.encode_v(plan, v)
    vp = oracle_lib.pack_v(vc, int(plan[0]['v_bits']), bool(v_layout))
    out, _ = oracle_lib.decode_attn(plan, oracle_lib.rotate_q(plan, qq), kp, kn, vp, vn,
                                    n_splits=3, k_layout=k_layout, v_layout=v_layout)
    # the record keeps norms, the rotated query and the codebooks in fp16; the torch
    # path keeps fp32 throughout (a wrong code or norm shows as > 1e-2 here)
    assert np.abs(out - ref.numpy()).max() < 4e-3
