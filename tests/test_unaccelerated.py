"""The unpacked (plain torch) quantise-reconstruct path, checked against the
packed path's CPU checker and against what the mathematics fixes."""
import numpy as np
import pytest
import torch
import torch.nn as nn

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


class _Attn(nn.Module):
    def __init__(self, nkv):
        super().__init__()
        self.k_proj = nn.Linear(64, nkv * 128, bias=True)
        self.v_proj = nn.Linear(64, nkv * 128, bias=False)


class _Layer(nn.Module):
    def __init__(self, nkv):
        super().__init__()
        self.self_attn = _Attn(nkv)


class _Model(nn.Module):
    def __init__(self, n_layers, nkv):
        super().__init__()
        self.model = nn.Module()
        self.model.layers = nn.ModuleList([_Layer(nkv) for _ in range(n_layers)])

    def forward(self, x, past_key_values=None):
        return x


def _quantizers(n_layers, nkv):
    gen = torch.Generator().manual_seed(2)
    data = {li: {'q': torch.randn(nkv, 512, 128, generator=gen) * torch.linspace(0.2, 3, 128),
                 'k': torch.randn(nkv, 128, 128, generator=gen) * torch.linspace(0.2, 3, 128)}
            for li in range(n_layers)}
    return ua.build_unaccelerated_quantizers(data, n_layers, nkv, 128, device='cpu')


def test_patch_wraps_projections_and_unpatch_restores():
    torch.manual_seed(0)
    m = _Model(2, 2)
    kq, vq = _quantizers(2, 2)
    assert kq[0][0].rotation_threshold == 1 and vq[1][1].bit_width == 3
    x = torch.randn(3, 7, 64)
    attn = m.model.layers[1].self_attn
    plain_k, plain_v = attn.k_proj(x), attn.v_proj(x)
    handles = ua.patch_model_kv(m, kq, vq, 128, 2)
    got_k, got_v = attn.k_proj(x), attn.v_proj(x)
    assert got_k.shape == plain_k.shape and got_k.dtype == plain_k.dtype
    for h in range(2):
        sl = slice(h * 128, (h + 1) * 128)
        assert torch.allclose(got_k[..., sl], kq[1][h].compress_decompress(plain_k[..., sl].float()), atol=1e-6)
        assert torch.allclose(got_v[..., sl], vq[1][h].compress_decompress(
            plain_v[..., sl].reshape(-1, 128).float()).reshape(3, 7, 128), atol=1e-6)
    cos = torch.nn.functional.cosine_similarity(got_k.flatten(), plain_k.flatten(), dim=0)
    assert 0.9 < float(cos.detach()) < 1.0
    ua.unpatch_model_kv(handles)
    assert torch.equal(attn.k_proj(x), plain_k) and isinstance(attn.k_proj, nn.Linear)


class _Cache:
    def __init__(self, n_layers, B, nkv, T):
        g = torch.Generator().manual_seed(1)
        self.key_cache = [torch.randn(B, nkv, T, 128, generator=g).half() for _ in range(n_layers)]
        self.value_cache = [torch.randn(B, nkv, T, 128, generator=g).half() for _ in range(n_layers)]


def test_buffered_patch_flushes_only_tokens_that_left_the_window():
    m = _Model(2, 2)
    kq, vq = _quantizers(2, 2)
    patch = ua.patch_model_kv_buffered(m, kq, vq, 128, 2, 2, recent_window=16, n_sink_token=4)
    cache = _Cache(2, 2, 2, 4 + 16 + 3)
    before_k = [k.clone() for k in cache.key_cache]
    before_v = [v.clone() for v in cache.value_cache]
    m(torch.zeros(1), past_key_values=cache)
    for li in range(2):
        k, v = cache.key_cache[li], cache.value_cache[li]
        changed = (k != before_k[li]).any(dim=-1).any(dim=0).any(dim=0)
        assert changed.tolist() == [False] * 4 + [True] * 3 + [False] * 16
        assert torch.equal(v[:, :, :4], before_v[li][:, :, :4]) and torch.equal(v[:, :, 7:], before_v[li][:, :, 7:])
        ref = kq[li][1].compress_decompress(before_k[li][:, 1, 4:7].reshape(-1, 128).float())
        assert torch.equal(k[:, 1, 4:7].reshape(-1, 128), ref.half())
        assert patch.state[li]["n_flushed"] == 3
    snap = [k.clone() for k in cache.key_cache]
    m(torch.zeros(1), past_key_values=cache)               # nothing new left the window
    assert all(torch.equal(a, b) for a, b in zip(snap, cache.key_cache))
    patch.reset()
    assert patch.state[0]["n_flushed"] == 0
    patch.remove()
    m(torch.zeros(1), past_key_values=cache)
    assert all(torch.equal(a, b) for a, b in zip(snap, cache.key_cache))


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
