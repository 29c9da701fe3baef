"""Model-level drivers on a tiny random Qwen2 model: layer-major prefill into the packed
cache, production decode steps, fp16 dense baseline (GPU only)."""
import pytest
import torch

pytestmark = pytest.mark.gpu


def test_packed_decode_follows_the_dense_model_on_a_tiny_qwen2():
    pytest.importorskip("transformers")
    from blockgtq_amd import e2e
    # generous bit widths: the packed path must then track the dense model closely
    out, logits = e2e.run("tiny", batch=2, prompt_len=200, new_tokens=6, k_bits=6.0, v_bits=4,
                          max_bits=8, n_calib=128, return_logits=True)
    assert out["layers"] == 2 and out["decode_tokens_per_s"] > 0 and out["prefill_pack_ms"] > 0
    assert out["packed_cache_bytes"] < out["fp16_cache_bytes"]
    a, b = logits["packed_step0"].flatten(), logits["fp16_step0"].flatten()
    assert torch.isfinite(a).all()
    # same prompt, same first token: the step-0 logits of the two paths differ only by the
    # quantisation of the cached K/V
    cos = torch.nn.functional.cosine_similarity(a, b, dim=0).item()
    assert cos > 0.98, cos


def test_graph_replay_of_the_decode_step_equals_eager_steps():
    """The whole decode step recorded once and replayed must produce, replay after
    replay, what eager steps produce: same greedy tokens, same logits."""
    pytest.importorskip("transformers")
    from blockgtq_amd import e2e
    kw = dict(batch=2, prompt_len=150, new_tokens=14, k_bits=4.0, v_bits=3, max_bits=6, n_calib=128,
              return_logits=True, fp16_baseline=False)
    out_g, lg = e2e.run("tiny", graph=True, **kw)
    out_e, le = e2e.run("tiny", graph=False, **kw)
    assert out_g["decode_mode"].startswith("HIP graph") and out_e["decode_mode"] == "eager"
    assert torch.equal(lg["packed_step0"], le["packed_step0"])
    assert lg["tokens"].shape == (2, 14) and torch.equal(lg["tokens"], le["tokens"])
    for i in range(3):                                  # graph steps 0..2 are eager steps 8..10
        assert torch.allclose(lg[f"graph_step{i}"], le[f"eager_step{8 + i}"], atol=2e-2, rtol=0)


@pytest.mark.slow
def test_qwen25_3b_geometry_at_its_stated_size(oracle_lib):
    """Qwen2.5-3B geometry (36 layers, 16 query / 2 KV heads), batch 4, 8192-token prompt, 256 new
    tokens, random-init weights.  On the way the run is tapped: the packed K and V records of the
    last prompt token of two layers must equal the checker's bytes for the fp16 K/V the layer
    handed over, the first decode step's attention output of one layer must be within 2e-3 of the
    checker's attention over the packed cache as it stood, and the graph-replayed steps must pick
    the tokens that eager steps pick."""
    pytest.importorskip("transformers")
    import numpy as np
    from blockgtq_amd import e2e, ops
    from blockgtq_amd.production_cache import BlockGTQProductionCache as Cache
    B, P, N = 4, 8192, 256
    tap = {"enc": {}, "step0": None, "cache": None}
    enc0, att0 = Cache._encode_batched, Cache.encode_and_attend

    def enc(self, li, k, v, t_pos):
        if k.shape[2] > 1 and li in (0, self.n_layers - 1) and isinstance(t_pos, int) and t_pos + k.shape[2] == P:
            tap["enc"][li] = (k[:, :, -1].half().cpu().numpy(), v[:, :, -1].half().cpu().numpy())
        return enc0(self, li, k, v, t_pos)

    def att(self, li, q, k, v):
        out = att0(self, li, q, k, v)
        if li == 17 and tap["step0"] is None:
            tap["cache"] = self
            tap["step0"] = (q[:, :, 0].half().clone(), out[:, :, 0].float().cpu().numpy())
        return out

    Cache._encode_batched, Cache.encode_and_attend = enc, att
    try:
        out_g, lg = e2e.run("qwen2.5-3b", batch=B, prompt_len=P, new_tokens=N, return_logits=True,
                            fp16_baseline=False, graph=True)
    finally:
        Cache._encode_batched, Cache.encode_and_attend = enc0, att0
    assert out_g["layers"] == 36 and out_g["decode_mode"].startswith("HIP graph")
    cache = tap["cache"]
    assert cache is not None and set(tap["enc"]) == {0, 35}
    # (1) records of the last prompt token
    for li, (k_last, v_last) in tap["enc"].items():
        plans = cache.batched_args[li]['plans_np']
        for h in range(2):
            pl = plans[h:h + 1]
            codes, raw, corr = oracle_lib.encode_k(pl, k_last[:, h])
            own = int(pl['k_row_bytes'][0])
            ng = max(int(pl['n_seg'][0]), 1)
            assert np.array_equal(cache.k_packed[li, :, h, P - 1, :own].cpu().numpy(), oracle_lib.pack_k(pl, codes, 0))
            assert np.array_equal(cache.k_norms[li, :, h, P - 1, :ng].cpu().numpy().view(np.uint16),
                                  oracle_lib.f2h(raw[:, :ng]).view(np.uint16))
            vc, vn = oracle_lib.encode_v(pl, v_last[:, h])
            assert np.array_equal(cache.v_packed[li, :, h, P - 1].cpu().numpy(), oracle_lib.pack_v(vc, 3, False))
            assert np.array_equal(cache.v_norms[li, :, h, P - 1].cpu().numpy().view(np.uint16), vn.view(np.uint16))
    # (2) attention of the first decode step, layer 17: the cache is append-only, so its first
    # P + 1 records are what that step saw
    q, got = tap["step0"]
    li = 17
    plans = cache.batched_args[li]['plans_np']
    q_rot = ops.rotate_q(cache.batched_args[li]['plans'], q.contiguous(), 2).cpu().numpy()
    T = P + 1
    for b, h in ((0, 0), (3, 1)):
        pl = plans[h:h + 1]
        own, ng = int(pl['k_row_bytes'][0]), max(int(pl['n_seg'][0]), 1)
        ref, _ = oracle_lib.decode_attn(pl, q_rot[b, h * 8:(h + 1) * 8],
                                        cache.k_packed[li, b, h, :T, :own].cpu().numpy(),
                                        cache.k_norms[li, b, h, :T, :ng].cpu().numpy(),
                                        cache.v_packed[li, b, h, :T].cpu().numpy(),
                                        cache.v_norms[li, b, h, :T].cpu().numpy())
        assert np.abs(got[b, h * 8:(h + 1) * 8] - ref).max() < 2e-3
    del cache, tap
    torch.cuda.empty_cache()
    # (3) the same run without the graph picks the same tokens
    out_e, le = e2e.run("qwen2.5-3b", batch=B, prompt_len=P, new_tokens=N, return_logits=True,
                        fp16_baseline=False, graph=False)
    assert out_e["decode_mode"] == "eager"
    assert lg["tokens"].shape == (B, N) and torch.equal(lg["tokens"], le["tokens"])
