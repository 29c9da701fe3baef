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
