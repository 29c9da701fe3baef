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
