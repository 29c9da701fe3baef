"""Layer-major prefill into a packed cache.

All prompt tokens go through one transformer layer at a time: QKV + RoPE for
the whole prompt, one quantise-and-pack launch per K and V, attention, MLP.
No fp16 KV cache of the full model is ever materialised.  Reference behaviour:
blockgtq/prefill.py:24-111.

Attention inside the prompt runs as dense causal SDPA on the layer's own fp16
K/V (which are at hand at that point), not on the dequantised packed cache as
the reference's prefill kernel does; the packed records written are identical.
"""
import torch
import torch.nn.functional as F

from .packed_kv_manager import run_decoder_stack


@torch.no_grad()
def layer_major_prefill(model, cache, prompt_ids, block_q=32, block_t=128):
    """Populate ``cache`` for positions ``[0, T)`` and set ``cache.seq_len = T``.

    ``prompt_ids`` is (B, T); B must match the cache's batch size.
    """
    B, T = prompt_ids.shape
    pos = torch.arange(T, device=prompt_ids.device).unsqueeze(0).expand(B, -1)
    hidden = model.model.embed_tokens(prompt_ids)

    def attend(li, q, k, v):
        cache._encode_batched(li, k, v, 0)
        return F.scaled_dot_product_attention(q, k, v, is_causal=True, scale=cache.scale,
                                              enable_gqa=True)

    hidden = run_decoder_stack(model, hidden, pos, cache.nq, cache.nkv, cache.hd, attend)
    cache.seq_len = T
    return hidden


__all__ = ["layer_major_prefill"]
