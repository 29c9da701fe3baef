"""Model glue around ``BlockGTQProductionCache`` for Llama-style HF models
(``model.model.embed_tokens / layers / norm``, ``model.lm_head``).

Reference behaviour: blockgtq/production_decode.py:11-99.
"""
import torch

from .packed_kv_manager import run_decoder_stack


@torch.no_grad()
def production_decode_step(model, input_ids, position_ids, cache):
    """One decode step: embed -> per layer (norm, QKV, RoPE, packed encode +
    attention, MLP) -> final norm + lm_head.  Returns logits (B, 1, vocab)."""
    hidden = model.model.embed_tokens(input_ids)
    hidden = run_decoder_stack(model, hidden, position_ids, cache.nq, cache.nkv, cache.hd,
                               cache.encode_and_attend)
    cache.increment_seq_len()
    return model.lm_head(model.model.norm(hidden))


@torch.no_grad()
def production_prefill(model, input_ids, cache, chunk_encode=64):
    """Prefill with the model's own attention, then pack its fp16 K/V.

    Runs the HF forward with a ``DynamicCache``, reads the post-RoPE K/V of
    every layer back and encodes them into ``cache`` in slices of
    ``chunk_encode`` tokens.  Returns the prompt logits.
    """
    from transformers import DynamicCache

    prompt_len = input_ids.shape[1]
    position_ids = torch.arange(prompt_len, device=input_ids.device).unsqueeze(0)
    hf_cache = DynamicCache()
    out = model(input_ids, position_ids=position_ids, past_key_values=hf_cache, use_cache=True)
    for li in range(cache.n_layers):
        k, v = _layer_kv(hf_cache, li)
        for lo in range(0, prompt_len, chunk_encode):
            hi = min(lo + chunk_encode, prompt_len)
            cache._encode_batched(li, k[:, :, lo:hi], v[:, :, lo:hi], lo)
    cache.seq_len = prompt_len
    del hf_cache
    return out.logits


def _layer_kv(hf_cache, li):
    """K, V (B, n_kv, T, D) of layer ``li`` from either DynamicCache generation."""
    if hasattr(hf_cache, 'key_cache'):
        return hf_cache.key_cache[li], hf_cache.value_cache[li]
    layer = hf_cache.layers[li]
    return layer.keys, layer.values


__all__ = ["production_decode_step", "production_prefill"]
