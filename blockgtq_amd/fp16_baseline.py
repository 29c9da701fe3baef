"""Uncompressed fp16 KV cache + decode glue, the dense baseline the packed
path is compared with (blockgtq/fp16_baseline.py:16-96)."""
import math

import torch
import torch.nn.functional as F

from .packed_kv_manager import run_decoder_stack


class FP16KVCache:
    def __init__(self, n_layers, nkv, nq, hd, max_T, device='cuda', batch_size=1,
                 dtype=torch.float16):
        self.n_layers, self.nkv, self.nq, self.hd = n_layers, nkv, nq, hd
        self.gqa = nq // nkv
        self.scale = 1.0 / math.sqrt(hd)
        self.seq_len = 0
        shape = (n_layers, batch_size, nkv, max_T, hd)
        self.k_cache = torch.zeros(shape, dtype=dtype, device=device)
        self.v_cache = torch.zeros(shape, dtype=dtype, device=device)

    def attend(self, layer_idx, q, k, v):
        """Store K/V at the current position and run dense SDPA over the prefix."""
        li, t = layer_idx, self.seq_len
        S = k.shape[2]
        self.k_cache[li, :, :, t:t + S] = k
        self.v_cache[li, :, :, t:t + S] = v
        T = t + S
        k_all = self.k_cache[li, :, :, :T]
        v_all = self.v_cache[li, :, :, :T]
        return F.scaled_dot_product_attention(
            q.to(k_all.dtype), k_all, v_all, is_causal=(S > 1 and t == 0),
            scale=self.scale, enable_gqa=True)

    def increment(self, by=1):
        self.seq_len += by

    def cache_memory_bytes(self) -> int:
        return 2 * self.k_cache.shape[0] * self.k_cache.shape[1] * self.nkv * self.seq_len * self.hd * 2


@torch.no_grad()
def fp16_decode_step(model, input_ids, position_ids, cache):
    hidden = model.model.embed_tokens(input_ids)
    hidden = run_decoder_stack(model, hidden, position_ids, cache.nq, cache.nkv, cache.hd,
                               cache.attend)
    cache.increment(input_ids.shape[1])
    return model.lm_head(model.model.norm(hidden))


__all__ = ["FP16KVCache", "fp16_decode_step"]
