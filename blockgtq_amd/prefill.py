"""Layer-major prefill into a packed cache.

All prompt tokens go through one transformer layer at a time: QKV + RoPE for
the whole prompt, one quantise-and-pack launch per K and V, causal attention
over the records just written, MLP.  No fp16 KV cache of the full model is
ever materialised.  Reference behaviour: blockgtq/prefill.py:24-111.

As in the reference, attention inside the prompt sees the *quantised* keys and
values (what later decode steps will see), not the layer's fp16 K/V: the
queries are permuted + rotated into each head's packed space with one batched
GEMM and ``bgtq_prefill_attn`` attends straight over the records (tiles are
dequantised inside the kernel; no fp16 K/V of the layer is written).  Argument
sets that kernel does not take go through one dequantisation pass
(``bgtq_dequant_kv``) and the library's fused causal attention.
"""
import torch

from . import ops
from .packed_kv_manager import run_decoder_stack


def _layer_matrices(cache, li):
    """Per-KV-head query transform (D, D) = permutation then rotation, and V
    un-rotation (D, D), stacked over the heads of layer ``li`` (built once)."""
    store = cache.__dict__.setdefault('_prefill_mats', {})
    if li not in store:
        qm, vm = [], []
        for q8 in cache.quantizers[li]:
            m = torch.zeros(cache.hd, cache.hd, dtype=torch.float32, device=q8._block_rot_T.device)
            m[q8._head_perm] = q8._block_rot_T.float()           # q[:, head_perm] @ R^T == q @ m
            qm.append(m)
            vm.append(q8._v_rot.float())
        store[li] = (torch.stack(qm), torch.stack(vm))
    return store[li]


@torch.no_grad()
def packed_prefill_attention(cache, li, q, T, q_pos_offset=0):
    """Causal attention of q (B, n_q, S, D) over records ``[0, T)`` of layer ``li``
    of a ``BlockGTQProductionCache``; returns (B, n_q, S, D) fp16."""
    B, n_q, S, D = q.shape
    q_mat, v_rot = _layer_matrices(cache, li)
    if cache.quantizers[li][0]._q_perm_baked:
        q_rot = q.to(torch.float16)
    else:
        qg = q.reshape(B, cache.nkv, cache.gqa * S, D).float()
        q_rot = (qg @ q_mat.unsqueeze(0)).to(torch.float16).reshape(B, n_q, S, D)
    plans = cache.batched_args[li]['plans']
    return ops.prefill_attention_records(
        plans, q_rot, cache.k_packed[li], cache.k_norms[li], cache.v_packed[li], cache.v_norms[li], T,
        k_layout=cache._k_layout, v_layout=cache._v_layout, scale=cache.scale, is_causal=True,
        q_pos_offset=q_pos_offset, k_row_width=cache.k_bytes_per_tok, v_row_width=cache.vpb)


@torch.no_grad()
def layer_major_prefill(model, cache, prompt_ids, block_q=32, block_t=128):
    """Populate ``cache`` for positions ``[0, T)`` and set ``cache.seq_len = T``.

    ``prompt_ids`` is (B, T); B must match the cache's batch size.  ``block_q``
    and ``block_t`` tuned the reference's kernel and are ignored.
    """
    B, T = prompt_ids.shape
    pos = torch.arange(T, device=prompt_ids.device).unsqueeze(0).expand(B, -1)
    hidden = model.model.embed_tokens(prompt_ids)

    def attend(li, q, k, v):
        cache._encode_batched(li, k, v, 0)
        return packed_prefill_attention(cache, li, q, T)

    hidden = run_decoder_stack(model, hidden, pos, cache.nq, cache.nkv, cache.hd, attend)
    cache.seq_len = T
    return hidden


__all__ = ["layer_major_prefill", "packed_prefill_attention"]
