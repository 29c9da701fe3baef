"""Calibration helpers: collect Q/K activations, build per-head quantizers.

Turns a Llama-style HF model plus calibration token ids (or ready-made
activation tensors) into the ``(quantizers, batched_args, kernel_args)`` triple
``BlockGTQProductionCache`` takes.  Reference behaviour:
blockgtq/calibration.py:35-181.
"""
import torch

from .quantizer import BlockGTQQuantizer, build_batched_encode_args


@torch.no_grad()
def collect_qk_activations(model, enc, device, n_calib_tokens=256,
                           post_rope=True, effective_len=None):
    """Per-layer ``{'q': (nkv, gqa*T, hd), 'k': (nkv, T, hd)}`` from forward hooks
    on ``q_proj`` / ``k_proj``; with ``post_rope`` RoPE is applied afterwards at
    the calibration positions (stretched to ``[0, effective_len)`` if given)."""
    ids = enc[:, :n_calib_tokens].to(device)
    cfg = model.config
    nq = cfg.num_attention_heads
    hd = getattr(cfg, 'head_dim', None) or cfg.hidden_size // nq
    nkv = getattr(cfg, 'num_key_value_heads', nq)
    gqa = nq // nkv
    T = ids.size(1)
    position_ids = None
    if effective_len is not None:
        if effective_len < T:
            raise ValueError(f"effective_len ({effective_len}) must be >= n_calib_tokens ({T})")
        step = effective_len // T
        position_ids = torch.arange(0, T * step, step, device=device).unsqueeze(0)

    layer_data, handles = {}, []
    for li, layer in enumerate(model.model.layers):
        layer_data[li] = {}

        def k_hook(mod, inp, out, li=li):
            layer_data[li]['k'] = out.detach().reshape(-1, nkv, hd).permute(1, 0, 2)

        def q_hook(mod, inp, out, li=li):
            qg = out.detach().reshape(-1, nkv, gqa, hd)
            layer_data[li]['q'] = qg.permute(1, 2, 0, 3).reshape(nkv, -1, hd)

        handles.append(layer.self_attn.k_proj.register_forward_hook(k_hook))
        handles.append(layer.self_attn.q_proj.register_forward_hook(q_hook))
    try:
        model(ids) if position_ids is None else model(ids, position_ids=position_ids)
    finally:
        for h in handles:
            h.remove()

    if post_rope:
        from transformers.models.llama.modeling_llama import apply_rotary_pos_emb
        rope = (getattr(model.model.layers[0].self_attn, 'rotary_emb', None)
                or model.model.rotary_emb)
        if position_ids is None:
            position_ids = torch.arange(T, device=device).unsqueeze(0)
        cos, sin = rope(torch.zeros(1, 1, T, hd, device=device, dtype=torch.float16), position_ids)
        for li, d in layer_data.items():
            k, q = d['k'], d['q']
            q3 = q.reshape(-1, k.shape[1], hd).unsqueeze(0).to(cos.dtype)
            k4 = k.unsqueeze(0).to(cos.dtype)
            q_r, _ = apply_rotary_pos_emb(q3, q3, cos, sin)
            _, k_r = apply_rotary_pos_emb(k4, k4, cos, sin)
            d['q'] = q_r[0].reshape(nkv, -1, hd).to(q.dtype)
            d['k'] = k_r[0].to(k.dtype)
    return layer_data


def build_quantizers(layer_data, n_layers, nkv, hd, k_avg_bits=3.0, v_bits=3,
                     k_nibble=True, device='cuda', min_bits=1, max_bits=8,
                     rotation_threshold=2):
    """``(quantizers[li][hi], batched_args[li], kernel_args[li][hi])`` from
    ``layer_data[li] = {'q': (nkv, Nq, hd), 'k': (nkv, Nk, hd)}``."""
    quantizers = [[None] * nkv for _ in range(n_layers)]
    kernel_args = [[None] * nkv for _ in range(n_layers)]
    batched_args = [None] * n_layers
    for li in range(n_layers):
        for hi in range(nkv):
            q8 = BlockGTQQuantizer(head_dim=hd, avg_bits=k_avg_bits, device=device,
                                   min_bits=min_bits, max_bits=max_bits,
                                   rotation_threshold=rotation_threshold)
            q8.calibrate(layer_data[li]['q'][hi], layer_data[li]['k'][hi])
            q8.init_v_quantizer(v_bits=v_bits, seed=42 + hi)
            quantizers[li][hi] = q8
            kernel_args[li][hi] = q8.build_kernel_args()
        batched_args[li] = build_batched_encode_args(quantizers[li], device=device)
    return quantizers, batched_args, kernel_args


def bake_q_rotations(model, quantizers, n_layers, nkv, nq):
    """Fold every head's permutation + rotation into ``q_proj`` (in place)."""
    for li in range(n_layers):
        attn = model.model.layers[li].self_attn
        for hi in range(nkv):
            quantizers[li][hi].bake_permutation_into_qproj(
                attn.q_proj.weight.data, kv_head_idx=hi, n_kv_heads=nkv, n_q_heads=nq,
                q_proj_bias=getattr(attn.q_proj, 'bias', None))


__all__ = ["collect_qk_activations", "build_quantizers", "bake_q_rotations"]
