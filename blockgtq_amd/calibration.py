"""Calibration helpers: collect Q/K activations, build per-head quantizers.

Turns a Llama-style HF model plus calibration token ids (or ready-made
activation tensors) into the ``(quantizers, batched_args, kernel_args)`` triple
``BlockGTQProductionCache`` takes.  Reference behaviour:
blockgtq/calibration.py:35-181.
"""
import numpy as np
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


_CALIB_FORMAT = 1


def save_calibration(path, quantizers) -> None:
    """Write the calibration result of ``quantizers[li][hi]`` to ``path`` (``.npz``).

    Everything a head's tables hold follows from its per-block bit allocation and the
    constructor arguments (rotations and codebooks are seeded), so that is all the file
    keeps: a few hundred bytes a head instead of the activations the reference stores
    and recalibrates from on every run (examples/build_calib_cache.py:238-298)."""
    n_layers, nkv = len(quantizers), len(quantizers[0])
    q0 = quantizers[0][0]
    alloc = np.zeros((n_layers, nkv, q0.head_dim // 2), dtype=np.int16)
    v_seed = np.zeros((n_layers, nkv), dtype=np.int64)
    params = np.zeros((n_layers, nkv, 6), dtype=np.float64)
    for li in range(n_layers):
        for hi in range(nkv):
            q8 = quantizers[li][hi]
            assert q8._calibrated and hasattr(q8, '_v_bits'), \
                f"layer {li} head {hi}: calibrate() and init_v_quantizer() first"
            assert q8.head_dim == q0.head_dim and q8.v_bits == q0.v_bits
            alloc[li, hi] = q8.bit_allocation.cpu().numpy()
            v_seed[li, hi] = q8._v_seed
            params[li, hi] = (q8.avg_bits, q8.rotation_threshold, q8.min_bits, q8.max_bits,
                              q8.rope_base, q8.n_bins)
    np.savez(path, format=np.int64(_CALIB_FORMAT), head_dim=np.int64(q0.head_dim),
             v_bits=np.int64(q0.v_bits), bit_allocation=alloc, v_seed=v_seed, params=params)


def load_calibration(path, device='cuda'):
    """``(quantizers, batched_args, kernel_args)`` as ``build_quantizers`` returns them,
    rebuilt from a file written by ``save_calibration``; the device plans come out
    byte-identical to those of the quantizers that were saved."""
    with np.load(path, allow_pickle=False) as f:
        if int(f['format']) != _CALIB_FORMAT:
            raise ValueError(f"{path}: calibration format {int(f['format'])}, "
                             f"this build reads {_CALIB_FORMAT}")
        hd, v_bits = int(f['head_dim']), int(f['v_bits'])
        alloc, v_seed, params = f['bit_allocation'], f['v_seed'], f['params']
    n_layers, nkv = alloc.shape[:2]
    quantizers = [[None] * nkv for _ in range(n_layers)]
    kernel_args = [[None] * nkv for _ in range(n_layers)]
    batched_args = [None] * n_layers
    for li in range(n_layers):
        for hi in range(nkv):
            avg, thr, lo, hi_bits, base, bins = params[li, hi]
            q8 = BlockGTQQuantizer(head_dim=hd, avg_bits=float(avg), device=device,
                                   rotation_threshold=int(thr), min_bits=int(lo),
                                   max_bits=int(hi_bits), rope_base=float(base), n_bins=int(bins))
            q8.calibrate_from_allocation(torch.from_numpy(alloc[li, hi].astype(np.int64)))
            q8.init_v_quantizer(v_bits=v_bits, seed=int(v_seed[li, hi]))
            quantizers[li][hi] = q8
            kernel_args[li][hi] = q8.build_kernel_args()
        batched_args[li] = build_batched_encode_args(quantizers[li], device=device)
    return quantizers, batched_args, kernel_args


__all__ = ["collect_qk_activations", "build_quantizers", "bake_q_rotations",
           "save_calibration", "load_calibration"]
