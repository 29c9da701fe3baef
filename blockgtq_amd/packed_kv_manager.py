"""Packed KV cache manager with the true bit-packed layout.

Same public surface as the reference's ``BlockGTQKVManager``
(blockgtq/packed_kv_manager.py:28-453): per-(layer, KV head) quantizers, packed
storage ``(n_layers, B, n_kv, max_T, bytes)``, ``append_and_attend`` for decode.
K records are bit-packed by RoPE-block bit width with raw (uncorrected) fp16
group norms, V records are bit-packed at ``v_bits`` with one corrected fp16
norm per token.

What differs underneath: one encode launch writes all heads of a layer straight
into their cache slots, and one decode launch covers every (batch row, KV head,
partition); nothing loops over heads and nothing is captured into graphs
because no step needs a per-head kernel variant.  Per-row sequence lengths are
supported (``set_seq_lens``) for ragged batches; by default every row shares
``seq_len`` as in the reference.

With ``n_sink`` / ``recent_window`` set, the manager keeps the three-region
layout of the reference's buffered mode (blockgtq/unaccelerated.py:163-244, block
size 1): the first ``n_sink`` tokens and the most recent ``recent_window`` tokens
stay fp16 in a small per-layer buffer, everything between lives in the packed
cache.  Every append moves the token that falls out of the window into the packed
cache; attention runs over the packed part and the buffer and merges the two.
"""
import math

import torch

from . import ops, plan as _plan
from .quantizer import (BlockGTQQuantizer, build_batched_encode_args,
                        encode_k_into, encode_v_into)
from .v_packing import packed_v_bytes


class BlockGTQKVManager:
    def __init__(self, n_layers: int, n_q_heads: int, n_kv_heads: int,
                 head_dim: int, max_seq_len: int, batch_size: int = 1,
                 k_avg_bits: float = 3.0, v_bits: int = 3, device='cuda',
                 min_bits: int = 1, max_bits: int = 8, rotation_threshold: int = 2,
                 n_sink: int = 0, recent_window: int = 0):
        self.n_layers = n_layers
        self.n_q = n_q_heads
        self.n_kv = n_kv_heads
        self.hd = head_dim
        self.max_T = max_seq_len
        self.B = batch_size
        self.k_avg_bits = k_avg_bits
        self.v_bits = v_bits
        self.device = device
        self.min_bits, self.max_bits = min_bits, max_bits
        self.rotation_threshold = rotation_threshold
        self.gqa_ratio = n_q_heads // n_kv_heads
        self.scale = 1.0 / math.sqrt(head_dim)
        self.seq_len = 0
        self._seq_lens = None          # int32 (B,) device tensor when rows are ragged
        self._lens_src, self._lens_S, self._lens_plus = None, 0, None   # cached _seq_lens + S

        self.quantizers = [[None] * n_kv_heads for _ in range(n_layers)]
        self._kernel_args = [[None] * n_kv_heads for _ in range(n_layers)]
        self._batched_args = [None] * n_layers
        self._max_k_packed_bytes = 0
        self._max_n_groups = 0
        self._k_packed = self._k_norms = self._v_packed = self._v_norms = None
        self._ws = ops.Workspace()
        self.n_splits = 0              # partitions per (row, KV head); 0 = library default
        # with-buffer mode: fp16 sink tokens + ring of recent tokens, (L, B, n_kv, n_sink + window, D)
        self.n_sink, self.window = int(n_sink), int(recent_window)
        self.buffered = self.window > 0
        if self.n_sink and not self.buffered:
            raise ValueError("n_sink needs recent_window > 0")
        self._buf_k = self._buf_v = None
        self._step_src, self._step_idx = None, None     # per-step index tensors of the buffered append

    # ------------------------------------------------------------ calibration
    def calibrate(self, layer_idx: int, q_data: torch.Tensor, k_data: torch.Tensor):
        """q_data, k_data: (N, D) shared by all heads or (n_kv, N, D) per head."""
        if q_data.dim() == 2:
            q_data = q_data.unsqueeze(0).expand(self.n_kv, -1, -1)
            k_data = k_data.unsqueeze(0).expand(self.n_kv, -1, -1)
        for hi in range(self.n_kv):
            q8 = BlockGTQQuantizer(head_dim=self.hd, avg_bits=self.k_avg_bits,
                                   rotation_threshold=self.rotation_threshold,
                                   min_bits=self.min_bits, max_bits=self.max_bits,
                                   device=self.device)
            q8.calibrate(q_data[hi], k_data[hi])
            q8.init_v_quantizer(v_bits=self.v_bits, seed=42 + hi)
            self._install(layer_idx, hi, q8)
        self._finish_layer(layer_idx)

    def set_quantizers(self, layer_idx: int, quantizers):
        """Install already calibrated quantizers (with V initialised) for a layer."""
        for hi, q8 in enumerate(quantizers):
            self._install(layer_idx, hi, q8)
        self._finish_layer(layer_idx)

    def _install(self, li, hi, q8):
        self.quantizers[li][hi] = q8
        ka = q8.build_kernel_args()
        self._kernel_args[li][hi] = ka
        self._max_k_packed_bytes = max(self._max_k_packed_bytes, ka['total_packed_bytes'])
        self._max_n_groups = max(self._max_n_groups, q8._n_groups)

    def _finish_layer(self, li):
        self._batched_args[li] = build_batched_encode_args(self.quantizers[li], device=self.device)

    # ---------------------------------------------------------------- storage
    def _ensure_storage(self):
        if self._k_packed is not None:
            return
        # Rows start on a dword and keep clear of the strides that collide in LDS; the V
        # cache is a view of the first _vpb bytes of its (possibly wider) rows.
        # every layer's K cache has its own row width (the widest record of that layer)
        self._k_rows = [_plan.cache_row_bytes(max(ba['max_tpb'], 1) if ba is not None else self._max_k_packed_bytes)
                        for ba in self._batched_args]
        self._k_row = max(self._k_rows)
        self._vpb = packed_v_bytes(self.hd, self.v_bits)
        ng = max(self._max_n_groups, 1)
        shape = (self.n_layers, self.B, self.n_kv, self.max_T)
        dev = self.device
        self._k_packed = [torch.zeros(*shape[1:], w, dtype=torch.uint8, device=dev) for w in self._k_rows]
        self._k_norms = torch.zeros(*shape, ng, dtype=torch.float16, device=dev)
        self._v_row = _plan.cache_row_bytes(self._vpb)
        self._v_packed = torch.zeros(*shape, self._v_row, dtype=torch.uint8, device=dev)[..., :self._vpb]
        self._v_norms = torch.zeros(*shape, dtype=torch.float16, device=dev)
        if self.buffered:
            bshape = (self.n_layers, self.B, self.n_kv, self.n_sink + self.window, self.hd)
            self._buf_k = torch.zeros(bshape, dtype=torch.float16, device=dev)
            self._buf_v = torch.zeros(bshape, dtype=torch.float16, device=dev)

    def set_seq_lens(self, seq_lens):
        """Per-row visible lengths (ragged batch); ``None`` returns to one shared length."""
        if seq_lens is None:
            self._seq_lens = None
            return
        t = torch.as_tensor(seq_lens, dtype=torch.int32).to(self.device)
        assert t.numel() == self.B
        self._seq_lens = t
        self.seq_len = int(t.max().item())

    def _encode_kv(self, layer_idx: int, k: torch.Tensor, v: torch.Tensor, t_pos):
        """Encode k, v (B, n_kv, S, D) into the cache at ``t_pos`` (int or int32 (B,))."""
        self._ensure_storage()
        li = layer_idx
        plans = self._batched_args[li]['plans']
        k16 = k if k.dtype == torch.float16 else k.to(torch.float16)
        v16 = v if v.dtype == torch.float16 else v.to(torch.float16)
        if k16.stride(-1) != 1:
            k16 = k16.contiguous()
        if v16.stride(-1) != 1:
            v16 = v16.contiguous()
        if k16.shape[0] * k16.shape[2] <= 64:          # a decode append: K and V in one launch
            ops.decode_prepare(plans, k16, v16, None, self._k_packed[li], self._k_norms[li],
                               self._v_packed[li], self._v_norms[li], t_pos, self._k_rows[li],
                               self._k_norms.shape[-1], self._vpb, self.n_kv,
                               _plan.K_BITPACKED, _plan.V_BITPACKED)
            return
        encode_k_into(plans, k16, self._k_packed[li], self._k_norms[li], t_pos,
                      self._k_rows[li], self._k_norms.shape[-1], _plan.K_BITPACKED)
        encode_v_into(plans, v16, self._v_packed[li], self._v_norms[li], t_pos,
                      self._vpb, _plan.V_BITPACKED)

    def init_from_cache(self, past_key_value):
        """Pack an fp16 prefill cache: K, V (B, n_kv, T, D) per layer, read from
        ``.key_cache[li]`` / ``.value_cache[li]`` (blockgtq/packed_kv_manager.py:259) or,
        for a ``DynamicCache`` that no longer has those lists, from ``.layers[li].keys / .values``."""
        from .production_decode import _layer_kv
        T = 0
        for li in range(self.n_layers):
            k, v = _layer_kv(past_key_value, li)
            T = k.shape[2]
            self._encode_kv(li, k, v, 0)
        self.seq_len = T

    # ------------------------------------------------------- with-buffer mode
    @torch.no_grad()
    def fill_buffered(self, layer_idx: int, k: torch.Tensor, v: torch.Tensor, lens=None):
        """Load a layer's prefix in with-buffer mode.  k, v (B, n_kv, Tmax, D) post-RoPE; row b
        holds ``lens[b]`` tokens (all ``Tmax`` when ``lens`` is None), each at least
        ``n_sink + recent_window`` long.  Call ``set_seq_lens(lens)`` afterwards."""
        assert self.buffered
        self._ensure_storage()
        li, ns, w = layer_idx, self.n_sink, self.window
        B, _, Tmax, _ = k.shape
        dev = k.device
        lens_t = (torch.full((B,), Tmax, dtype=torch.long, device=dev) if lens is None
                  else torch.as_tensor(lens, dtype=torch.long).to(dev))
        assert int(lens_t.min()) >= ns + w and int(lens_t.max()) <= Tmax
        k16, v16 = k.to(torch.float16), v.to(torch.float16)
        if Tmax - w > ns:          # tokens between sink and window, packed index = position - n_sink
            self._encode_kv(li, k16[:, :, ns:Tmax - w], v16[:, :, ns:Tmax - w], 0)
        self._buf_k[li, :, :, :ns] = k16[:, :, :ns]
        self._buf_v[li, :, :, :ns] = v16[:, :, :ns]
        pos = lens_t[:, None] - w + torch.arange(w, device=dev)[None, :]           # (B, w) positions
        slot = ns + (pos - ns) % w
        ar = torch.arange(B, device=dev)[:, None]
        self._buf_k[li][ar, :, slot] = k16[ar, :, pos]
        self._buf_v[li][ar, :, slot] = v16[ar, :, pos]

    def _buffered_step_indices(self):
        """Index tensors of one buffered append, shared by all layers of a step."""
        if self._step_src is self._seq_lens:
            return self._step_idx
        ns, w = self.n_sink, self.window
        p = self._seq_lens.to(torch.long)                  # position of the token being appended
        rel = p - ns
        slot = torch.where(p < ns, p, ns + rel.clamp(min=0) % w)
        flush = rel >= w                                    # the slot holds a token that leaves the window
        scratch_row = self.max_T - 1                        # records of rows that flush nothing go here
        t_flush = torch.where(flush, rel - w, torch.full_like(rel, scratch_row)).to(torch.int32)
        packed_len = (p + 1 - ns - w).clamp(min=0).to(torch.int32)
        buf_len = (p + 1).clamp(max=ns + w).to(torch.int32)
        ar = torch.arange(self.B, device=p.device)
        self._step_src = self._seq_lens
        self._step_idx = (ar, slot.to(torch.int32), t_flush, packed_len, buf_len)
        return self._step_idx

    @torch.no_grad()
    def _append_and_attend_buffered(self, li, q, k_new, v_new):
        assert k_new.shape[2] == 1, "with-buffer decode appends one token per sequence"
        self._ensure_storage()
        if self._seq_lens is None:
            self.set_seq_lens([self.seq_len] * self.B)
        assert self.seq_len + 1 - self.n_sink - self.window < self.max_T - 1
        ar, slot, t_flush, packed_len, buf_len = self._buffered_step_indices()
        plans = self._batched_args[li]['plans']
        B = q.shape[0]
        q3 = q.reshape(B, self.n_q, self.hd).to(torch.float16).contiguous()
        bk, bv = self._buf_k[li], self._buf_v[li]
        # the tokens leaving the window come out (B, n_kv, 1, D), this step's tokens go in
        old_k, old_v = ops.window_swap(bk, bv, k_new[:, :, 0].to(torch.float16),
                                       v_new[:, :, 0].to(torch.float16), slot)
        q_rot = ops.decode_prepare(
            plans, old_k, old_v, q3, self._k_packed[li], self._k_norms[li],
            self._v_packed[li], self._v_norms[li], t_flush, self._k_rows[li],
            self._k_norms.shape[-1], self._vpb, self.n_kv, _plan.K_BITPACKED, _plan.V_BITPACKED)
        ext_out, ext_lse = ops.window_attention(q3, bk, bv, buf_len, self.n_kv, self.scale)
        T = max(self.seq_len + 1 - self.n_sink - self.window, 1)
        out = ops.decode_attention(
            plans, q_rot, self._k_packed[li], self._k_norms[li],
            self._v_packed[li], self._v_norms[li], T, seq_lens=packed_len, n_splits=self.n_splits,
            k_layout=_plan.K_BITPACKED, v_layout=_plan.V_BITPACKED, scale=self.scale,
            k_row_width=self._k_rows[li], v_row_width=self._vpb, workspace=self._ws,
            extra_out=ext_out, extra_lse=ext_lse)
        return out.unsqueeze(2)

    # ----------------------------------------------------------------- decode
    @torch.no_grad()
    def append_and_attend(self, layer_idx: int, q: torch.Tensor,
                          k_new: torch.Tensor, v_new: torch.Tensor) -> torch.Tensor:
        """q (B, n_q, 1, D), k_new / v_new (B, n_kv, S, D) -> (B, n_q, 1, D) fp16."""
        if self.buffered:
            return self._append_and_attend_buffered(layer_idx, q, k_new, v_new)
        li = layer_idx
        S = k_new.shape[2]
        t_pos = self._seq_lens if self._seq_lens is not None else self.seq_len
        T = self.seq_len + S
        plans = self._batched_args[li]['plans']
        B = q.shape[0]
        q3 = q.reshape(B, self.n_q, self.hd)
        if q3.dtype != torch.float16:
            q3 = q3.to(torch.float16)
        if self.quantizers[li][0]._q_perm_baked:
            self._encode_kv(li, k_new, v_new, t_pos)
        else:
            # encode K, V and rotate the queries in one launch
            self._ensure_storage()
            k16 = k_new if k_new.dtype == torch.float16 else k_new.to(torch.float16)
            v16 = v_new if v_new.dtype == torch.float16 else v_new.to(torch.float16)
            k16 = k16 if k16.stride(-1) == 1 else k16.contiguous()
            v16 = v16 if v16.stride(-1) == 1 else v16.contiguous()
            q3 = ops.decode_prepare(
                plans, k16, v16, q3.contiguous(), self._k_packed[li], self._k_norms[li],
                self._v_packed[li], self._v_norms[li], t_pos, self._k_rows[li],
                self._k_norms.shape[-1], self._vpb, self.n_kv, _plan.K_BITPACKED, _plan.V_BITPACKED)
        lens = None
        if self._seq_lens is not None:
            if self._lens_src is not self._seq_lens or self._lens_S != S:   # one add per step, not per layer
                self._lens_src, self._lens_S, self._lens_plus = self._seq_lens, S, self._seq_lens + S
            lens = self._lens_plus
        out = ops.decode_attention(
            plans, q3.contiguous(), self._k_packed[li], self._k_norms[li],
            self._v_packed[li], self._v_norms[li], T, seq_lens=lens, n_splits=self.n_splits,
            k_layout=_plan.K_BITPACKED, v_layout=_plan.V_BITPACKED, scale=self.scale,
            k_row_width=self._k_rows[li], v_row_width=self._vpb, workspace=self._ws)
        return out.unsqueeze(2)

    def increment_seq_len(self):
        self.seq_len += 1
        if self._seq_lens is not None:
            self._seq_lens = self._seq_lens + 1

    def bake_q_permutations(self, model, n_kv_heads: int, n_q_heads: int):
        """Fold every head's permutation + rotation into ``q_proj`` (in place)."""
        for li, layer in enumerate(_get_model_layers(model)[:self.n_layers]):
            attn = layer.self_attn
            for hi in range(self.n_kv):
                self.quantizers[li][hi].bake_permutation_into_qproj(
                    attn.q_proj.weight.data, kv_head_idx=hi, n_kv_heads=n_kv_heads,
                    n_q_heads=n_q_heads, q_proj_bias=getattr(attn.q_proj, 'bias', None))

    # ------------------------------------------------------------- accounting
    def cache_memory_bytes(self) -> int:
        """Bytes the packed cache holds for the current length (padding included)."""
        self._ensure_storage()
        per_token = sum(self._k_rows) + self.n_layers * (self._v_row + self._k_norms.shape[-1] * 2 + 2)
        return self.seq_len * self.n_kv * self.B * per_token

    def fp16_cache_bytes(self) -> int:
        return self.n_layers * self.B * self.n_kv * self.seq_len * self.hd * 2 * 2


def _get_model_layers(model):
    if hasattr(model, 'model') and hasattr(model.model, 'layers'):
        return list(model.model.layers)
    raise ValueError("Cannot find model layers - expected model.model.layers")


def _project_qkv(model, layer, hidden, position_ids, n_q, n_kv, hd):
    """input_layernorm -> q/k/v projections -> (B, H, S, hd) -> RoPE."""
    from transformers.models.llama.modeling_llama import apply_rotary_pos_emb
    attn = layer.self_attn
    B, S, _ = hidden.shape
    q = attn.q_proj(hidden).view(B, S, n_q, hd).transpose(1, 2)
    k = attn.k_proj(hidden).view(B, S, n_kv, hd).transpose(1, 2)
    v = attn.v_proj(hidden).view(B, S, n_kv, hd).transpose(1, 2)
    if hasattr(attn, 'q_norm') and attn.q_norm is not None:      # Qwen3-style per-head norm
        q, k = attn.q_norm(q), attn.k_norm(k)
    rope = getattr(attn, 'rotary_emb', None) or model.model.rotary_emb
    cos, sin = rope(v, position_ids)
    q, k = apply_rotary_pos_emb(q, k, cos, sin)
    return q, k, v


def run_decoder_stack(model, hidden, position_ids, n_q, n_kv, hd, attend):
    """Llama-style decoder loop with the attention replaced by ``attend(li, q, k, v)``
    returning (B, n_q, S, hd); shared by every decode/prefill driver of this package."""
    for li, layer in enumerate(_get_model_layers(model)):
        residual = hidden
        x = layer.input_layernorm(hidden)
        q, k, v = _project_qkv(model, layer, x, position_ids, n_q, n_kv, hd)
        B, _, S, _ = q.shape
        a = attend(li, q, k, v).to(x.dtype)
        a = a.transpose(1, 2).reshape(B, S, n_q * hd)
        hidden = residual + layer.self_attn.o_proj(a)
        residual = hidden
        hidden = residual + layer.mlp(layer.post_attention_layernorm(hidden))
    return hidden


@torch.no_grad()
def decode_step(model, input_ids, position_ids, kv_manager: BlockGTQKVManager):
    """One decode step through all layers; returns logits (B, 1, vocab)."""
    hidden = model.model.embed_tokens(input_ids)
    hidden = run_decoder_stack(model, hidden, position_ids, kv_manager.n_q, kv_manager.n_kv,
                               kv_manager.hd, kv_manager.append_and_attend)
    kv_manager.increment_seq_len()
    return model.lm_head(model.model.norm(hidden))
