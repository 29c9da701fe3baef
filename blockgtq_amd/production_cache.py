"""Production packed KV cache: mixed nibble K layout, nibble V layout by default.

Same constructor and attributes as the reference's ``BlockGTQProductionCache``
(blockgtq/production_cache.py:35-283).  ``k_nibble=True`` stores K as nibbles
for bit widths <= 4 followed by raw bytes for widths 5-8 with norm-corrected
group norms; ``k_nibble=False`` selects the bit-packed record with raw norms.
``v_nibble`` likewise picks 4-bit or ``v_bits``-bit V records.

Encode writes all KV heads of a layer into their cache slots with one K launch
and one V launch; decode is one attention launch over every (batch row, KV
head, partition) plus one merge launch.  ``batch_size`` (default 1, the only
value the reference supports) sizes the batch axis of the storage.
"""
import math

import torch

from . import ops, plan as _plan
from .quantizer import encode_k_into, encode_v_into
from .v_packing import packed_v_bytes


class BlockGTQProductionCache:
    def __init__(self, quantizers, batched_args, kernel_args,
                 n_layers, nkv, nq, hd, max_T, v_bits=3,
                 k_nibble=True, v_nibble=True, device='cuda', batch_size=1):
        self.quantizers = quantizers
        self.batched_args = batched_args
        self.kernel_args = kernel_args
        self.n_layers, self.nkv, self.nq, self.hd = n_layers, nkv, nq, hd
        self.gqa = nq // nkv
        self.v_bits = v_bits
        self.k_nibble, self.v_nibble = k_nibble, v_nibble
        self.device = device
        self.B = batch_size
        self.scale = 1.0 / math.sqrt(hd)
        self.seq_len = 0
        self._seq_lens = None
        self._lens2 = None
        self._static_T = None          # launch bound used instead of seq_len in graph mode
        self.max_T = max_T

        self.max_ng = max(max(quantizers[li][hi]._n_groups
                              for li in range(n_layers) for hi in range(nkv)), 1)
        own = max(ba['max_mixed_bytes'] if k_nibble else ba['max_tpb'] for ba in batched_args)
        # rows start on a dword and avoid the strides that collide in LDS
        self.k_bytes_per_tok = _plan.cache_row_bytes(own)
        self.vpb = hd // 2 if v_nibble else packed_v_bytes(hd, v_bits)
        self._k_layout = _plan.K_MIXED if k_nibble else _plan.K_BITPACKED
        self._v_layout = _plan.V_NIBBLE if v_nibble else _plan.V_BITPACKED

        shape = (n_layers, batch_size, nkv, max_T)
        self.k_packed = torch.zeros(*shape, self.k_bytes_per_tok, dtype=torch.uint8, device=device)
        self.k_norms = torch.zeros(*shape, self.max_ng, dtype=torch.float16, device=device)
        self._v_row = _plan.cache_row_bytes(self.vpb)      # v_packed is a view of the first vpb bytes
        self.v_packed = torch.zeros(*shape, self._v_row, dtype=torch.uint8, device=device)[..., :self.vpb]
        self.v_norms = torch.zeros(*shape, dtype=torch.float16, device=device)
        self._ws = ops.Workspace()
        self.n_splits = 0              # partitions per (row, KV head); 0 = library default
        # K cell search: the reference's 256-bin table (blockgtq/quantizer.py:841-850);
        # plan.QUANT_EXACT gives the nearest centroid of the unpacked torch path
        self.quant_mode = _plan.QUANT_LUT256

    # ---------------------------------------------------------------- encode
    def _encode_batched(self, layer_idx, k, v, t_pos):
        """Encode k, v (B, n_kv, S, D) into positions ``[t_pos, t_pos + S)``."""
        li = layer_idx
        plans = self.batched_args[li]['plans']
        k16 = k if k.dtype == torch.float16 else k.to(torch.float16)
        v16 = v if v.dtype == torch.float16 else v.to(torch.float16)
        if k16.stride(-1) != 1:
            k16 = k16.contiguous()
        if v16.stride(-1) != 1:
            v16 = v16.contiguous()
        encode_k_into(plans, k16, self.k_packed[li], self.k_norms[li], t_pos,
                      self.k_bytes_per_tok, self.max_ng, self._k_layout, self.quant_mode)
        encode_v_into(plans, v16, self.v_packed[li], self.v_norms[li], t_pos,
                      self.vpb, self._v_layout)

    _encode_graphed = _encode_batched      # single-token appends take the same path

    def set_seq_lens(self, seq_lens):
        """Per-row visible lengths for a ragged batch (``None``: one shared length).
        The cache keeps its own copy and advances it in place."""
        if seq_lens is None:
            self._seq_lens = None
            self._lens2 = None
            self._static_T = None
            return
        t = torch.as_tensor(seq_lens, dtype=torch.int32).to(self.device)
        assert t.numel() == self.B
        self._set_device_lengths(t)
        self.seq_len = int(t.max().item())

    def _set_device_lengths(self, lens):
        """Row 0: tokens in the cache per batch row (the append position); row 1: one more (what a
        single-token step attends over).  Both advance together, so a step launches no arithmetic
        on the lengths."""
        self._lens2 = torch.stack([lens.to(torch.int32), lens.to(torch.int32) + 1]).contiguous()
        self._seq_lens = self._lens2[0]

    def use_device_lengths(self):
        """Keep the lengths on the device only, so that a decode step contains no
        host-side number that changes from step to step and can be recorded into a
        HIP graph once and replayed: append positions and visible lengths come from
        the device copy, launches are sized for ``max_T``.  ``seq_len`` on the host
        then counts the steps issued, not replays."""
        if self._seq_lens is None:
            self._set_device_lengths(torch.full((self.B,), self.seq_len, dtype=torch.int32, device=self.device))
        self._static_T = self.max_T

    # ---------------------------------------------------------------- decode
    @torch.no_grad()
    def encode_and_attend(self, layer_idx, q, k, v):
        """q (B, n_q, 1, hd), k / v (B, n_kv, S, hd) post-RoPE -> (B, n_q, 1, hd) fp16."""
        li = layer_idx
        S = k.shape[2]
        t_pos = self._seq_lens if self._seq_lens is not None else self.seq_len
        T = self._static_T if self._static_T is not None else self.seq_len + S
        plans = self.batched_args[li]['plans']
        B = q.shape[0]
        q3 = q.reshape(B, self.nq, self.hd)
        if q3.dtype != torch.float16:
            q3 = q3.to(torch.float16)
        if self.quantizers[li][0]._q_perm_baked:
            self._encode_batched(li, k, v, t_pos)
        else:                        # encode K, V and rotate the queries in one launch
            k16 = k if k.dtype == torch.float16 else k.to(torch.float16)
            v16 = v if v.dtype == torch.float16 else v.to(torch.float16)
            k16 = k16 if k16.stride(-1) == 1 else k16.contiguous()
            v16 = v16 if v16.stride(-1) == 1 else v16.contiguous()
            q3 = ops.decode_prepare(
                plans, k16, v16, q3.contiguous(), self.k_packed[li], self.k_norms[li],
                self.v_packed[li], self.v_norms[li], t_pos, self.k_bytes_per_tok, self.max_ng,
                self.vpb, self.nkv, self._k_layout, self._v_layout, self.quant_mode)
        lens = None if self._seq_lens is None else self._lens2[1] if S == 1 else self._seq_lens + S
        out = ops.decode_attention(
            plans, q3.contiguous(), self.k_packed[li], self.k_norms[li],
            self.v_packed[li], self.v_norms[li], T, seq_lens=lens, n_splits=self.n_splits,
            k_layout=self._k_layout, v_layout=self._v_layout, scale=self.scale,
            k_row_width=self.k_bytes_per_tok, v_row_width=self.vpb, workspace=self._ws)
        return out.unsqueeze(2)

    def increment_seq_len(self, by=1):
        self.seq_len += by
        if self._seq_lens is not None:
            self._lens2.add_(by)

    # ------------------------------------------------------------ accounting
    def cache_memory_bytes(self) -> int:
        n = self.seq_len * self.nkv * self.n_layers * self.B
        return n * (self.k_bytes_per_tok + self._v_row + self.max_ng * 2 + 2)

    def fp16_cache_bytes(self) -> int:
        return self.n_layers * self.B * self.nkv * self.seq_len * self.hd * 2 * 2
