"""Torch-facing wrappers of the decode entry points of the C ABI.

These take cache-shaped tensors (batch, KV head, token, ...) and launch one
kernel for every (batch row, KV head, partition) plus one merge kernel; the
per-KV-head Python loop of the reference (blockgtq/production_cache.py:234-262)
has no counterpart here.
"""
import math
import warnings
from typing import Optional

import torch

from . import _capi, plan as _plan


class Workspace:
    """Reusable fp32 partial buffers for (B, n_q, n_splits) so a decode step
    allocates nothing after the first call."""

    def __init__(self):
        self._buf = None

    def get(self, B, n_q, n_splits, device):
        need = B * n_q * n_splits * (_plan.HEAD_DIM + 1)
        if self._buf is None or self._buf.numel() < need or self._buf.device != torch.device(device):
            self._buf = torch.empty(need, dtype=torch.float32, device=device)
        out = self._buf[:B * n_q * n_splits * _plan.HEAD_DIM]
        lse = self._buf[B * n_q * n_splits * _plan.HEAD_DIM:need]
        return out, lse


_default_ws = Workspace()


def default_splits(B: int, n_kv: int, T: int) -> int:
    return _capi.lib().bgtq_default_splits(int(B), int(n_kv), int(T))


@torch.no_grad()
def rotate_q(plans: torch.Tensor, q: torch.Tensor, n_kv: int) -> torch.Tensor:
    """q (B, n_q, D) fp16 -> permuted + rotated into each KV head's packed space."""
    _capi.require_cuda(q, "q")
    assert q.dim() == 3 and q.dtype == torch.float16 and q.stride(-1) == 1
    B, n_q, _ = q.shape
    out = torch.empty((B, n_q, _plan.HEAD_DIM), dtype=torch.float16, device=q.device)
    _capi.check(_capi.lib().bgtq_rotate_q(
        _capi.ptr(plans), _capi.ptr(q), q.stride(0), q.stride(1),
        _capi.ptr(out), out.stride(0), out.stride(1),
        B, n_kv, n_q // n_kv, _capi.stream_ptr(q.device)), "bgtq_rotate_q")
    return out


GENERIC_PATH, MFMA_PATH = 1, 2      # values of bgtq_last_decode_path()
_paths_seen: dict = {}              # cache geometry -> kernel that bgtq_decode_attn chose for it


def last_decode_path() -> int:
    """Which kernel this process's last ``bgtq_decode_attn`` launched: 1 generic, 2 matrix-core."""
    return _capi.lib().bgtq_last_decode_path()


@torch.no_grad()
def decode_attention(plans: torch.Tensor, q_rot: torch.Tensor,
                     k_packed: torch.Tensor, k_norms: torch.Tensor,
                     v_packed: torch.Tensor, v_norms: torch.Tensor,
                     T: int, *, seq_lens: Optional[torch.Tensor] = None,
                     n_splits: int = 0, k_layout: int = _plan.K_BITPACKED,
                     v_layout: int = _plan.V_BITPACKED, scale: Optional[float] = None,
                     k_row_width: Optional[int] = None, v_row_width: Optional[int] = None,
                     unrotate: bool = True, return_lse: bool = False,
                     extra_out: Optional[torch.Tensor] = None,
                     extra_lse: Optional[torch.Tensor] = None,
                     workspace: Optional[Workspace] = None):
    """Decode attention of one layer over the packed cache.

    q_rot (B, n_q, D) fp16 rotated queries; k_packed (B, n_kv, >=T, Kb) uint8;
    k_norms (B, n_kv, >=T, G) fp16; v_packed (B, n_kv, >=T, Vb) uint8; v_norms
    (B, n_kv, >=T) fp16.  ``T`` tokens are visible for every batch row unless
    ``seq_lens`` (int32 device tensor, B) gives per-row counts (then ``T`` must
    be their maximum).  Returns (B, n_q, D) fp16 [and the total lse (B, n_q)].
    """
    _capi.require_cuda(q_rot, "q_rot")
    assert q_rot.dim() == 3 and q_rot.dtype == torch.float16 and q_rot.stride(-1) == 1
    assert k_packed.dtype == torch.uint8 and k_packed.stride(-1) == 1
    assert v_packed.dtype == torch.uint8 and v_packed.stride(-1) == 1
    assert k_norms.dtype == torch.float16 and k_norms.stride(-1) == 1
    assert v_norms.dtype == torch.float16
    B, n_q, D = q_rot.shape
    n_kv = k_packed.shape[1]
    gqa = n_q // n_kv
    assert k_packed.shape[2] >= T and v_packed.shape[2] >= T
    if seq_lens is not None:
        assert seq_lens.dtype == torch.int32 and seq_lens.is_cuda and seq_lens.numel() == B
    scale = 1.0 / math.sqrt(D) if scale is None else float(scale)
    k_row_width = k_packed.shape[-1] if k_row_width is None else k_row_width
    v_row_width = v_packed.shape[-1] if v_row_width is None else v_row_width
    L = _capi.lib()
    if n_splits <= 0:
        n_splits = L.bgtq_default_splits(B, n_kv, max(T, 1))
        if seq_lens is not None:
            # ragged rows: smaller partitions let the short rows' compute units pick up
            # pieces of the long rows
            n_splits = max(n_splits, min(4 * n_splits, (T + 511) // 512))
    ws = workspace or _default_ws
    part_out, part_lse = ws.get(B, n_q, n_splits, q_rot.device)
    st = _capi.stream_ptr(q_rot.device)
    _capi.check(L.bgtq_decode_attn(
        _capi.ptr(plans), _capi.ptr(q_rot), q_rot.stride(0), q_rot.stride(1),
        _capi.ptr(k_packed), k_packed.stride(0), k_packed.stride(1), k_packed.stride(2), k_row_width,
        _capi.ptr(k_norms), k_norms.stride(0), k_norms.stride(1), k_norms.stride(2),
        _capi.ptr(v_packed), v_packed.stride(0), v_packed.stride(1), v_packed.stride(2), v_row_width,
        _capi.ptr(v_norms), v_norms.stride(0), v_norms.stride(1), v_norms.stride(2),
        _capi.ptr(seq_lens), int(T), B, n_kv, gqa, n_splits,
        _capi.ptr(part_out), _capi.ptr(part_lse), k_layout, v_layout, scale, st),
        "bgtq_decode_attn")
    shape_key = (n_kv, gqa, k_packed.stride(2), v_packed.stride(2), k_norms.stride(2), k_layout, v_layout)
    if shape_key not in _paths_seen:
        _paths_seen[shape_key] = path = L.bgtq_last_decode_path()
        if path == GENERIC_PATH:
            warnings.warn(f"bgtq_decode_attn runs its generic kernel (several times slower than the matrix-core "
                          f"one) for n_kv={n_kv}, gqa={gqa}, K rows {k_packed.stride(2)} B, V rows "
                          f"{v_packed.stride(2)} B: the fast kernel takes gqa <= 16, K rows that follow each "
                          f"other at a multiple of 4 bytes (4..128), V rows of 16..64 bytes at most 4 bytes apart",
                          RuntimeWarning, stacklevel=2)
    out = torch.empty((B, n_q, D), dtype=torch.float16, device=q_rot.device)
    lse = torch.empty((B, n_q), dtype=torch.float32, device=q_rot.device) if return_lse else None
    n_extra = 0
    if extra_out is not None:
        assert extra_out.dtype == torch.float32 and extra_lse.dtype == torch.float32
        assert extra_out.is_contiguous() and extra_lse.is_contiguous()
        n_extra = extra_lse.shape[-1] if extra_lse.dim() == 3 else 1
    _capi.check(L.bgtq_lse_reduce(
        _capi.ptr(plans), _capi.ptr(part_out), _capi.ptr(part_lse), n_splits,
        _capi.ptr(extra_out), _capi.ptr(extra_lse), n_extra,
        B, n_kv, gqa, int(unrotate), _capi.ptr(out), out.stride(0), out.stride(1),
        _capi.ptr(lse), st), "bgtq_lse_reduce")
    return (out, lse) if return_lse else out


def decode_prepare(plans: torch.Tensor, k: torch.Tensor, v: torch.Tensor, q: torch.Tensor,
                   k_packed: torch.Tensor, k_norms: torch.Tensor, v_packed: torch.Tensor,
                   v_norms: torch.Tensor, t_pos, k_row_width: int, norm_width: int,
                   v_row_width: int, n_kv: int, k_layout: int, v_layout: int,
                   quant_mode: int = _plan.QUANT_LUT256) -> torch.Tensor:
    """One launch for everything a decode step does before attention: encode
    ``k`` / ``v`` (B, n_kv, S, D) fp16 into the cache views at ``t_pos`` (int or
    int32 device tensor (B,)) and rotate ``q`` (B, n_q, D) fp16.  Returns the
    rotated queries; same results as ``encode_k_into`` + ``encode_v_into`` + ``rotate_q``.
    ``q`` may be None (queries rotated elsewhere): K and V are appended in one launch and
    None is returned."""
    _capi.require_cuda(k, "k")
    for t in (k, v) + ((q,) if q is not None else ()):
        assert t.dtype == torch.float16 and t.stride(-1) == 1
    assert k_packed.dtype == torch.uint8 and v_packed.dtype == torch.uint8
    assert k_norms.dtype == torch.float16 and v_norms.dtype == torch.float16
    B, H, S, _ = k.shape
    n_q = q.shape[1] if q is not None else n_kv
    q_rot = torch.empty((B, n_q, q.shape[2]), dtype=torch.float16, device=q.device) if q is not None else None
    if isinstance(t_pos, torch.Tensor):
        assert t_pos.dtype == torch.int32 and t_pos.is_cuda
        tp, ts = _capi.ptr(t_pos), 0
    else:
        tp, ts = None, int(t_pos)
    from .quantizer import _cache_capacity
    max_T = _cache_capacity(t_pos, S, k_packed, k_norms, v_packed, v_norms)
    L = _capi.lib()
    _capi.check(L.bgtq_decode_prepare(
        _capi.ptr(plans), _capi.ptr(k), k.stride(0), k.stride(1), k.stride(2),
        _capi.ptr(v), v.stride(0), v.stride(1), v.stride(2), B, H, S,
        _capi.ptr(k_packed), k_packed.stride(0), k_packed.stride(1), k_packed.stride(2), k_row_width,
        _capi.ptr(k_norms), k_norms.stride(0), k_norms.stride(1), k_norms.stride(2), norm_width,
        _capi.ptr(v_packed), v_packed.stride(0), v_packed.stride(1), v_packed.stride(2), v_row_width,
        _capi.ptr(v_norms), v_norms.stride(0), v_norms.stride(1), v_norms.stride(2),
        tp, ts, max_T, k_layout, v_layout, quant_mode,
        _capi.ptr(q), q.stride(0) if q is not None else 0, q.stride(1) if q is not None else 0,
        _capi.ptr(q_rot), q_rot.stride(0) if q is not None else 0, q_rot.stride(1) if q is not None else 0,
        n_q // n_kv, _capi.stream_ptr(k.device)), "bgtq_decode_prepare")
    return q_rot


@torch.no_grad()
def window_attention(q: torch.Tensor, kbuf: torch.Tensor, vbuf: torch.Tensor,
                     lens: Optional[torch.Tensor], n_kv: int, scale: Optional[float] = None):
    """Dense fp16 attention partial over buffered (unquantised) tokens.

    q (B, n_q, D) fp16 ORIGINAL queries; kbuf / vbuf (B, n_kv, W, D) fp16 with a
    common layout; ``lens`` int32 device tensor (B,) of valid rows or None.
    Returns (partial (B, n_q, D) fp32, lse (B, n_q) fp32) for ``decode_attention``'s
    ``extra_out`` / ``extra_lse``."""
    _capi.require_cuda(q, "q")
    assert q.dtype == torch.float16 and q.stride(-1) == 1
    assert kbuf.dtype == torch.float16 and vbuf.dtype == torch.float16
    assert kbuf.shape == vbuf.shape and kbuf.stride() == vbuf.stride() and kbuf.stride(-1) == 1
    B, n_q, D = q.shape
    W = kbuf.shape[2]
    scale = 1.0 / math.sqrt(D) if scale is None else float(scale)
    po = torch.empty((B, n_q, D), dtype=torch.float32, device=q.device)
    pl = torch.empty((B, n_q), dtype=torch.float32, device=q.device)
    _capi.check(_capi.lib().bgtq_window_attn(
        _capi.ptr(q), q.stride(0), q.stride(1), _capi.ptr(kbuf), _capi.ptr(vbuf),
        kbuf.stride(0), kbuf.stride(1), kbuf.stride(2), _capi.ptr(lens), W,
        B, n_kv, n_q // n_kv, scale, _capi.ptr(po), _capi.ptr(pl), _capi.stream_ptr(q.device)),
        "bgtq_window_attn")
    return po, pl


def window_swap(kbuf: torch.Tensor, vbuf: torch.Tensor, new_k: torch.Tensor, new_v: torch.Tensor,
                slot: torch.Tensor):
    """Ring update of the with-buffer append in one launch: for every batch row the fp16
    token in slot ``slot[b]`` of ``kbuf`` / ``vbuf`` (B, n_kv, W, D) is returned and replaced by
    ``new_k`` / ``new_v`` (B, n_kv, D).  ``slot`` int32 device tensor (B,); rows whose slot lies
    outside [0, W) move nothing and return zeros.  Returns (old_k, old_v), each (B, n_kv, 1, D)."""
    _capi.require_cuda(kbuf, "kbuf")
    for t in (kbuf, vbuf, new_k, new_v):
        assert t.dtype == torch.float16 and t.stride(-1) == 1
    assert kbuf.shape == vbuf.shape and kbuf.stride() == vbuf.stride()
    assert new_k.shape == new_v.shape and new_k.stride() == new_v.stride()
    assert slot.dtype == torch.int32 and slot.is_contiguous()
    B, n_kv, W, D = kbuf.shape
    assert new_k.shape == (B, n_kv, D)
    old_k = torch.empty((B, n_kv, 1, D), dtype=torch.float16, device=kbuf.device)
    old_v = torch.empty_like(old_k)
    _capi.check(_capi.lib().bgtq_window_swap(
        _capi.ptr(kbuf), _capi.ptr(vbuf), kbuf.stride(0), kbuf.stride(1), kbuf.stride(2),
        _capi.ptr(new_k), _capi.ptr(new_v), new_k.stride(0), new_k.stride(1),
        _capi.ptr(slot), W, B, n_kv, _capi.ptr(old_k), _capi.ptr(old_v),
        _capi.stream_ptr(kbuf.device)), "bgtq_window_swap")
    return old_k, old_v


@torch.no_grad()
def dequant_kv(plans: torch.Tensor, k_packed: torch.Tensor, k_norms: torch.Tensor,
               v_packed: torch.Tensor, v_norms: torch.Tensor, T: int, *,
               k_layout: int = _plan.K_BITPACKED, v_layout: int = _plan.V_BITPACKED,
               k_row_width: Optional[int] = None, v_row_width: Optional[int] = None):
    """The first ``T`` records of a layer's packed cache as fp16 tensors.

    Inputs as for ``decode_attention``.  Returns ``(k_hat, v_hat)``, both
    (B, n_kv, T, D) fp16: K in the packed-dim order and rotated space of the
    records (what ``rotate_q`` queries multiply with), V in its rotated space."""
    _capi.require_cuda(k_packed, "k_packed")
    assert k_packed.dtype == torch.uint8 and k_packed.stride(-1) == 1
    assert v_packed.dtype == torch.uint8 and v_packed.stride(-1) == 1
    assert k_norms.dtype == torch.float16 and v_norms.dtype == torch.float16
    B, n_kv = k_packed.shape[:2]
    assert k_packed.shape[2] >= T and v_packed.shape[2] >= T
    k_row_width = k_packed.shape[-1] if k_row_width is None else k_row_width
    v_row_width = v_packed.shape[-1] if v_row_width is None else v_row_width
    ko = torch.empty((B, n_kv, T, _plan.HEAD_DIM), dtype=torch.float16, device=k_packed.device)
    vo = torch.empty_like(ko)
    _capi.check(_capi.lib().bgtq_dequant_kv(
        _capi.ptr(plans),
        _capi.ptr(k_packed), k_packed.stride(0), k_packed.stride(1), k_packed.stride(2), k_row_width,
        _capi.ptr(k_norms), k_norms.stride(0), k_norms.stride(1), k_norms.stride(2),
        _capi.ptr(v_packed), v_packed.stride(0), v_packed.stride(1), v_packed.stride(2), v_row_width,
        _capi.ptr(v_norms), v_norms.stride(0), v_norms.stride(1), v_norms.stride(2),
        B, n_kv, T, k_layout, v_layout,
        _capi.ptr(ko), ko.stride(0), ko.stride(1), ko.stride(2),
        _capi.ptr(vo), vo.stride(0), vo.stride(1), vo.stride(2),
        _capi.stream_ptr(k_packed.device)), "bgtq_dequant_kv")
    return ko, vo


UNSUPPORTED = -2          # BGTQ_EUNSUPPORTED: the fast kernel does not take this argument set


@torch.no_grad()
def prefill_attention_packed(plans: torch.Tensor, q_rot: torch.Tensor, k_packed: torch.Tensor,
                             k_norms: torch.Tensor, v_packed: torch.Tensor, v_norms: torch.Tensor,
                             T: int, *, k_layout: int = _plan.K_BITPACKED, v_layout: int = _plan.V_BITPACKED,
                             scale: Optional[float] = None, is_causal: bool = True, q_pos_offset: int = 0,
                             unrotate: bool = True, k_row_width: Optional[int] = None,
                             v_row_width: Optional[int] = None) -> Optional[torch.Tensor]:
    """Attention of many query tokens straight over the packed cache (``bgtq_prefill_attn``).

    q_rot (B, n_q, S, D) fp16 rotated queries; cache tensors as for ``decode_attention``.
    Query token s sees records ``t <= q_pos_offset + s`` when ``is_causal``.  Returns
    (B, n_q, S, D) fp16, or ``None`` when the kernel does not take this argument set
    (``prefill_attention_records`` copies records into rows the kernel can walk first)."""
    _capi.require_cuda(k_packed, "k_packed")
    assert q_rot.dtype == torch.float16 and q_rot.dim() == 4 and q_rot.stride(-1) == 1
    assert k_packed.dtype == torch.uint8 and k_packed.stride(-1) == 1
    assert v_packed.dtype == torch.uint8 and v_packed.stride(-1) == 1
    assert k_norms.dtype == torch.float16 and v_norms.dtype == torch.float16
    B, n_q, S, D = q_rot.shape
    n_kv = k_packed.shape[1]
    assert D == _plan.HEAD_DIM and n_q % n_kv == 0 and k_packed.shape[2] >= T
    k_row_width = k_packed.shape[-1] if k_row_width is None else k_row_width
    v_row_width = v_packed.shape[-1] if v_row_width is None else v_row_width
    scale = 1.0 / math.sqrt(D) if scale is None else float(scale)
    out = torch.empty((B, n_q, S, D), dtype=torch.float16, device=q_rot.device)
    code = _capi.lib().bgtq_prefill_attn(
        _capi.ptr(plans), _capi.ptr(q_rot), q_rot.stride(0), q_rot.stride(1), q_rot.stride(2),
        _capi.ptr(k_packed), k_packed.stride(0), k_packed.stride(1), k_packed.stride(2), k_row_width,
        _capi.ptr(k_norms), k_norms.stride(0), k_norms.stride(1), k_norms.stride(2),
        _capi.ptr(v_packed), v_packed.stride(0), v_packed.stride(1), v_packed.stride(2), v_row_width,
        _capi.ptr(v_norms), v_norms.stride(0), v_norms.stride(1), v_norms.stride(2),
        B, n_kv, n_q // n_kv, S, T, int(q_pos_offset), int(bool(is_causal)),
        k_layout, v_layout, scale, int(bool(unrotate)),
        _capi.ptr(out), out.stride(0), out.stride(1), out.stride(2), _capi.stream_ptr(q_rot.device))
    if code == UNSUPPORTED:
        return None
    _capi.check(code, "bgtq_prefill_attn")
    return out


def _packed_rows(rec: torch.Tensor, T: int, width: int, v_rows: bool = False) -> torch.Tensor:
    """The first ``T`` records of a (B, n_kv, >=T, >=width) uint8 cache tensor in the row layout the
    prompt-phase kernel takes (rows that follow each other at a stride of ``width`` rounded up to 4
    bytes; V rows of 32 or 64 bytes may sit 4 bytes apart): the tensor itself when it already has it,
    a copy otherwise."""
    row = (width + 3) // 4 * 4
    ok = rec.stride(2) == row or (v_rows and rec.stride(2) == row + 4)
    if ok and rec.stride(0) % 4 == 0 and rec.stride(1) % 4 == 0 and rec.data_ptr() % 4 == 0:
        return rec
    out = torch.zeros((rec.shape[0], rec.shape[1], T, row), dtype=torch.uint8, device=rec.device)
    out[..., :width] = rec[:, :, :T, :width]
    return out


@torch.no_grad()
def prefill_attention_records(plans, q_rot, k_packed, k_norms, v_packed, v_norms, T, *, k_layout=_plan.K_BITPACKED,
                              v_layout=_plan.V_BITPACKED, scale=None, is_causal=True, q_pos_offset=0,
                              unrotate=True, k_row_width=None, v_row_width=None) -> torch.Tensor:
    """``prefill_attention_packed`` for any tensor layout: records whose rows the kernel cannot walk
    (token stride other than the row width, odd alignment) are first copied into rows it can, queries
    are made contiguous; an argument set the kernel still refuses raises."""
    k_row_width = k_packed.shape[-1] if k_row_width is None else k_row_width
    v_row_width = v_packed.shape[-1] if v_row_width is None else v_row_width
    B, n_q, S, D = q_rot.shape
    if T == 0 or B == 0:
        return torch.zeros((B, n_q, S, D), dtype=torch.float16, device=q_rot.device)
    kp = _packed_rows(k_packed, T, k_row_width)
    vp = _packed_rows(v_packed, T, v_row_width, v_rows=True)
    vn = v_norms if v_norms.stride(-1) == 1 else v_norms.contiguous()
    out = prefill_attention_packed(plans, q_rot.contiguous(), kp, k_norms.contiguous() if k_norms.stride(-1) != 1 else k_norms,
                                   vp, vn, T, k_layout=k_layout, v_layout=v_layout, scale=scale, is_causal=is_causal,
                                   q_pos_offset=q_pos_offset, unrotate=unrotate,
                                   k_row_width=kp.stride(2), v_row_width=v_row_width)
    if out is None:
        raise RuntimeError("bgtq_prefill_attn does not take this argument set (more than 256 query heads per "
                           "KV head, a V record that is not 16, 32, 48 or 64 bytes, or more than 8 norm columns)")
    return out

