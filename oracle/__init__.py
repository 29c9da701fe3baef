"""CPU checker for the packed-KV path.  TEST INFRASTRUCTURE ONLY.

Only tests/, the smoke run and the CPU-baseline leg of bench.py import this
package; nothing under blockgtq_amd/ does.  The arithmetic lives in
``bgtq_oracle.c`` (see its header for the reference lines it restates and for
what pins it); this module builds that file with gcc, loads it with ctypes and
exposes numpy-in / numpy-out wrappers.
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "_build", "libbgtq_oracle.so")
D = 128
MAX_SEG = 8

_lib = None


def build(force=False):
    """Compile the checker with gcc (``make -C oracle``)."""
    if force and os.path.exists(LIB_PATH):
        os.remove(LIB_PATH)
    res = subprocess.run(["make", "-C", _HERE], capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError("oracle build failed:\n" + res.stdout + res.stderr)
    return LIB_PATH


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            build()
        _lib = ctypes.CDLL(LIB_PATH)
        _lib.orc_plan_sizeof.restype = ctypes.c_size_t
    return _lib


def _p(a):
    return a.ctypes.data_as(ctypes.c_void_p)


def _plan_ptr(plan):
    """plan: (1,) or () structured array of one bgtq_head_plan."""
    plan = np.ascontiguousarray(plan).reshape(-1)[:1]
    assert plan.dtype.itemsize == lib().orc_plan_sizeof(), "plan layout mismatch"
    return plan, _p(plan)


def _u16(a):
    """fp16 array -> contiguous uint16 view."""
    a = np.ascontiguousarray(a)
    if a.dtype == np.float16:
        a = a.view(np.uint16)
    assert a.dtype == np.uint16
    return a


i64 = ctypes.c_int64
ci = ctypes.c_int
cf = ctypes.c_float


def f2h(x):
    x = np.ascontiguousarray(x, dtype=np.float32)
    out = np.empty(x.shape, dtype=np.uint16)
    lib().orc_f2h(_p(x), _p(out), i64(x.size))
    return out


def h2f(x):
    x = _u16(x)
    out = np.empty(x.shape, dtype=np.float32)
    lib().orc_h2f(_p(x), _p(out), i64(x.size))
    return out


def encode_k(plan, k, quant_mode=0):
    """k: (N, 128) fp16 -> codes (N,128) u8 packed order, raw norms (N,8) f32,
    corrected norms (N,8) f32."""
    plan, pp = _plan_ptr(plan)
    k = _u16(k).reshape(-1, D)
    N = k.shape[0]
    codes = np.zeros((N, D), np.uint8)
    raw = np.zeros((N, MAX_SEG), np.float32)
    corr = np.zeros((N, MAX_SEG), np.float32)
    lib().orc_encode_k(pp, _p(k), i64(N), ci(quant_mode), _p(codes), _p(raw), _p(corr))
    return codes, raw, corr


def pack_k(plan, codes, layout=0, width=None):
    plan, pp = _plan_ptr(plan)
    codes = np.ascontiguousarray(codes, dtype=np.uint8).reshape(-1, D)
    N = codes.shape[0]
    own = int(plan['k_mixed_bytes'][0] if layout else plan['k_row_bytes'][0])
    width = own if width is None else width
    out = np.zeros((N, max(width, 1)), np.uint8)
    fn = lib().orc_pack_k_mixed if layout else lib().orc_pack_k_bits
    fn(pp, _p(codes), i64(N), _p(out), i64(out.shape[1]), ci(width))
    return out[:, :width]


def unpack_k(plan, packed, layout=0):
    plan, pp = _plan_ptr(plan)
    packed = np.ascontiguousarray(packed, dtype=np.uint8)
    N = packed.shape[0]
    # the unpacker may peek one byte past a record
    buf = np.zeros((N, packed.shape[1] + 2), np.uint8)
    buf[:, :packed.shape[1]] = packed
    codes = np.zeros((N, D), np.uint8)
    fn = lib().orc_unpack_k_mixed if layout else lib().orc_unpack_k_bits
    fn(pp, _p(buf), i64(N), i64(buf.shape[1]), _p(codes))
    return codes


def encode_v(plan, v):
    """v: (N,128) fp16 -> codes (N,128) u8, corrected norms (N,) fp16 (as uint16)."""
    plan, pp = _plan_ptr(plan)
    v = _u16(v).reshape(-1, D)
    N = v.shape[0]
    codes = np.zeros((N, D), np.uint8)
    norms = np.zeros(N, np.uint16)
    lib().orc_encode_v(pp, _p(v), i64(N), _p(codes), _p(norms))
    return codes, norms


def v_bytes(bits, nibble=False):
    bw = 4 if nibble else bits
    return {1: 16, 2: 32, 3: 48, 4: 64}[bw]


def pack_v(codes, v_bits, nibble=False):
    codes = np.ascontiguousarray(codes, dtype=np.uint8).reshape(-1, D)
    N = codes.shape[0]
    nb = v_bytes(v_bits, nibble)
    out = np.zeros((N, nb), np.uint8)
    lib().orc_pack_v(_p(codes), i64(N), ci(v_bits), ci(int(nibble)), _p(out), i64(nb))
    return out


def unpack_v(packed, v_bits, nibble=False):
    packed = np.ascontiguousarray(packed, dtype=np.uint8)
    N = packed.shape[0]
    buf = np.zeros((N, packed.shape[1] + 2), np.uint8)
    buf[:, :packed.shape[1]] = packed
    codes = np.zeros((N, D), np.uint8)
    lib().orc_unpack_v(_p(buf), i64(N), i64(buf.shape[1]), ci(v_bits), ci(int(nibble)), _p(codes))
    return codes


def rotate_q(plan, q):
    plan, pp = _plan_ptr(plan)
    q = _u16(q).reshape(-1, D)
    out = np.zeros_like(q)
    lib().orc_rotate_q(pp, _p(q), i64(q.shape[0]), _p(out))
    return out.view(np.float16)


def decode_attn(plan, q_rot, k_packed, k_norms, v_packed, v_norms, T=None, n_splits=1,
                k_layout=0, v_layout=0, scale=None, unrotate=True):
    """One (batch row, KV head).  q_rot (gqa,128) fp16; k_packed (T,Kb) u8;
    k_norms (T,G) fp16; v_packed (T,Vb) u8; v_norms (T,) fp16.
    Returns out (gqa,128) float32 and lse (gqa,) float32."""
    plan, pp = _plan_ptr(plan)
    q = _u16(q_rot).reshape(-1, D)
    gqa = q.shape[0]
    T = k_packed.shape[0] if T is None else T
    kp = np.zeros((k_packed.shape[0], k_packed.shape[1] + 2), np.uint8)
    kp[:, :k_packed.shape[1]] = k_packed
    vp = np.zeros((v_packed.shape[0], v_packed.shape[1] + 2), np.uint8)
    vp[:, :v_packed.shape[1]] = v_packed
    kn = _u16(k_norms)
    kn = kn.reshape(kn.shape[0], -1)
    vn = _u16(v_norms).reshape(-1)
    scale = 1.0 / np.sqrt(D) if scale is None else scale
    out = np.zeros((gqa, D), np.float32)
    lse = np.zeros(gqa, np.float32)
    lib().orc_decode_attn(pp, _p(q), ci(gqa), _p(kp), i64(kp.shape[1]), _p(kn), i64(kn.shape[1]),
                          _p(vp), i64(vp.shape[1]), _p(vn), i64(1),
                          i64(T), ci(n_splits), ci(k_layout), ci(v_layout), cf(scale),
                          ci(int(unrotate)), _p(out), _p(lse))
    return out, lse


def dequant_k(plan, codes, norms16):
    """K in the packed (permuted + rotated) space as float32 (N,128)."""
    plan, pp = _plan_ptr(plan)
    codes = np.ascontiguousarray(codes, dtype=np.uint8).reshape(-1, D)
    kn = _u16(norms16)
    kn = kn.reshape(codes.shape[0], -1)
    out = np.zeros((codes.shape[0], D), np.float32)
    lib().orc_dequant_k(pp, _p(codes), _p(kn), i64(kn.shape[1]), i64(codes.shape[0]), _p(out))
    return out


def dequant_v(plan, codes, norms16):
    """V in its rotated space as float32 (N,128)."""
    plan, pp = _plan_ptr(plan)
    codes = np.ascontiguousarray(codes, dtype=np.uint8).reshape(-1, D)
    vn = _u16(norms16).reshape(-1)
    out = np.zeros((codes.shape[0], D), np.float32)
    lib().orc_dequant_v(pp, _p(codes), _p(vn), i64(codes.shape[0]), _p(out))
    return out
