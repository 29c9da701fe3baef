"""GPU: the entry point that allocates nothing (bgtq_decode_attend_static) against
bgtq_decode_attn + bgtq_lse_reduce with a caller-provided workspace, through the C ABI.

Both run the same kernels on the same inputs, so the fp16 outputs and the fp32 log-sum-exps
must be bit-identical.  Two calls in a row share the library's fixed array; the second is
smaller (fewer rows, shorter context, fewer partitions), so stale entries of the first call
would show if the second read anything it did not write itself."""
import ctypes

import pytest
import torch

from blockgtq_amd import _capi, plan as P
from test_gpu_decode import _build

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _both(args, q_rot, kp, kn, vp, vn, T, n_kv, gqa, n_splits, lens=None):
    lib = _capi.lib()
    B = q_rot.shape[0]
    n_q = n_kv * gqa
    st = _capi.stream_ptr(q_rot.device)
    common = (_capi.ptr(args['plans']), _capi.ptr(q_rot), q_rot.stride(0), q_rot.stride(1),
              _capi.ptr(kp), kp.stride(0), kp.stride(1), kp.stride(2), kp.shape[-1],
              _capi.ptr(kn), kn.stride(0), kn.stride(1), kn.stride(2),
              _capi.ptr(vp), vp.stride(0), vp.stride(1), vp.stride(2), vp.shape[-1],
              _capi.ptr(vn), vn.stride(0), vn.stride(1), vn.stride(2),
              _capi.ptr(lens), T, B, n_kv, gqa, n_splits)
    scale = 1.0 / 128 ** 0.5
    # existing entry points, workspace from the caller
    ws = torch.empty(lib.bgtq_workspace_bytes(B, n_q, n_splits) // 4, dtype=torch.float32, device=DEV)
    part_out, part_lse = ws[:B * n_q * n_splits * 128], ws[B * n_q * n_splits * 128:]
    out0 = torch.empty(B, n_q, 128, dtype=torch.float16, device=DEV)
    lse0 = torch.empty(B, n_q, dtype=torch.float32, device=DEV)
    _capi.check(lib.bgtq_decode_attn(*common, _capi.ptr(part_out), _capi.ptr(part_lse), 0, 0, scale, st),
                "bgtq_decode_attn")
    _capi.check(lib.bgtq_lse_reduce(_capi.ptr(args['plans']), _capi.ptr(part_out), _capi.ptr(part_lse),
                                    n_splits, None, None, 0, B, n_kv, gqa, 1,
                                    _capi.ptr(out0), out0.stride(0), out0.stride(1), _capi.ptr(lse0), st),
                "bgtq_lse_reduce")
    # the entry point under test: everything preallocated, no workspace argument
    out1 = torch.full((B, n_q, 128), 9.0, dtype=torch.float16, device=DEV)
    lse1 = torch.full((B, n_q), 9.0, dtype=torch.float32, device=DEV)
    before = torch.cuda.memory_allocated()
    _capi.check(lib.bgtq_decode_attend_static(*common, 0, 0, scale, 1, _capi.ptr(out1), out1.stride(0),
                                              out1.stride(1), _capi.ptr(lse1), st),
                "bgtq_decode_attend_static")
    assert torch.cuda.memory_allocated() == before
    torch.cuda.synchronize()
    return out0, lse0, out1, lse1


def test_static_entry_matches_workspace_entry_twice_second_call_smaller():
    # first call: 3 rows x 2 KV heads x 8 query heads each, 700 tokens, 6 partitions
    a = _build(192, 1, 5, 3, 2, 8, 3, 700, seed=21)
    o0, l0, o1, l1 = _both(a[0], *a[2:], 700, 2, 8, 6)
    assert torch.equal(o0, o1) and torch.equal(l0, l1)
    assert o0.float().abs().max() > 0
    # second call, smaller in every respect: 1 row x 1 KV head x 4 heads, 90 tokens, 2 partitions
    b = _build(192, 1, 5, 3, 1, 4, 1, 90, seed=22)
    o0, l0, o1, l1 = _both(b[0], *b[2:], 90, 1, 4, 2)
    assert torch.equal(o0, o1) and torch.equal(l0, l1)
    # ragged lengths through the same entry point
    lens = torch.tensor([700, 33, 0], dtype=torch.int32, device=DEV)
    o0, l0, o1, l1 = _both(a[0], *a[2:], 700, 2, 8, 5, lens=lens)
    assert torch.equal(o0, o1) and torch.equal(l0, l1)


def test_static_entry_refuses_sizes_beyond_its_array():
    lib = _capi.lib()
    a = _build(192, 1, 5, 3, 1, 4, 1, 70, seed=23)
    args, _, q_rot, kp, kn, vp, vn = a
    out = torch.empty(1, 4, 128, dtype=torch.float16, device=DEV)
    # B * n_q * n_splits * 129 * 4 bytes > 8 MiB: claimed batch of 4096 rows x 4 heads x 2 partitions
    rc = lib.bgtq_decode_attend_static(
        _capi.ptr(args['plans']), _capi.ptr(q_rot), 0, q_rot.stride(1),
        _capi.ptr(kp), 0, kp.stride(1), kp.stride(2), kp.shape[-1],
        _capi.ptr(kn), 0, kn.stride(1), kn.stride(2),
        _capi.ptr(vp), 0, vp.stride(1), vp.stride(2), vp.shape[-1],
        _capi.ptr(vn), 0, vn.stride(1), vn.stride(2),
        None, 70, 4096, 1, 4, 2, 0, 0, 0.0884, 1, _capi.ptr(out), 0, out.stride(1), None,
        _capi.stream_ptr(out.device))
    assert rc == -3
    assert "maximum" in lib.bgtq_strerror(rc).decode()


def test_static_entry_replays_in_a_graph_after_one_eager_call():
    """The first call on a device looks up the array's address and sets kernel attributes (no
    stream operations), so it is made eagerly; after that the entry point can be captured.  Every
    replay, with eager work between the replays, must reproduce the eager result bit for bit."""
    lib = _capi.lib()
    args, _, q_rot, kp, kn, vp, vn = _build(192, 1, 5, 3, 2, 8, 2, 500, seed=25)
    B, n_kv, gqa, T, ns = 2, 2, 8, 500, 4
    scale = 1.0 / 128 ** 0.5
    out_e = torch.empty(B, n_kv * gqa, 128, dtype=torch.float16, device=DEV)
    out_g = torch.zeros_like(out_e)

    def call(out):
        _capi.check(lib.bgtq_decode_attend_static(
            _capi.ptr(args['plans']), _capi.ptr(q_rot), q_rot.stride(0), q_rot.stride(1),
            _capi.ptr(kp), kp.stride(0), kp.stride(1), kp.stride(2), kp.shape[-1],
            _capi.ptr(kn), kn.stride(0), kn.stride(1), kn.stride(2),
            _capi.ptr(vp), vp.stride(0), vp.stride(1), vp.stride(2), vp.shape[-1],
            _capi.ptr(vn), vn.stride(0), vn.stride(1), vn.stride(2),
            None, T, B, n_kv, gqa, ns, 0, 0, scale, 1, _capi.ptr(out), out.stride(0), out.stride(1), None,
            _capi.stream_ptr(q_rot.device)), "bgtq_decode_attend_static")

    call(out_e)                                   # eager warm-up: address look-up, attributes
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        call(out_g)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        call(out_g)
    for i in range(3):
        out_g.zero_()
        (q_rot.float() * (i + 1)).sum().item()    # the program's own eager work and a synchronisation
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out_g, out_e), i
