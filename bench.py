#!/usr/bin/env python3
"""Headline benchmark: packed decode attention, K3V3, 32k context, one MI355X.

A step is one decode step of the hot path over all layers of the workload:
per layer, append one token per sequence through the quantise-and-pack kernels,
rotate the queries, run the fused unpack + dequant + split-T attention over the
packed cache and merge the partitions.  The whole step is captured once into a
HIP graph and replayed, the packed cache is resident in HBM before timing, and
the timed region is bracketed by device synchronisation.

Prints ONE JSON line.  ``value`` is microseconds per layer per step (lower is
better); ``roofline`` prices the attention kernel alone against the 8 TB/s HBM
peak over the bytes it must touch by construction; ``cpu_baseline`` times the
CPU checker (the scalar C restatement under oracle/, parallel over the host
cores) on a bounded sample of the same packed cache.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0
# HBM bytes per attention launch from FETCH_SIZE / WRITE_SIZE counter runs scaled by a copy
# kernel of known size (profiles/decode_mfma_kernel_*_hbm_traffic.txt); valid for the
# workload's own context, batch and default partition count only.
MEASURED_TRAFFIC_BYTES = {"qwen3b_b8_32k_k3v3": 66.12e6, "llama8b_4k_k3v3": 7.01e6,
                          "llama8b_128k_k2v2": 88.68e6, "qwen3_8b_b32_ragged_buffered": 267.36e6}


def parse():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--workload", default="qwen3b_b8_32k_k3v3")
    ap.add_argument("--layers", type=int, default=0, help="override layer count (0 = workload's)")
    ap.add_argument("--context", type=int, default=0, help="override context length")
    ap.add_argument("--splits", type=int, default=0, help="partitions per (row, KV head); 0 = auto")
    ap.add_argument("--no-graph", action="store_true", help="launch eagerly instead of replaying a graph")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--cpu-seconds", type=float, default=15.0)
    return ap.parse_args()


def cpu_baseline(mgr, w, q_rot_layer0, seconds, packed_lens):
    """Time the CPU checker on (batch row, KV head) pairs of layer 0 until about
    ``seconds`` of wall time are spent; scale to a full layer.  ``packed_lens[b]`` is
    the number of packed tokens row b attends to."""
    import numpy as np
    import oracle
    from concurrent.futures import ThreadPoolExecutor

    oracle.build()
    cores = min(os.cpu_count() or 1, 16)
    T = max(packed_lens)
    li = 0
    kp = mgr._k_packed[li][:, :, :T].cpu().numpy()
    kn = mgr._k_norms[li, :, :, :T].cpu().numpy()
    vp = mgr._v_packed[li, :, :, :T].cpu().numpy()
    vn = mgr._v_norms[li, :, :, :T].cpu().numpy()
    qr = q_rot_layer0.cpu().numpy()
    plans = mgr._batched_args[li]['plans_np']
    gqa = mgr.gqa_ratio
    pairs = [(b, h) for b in range(w.batch) for h in range(w.n_kv)]

    def one(bh):
        b, h = bh
        q8 = mgr.quantizers[li][h]
        n = packed_lens[b]
        oracle.decode_attn(plans[h:h + 1], qr[b, h * gqa:(h + 1) * gqa],
                           kp[b, h][:n, :q8._total_packed_bytes], kn[b, h][:n, :max(q8._n_groups, 1)],
                           vp[b, h][:n], vn[b, h][:n], n_splits=1)

    one(pairs[0])                                   # page in
    done, t0 = 0, time.perf_counter()
    with ThreadPoolExecutor(cores) as ex:           # ctypes releases the GIL
        while time.perf_counter() - t0 < seconds and done < 4 * len(pairs):
            batch = [pairs[(done + i) % len(pairs)] for i in range(cores)]
            list(ex.map(one, batch))
            done += len(batch)
    dt = time.perf_counter() - t0
    per_layer_us = dt / done * len(pairs) * 1e6
    return {"value": per_layer_us, "unit": "us/layer/step", "cores": cores, "kind": "port",
            "sample": f"{done} (batch row, KV head) packed-attention calls of layer 0 at up to T={T} "
                      f"({done / len(pairs):.2f} layer-steps), scalar C checker, {cores} threads"}


def main():
    args = parse()
    if args.gpus != 1:
        print("bench.py measures the single-GPU packed decode path; this build has no "
              "multi-GPU leg (every box has one GPU). Run with --gpus 1.", file=sys.stderr)
        sys.exit(2)
    import torch
    from blockgtq_amd import _capi, ops, plan as _plan
    from blockgtq_amd import workloads as wl

    if not torch.cuda.is_available():
        print("bench.py needs a GPU", file=sys.stderr)
        sys.exit(2)
    _capi.lib()
    dev = "cuda:0"
    torch.cuda.set_device(0)
    w = wl.WORKLOADS[args.workload]
    if args.context:
        w.context = args.context
    L = args.layers or w.n_layers

    t_setup = time.perf_counter()
    mgr, energies = wl.build_manager(w, dev, max_T=w.context + 8, n_layers=L)
    wl.fill_cache(mgr, w, energies, dev)
    torch.cuda.synchronize()
    setup_s = time.perf_counter() - t_setup
    T = mgr.seq_len
    seq_lens = w.seq_lens or [T] * w.batch

    qs = [wl.draw_q(w, li, dev, T) for li in range(L)]
    kvs = [wl.draw_kv(w, energies[li], 1, 10_000_000 + li, dev, pos0=T) for li in range(L)]
    n_splits = args.splits or ops.default_splits(w.batch, w.n_kv, T + 1)
    if not args.splits and (w.seq_lens is not None or w.window):
        n_splits = max(n_splits, min(4 * n_splits, (T + 511) // 512))      # ragged rows: finer partitions
    if mgr.buffered and mgr._seq_lens is None:
        mgr.set_seq_lens(seq_lens)
    mgr.n_splits = n_splits
    outs = [None] * L

    def step():
        # append at position T (the same slot every step, so the context stays fixed)
        for li in range(L):
            outs[li] = mgr.append_and_attend(li, qs[li], kvs[li][0], kvs[li][1])

    # --- warm up eagerly, then capture the step once -----------------------
    step()
    torch.cuda.synchronize()
    graph = None
    if not args.no_graph:
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            step()
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            step()
    run = graph.replay if graph is not None else step

    for _ in range(args.warmup):
        run()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        run()
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    ms_per_step = wall / args.steps * 1e3
    us_per_layer = ms_per_step * 1e3 / L

    # --- attention kernel alone: average launch duration by HIP events -----
    plans0 = [mgr._batched_args[li]['plans'] for li in range(L)]
    q_rots = [ops.rotate_q(plans0[li], qs[li].reshape(w.batch, w.n_q, w.head_dim).contiguous(), w.n_kv)
              for li in range(L)]
    part_out, part_lse = mgr._ws.get(w.batch, w.n_q, n_splits, dev)
    lib = _capi.lib()
    # tokens of the packed cache each row attends to once this step's token is in
    fp16_rows = (mgr.n_sink + mgr.window) if mgr.buffered else 0
    packed_lens = [max(t + 1 - fp16_rows, 0) for t in seq_lens]
    ragged = mgr.buffered or w.seq_lens is not None
    lens_dev = torch.tensor(packed_lens, dtype=torch.int32, device=dev) if ragged else None
    Tk = max(packed_lens)

    def attn_only(li):
        _capi.check(lib.bgtq_decode_attn(
            _capi.ptr(plans0[li]), _capi.ptr(q_rots[li]), q_rots[li].stride(0), q_rots[li].stride(1),
            _capi.ptr(mgr._k_packed[li]), *mgr._k_packed[li].stride()[:3], mgr._k_rows[li],
            _capi.ptr(mgr._k_norms[li]), *mgr._k_norms[li].stride()[:3],
            _capi.ptr(mgr._v_packed[li]), *mgr._v_packed[li].stride()[:3], mgr._vpb,
            _capi.ptr(mgr._v_norms[li]), *mgr._v_norms[li].stride()[:3],
            _capi.ptr(lens_dev), Tk, w.batch, w.n_kv, mgr.gqa_ratio, n_splits,
            _capi.ptr(part_out), _capi.ptr(part_lse), _plan.K_BITPACKED, _plan.V_BITPACKED,
            mgr.scale, _capi.stream_ptr()), "bgtq_decode_attn")

    def attn_all():
        for li in range(L):
            attn_only(li)

    attn_all()
    torch.cuda.synchronize()
    # One launch per layer back to back between two events on the launch stream, (a) launched
    # eagerly and (b) as a graph like the step above.  Both are the kernel's average duration plus
    # whatever gap the launch path leaves between two kernels: (a) turns host-bound when the
    # host's launch cost exceeds the kernel (a profiler multiplies it), (b) leaves long gaps
    # between short kernels.  The smaller of the two is reported.
    reps = max(1, args.steps // 2)

    def timed(run_once):
        ev0, ev1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        ev0.record()                   # same (current) stream the kernels go to
        for _ in range(reps):
            run_once()
        ev1.record()
        torch.cuda.synchronize()
        return ev0.elapsed_time(ev1) * 1e3 / (reps * L)

    attn_us = timed(attn_all)
    if graph is not None:
        attn_graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(attn_graph):
            attn_all()
        attn_graph.replay()
        torch.cuda.synchronize()
        attn_us = min(attn_us, timed(attn_graph.replay))
    alg_bytes = sum(wl.algorithmic_bytes_per_layer(mgr, li, [t + 1 for t in seq_lens])
                    for li in range(L)) / L
    achieved = alg_bytes / (attn_us * 1e-6) / 1e9

    tokens_per_s = w.batch / (ms_per_step * 1e-3)
    out = {
        "metric": "decode_attn_us_per_layer_per_step",
        "value": round(us_per_layer, 3),
        "unit": "us/layer/step",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 4),
        "higher_is_better": False, "scaling": "weak", "vs_baseline": None,
        "dtype": "u8 codes -> fp16 operands, fp32 accumulate", "data": "synthetic",
        "config": {"workload": w.name, "layers": L, "n_q_heads": w.n_q, "n_kv_heads": w.n_kv,
                   "head_dim": w.head_dim, "batch": w.batch, "context": T,
                   "k_bits_avg": w.k_bits, "v_bits": w.v_bits, "n_splits": n_splits,
                   "k_layout": "bit-packed", "v_layout": "bit-packed",
                   "fp16_sink_tokens": mgr.n_sink, "fp16_recent_window": mgr.window,
                   "step": "append(encode K,V) + rotate Q + attention + merge, per layer",
                   "graph": graph is not None},
        "tokens_per_s": round(tokens_per_s, 1),
        "attn_kernel_us_per_layer": round(attn_us, 3),
        "hbm_gbs_step": round(alg_bytes / (us_per_layer * 1e-6) / 1e9, 1),
        "setup_s": round(setup_s, 1),
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS,
                     "unit": "GB/s", "frac": round(achieved / HBM_PEAK_GBS, 4),
                     "traffic": (MEASURED_TRAFFIC_BYTES.get(w.name)
                                 if not (args.context or args.splits) else None),
                     "kernel": "decode attention",
                     "algorithmic_bytes_per_launch": int(alg_bytes),
                     "avg_launch_us": round(attn_us, 3)},
    }
    if not args.no_cpu:
        out["cpu_baseline"] = cpu_baseline(mgr, w, q_rots[0], args.cpu_seconds, packed_lens)
    else:
        out["cpu_baseline"] = None
    print(json.dumps(out))


if __name__ == "__main__":
    main()
