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
unpacked torch path (quantise -> reconstruct per KV head, then fp32 attention
with GQA expansion) on the host cores on a bounded sample of the same workload.
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
# of known size: blockgtq_amd/measured_traffic.json, one entry per workload, each naming the
# kernel revision it was measured on and the summary under profiles/ that holds the readings.
TRAFFIC_TABLE = os.path.join(ROOT, "blockgtq_amd", "measured_traffic.json")


def measured_traffic(workload, kernel_revision, default_shape):
    """Bytes per launch for ``workload`` if the table has a figure taken on this kernel revision
    at the workload's own context and partition count, else None."""
    if not default_shape:
        return None
    try:
        with open(TRAFFIC_TABLE) as f:
            entry = json.load(f)["entries"].get(workload)
    except (OSError, ValueError, KeyError):
        return None
    if not entry or entry.get("decode_kernel_revision") != kernel_revision:
        return None
    return entry["hbm_bytes_per_launch"]


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
    ap.add_argument("--layout", choices=["bitpacked", "nibble"], default="bitpacked",
                    help="record layout of the packed cache: bit-packed K and V (the headline), or the "
                         "production cache's default (K as nibbles + raw bytes with corrected norms, V as nibbles)")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--cpu-seconds", type=float, default=15.0)
    return ap.parse_args()


def _cpu_model():
    try:
        with open("/proc/cpuinfo") as f:
            for line in f:
                if line.startswith("model name"):
                    return line.split(":", 1)[1].strip()
    except OSError:
        pass
    return "unknown CPU"


def cpu_baseline(mgr, w, energies, seconds, seq_lens):
    """The unpacked torch path on the host cores, layer 0 of the same workload: per KV head
    quantise -> reconstruct K (Block-GTQ, the packed cache's own bit allocation) and V (TQ-MSE)
    into full-width fp32, then fp32 scaled-dot-product attention of one decode query per
    sequence with the KV heads expanded to their query groups.  Two figures: attention over
    an already reconstructed cache, and reconstruction + attention (what a CPU holding only
    quantised data pays per step).  Median of 10 runs after 2 warm-ups, on as many batch
    rows as the time budget allows, scaled to the whole batch."""
    import statistics
    import torch
    from blockgtq_amd import unaccelerated as ua
    from blockgtq_amd import workloads as wl

    threads = torch.get_num_threads()                # the process's CPU share (OMP_NUM_THREADS)
    q8s = mgr.quantizers[0]
    kqs, vqs = ua.quantizers_from_allocations(
        [q8.bit_allocation for q8 in q8s], w.head_dim, w.v_bits, [42 + h for h in range(w.n_kv)],
        rotation_threshold=q8s[0].rotation_threshold, min_bits=w.min_bits, max_bits=w.max_bits, device="cpu")
    T = max(seq_lens)
    one_row = wl.Workload(**{**w.__dict__, "batch": 1})

    def draw_row(b):
        k, v = wl.draw_kv(one_row, energies[0], seq_lens[b], 500_000 + b, "cpu")
        q = wl.draw_q(one_row, 0, "cpu", seq_lens[b])
        return q[:, :, 0], k, v

    def full(row):
        q, k, v = row
        return ua.decode_attention(q, *ua.round_trip_heads(kqs, vqs, k, v), scale=mgr.scale)

    rows = [draw_row(0)]
    t0 = time.perf_counter()
    full(rows[0])
    t_row = time.perf_counter() - t0
    n_rows = max(1, min(w.batch, int(seconds / (13.0 * max(t_row, 1e-4)))))
    rows += [draw_row(b) for b in range(1, n_rows)]
    recon = [ua.round_trip_heads(kqs, vqs, k, v) for _, k, v in rows]

    def median_us(fn):
        for _ in range(2):
            fn()
        times = []
        for _ in range(10):
            t = time.perf_counter()
            fn()
            times.append(time.perf_counter() - t)
        return statistics.median(times) * 1e6 * w.batch / n_rows

    both = median_us(lambda: [full(r) for r in rows])
    attn = median_us(lambda: [ua.decode_attention(r[0], kh, vh, scale=mgr.scale) for r, (kh, vh) in zip(rows, recon)])
    return {"value": round(both, 1), "unit": "us/layer/step", "cores": threads, "kind": "port",
            "attention_only_us": round(attn, 1),
            "sample": f"layer 0, {n_rows} of {w.batch} batch rows at their own context (up to T={T}), scaled to the "
                      f"batch; value = reconstruct K (Block-GTQ) and V (TQ-MSE) per KV head + fp32 SDPA with "
                      f"GQA expansion, attention_only_us = SDPA over an already reconstructed cache; torch "
                      f"{torch.__version__.split('+')[0]}, {threads} threads of {os.cpu_count()} logical CPUs "
                      f"({_cpu_model()}); median of 10 after 2 warm-ups"}


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
    nibble = args.layout == "nibble"
    if nibble:
        if mgr.buffered or w.seq_lens is not None:
            print("--layout nibble is measured on the plain (unbuffered, equal-length) workloads", file=sys.stderr)
            sys.exit(2)
        # the production cache in its default layout, on the same quantizers
        from blockgtq_amd.production_cache import BlockGTQProductionCache
        cache = BlockGTQProductionCache(mgr.quantizers, mgr._batched_args, mgr._kernel_args, L, w.n_kv, w.n_q,
                                        w.head_dim, w.context + 8, v_bits=w.v_bits, k_nibble=True, v_nibble=True,
                                        device=dev, batch_size=w.batch)
        for li in range(L):
            for lo in range(0, w.context, 8192):
                n = min(8192, w.context - lo)
                k, v = wl.draw_kv(w, energies[li], n, li * 4096 + lo // 8192, dev, pos0=lo)
                cache._encode_batched(li, k, v, lo)
        cache.seq_len = w.context
        store = {"k": cache.k_packed, "kn": cache.k_norms, "v": cache.v_packed, "vn": cache.v_norms,
                 "k_rows": [cache.k_bytes_per_tok] * L, "vpb": cache.vpb,
                 "k_layout": cache._k_layout, "v_layout": cache._v_layout, "ws": cache._ws}
    else:
        wl.fill_cache(mgr, w, energies, dev)
        store = {"k": mgr._k_packed, "kn": mgr._k_norms, "v": mgr._v_packed, "vn": mgr._v_norms,
                 "k_rows": mgr._k_rows, "vpb": mgr._vpb,
                 "k_layout": _plan.K_BITPACKED, "v_layout": _plan.V_BITPACKED, "ws": mgr._ws}
    torch.cuda.synchronize()
    setup_s = time.perf_counter() - t_setup
    T = w.context if nibble else mgr.seq_len
    seq_lens = w.seq_lens or [T] * w.batch

    qs = [wl.draw_q(w, li, dev, T) for li in range(L)]
    kvs = [wl.draw_kv(w, energies[li], 1, 10_000_000 + li, dev, pos0=T) for li in range(L)]
    n_splits = args.splits or ops.default_splits(w.batch, w.n_kv, T + 1)
    if not args.splits and (w.seq_lens is not None or w.window):
        n_splits = max(n_splits, min(4 * n_splits, (T + 511) // 512))      # ragged rows: finer partitions
    if mgr.buffered and mgr._seq_lens is None:
        mgr.set_seq_lens(seq_lens)
    mgr.n_splits = n_splits
    if nibble:
        cache.n_splits = n_splits
    outs = [None] * L

    def step():
        # append at position T (the same slot every step, so the context stays fixed)
        for li in range(L):
            if nibble:
                outs[li] = cache.encode_and_attend(li, qs[li], kvs[li][0], kvs[li][1])
            else:
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
    part_out, part_lse = store["ws"].get(w.batch, w.n_q, n_splits, dev)
    lib = _capi.lib()
    # tokens of the packed cache each row attends to once this step's token is in
    fp16_rows = (mgr.n_sink + mgr.window) if mgr.buffered else 0
    packed_lens = [max(t + 1 - fp16_rows, 0) for t in seq_lens]
    ragged = mgr.buffered or w.seq_lens is not None
    lens_dev = torch.tensor(packed_lens, dtype=torch.int32, device=dev) if ragged else None
    Tk = max(packed_lens)

    def attn_only(li):
        kp, kn, vp, vn = store["k"][li], store["kn"][li], store["v"][li], store["vn"][li]
        _capi.check(lib.bgtq_decode_attn(
            _capi.ptr(plans0[li]), _capi.ptr(q_rots[li]), q_rots[li].stride(0), q_rots[li].stride(1),
            _capi.ptr(kp), *kp.stride()[:3], store["k_rows"][li],
            _capi.ptr(kn), *kn.stride()[:3],
            _capi.ptr(vp), *vp.stride()[:3], store["vpb"],
            _capi.ptr(vn), *vn.stride()[:3],
            _capi.ptr(lens_dev), Tk, w.batch, w.n_kv, mgr.gqa_ratio, n_splits,
            _capi.ptr(part_out), _capi.ptr(part_lse), store["k_layout"], store["v_layout"],
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
    alg_bytes = sum(wl.algorithmic_bytes_per_layer(mgr, li, [t + 1 for t in seq_lens], nibble)
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
                   "k_layout": "nibbles + raw bytes" if nibble else "bit-packed",
                   "v_layout": "nibbles" if nibble else "bit-packed",
                   "fp16_sink_tokens": mgr.n_sink, "fp16_recent_window": mgr.window,
                   "step": "append(encode K,V) + rotate Q + attention + merge, per layer",
                   "graph": graph is not None},
        "tokens_per_s": round(tokens_per_s, 1),
        "attn_kernel_us_per_layer": round(attn_us, 3),
        "hbm_gbs_step": round(alg_bytes / (us_per_layer * 1e-6) / 1e9, 1),
        "setup_s": round(setup_s, 1),
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS,
                     "unit": "GB/s", "frac": round(achieved / HBM_PEAK_GBS, 4),
                     "traffic": measured_traffic(w.name, lib.bgtq_decode_kernel_revision(),
                                                 not (args.context or args.splits or nibble)),
                     "kernel": "decode attention",
                     "algorithmic_bytes_per_launch": int(alg_bytes),
                     "avg_launch_us": round(attn_us, 3)},
    }
    if not args.no_cpu:
        out["cpu_baseline"] = cpu_baseline(mgr, w, energies, args.cpu_seconds, [t + 1 for t in seq_lens])
    else:
        out["cpu_baseline"] = None
    print(json.dumps(out))


if __name__ == "__main__":
    main()
