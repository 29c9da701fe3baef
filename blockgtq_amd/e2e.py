"""End-to-end packed decode on a randomly initialised Qwen2-style model.

Builds the model from a local config (no hub access), calibrates the per-head
quantizers on the model's own Q/K activations for random tokens, prefills a
prompt layer by layer through the quantise-and-pack path, then decodes greedily
from the packed cache; the same prompt and token budget run through a dense
fp16 KV cache for comparison.  ``python -m blockgtq_amd.e2e --help``.

Mirrors what the reference's bench/bench_decode_e2e.py measures (prefill pack
time, decode tokens/s, per-layer attention time against fp16 attention) with
synthetic weights and token ids.
"""
import argparse
import json
import time

import torch

MODELS = {
    # geometry of Qwen2.5-3B (config.json of the public checkpoint)
    "qwen2.5-3b": dict(vocab_size=151936, hidden_size=2048, intermediate_size=11008,
                       num_hidden_layers=36, num_attention_heads=16, num_key_value_heads=2,
                       max_position_embeddings=32768, rope_theta=1e6, rms_norm_eps=1e-6,
                       tie_word_embeddings=True),
    # small stand-in with the same head geometry for tests
    "tiny": dict(vocab_size=1024, hidden_size=512, intermediate_size=1024,
                 num_hidden_layers=2, num_attention_heads=4, num_key_value_heads=2,
                 max_position_embeddings=8192, rope_theta=1e6, rms_norm_eps=1e-6,
                 tie_word_embeddings=True),
}


def build_model(name, device, dtype=torch.bfloat16, seed=1234, n_layers=None):
    """Random-init Qwen2 causal LM of geometry ``name`` on ``device``."""
    from transformers import Qwen2Config, Qwen2ForCausalLM
    kw = dict(MODELS[name])
    if n_layers:
        kw["num_hidden_layers"] = n_layers
    cfg = Qwen2Config(**kw)
    torch.manual_seed(seed)
    with torch.device(device):
        model = Qwen2ForCausalLM(cfg)
    return model.to(dtype).eval()


class _Timer:
    """Accumulates device time of bracketed regions with events on the current stream."""

    def __init__(self):
        self.pairs = []

    def __call__(self, fn, *a, **kw):
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        out = fn(*a, **kw)
        e1.record()
        self.pairs.append((e0, e1))
        return out

    def total_ms(self):
        torch.cuda.synchronize()
        return sum(a.elapsed_time(b) for a, b in self.pairs)


@torch.no_grad()
def run(model_name="qwen2.5-3b", batch=4, prompt_len=8192, new_tokens=256, k_bits=3.0, v_bits=3,
        device="cuda:0", seed=1234, n_layers=None, n_calib=256, fp16_baseline=True,
        max_bits=5, return_logits=False, graph=True):
    from . import _capi
    from .calibration import build_quantizers, collect_qk_activations
    from .fp16_baseline import FP16KVCache, fp16_decode_step
    from .packed_kv_manager import run_decoder_stack
    from .prefill import layer_major_prefill
    from .production_cache import BlockGTQProductionCache
    from .production_decode import production_decode_step

    _capi.lib()
    torch.cuda.set_device(device)
    model = build_model(model_name, device, seed=seed, n_layers=n_layers)
    cfg = model.config
    L, nq, nkv = cfg.num_hidden_layers, cfg.num_attention_heads, cfg.num_key_value_heads
    hd = cfg.hidden_size // nq
    gen = torch.Generator().manual_seed(seed)
    prompt = torch.randint(0, cfg.vocab_size, (batch, prompt_len), generator=gen).to(device)
    calib = torch.randint(0, cfg.vocab_size, (1, n_calib), generator=gen)

    t0 = time.perf_counter()
    layer_data = collect_qk_activations(model, calib, device, n_calib_tokens=n_calib)
    layer_data = {li: {k: v.float().cpu() for k, v in d.items()} for li, d in layer_data.items()}
    quantizers, batched_args, kernel_args = build_quantizers(
        layer_data, L, nkv, hd, k_avg_bits=k_bits, v_bits=v_bits, k_nibble=False, device=device,
        min_bits=1, max_bits=max_bits)
    calib_s = time.perf_counter() - t0

    max_T = prompt_len + new_tokens + 8
    cache = BlockGTQProductionCache(quantizers, batched_args, kernel_args, L, nkv, nq, hd, max_T,
                                    v_bits=v_bits, k_nibble=False, v_nibble=False, device=device,
                                    batch_size=batch)
    # ---- prefill: whole prompt through one layer at a time, K/V packed on the way ----------
    pack = _Timer()
    enc = cache._encode_batched
    cache._encode_batched = lambda *a, **kw: pack(enc, *a, **kw)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    hidden = layer_major_prefill(model, cache, prompt)
    logits = model.lm_head(model.model.norm(hidden[:, -1:]))
    torch.cuda.synchronize()
    prefill_ms = (time.perf_counter() - t0) * 1e3
    pack_ms = pack.total_ms()
    cache._encode_batched = enc
    first = logits.argmax(-1)
    if return_logits:
        out_logits = {"packed_prefill": logits.float().cpu()}

    # ---- packed decode -----------------------------------------------------------------------
    # The first steps run eagerly (per-layer attention time comes from them); the rest is one
    # HIP graph of the whole step (model layers, append, attention, merge, greedy pick, position
    # and length updates) replayed once per token.
    attn = _Timer()
    ea = cache.encode_and_attend
    n_eager = min(8, new_tokens) if graph else new_tokens
    tok, toks = first, []
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for i in range(n_eager):
        timed = i >= n_eager - 8              # per-layer attention time from the last eager steps
        cache.encode_and_attend = (lambda *a, **kw: attn(ea, *a, **kw)) if timed else ea
        pos = torch.full((batch, 1), prompt_len + i, device=device, dtype=torch.long)
        step_logits = production_decode_step(model, tok, pos, cache)
        if return_logits and i == 0:
            out_logits["packed_step0"] = step_logits.float().cpu()
        if return_logits and not graph:
            out_logits[f"eager_step{i}"] = step_logits.float().cpu()
        tok = step_logits.argmax(-1)
        toks.append(tok)
    torch.cuda.synchronize()
    eager_s = time.perf_counter() - t0
    cache.encode_and_attend = ea
    attn_us = attn.total_ms() * 1e3 / (min(8, n_eager) * L)
    graph_s, n_graph = 0.0, new_tokens - n_eager
    if n_graph > 0:
        cache.use_device_lengths()
        ids = tok.clone()
        pos = torch.full((batch, 1), prompt_len + n_eager, device=device, dtype=torch.long)
        logits_buf = [None]

        def step():
            lg = production_decode_step(model, ids, pos, cache)
            logits_buf[0] = lg
            ids.copy_(lg.argmax(-1))
            pos.add_(1)

        state = (ids.clone(), pos.clone(), cache._lens2.clone(), cache.seq_len)
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            for _ in range(2):
                step()
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g):
            step()
        ids.copy_(state[0]); pos.copy_(state[1]); cache._lens2.copy_(state[2])
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for i in range(n_graph):
            g.replay()
            toks.append(ids.clone())
            if return_logits and i < 3:
                out_logits[f"graph_step{i}"] = logits_buf[0].float().cpu()
        torch.cuda.synchronize()
        graph_s = time.perf_counter() - t0
        cache.seq_len = state[3] + n_graph
    if return_logits:
        out_logits["tokens"] = torch.cat(toks, 1).cpu()
    decode_s = eager_s + graph_s
    out = {
        "model": model_name, "layers": L, "batch": batch, "prompt_len": prompt_len,
        "new_tokens": new_tokens, "k_bits_avg": k_bits, "v_bits": v_bits,
        "data": "random-init bf16 weights, uniform random token ids", "calibration_s": round(calib_s, 1),
        "prefill_ms": round(prefill_ms, 1), "prefill_pack_ms": round(pack_ms, 2),
        "decode_tokens_per_s": round(batch * (n_graph / graph_s if n_graph else new_tokens / decode_s), 1),
        "decode_ms_per_step": round((graph_s / n_graph if n_graph else decode_s / new_tokens) * 1e3, 3),
        "decode_mode": "HIP graph of the whole step" if n_graph else "eager",
        # eagerly launched steps: all of them without the graph, else only the first 8 (which also
        # carry the one-off costs of a first call), so the figure is only comparable in the first case
        ("decode_tokens_per_s_eager" if not n_graph else "first_steps_eager_tokens_per_s"):
            round(batch * n_eager / eager_s, 1),
        "eager_attn_us_per_layer": round(attn_us, 2),
        "packed_cache_bytes": cache.cache_memory_bytes(), "fp16_cache_bytes": cache.fp16_cache_bytes(),
    }
    del cache

    if fp16_baseline:
        dense = FP16KVCache(L, nkv, nq, hd, max_T, device=device, batch_size=batch, dtype=torch.bfloat16)
        pos = torch.arange(prompt_len, device=device).unsqueeze(0).expand(batch, -1)
        hidden = run_decoder_stack(model, model.model.embed_tokens(prompt), pos, nq, nkv, hd, dense.attend)
        dense.increment(prompt_len)
        dense_logits = model.lm_head(model.model.norm(hidden[:, -1:]))
        tok = dense_logits.argmax(-1)
        attn = _Timer()
        da = dense.attend
        toks = []
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for i in range(new_tokens):
            dense.attend = (lambda *a, **kw: attn(da, *a, **kw)) if i >= new_tokens - 8 else da
            pos = torch.full((batch, 1), prompt_len + i, device=device, dtype=torch.long)
            step_logits = fp16_decode_step(model, first if i == 0 else tok, pos, dense)
            if return_logits and i == 0:
                out_logits["fp16_step0"] = step_logits.float().cpu()
            tok = step_logits.argmax(-1)
            toks.append(tok)
        torch.cuda.synchronize()
        dense_s = time.perf_counter() - t0
        out["fp16_decode_tokens_per_s"] = round(batch * new_tokens / dense_s, 1)
        out["fp16_attn_us_per_layer"] = round(attn.total_ms() * 1e3 / (8 * L), 2)
    return (out, out_logits) if return_logits else out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--model", default="qwen2.5-3b", choices=sorted(MODELS))
    ap.add_argument("--batch", type=int, default=4)
    ap.add_argument("--prompt-len", type=int, default=8192)
    ap.add_argument("--new-tokens", type=int, default=256)
    ap.add_argument("--k-bits", type=float, default=3.0)
    ap.add_argument("--v-bits", type=int, default=3)
    ap.add_argument("--layers", type=int, default=0)
    ap.add_argument("--no-fp16", action="store_true")
    ap.add_argument("--no-graph", action="store_true", help="decode eagerly instead of replaying a HIP graph")
    a = ap.parse_args()
    print(json.dumps(run(a.model, a.batch, a.prompt_len, a.new_tokens, a.k_bits, a.v_bits,
                         n_layers=a.layers or None, fp16_baseline=not a.no_fp16, graph=not a.no_graph)))


if __name__ == "__main__":
    main()
