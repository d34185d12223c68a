"""Decode and prefill throughput of the Llama-3.1-8B shape with random weights.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

One JSON line on stdout. ``value`` is decoded tokens per second at batch 8: a
step is one decode step of the real generation path (step function, argmax on
the GPU, every step's tokens back on the host; as in the generation loop, a step
takes its tokens from where the last one left them on the GPU, so the host reads
one step's tokens while the next step runs). Prompts have
unequal, seeded lengths of 128-2048 tokens; the context length is 4096.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

# published peaks of MI355X
HBM_GBS = 8000.0
PEAK_TFLOPS = {"bf16": 2500.0, "fp16": 2500.0, "fp8": 5000.0, "fp32": 157.3}

from transformer_amd.config.shapes import LLAMA2_7B, LLAMA3_70B, LLAMA31_8B, SHAPES  # noqa: E402,F401

# prompt lengths of the decode batch that each configuration is quoted with
PROMPTS = {"8b": (128, 2048), "7b": (64, 1024), "70b": (2048, 2048)}
CONTEXT = 4096
PROMPT_MIN, PROMPT_MAX = 128, 2048
PREFILL_TOKENS = 2048


def prefill_flops(cfg, T):
    """Matrix products of T prompt tokens, causal attention, one row of the output matrix."""
    d, nh, nkv, dh, di = cfg.hidden, cfg.num_heads, cfg.num_kv_heads, cfg.head_dim, cfg.intermediate
    per_layer = 2 * T * d * (nh + 2 * nkv) * dh + 2 * T * nh * dh * d + 2 * T * d * 2 * di + 2 * T * di * d
    attn = 2 * 2 * nh * dh * (T * (T + 1) // 2)
    return cfg.num_layers * (per_layer + attn) + 2 * d * cfg.vocab


def decode_bytes(model, cfg, contexts):
    """What a decode step has to read: every weight it uses, once, and the cache of
    the live sequences."""
    import torch
    w = model.weight_bytes()
    if model.w["embed"].data_ptr() != model.w["head"].data_ptr():
        w -= model.w["embed"].numel() * model.w["embed"].element_size()   # only rows are read
    item = torch.empty((), dtype=model.dtype).element_size()
    return w + sum(contexts) * cfg.kv_bytes_per_token(item)


def time_decode(model, cfg, batch, steps, warmup, seed, prompt_min=PROMPT_MIN, prompt_max=PROMPT_MAX):
    import numpy as np
    import torch
    from transformer_amd import Entry
    from transformer_amd.sampling.sampler import Sampler
    rng = np.random.default_rng(seed)
    lens = [int(x) for x in rng.integers(prompt_min, prompt_max + 1, batch)]
    total = warmup + steps
    cache = model.new_cache(sum(-(-(n + total + 2) // 64) * 64 for n in lens), max_slots=batch)
    slots = [cache.alloc_slot() for _ in lens]
    sampler = Sampler(device=model.device)
    # prompts, a few sequences per step to bound the scratch memory
    toks = [[int(t) for t in rng.integers(0, cfg.vocab, n)] for n in lens]
    first = []
    for i in range(0, batch, 8):
        lg = model.step(cache, [Entry(s, t, (len(t) - 1,)) for s, t in zip(slots[i:i + 8], toks[i:i + 8])])
        first += sampler.choose(lg, range(i, i + len(lg)), [0] * len(lg))
    # the generation loop's way of stepping: the next step starts from the tokens where the
    # GPU left them, and the host reads each step's tokens while the next one runs
    lg = model.step(cache, [Entry(s, (t,), (0,)) for s, t in zip(slots, first)])
    flying = sampler.choose_async(lg, range(batch), [1] * batch)
    entries = [Entry(s, (0,), (0,)) for s in slots]
    produced = []

    def one():
        nonlocal flying
        lg = model.step(cache, entries, device_tokens=flying.device)
        nxt = sampler.choose_async(lg, range(batch), [0] * batch)
        produced.append(flying.result())
        flying = nxt

    for _ in range(warmup):
        one()
    flying.result()
    torch.cuda.synchronize()
    ctx_mid = [cache.length(s) + steps // 2 for s in slots]
    t0 = time.perf_counter()
    for _ in range(steps):
        one()
    flying.result()
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    for s in slots:
        cache.free_slot(s)
    del cache
    torch.cuda.empty_cache()
    return dt, ctx_mid


def time_prefill(model, cfg, reps, seed, tokens=PREFILL_TOKENS):
    import numpy as np
    import torch
    from transformer_amd import Entry
    rng = np.random.default_rng(seed)
    toks = [int(t) for t in rng.integers(0, cfg.vocab, tokens)]
    cache = model.new_cache(-(-tokens // 64) * 64, max_slots=1)
    times = []
    for r in range(reps + 1):
        s = cache.alloc_slot()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        model.step(cache, [Entry(s, toks, (tokens - 1,))])
        torch.cuda.synchronize()
        dt = time.perf_counter() - t0
        cache.free_slot(s)
        if r > 0:                       # the first run warms the library's kernel choice
            times.append(dt)
    del cache
    torch.cuda.empty_cache()
    return sorted(times)[len(times) // 2]          # the median


def read_probe_gbs(device, nbytes=1 << 30, workgroups=2048, reps=5):
    """GB/s of a kernel that only reads: the machine's own ceiling for the weight streams of a
    decode step (the roofline of the line is the published 8 TB/s; this says how much of the
    distance to it is the memory system's)."""
    import torch
    from transformer_amd import kernels
    buf = torch.zeros(nbytes // 4, dtype=torch.int32, device=device)
    sink = torch.zeros(256, dtype=torch.int32, device=device)
    best = float("inf")
    for _ in range(reps + 1):
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        kernels.read_probe(buf, workgroups, sink)
        e1.record()
        torch.cuda.synchronize()
        best = min(best, e0.elapsed_time(e1) * 1e-3)
    return nbytes / best / 1e9


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=128)
    ap.add_argument("--warmup", type=int, default=16)
    ap.add_argument("--batch", type=int, default=8)
    ap.add_argument("--layers", type=int, default=None, help="build fewer layers than the model has")
    ap.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "float32"])
    ap.add_argument("--shape", default="8b", choices=sorted(SHAPES),
                    help="layer sizes: the headline model (8b), Llama-2-7B (7b) or Llama-3-70B (70b)")
    ap.add_argument("--prompt-min", type=int, default=None, help="shortest prompt of the decode batch")
    ap.add_argument("--prompt-max", type=int, default=None, help="longest prompt of the decode batch")
    ap.add_argument("--no-points", action="store_true", help="skip batch 1 and 64 and the prefill")
    ap.add_argument("--probe", action="store_true",
                    help="also measure what a kernel that only reads gets from this machine's memory "
                         "and add it to the line (\"probe\")")
    ap.add_argument("--prefill-tokens", type=int, default=PREFILL_TOKENS,
                    help="tokens of the prompt whose step is timed (the line's \"prefill\")")
    ap.add_argument("--prefill-only", action="store_true",
                    help="run only the 2,048-token prefill (for profiling); prints its own line")
    a = ap.parse_args()
    if a.gpus != 1:
        print(f"bench.py measures one GPU; --gpus {a.gpus} is not supported by this engine")
        return 2
    import torch
    import transformer_amd as ta
    shape_name, shape = SHAPES[a.shape]
    if a.prompt_min is None:
        a.prompt_min = PROMPTS[a.shape][0]
    if a.prompt_max is None:
        a.prompt_max = max(PROMPTS[a.shape][1], a.prompt_min)
    # longer prompts than the shape's context are a measurement of their own: let positions reach them
    room = max(a.prompt_max + 2 * (a.steps + a.warmup) + 8, a.prefill_tokens)
    shape = {**shape, "max_position_embeddings": max(shape["max_position_embeddings"], room)}
    cfg = ta.LlamaConfig.from_dict(shape)
    layers = a.layers or cfg.num_layers
    model = ta.random_model(cfg, seed=0, dtype=a.dtype, num_layers=layers)
    mcfg = model.config
    torch.cuda.synchronize()
    dkey = "bf16" if a.dtype == "bfloat16" else "fp32"

    if a.prefill_only:
        pt = time_prefill(model, mcfg, reps=max(1, a.steps), seed=2, tokens=a.prefill_tokens)
        fl = prefill_flops(mcfg, a.prefill_tokens)
        print(json.dumps({"prefill_ms": round(pt * 1e3, 3), "tokens": a.prefill_tokens,
                          "tok_per_s": round(a.prefill_tokens / pt, 1),
                          "frac": round(fl / pt / (PEAK_TFLOPS[dkey] * 1e12), 4)}))
        return 0
    dt, ctx = time_decode(model, mcfg, a.batch, a.steps, a.warmup, seed=1, prompt_min=a.prompt_min,
                          prompt_max=a.prompt_max)
    ms = dt / a.steps * 1e3
    value = a.batch * a.steps / dt
    nbytes = decode_bytes(model, mcfg, ctx)
    achieved = nbytes / (dt / a.steps) / 1e9
    line = {
        "metric": f"decode tok/s @ batch {a.batch}; {shape_name} shape", "value": round(value, 2),
        "unit": "tok/s", "n_gpus": 1, "steps": a.steps, "warmup": a.warmup,
        "ms_per_step": round(ms, 4), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": dkey, "data": "synthetic",
        "config": {"model": f"{shape_name} shape, random weights N(0,0.02)",
                   "layers": layers, "layers_of_model": cfg.num_layers, "hidden": cfg.hidden,
                   "heads": cfg.num_heads, "kv_heads": cfg.num_kv_heads, "head_dim": cfg.head_dim,
                   "intermediate": cfg.intermediate, "vocab": cfg.vocab,
                   "rope_theta": cfg.rope_theta, "rms_eps": cfg.rms_eps,
                   "global_batch": a.batch, "seq_len": max(CONTEXT, a.prompt_max + a.steps + a.warmup),
                   "prompt_min": a.prompt_min, "prompt_max": a.prompt_max, "mean_context": round(sum(ctx) / len(ctx), 1),
                   "prefill_tokens": a.prefill_tokens, "parallelism": "single GPU",
                   "sampling": "greedy"},
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_GBS,
                     "unit": "GB/s", "frac": round(achieved / HBM_GBS, 4)},
    }
    if a.probe:
        gbs = read_probe_gbs(model.device)
        line["probe"] = {"read_gbs": round(gbs, 1), "achieved_of_read": round(achieved / gbs, 4),
                         "what": "1 GiB read by 2048 workgroups with non-temporal loads, best of 5"}
    if not a.no_points:
        pt = time_prefill(model, mcfg, reps=5, seed=2, tokens=a.prefill_tokens)
        fl = prefill_flops(mcfg, a.prefill_tokens)
        line["prefill"] = {"value": round(a.prefill_tokens / pt, 1), "tokens": a.prefill_tokens,
                           "ms": round(pt * 1e3, 3),
                           "frac": round(fl / pt / (PEAK_TFLOPS[dkey] * 1e12), 4)}
        points = {}
        for b, st in ((1, max(16, a.steps // 2)), (64, max(16, a.steps // 2))):
            d2, _ = time_decode(model, mcfg, b, st, max(4, a.warmup // 2), seed=3 + b,
                                prompt_min=a.prompt_min, prompt_max=a.prompt_max)
            points[f"decode_b{b}"] = round(b * st / d2, 2)
        line["points"] = points
    print(json.dumps(line))
    return 0


if __name__ == "__main__":
    sys.exit(main())
