"""Decode and prefill throughput of the Llama-3.1-8B shape with random weights.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

One JSON line on stdout. ``value`` is decoded tokens per second at batch 8: a
step is one decode step of the generation loop itself (``run_batches`` over the
engine's stepper: step function, argmax on the GPU, every step's tokens back on
the host while the next step runs). Prompts have unequal, seeded lengths of
128-2048 tokens; the context length is 4096. ``points`` holds the same at batch 1
and 64, at a long context, for other prompt lengths and for the Llama-2-7B shape,
each with its time, context and fraction of the roofline.
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
    """Times ``steps`` decode steps of the generation loop itself: ``run_batches`` over a
    ``ModelStepper`` (all prompts in one step, then one token per sequence and step, the next
    step started before the last one's tokens have reached the host), greedy, no stop token.
    The stepper is the engine's own with a clock added: before the first timed step is started
    and before the step after the last timed one, it waits for the GPU and reads the time, so
    exactly ``steps`` steps lie between the two readings, after ``warmup`` untimed ones.
    Returns (seconds, each sequence's context half-way, the loop's own Timing)."""
    import numpy as np
    import torch
    from transformer_amd.engine.generate import ModelStepper, run_batches
    from transformer_amd.sampling.sampler import Sampler
    rng = np.random.default_rng(seed)
    lens = [int(x) for x in rng.integers(prompt_min, prompt_max + 1, batch)]
    new_tokens = warmup + steps + 2
    cache = model.new_cache(sum(-(-(n + new_tokens) // 64) * 64 for n in lens), max_slots=batch)
    prompts = [[int(t) for t in rng.integers(0, cfg.vocab, n)] for n in lens]

    class Clocked(ModelStepper):
        def __init__(self, *args):
            super().__init__(*args)
            self.calls, self.marks, self.lengths = 0, [], None

        def step_async(self, items, previous=None, take=None):
            if self.calls in (1 + warmup, 1 + warmup + steps):      # call 0 runs the prompts
                torch.cuda.synchronize()
                self.marks.append(time.perf_counter())
                if self.lengths is None:
                    self.lengths = [self.cache.length(slot) for slot, *_ in items]
            self.calls += 1
            return super().step_async(items, previous, take)

    stepper = Clocked(model, cache, Sampler(device=model.device))
    result = run_batches(stepper, prompts, new_tokens, (), cache.num_pages * 64, batch,
                         max_position=model.spec.max_position)
    torch.cuda.synchronize()
    if len(stepper.marks) != 2 or len(result.batches) != 1 or \
            any(len(t) != new_tokens for t in result.tokens):
        raise RuntimeError("the generation loop did not run the steps that were to be timed")
    dt = stepper.marks[1] - stepper.marks[0]
    ctx_mid = [n + steps // 2 for n in stepper.lengths]
    del cache, stepper
    torch.cuda.empty_cache()
    return dt, ctx_mid, result.timing


def decode_point(model, cfg, batch, steps, warmup, seed, prompt_min, prompt_max):
    """One decode measurement with everything its roofline needs."""
    dt, ctx, timing = time_decode(model, cfg, batch, steps, warmup, seed, prompt_min, prompt_max)
    nbytes = decode_bytes(model, cfg, ctx)
    gbs = nbytes / (dt / steps) / 1e9
    return {"tok_s": round(batch * steps / dt, 2), "ms_per_step": round(dt / steps * 1e3, 4),
            "mean_context": round(sum(ctx) / len(ctx), 1), "gbs": round(gbs, 1),
            "frac": round(gbs / HBM_GBS, 4),
            # the loop's own table: every single-token step it ran, the recording of the first among them
            "loop_tok_s": round(timing.decode_tokens / max(timing.decode_seconds, 1e-9), 2)}


def time_prefill(model, cfg, reps, seed, tokens=PREFILL_TOKENS, lengths=None):
    """Median seconds of one step that runs a prompt of ``tokens`` tokens (or prompts of
    ``lengths``, together in one step) and returns the logits of each prompt's last place."""
    import numpy as np
    import torch
    from transformer_amd import Entry
    rng = np.random.default_rng(seed)
    lengths = list(lengths) if lengths is not None else [tokens]
    toks = [[int(t) for t in rng.integers(0, cfg.vocab, n)] for n in lengths]
    cache = model.new_cache(sum(-(-n // 64) * 64 for n in lengths), max_slots=len(lengths))
    times = []
    for r in range(reps + 1):
        slots = [cache.alloc_slot() for _ in lengths]
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        model.step(cache, [Entry(s, t, (len(t) - 1,)) for s, t in zip(slots, toks)])
        torch.cuda.synchronize()
        dt = time.perf_counter() - t0
        for s_ in slots:
            cache.free_slot(s_)
        if r > 0:                       # the first run warms the library's kernel choice
            times.append(dt)
    del cache
    torch.cuda.empty_cache()
    return sorted(times)[len(times) // 2]          # the median


def prefill_point(model, cfg, dkey, reps, seed, tokens=None, lengths=None):
    lengths = list(lengths) if lengths is not None else [tokens]
    pt = time_prefill(model, cfg, reps, seed, lengths=lengths)
    fl = sum(prefill_flops(cfg, n) for n in lengths)
    total = sum(lengths)
    return {"value": round(total / pt, 1), "tokens": total, "ms": round(pt * 1e3, 3),
            "frac": round(fl / pt / (PEAK_TFLOPS[dkey] * 1e12), 4)}


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
    ap.add_argument("--no-extra", action="store_true",
                    help="skip the further points (long context, other prompt lengths, the 7B shape)")
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
    if a.shape == "8b" and not (a.no_points or a.no_extra or a.prefill_only):
        room = max(room, 8192 + 64)          # the further points reach 8 k tokens
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
    main_point = decode_point(model, mcfg, a.batch, a.steps, a.warmup, 1, a.prompt_min, a.prompt_max)
    line = {
        "metric": f"decode tok/s @ batch {a.batch}; {shape_name} shape", "value": main_point["tok_s"],
        "unit": "tok/s", "n_gpus": 1, "steps": a.steps, "warmup": a.warmup,
        "ms_per_step": main_point["ms_per_step"], "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": dkey, "data": "synthetic",
        "config": {"model": f"{shape_name} shape, random weights N(0,0.02)",
                   "layers": layers, "layers_of_model": cfg.num_layers, "hidden": cfg.hidden,
                   "heads": cfg.num_heads, "kv_heads": cfg.num_kv_heads, "head_dim": cfg.head_dim,
                   "intermediate": cfg.intermediate, "vocab": cfg.vocab,
                   "rope_theta": cfg.rope_theta, "rms_eps": cfg.rms_eps,
                   "global_batch": a.batch, "seq_len": max(CONTEXT, a.prompt_max + a.steps + a.warmup),
                   "prompt_min": a.prompt_min, "prompt_max": a.prompt_max,
                   "mean_context": main_point["mean_context"],
                   "prefill_tokens": a.prefill_tokens, "parallelism": "single GPU",
                   "sampling": "greedy", "loop": "engine.generate.run_batches"},
        "roofline": {"bound": "hbm", "achieved": main_point["gbs"], "peak": HBM_GBS,
                     "unit": "GB/s", "frac": main_point["frac"]},
        "loop_tok_s": main_point["loop_tok_s"],
    }
    if a.probe:
        gbs = read_probe_gbs(model.device)
        line["probe"] = {"read_gbs": round(gbs, 1), "achieved_of_read": round(main_point["gbs"] / gbs, 4),
                         "what": "1 GiB read by 2048 workgroups with non-temporal loads, best of 5"}
    if not a.no_points:
        line["prefill"] = prefill_point(model, mcfg, dkey, 5, 2, tokens=a.prefill_tokens)
        # every point with what its roofline needs, flat: tokens a second under the point's
        # name, then <name>_ms (a step), _ctx (mean context), _gbs and _frac (of the HBM peak;
        # prefill points: of the matrix cores' peak)
        points = {}

        def add_decode(name, pt):
            points[name] = pt["tok_s"]
            points[name + "_ms"], points[name + "_ctx"] = pt["ms_per_step"], pt["mean_context"]
            points[name + "_gbs"], points[name + "_frac"] = pt["gbs"], pt["frac"]

        def add_prefill(name, pt):
            points[name] = pt["value"]
            points[name + "_ms"], points[name + "_tokens"], points[name + "_frac"] = pt["ms"], pt["tokens"], pt["frac"]

        few, short = max(16, a.steps // 2), max(4, a.warmup // 2)
        for b in (1, 64):
            add_decode(f"decode_b{b}", decode_point(model, mcfg, b, few, short, 3 + b, a.prompt_min, a.prompt_max))
        if not a.no_extra and a.shape == "8b":
            import numpy as np
            # a long context, short and long prompts, many short prompts in one step
            add_decode("decode_b8_ctx8k", decode_point(model, mcfg, 8, 16, 4, 11, 7000, 8000))
            add_prefill("prefill_512", prefill_point(model, mcfg, dkey, 5, 12, tokens=512))
            add_prefill("prefill_8192", prefill_point(model, mcfg, dkey, 3, 13, tokens=8192))
            mixed = [int(x) for x in np.random.default_rng(14).integers(32, 257, 16)]
            add_prefill("prefill_16_prompts_32_to_256", prefill_point(model, mcfg, dkey, 5, 14, lengths=mixed))
            # the Llama-2-7B shape (every head has keys of its own: four times the cache per token)
            del model
            torch.cuda.empty_cache()
            name7, shape7 = SHAPES["7b"]
            cfg7 = ta.LlamaConfig.from_dict(shape7)
            model = ta.random_model(cfg7, seed=0, dtype=a.dtype,
                                    num_layers=min(layers, cfg7.num_layers) if a.layers else None)
            add_decode("llama2_7b_decode_b16", decode_point(model, model.config, 16, 16, 4, 15, *PROMPTS["7b"]))
        line["points"] = points
    print(json.dumps(line))
    return 0


if __name__ == "__main__":
    sys.exit(main())
