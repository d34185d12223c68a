"""The bench's accounting against the figures worked out by hand for the headline shape."""
import importlib.util
import pathlib

import transformer_amd as ta

ROOT = pathlib.Path(__file__).resolve().parent.parent
spec = importlib.util.spec_from_file_location("bench", ROOT / "bench.py")
bench = importlib.util.module_from_spec(spec)
spec.loader.exec_module(bench)


def test_prefill_flops_and_bytes_of_the_headline_shape():
    cfg = ta.LlamaConfig.from_dict(bench.LLAMA31_8B)
    assert cfg.param_count() == 8_030_261_248
    fl = bench.prefill_flops(cfg, 2048)
    assert abs(fl / 1e12 - 29.69) < 0.05
    assert cfg.kv_bytes_per_token(2) == 131072
    # weights a decode step reads: every layer matrix and norm, the output matrix, not the embedding
    d, nh, nkv, dh, di, V = 4096, 32, 8, 128, 14336, 128256
    matrices = ((nh + 2 * nkv) * dh * d + d * nh * dh + 3 * di * d) * 2
    assert matrices == 436_207_616
    # 15,009,316,864 bytes of matrices; the 65 norm vectors are float32 here (1,064,960 bytes)
    assert 32 * matrices + V * d * 2 == 15_009_316_864
    assert bench.PEAK_TFLOPS["bf16"] == 2500.0 and bench.HBM_GBS == 8000.0


def test_other_shapes_parse():
    for name, (label, shape) in bench.SHAPES.items():
        cfg = ta.LlamaConfig.from_dict(shape)
        assert cfg.head_dim == 128
    assert ta.LlamaConfig.from_dict(bench.LLAMA3_70B).param_count() == 70_553_706_496
    assert ta.LlamaConfig.from_dict(bench.LLAMA2_7B).param_count() == 6_738_415_616


import pytest


@pytest.mark.gpu
def test_the_bench_times_the_generation_loop_itself():
    """``bench.time_decode`` drives ``run_batches`` over the engine's own stepper with a clock
    added: exactly ``steps`` steps lie between its two readings, after the prompts' step and
    ``warmup`` more; the contexts it reports are the sequences' lengths half-way through."""
    import numpy as np
    import gpu_util as G
    model = G.engine("D", "bfloat16")
    cfg = model.config
    steps, warmup, batch, seed = 6, 3, 3, 5
    dt, ctx, timing = bench.time_decode(model, cfg, batch, steps, warmup, seed, prompt_min=10, prompt_max=90)
    lens = [int(x) for x in np.random.default_rng(seed).integers(10, 91, batch)]
    assert ctx == [n + warmup + steps // 2 for n in lens]
    assert timing.prefill_tokens == sum(lens)
    assert timing.decode_steps == warmup + steps + 1 and timing.decode_tokens == batch * (warmup + steps + 1)
    assert 0 < dt < timing.prefill_seconds + timing.decode_seconds
    point = bench.decode_point(model, cfg, batch, steps, warmup, seed, 10, 90)
    assert set(point) == {"tok_s", "ms_per_step", "mean_context", "gbs", "frac", "loop_tok_s"}
    assert abs(point["tok_s"] - batch * 1e3 / point["ms_per_step"]) < 0.01 * point["tok_s"]
    nbytes = bench.decode_bytes(model, cfg, ctx)
    assert abs(point["gbs"] - nbytes / (point["ms_per_step"] * 1e-3) / 1e9) < 0.02 * point["gbs"]
