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
