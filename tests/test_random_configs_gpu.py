"""Randomly drawn tiny configurations (seeded): head sizes in steps of 16 up to 256, any number of
heads and of query heads per kv head, widths, feed-forward sizes and vocabularies that are odd or no
power of two, with and without biases, both rotation pairings, tied and untied output. Each is
loaded in float32 and in bfloat16 and compared with the plain implementation: a batch of unequal
prompts in one step, then six single tokens each. A size that a kernel cannot take has to be refused
with an error, never answered wrongly; none of these is refused."""
import tempfile

import numpy as np
import pytest

import gpu_util as G
import plain_llama as P

pytestmark = pytest.mark.gpu


def _draw(case):
    r = np.random.default_rng(case)
    dh = int(r.choice([16, 32, 48, 64, 80, 96, 112, 128, 160, 192, 256]))
    nkv = int(r.choice([1, 2, 3, 5]))
    group = int(r.choice([1, 2, 3, 4, 7, 16, 20] if dh <= 64 else [1, 2, 4, 5]))
    cfg = {"architectures": ["LlamaForCausalLM"], "model_type": "llama",
           "num_hidden_layers": int(r.integers(1, 4)),
           "hidden_size": int(r.choice([40, 72, 100, 136, 264, 520, 34, 50, 66, 130, 33, 257])),
           "num_attention_heads": nkv * group, "num_key_value_heads": nkv, "head_dim": dh,
           "intermediate_size": int(r.choice([56, 120, 200, 344, 30, 57, 129, 1030])),
           "vocab_size": int(r.choice([97, 300, 1001, 2050, 5, 33000])),
           "rope_theta": float(r.choice([1e4, 5e5])), "rms_norm_eps": float(r.choice([1e-6, 1e-5, 1e-3])),
           "tie_word_embeddings": bool(r.integers(0, 2)), "max_position_embeddings": 512,
           "attention_bias": bool(r.integers(0, 2)), "mlp_bias": bool(r.integers(0, 2))}
    if r.integers(0, 2):
        cfg["rope_style"] = "interleaved"
    lens = {dtype: [int(x) for x in r.integers(1, 150, size=int(r.integers(1, 6)))] for dtype in G.MODES}
    return cfg, lens, r


@pytest.mark.parametrize("first", [1000, 1008, 1016])
def test_random_configurations_against_the_plain_model(first):
    import transformer_amd as ta
    for case in range(first, first + 8):
        cfg, lens_of, r = _draw(case)
        for dtype in G.MODES:
            with tempfile.TemporaryDirectory(prefix="ta_rand_") as d:
                P.make_model_folder(d, cfg, case, storage=G.MODES[dtype])
                ref = P.PlainLlama(d)
                model = ta.load_model(d, dtype, "cuda:0")
            lens = lens_of[dtype]
            toks = [[int(t) for t in r.integers(0, cfg["vocab_size"], size=n + 6)] for n in lens]
            cache = model.new_cache(64 * sum(-(-(n + 6) // 64) for n in lens), max_slots=len(lens))
            G.poison(cache)
            slots = [cache.alloc_slot() for _ in lens]
            want = [ref.forward(t) for t in toks]
            what = f"case {case} {dtype} {cfg} prompts {lens}"
            got = model.step(cache, [ta.Entry(s, t[:n], [n - 1]) for s, t, n in zip(slots, toks, lens)])
            got = got.float().cpu().numpy()
            for i, n in enumerate(lens):
                assert np.abs(got[i] - want[i][n - 1]).max() < G.TOL[dtype], what
            for j in range(6):
                got = model.step(cache, [ta.Entry(s, [t[n + j]], [0]) for s, t, n in zip(slots, toks, lens)])
                got = got.float().cpu().numpy()
                for i, n in enumerate(lens):
                    assert np.abs(got[i] - want[i][n + j]).max() < G.TOL[dtype], (what, j)
            for s in slots:
                cache.free_slot(s)
            cache.pool.check()
