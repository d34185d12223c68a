"""Helpers shared by the GPU tests: tiny configurations, model folders made with
the plain implementation's own writer, tolerances."""
import functools
import tempfile

import numpy as np

import plain_llama as P

# A third tiny configuration: every size differs from A and B, nothing is a power of two.
TINY_C = {
    "architectures": ["LlamaForCausalLM"], "model_type": "llama",
    "num_hidden_layers": 4, "hidden_size": 160, "num_attention_heads": 10,
    "num_key_value_heads": 5, "head_dim": 48, "intermediate_size": 304,
    "vocab_size": 1000, "rope_theta": 100000.0, "rms_norm_eps": 1e-4,
    "tie_word_embeddings": False, "max_position_embeddings": 512, "mlp_bias": True,
}
# The headline model's attention geometry (head size 128, four query heads per kv head) at a
# tiny width: it takes the matrix-core attention kernels, prompts through LDS included.
TINY_D = {
    "architectures": ["LlamaForCausalLM"], "model_type": "llama",
    "num_hidden_layers": 2, "hidden_size": 192, "num_attention_heads": 8,
    "num_key_value_heads": 2, "head_dim": 128, "intermediate_size": 320,
    "vocab_size": 515, "rope_theta": 500000.0, "rms_norm_eps": 1e-5,
    "tie_word_embeddings": False, "max_position_embeddings": 1024,
}
# One layer at a width where the products of 17 to 64 rows leave their result in several planes
# (the weight is cut along k among workgroups) that the next norm adds: both the norm inside
# the block and the final norm over gathered rows meet such planes.
TINY_E = {
    "architectures": ["LlamaForCausalLM"], "model_type": "llama",
    "num_hidden_layers": 1, "hidden_size": 1024, "num_attention_heads": 8,
    "num_key_value_heads": 2, "head_dim": 128, "intermediate_size": 2816,
    "vocab_size": 2000, "rope_theta": 1000000.0, "rms_norm_eps": 1e-5,
    "tie_word_embeddings": False, "max_position_embeddings": 512,
}
# One narrow layer with a long feed-forward: its down projection has k = 8,192, the length from
# which steps and prompts of more than 64 rows hand it to the library cut along k into planes.
TINY_F = {
    "architectures": ["LlamaForCausalLM"], "model_type": "llama",
    "num_hidden_layers": 1, "hidden_size": 64, "num_attention_heads": 4,
    "num_key_value_heads": 2, "head_dim": 32, "intermediate_size": 8192,
    "vocab_size": 300, "rope_theta": 10000.0, "rms_norm_eps": 1e-5,
    "tie_word_embeddings": True, "max_position_embeddings": 256,
}
CONFIGS = {"A": (P.TINY_A, 0), "B": (P.TINY_B, 1), "C": (TINY_C, 2), "D": (TINY_D, 3),
           "E": (TINY_E, 4), "F": (TINY_F, 5)}
MODES = {"float32": "F32", "bfloat16": "BF16"}

# Largest allowed |engine - plain| on logits (tiny models: logits of order 1).
# float32: accumulation-order noise is ~1e-6. bfloat16: every activation is rounded
# to 8 bits of mantissa (2^-9 relative), a few dozen roundings per token.
TOL = {"float32": 2e-5, "bfloat16": 3e-2}
# Largest allowed difference between two ways of cutting or batching the same tokens.
TOL_SPLIT = {"float32": 2e-6, "bfloat16": 2e-2}

_keep = []


@functools.lru_cache(maxsize=None)
def folder(name, dtype, edit_name=None):
    cfg, seed = CONFIGS[name]
    d = tempfile.TemporaryDirectory(prefix=f"ta_{name}_{dtype}_")
    _keep.append(d)
    P.make_model_folder(d.name, cfg, seed, storage=MODES[dtype], edit=EDITS.get(edit_name))
    return d.name


def _sharp(w):
    """Scale q and k projections so that attention is peaked: a fault in any single
    key (a far one, one at a page's edge) then moves the logits visibly."""
    for n in w:
        if n.endswith("q_proj.weight") or n.endswith("k_proj.weight"):
            w[n] *= 6.0


EDITS = {None: None, "sharp": _sharp}


@functools.lru_cache(maxsize=None)
def plain(name, dtype, edit_name=None):
    return P.PlainLlama(folder(name, dtype, edit_name))


@functools.lru_cache(maxsize=None)
def engine(name, dtype, edit_name=None):
    import transformer_amd as ta
    return ta.load_model(folder(name, dtype, edit_name), dtype, "cuda:0")


def tokens(name, n, seed):
    cfg, _ = CONFIGS[name]
    return [int(t) for t in np.random.default_rng(seed).integers(0, cfg["vocab_size"], n)]


def poison(cache):
    """Fill the cache with NaN so that a read of a row no step wrote shows."""
    for t in cache.keys + cache.values:
        t.fill_(float("nan"))
