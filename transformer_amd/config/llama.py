"""Typed configuration of the Llama dense decoder.

Read from the keys of the architecture's own config.json, or from the
``llama.*`` metadata of a GGUF file with the defaults the reference applies
(models/llama/common/src/storage.rs:36-60): kv heads default
to heads (:54), head size to hidden/heads (:55), eps to 1e-5 (:58), theta to
1e4 (:59). The typed fields mirror LlamaMeta
(models/llama/common/src/lib.rs:20-40).
"""
from __future__ import annotations

import json
import math
from dataclasses import dataclass, field, asdict
from pathlib import Path
from typing import Optional, Tuple

from .spec import (AttentionSpec, BlockSpec, ConfigError, ModelSpec, NormSpec, PositionSpec,
                   RunSpec, SwiGLUSpec)

_ROPE_STYLES = ("half", "interleaved")


def _need(d: dict, key: str, typ):
    if key not in d or d[key] is None:
        raise ConfigError(f"config key '{key}' is required")
    v = d[key]
    if typ is int:
        if isinstance(v, bool) or not isinstance(v, int):
            raise ConfigError(f"config key '{key}' must be an integer, got {v!r}")
    elif typ is float:
        if isinstance(v, bool) or not isinstance(v, (int, float)):
            raise ConfigError(f"config key '{key}' must be a number, got {v!r}")
        v = float(v)
    return v


def _opt(d: dict, key: str, typ, default):
    if key not in d or d[key] is None:
        return default
    return _need(d, key, typ)


def _torch_dtype(v):
    if v is None:
        return None
    if not isinstance(v, str):
        raise ConfigError(f"torch_dtype must be a string such as \"bfloat16\", got {v!r}")
    return v[6:] if v.startswith("torch.") else v


@dataclass(frozen=True)
class LlamaConfig:
    num_layers: int
    hidden: int
    num_heads: int
    num_kv_heads: int
    head_dim: int
    intermediate: int
    vocab: int
    max_position: int
    rope_theta: float = 10000.0
    rms_eps: float = 1e-5
    rope_style: str = "half"
    tie_embeddings: Optional[bool] = None   # None: decided by the weight file
    attention_bias: bool = False
    mlp_bias: bool = False
    stop_ids: Tuple[int, ...] = field(default_factory=tuple)
    architecture: str = "LlamaForCausalLM"
    # config.json's torch_dtype: the type the checkpoint was trained or saved in. It chooses the
    # engine's type where a caller names none (float32 -> float32, anything else -> bfloat16)
    torch_dtype: Optional[str] = None

    # ------------------------------------------------------------------ checks
    def __post_init__(self):
        for name in ("num_layers", "hidden", "num_heads", "num_kv_heads", "head_dim",
                     "intermediate", "vocab", "max_position"):
            if getattr(self, name) <= 0:
                raise ConfigError(f"{name} must be positive, got {getattr(self, name)}")
        if self.num_heads % self.num_kv_heads:
            raise ConfigError(f"num_heads {self.num_heads} is not a multiple of "
                              f"num_kv_heads {self.num_kv_heads}")
        if self.head_dim % 2:
            raise ConfigError(f"head_dim {self.head_dim} must be even (rotary pairs)")
        if self.rope_style not in _ROPE_STYLES:
            raise ConfigError(f"rope_style must be one of {_ROPE_STYLES}, got {self.rope_style!r}")
        if not self.rope_theta > 0:
            raise ConfigError(f"rope_theta must be positive, got {self.rope_theta}")
        if not self.rms_eps >= 0:
            raise ConfigError(f"rms_norm_eps must be >= 0, got {self.rms_eps}")

    # ------------------------------------------------------------- config.json
    @classmethod
    def from_dict(cls, d: dict) -> "LlamaConfig":
        hidden = _need(d, "hidden_size", int)
        heads = _need(d, "num_attention_heads", int)
        if heads <= 0:
            raise ConfigError("num_attention_heads must be positive")
        act = d.get("hidden_act", "silu")
        if act != "silu":
            raise ConfigError(f"hidden_act {act!r} is not supported (only 'silu')")
        if d.get("rope_scaling") is not None:
            raise ConfigError("rope_scaling is not supported: the reference reads no "
                              "rope scaling key; set it to null")
        eos = d.get("eos_token_id")
        if eos is None:
            stops = ()
        elif isinstance(eos, int) and not isinstance(eos, bool):
            stops = (eos,)
        elif isinstance(eos, (list, tuple)) and all(isinstance(e, int) for e in eos):
            stops = tuple(eos)
        else:
            raise ConfigError(f"eos_token_id must be an integer or a list of integers, got {eos!r}")
        tie = d.get("tie_word_embeddings")
        if tie is not None and not isinstance(tie, bool):
            raise ConfigError("tie_word_embeddings must be true, false or absent")
        arch = d.get("architectures") or [d.get("model_type", "llama")]
        return cls(
            num_layers=_need(d, "num_hidden_layers", int),
            hidden=hidden,
            num_heads=heads,
            num_kv_heads=_opt(d, "num_key_value_heads", int, heads),
            head_dim=_opt(d, "head_dim", int, hidden // heads),
            intermediate=_need(d, "intermediate_size", int),
            vocab=_need(d, "vocab_size", int),
            max_position=_need(d, "max_position_embeddings", int),
            rope_theta=_opt(d, "rope_theta", float, 1e4),
            rms_eps=_opt(d, "rms_norm_eps", float, 1e-5),
            rope_style=d.get("rope_style", "half"),
            tie_embeddings=tie,
            attention_bias=bool(d.get("attention_bias", False)),
            mlp_bias=bool(d.get("mlp_bias", False)),
            stop_ids=stops,
            architecture=arch[0],
            torch_dtype=_torch_dtype(d.get("torch_dtype", d.get("dtype"))),
        )

    @classmethod
    def from_json(cls, path) -> "LlamaConfig":
        p = Path(path)
        if p.is_dir():
            p = p / "config.json"
        try:
            d = json.loads(p.read_text())
        except FileNotFoundError:
            raise ConfigError(f"no config.json at {p}") from None
        except json.JSONDecodeError as e:
            raise ConfigError(f"{p}: not valid JSON ({e})") from None
        if not isinstance(d, dict):
            raise ConfigError(f"{p}: top level must be an object")
        return cls.from_dict(d)

    def to_dict(self) -> dict:
        """The config.json this configuration is read back from."""
        d = {
            "architectures": [self.architecture],
            "model_type": "llama",
            "num_hidden_layers": self.num_layers,
            "hidden_size": self.hidden,
            "num_attention_heads": self.num_heads,
            "num_key_value_heads": self.num_kv_heads,
            "head_dim": self.head_dim,
            "intermediate_size": self.intermediate,
            "vocab_size": self.vocab,
            "max_position_embeddings": self.max_position,
            "rope_theta": self.rope_theta,
            "rms_norm_eps": self.rms_eps,
            "rope_style": self.rope_style,
            "hidden_act": "silu",
            "attention_bias": self.attention_bias,
            "mlp_bias": self.mlp_bias,
            "rope_scaling": None,
        }
        if self.tie_embeddings is not None:
            d["tie_word_embeddings"] = self.tie_embeddings
        if self.torch_dtype is not None:
            d["torch_dtype"] = self.torch_dtype
        if self.stop_ids:
            d["eos_token_id"] = list(self.stop_ids) if len(self.stop_ids) > 1 else self.stop_ids[0]
        return d

    # -------------------------------------------------------------------- GGUF
    @classmethod
    def from_gguf_metadata(cls, meta: dict, vocab_rows: Optional[int] = None) -> "LlamaConfig":
        """``meta``: GGUF key -> value. Keys and defaults as
        models/llama/common/src/storage.rs:31-60 reads them.
        The vocabulary is the length of tokenizer.ggml.tokens (:48); a file
        without a tokenizer gives the rows of token_embd.weight instead."""
        arch = meta.get("general.architecture")
        if arch is None:
            raise ConfigError("GGUF metadata key 'general.architecture' is required")

        def key(k):
            return f"{arch}.{k}"

        def need(k):
            if key(k) not in meta:
                raise ConfigError(f"GGUF metadata key '{key(k)}' is required")
            return meta[key(k)]

        hidden = int(need("embedding_length"))
        heads = int(need("attention.head_count"))
        toks = meta.get("tokenizer.ggml.tokens")
        vocab = len(toks) if toks is not None else vocab_rows
        if vocab is None:
            raise ConfigError("GGUF file has neither tokenizer.ggml.tokens nor token_embd.weight")
        eos = meta.get("tokenizer.ggml.eos_token_id")
        return cls(
            num_layers=int(need("block_count")),
            hidden=hidden,
            num_heads=heads,
            num_kv_heads=int(meta.get(key("attention.head_count_kv"), heads)),
            head_dim=int(meta.get(key("rope.dimension_count"), hidden // heads)),
            intermediate=int(need("feed_forward_length")),
            vocab=int(vocab),
            max_position=int(need("context_length")),
            rope_theta=float(meta.get(key("rope.freq_base"), 1e4)),
            rms_eps=float(meta.get(key("attention.layer_norm_rms_epsilon"), 1e-5)),
            rope_style="interleaved",
            tie_embeddings=None,
            # the reference has a qkv bias for another architecture name only (storage.rs:45)
            attention_bias=False,
            stop_ids=(int(eos),) if eos is not None else (),
            architecture=str(arch),
        )

    # ------------------------------------------------------------ model layout
    def model_spec(self) -> ModelSpec:
        """Every block spelled out; Llama's blocks are all alike."""
        position = PositionSpec(head_dim=self.head_dim, theta=self.rope_theta,
                                style=self.rope_style)
        block = BlockSpec(
            norm1=NormSpec(size=self.hidden, eps=self.rms_eps),
            mixer=AttentionSpec(hidden=self.hidden, num_heads=self.num_heads,
                                num_kv_heads=self.num_kv_heads, head_dim=self.head_dim,
                                scale=1.0 / math.sqrt(self.head_dim), position=position,
                                window=None, qkv_bias=self.attention_bias,
                                out_bias=self.attention_bias),
            norm2=NormSpec(size=self.hidden, eps=self.rms_eps),
            ffn=SwiGLUSpec(hidden=self.hidden, intermediate=self.intermediate,
                           bias=self.mlp_bias),
        )
        spec = ModelSpec(
            vocab=self.vocab, hidden=self.hidden,
            blocks=tuple(block for _ in range(self.num_layers)),
            schedule=tuple(RunSpec(block=i) for i in range(self.num_layers)),
            final_norm=NormSpec(size=self.hidden, eps=self.rms_eps),
            tie_embeddings=self.tie_embeddings, max_position=self.max_position,
            stop_ids=self.stop_ids,
        )
        spec.validate()
        return spec

    # --------------------------------------------------------------- accounting
    def default_engine_dtype(self) -> str:
        """The engine type for a caller that names none."""
        return "float32" if self.torch_dtype == "float32" else "bfloat16"

    def with_layers(self, n: int) -> "LlamaConfig":
        """The same model with its first ``n`` layers only (measurements that have to fit a
        smaller memory or time). Any typed configuration may offer this; ``random_model`` asks
        for it when a caller wants fewer layers."""
        import dataclasses
        return dataclasses.replace(self, num_layers=int(n))

    def param_count(self) -> int:
        d, nh, nkv, dh, di = self.hidden, self.num_heads, self.num_kv_heads, self.head_dim, self.intermediate
        per = (nh + 2 * nkv) * dh * d + d * nh * dh + 3 * di * d + 2 * d
        head = 0 if self.tie_embeddings else self.vocab * d
        return self.num_layers * per + self.vocab * d + d + head

    def kv_bytes_per_token(self, itemsize: int) -> int:
        return self.num_layers * 2 * self.num_kv_heads * self.head_dim * itemsize

    def flat(self) -> dict:
        return {k: v for k, v in asdict(self).items() if not isinstance(v, (tuple, list))}
