"""The Llama dense decoder as a registry entry: its configuration, its blocks
and where its parameters are found in a weight file.

safetensors names are the architecture's own (``model.layers.N.self_attn.q_proj``
and so on); q/k/v and gate/up are stored apart there and are joined by rows into
the merged matrices in the reference's order: q heads, k heads, v heads
(models/llama/common/src/lib.rs:132-137, compute.rs:227) and gate
rows, up rows (lib.rs:154-157, compute.rs:286).

GGUF names are the ones the reference reads
(models/llama/common/src/storage.rs:32-34, :63-78, :84):
``blk.N.attn_qkv`` and ``blk.N.ffn_gate_up`` already merged by its conversion
step (docs/user-guide/doc.md:128-140), or the unmerged ``attn_q/k/v`` and
``ffn_gate/up`` that the conversion starts from. The output matrix falls back
to the embedding table when the file has none (storage.rs:84).
"""
from __future__ import annotations

from typing import Dict

from ..config.llama import LlamaConfig
from ..config.registry import Architecture, register_architecture
from ..weights.loader import Piece, Source


def _one(name, shape, **kw):
    return Source(options=((Piece(name, tuple(shape)),),), **kw)


def llama_weight_sources(cfg: LlamaConfig, file_format: str) -> Dict[str, Source]:
    d, nh, nkv, dh, di, V = (cfg.hidden, cfg.num_heads, cfg.num_kv_heads, cfg.head_dim,
                             cfg.intermediate, cfg.vocab)
    nq, nk = nh * dh, nkv * dh
    src: Dict[str, Source] = {}
    if file_format == "safetensors":
        src["embed.weight"] = _one("model.embed_tokens.weight", (V, d))
        src["final_norm.weight"] = _one("model.norm.weight", (d,))
        head = (Piece("lm_head.weight", (V, d)),)
        if cfg.tie_embeddings is True:
            src["head.weight"] = Source(options=(), stand_in="embed.weight",
                                        ignored=("lm_head.weight",))
        elif cfg.tie_embeddings is False:
            src["head.weight"] = Source(options=(head,))
        else:
            src["head.weight"] = Source(options=(head,), stand_in="embed.weight")
        for i in range(cfg.num_layers):
            f, p = f"model.layers.{i}.", f"blocks.{i}."
            src[p + "norm1.weight"] = _one(f + "input_layernorm.weight", (d,))
            src[p + "norm2.weight"] = _one(f + "post_attention_layernorm.weight", (d,))
            src[p + "mixer.qkv.weight"] = Source(options=((
                Piece(f + "self_attn.q_proj.weight", (nq, d)),
                Piece(f + "self_attn.k_proj.weight", (nk, d)),
                Piece(f + "self_attn.v_proj.weight", (nk, d))),))
            src[p + "mixer.out.weight"] = _one(f + "self_attn.o_proj.weight", (d, nq))
            src[p + "ffn.gate_up.weight"] = Source(options=((
                Piece(f + "mlp.gate_proj.weight", (di, d)),
                Piece(f + "mlp.up_proj.weight", (di, d))),))
            src[p + "ffn.down.weight"] = _one(f + "mlp.down_proj.weight", (d, di))
            if cfg.attention_bias:
                src[p + "mixer.qkv.bias"] = Source(options=((
                    Piece(f + "self_attn.q_proj.bias", (nq,)),
                    Piece(f + "self_attn.k_proj.bias", (nk,)),
                    Piece(f + "self_attn.v_proj.bias", (nk,))),))
                src[p + "mixer.out.bias"] = _one(f + "self_attn.o_proj.bias", (d,))
            if cfg.mlp_bias:
                src[p + "ffn.gate_up.bias"] = Source(options=((
                    Piece(f + "mlp.gate_proj.bias", (di,)),
                    Piece(f + "mlp.up_proj.bias", (di,))),))
                src[p + "ffn.down.bias"] = _one(f + "mlp.down_proj.bias", (d,))
        return src
    if file_format == "gguf":
        src["embed.weight"] = _one("token_embd.weight", (V, d))
        src["final_norm.weight"] = _one("output_norm.weight", (d,))
        src["head.weight"] = Source(options=((Piece("output.weight", (V, d)),),),
                                    stand_in="embed.weight")
        for i in range(cfg.num_layers):
            f, p = f"blk.{i}.", f"blocks.{i}."
            src[p + "norm1.weight"] = _one(f + "attn_norm.weight", (d,))
            src[p + "norm2.weight"] = _one(f + "ffn_norm.weight", (d,))
            src[p + "mixer.qkv.weight"] = Source(options=(
                (Piece(f + "attn_qkv.weight", (nq + 2 * nk, d)),),
                (Piece(f + "attn_q.weight", (nq, d)), Piece(f + "attn_k.weight", (nk, d)),
                 Piece(f + "attn_v.weight", (nk, d)))))
            src[p + "mixer.out.weight"] = _one(f + "attn_output.weight", (d, nq))
            src[p + "ffn.gate_up.weight"] = Source(options=(
                (Piece(f + "ffn_gate_up.weight", (2 * di, d)),),
                (Piece(f + "ffn_gate.weight", (di, d)), Piece(f + "ffn_up.weight", (di, d)))))
            src[p + "ffn.down.weight"] = _one(f + "ffn_down.weight", (d, di))
            if cfg.attention_bias:
                src[p + "mixer.qkv.bias"] = Source(options=(
                    (Piece(f + "attn_qkv.bias", (nq + 2 * nk,)),),
                    (Piece(f + "attn_q.bias", (nq,)), Piece(f + "attn_k.bias", (nk,)),
                     Piece(f + "attn_v.bias", (nk,)))))
                src[p + "mixer.out.bias"] = _one(f + "attn_output.bias", (d,))
        return src
    raise ValueError(f"unknown weight file format {file_format!r}")


LLAMA = Architecture(
    name="LlamaForCausalLM",
    config_from_dict=LlamaConfig.from_dict,
    config_from_gguf=LlamaConfig.from_gguf_metadata,
    model_spec=lambda cfg: cfg.model_spec(),
    weight_sources=llama_weight_sources,
)

register_architecture(LLAMA, "llama")
