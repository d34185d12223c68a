"""Writes a Llama model folder (safetensors names) out as one GGUF file with the
tensor names and metadata keys the reference reads
(models/llama/common/src/storage.rs:31-84).

GGUF Llama files rotate adjacent pairs (2j, 2j+1) where safetensors files rotate
(j, j + head_dim/2), so the rows of the q and k projections are reordered inside
every head: new row 2j is old row j, new row 2j+1 is old row j + head_dim/2. A
model then gives the same logits from either file. ``merged`` writes the qkv and
gate_up matrices the way the reference's conversion step leaves them
(docs/user-guide/doc.md:128-134); otherwise they stay apart.
"""
from __future__ import annotations

from pathlib import Path

import torch

from ..config.llama import LlamaConfig
from ..weights.gguf_io import write_gguf
from ..weights.safetensors_io import TensorFolder


def half_to_interleaved(w: torch.Tensor, num_heads: int, head_dim: int) -> torch.Tensor:
    """Reorders the rows (axis 0) of a q or k projection, or of its bias."""
    rest = w.shape[1:]
    v = w.reshape(num_heads, 2, head_dim // 2, *rest)       # [head, half, j, ...]
    return v.transpose(1, 2).reshape(num_heads * head_dim, *rest).contiguous()


def export_gguf(folder, out_path, merged: bool = True, norm_dtype=torch.float32) -> Path:
    folder = Path(folder)
    cfg = LlamaConfig.from_json(folder)
    if cfg.attention_bias or cfg.mlp_bias:
        raise ValueError("the reference's Llama GGUF layout has no bias tensors; this model has "
                         "attention_bias or mlp_bias set")
    f = TensorFolder(folder)
    nh, nkv, dh = cfg.num_heads, cfg.num_kv_heads, cfg.head_dim
    permute = cfg.rope_style == "half"
    meta = {
        "general.architecture": "llama",
        "general.name": folder.name,
        "llama.context_length": cfg.max_position,
        "llama.embedding_length": cfg.hidden,
        "llama.block_count": cfg.num_layers,
        "llama.feed_forward_length": cfg.intermediate,
        "llama.attention.head_count": nh,
        "llama.attention.head_count_kv": nkv,
        "llama.rope.dimension_count": dh,
        "llama.attention.layer_norm_rms_epsilon": float(cfg.rms_eps),
        "llama.rope.freq_base": float(cfg.rope_theta),
    }
    if cfg.stop_ids:
        meta["tokenizer.ggml.eos_token_id"] = int(cfg.stop_ids[0])
    out = {"token_embd.weight": f.read("model.embed_tokens.weight"),
           "output_norm.weight": f.read("model.norm.weight").to(norm_dtype)}
    if "lm_head.weight" in f:
        out["output.weight"] = f.read("lm_head.weight")
    for i in range(cfg.num_layers):
        p, b = f"model.layers.{i}.", f"blk.{i}."
        q, k, v = (f.read(p + f"self_attn.{n}_proj.weight") for n in "qkv")
        if permute:
            q, k = half_to_interleaved(q, nh, dh), half_to_interleaved(k, nkv, dh)
        out[b + "attn_norm.weight"] = f.read(p + "input_layernorm.weight").to(norm_dtype)
        out[b + "ffn_norm.weight"] = f.read(p + "post_attention_layernorm.weight").to(norm_dtype)
        gate, up = f.read(p + "mlp.gate_proj.weight"), f.read(p + "mlp.up_proj.weight")
        if merged:
            out[b + "attn_qkv.weight"] = torch.cat([q, k, v])
            out[b + "ffn_gate_up.weight"] = torch.cat([gate, up])
        else:
            out[b + "attn_q.weight"], out[b + "attn_k.weight"], out[b + "attn_v.weight"] = q, k, v
            out[b + "ffn_gate.weight"], out[b + "ffn_up.weight"] = gate, up
        out[b + "attn_output.weight"] = f.read(p + "self_attn.o_proj.weight")
        out[b + "ffn_down.weight"] = f.read(p + "mlp.down_proj.weight")
    write_gguf(out_path, meta, out)
    f.close()
    return Path(out_path)
