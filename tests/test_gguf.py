"""GGUF: the container, the metadata keys the reference reads, tensor names merged
and apart, and the row order that makes both rotary pairings agree."""
import numpy as np
import pytest
import torch

import plain_llama as P
from transformer_amd.api import open_model_source
from transformer_amd.engine.params import declared_params
from transformer_amd.architectures.llama_gguf_export import export_gguf, half_to_interleaved
from transformer_amd.weights.gguf_io import GGUFError, GGUFFile, write_gguf
from transformer_amd.weights.loader import WeightsError, load_parameters, plan_binding


def test_container_round_trip(tmp_path):
    meta = {"general.architecture": "llama", "llama.block_count": 3, "x.flag": True,
            "x.eps": 1e-5, "x.names": ["a", "bc"], "x.ids": [1, 2, 3], "x.big": 2 ** 40}
    t = {"a.weight": torch.randn(3, 5), "b.weight": torch.randn(7).to(torch.bfloat16),
         "c.weight": torch.randn(2, 3, 4).to(torch.float16)}
    write_gguf(tmp_path / "m.gguf", meta, t)
    f = GGUFFile(tmp_path / "m.gguf")
    assert f.metadata["llama.block_count"] == 3 and f.metadata["x.flag"] is True
    assert abs(f.metadata["x.eps"] - 1e-5) < 1e-12 and f.metadata["x.names"] == ["a", "bc"]
    assert f.metadata["x.ids"] == [1, 2, 3] and f.metadata["x.big"] == 2 ** 40
    for k, v in t.items():
        assert f.shape(k) == tuple(v.shape) and torch.equal(f.read(k), v)
    (tmp_path / "bad.gguf").write_bytes(b"GGML" + b"\0" * 40)
    with pytest.raises(GGUFError, match="not a GGUF"):
        GGUFFile(tmp_path / "bad.gguf")


def test_half_to_interleaved_is_the_pairing_change():
    dh, nh = 8, 2
    w = torch.arange(nh * dh, dtype=torch.float32).reshape(nh * dh, 1)
    p = half_to_interleaved(w, nh, dh)[:, 0].tolist()
    assert p[:8] == [0, 4, 1, 5, 2, 6, 3, 7] and p[8:] == [8, 12, 9, 13, 10, 14, 11, 15]
    # rotating the reordered rows interleaved equals reordering the rows rotated by halves
    rng = np.random.default_rng(0)
    t = rng.normal(size=(3, nh, dh))
    pos = [0, 5, 9]
    a = P.rope(t, pos, 1e4, "half")
    tp = half_to_interleaved(torch.tensor(t).permute(1, 2, 0).reshape(nh * dh, 3), nh, dh)
    b = P.rope(tp.reshape(nh, dh, 3).permute(2, 0, 1).numpy(), pos, 1e4, "interleaved")
    ap = half_to_interleaved(torch.tensor(a).permute(1, 2, 0).reshape(nh * dh, 3), nh, dh)
    assert np.allclose(b, ap.reshape(nh, dh, 3).permute(2, 0, 1).numpy())


@pytest.mark.parametrize("merged", [True, False])
def test_exported_file_binds_with_the_references_names(tmp_path, merged):
    P.make_model_folder(tmp_path / "st", P.TINY_A, 0, storage="BF16")
    path = export_gguf(tmp_path / "st", tmp_path / "m.gguf", merged=merged)
    arch, cfg, f = open_model_source(path)
    assert arch.name == "LlamaForCausalLM" and cfg.rope_style == "interleaved"
    assert (cfg.num_layers, cfg.hidden, cfg.num_kv_heads, cfg.head_dim, cfg.vocab) == (2, 64, 2, 16, 256)
    assert cfg.rope_theta == 10000.0 and abs(cfg.rms_eps - 1e-5) < 1e-9 and cfg.max_position == 128
    names = set(f.names())
    assert ("blk.0.attn_qkv.weight" in names) == merged and ("blk.0.attn_q.weight" in names) != merged
    params = declared_params(arch.model_spec(cfg))
    t = load_parameters(params, arch.weight_sources(cfg, "gguf"), f, torch.float32, "cpu")
    st = P.read_safetensors(tmp_path / "st" / "model.safetensors")
    qkv = t["blocks.1.mixer.qkv.weight"].double().numpy()
    assert np.array_equal(qkv[64 + 32:], st["model.layers.1.self_attn.v_proj.weight"])      # v rows last
    q = half_to_interleaved(torch.tensor(st["model.layers.1.self_attn.q_proj.weight"]), 4, 16).numpy()
    assert np.array_equal(qkv[:64], q)
    assert t["blocks.0.norm1.weight"].dtype == torch.float32
    assert t["head.weight"] is not t["embed.weight"]


def test_gguf_problems_are_listed(tmp_path):
    tied = {**P.TINY_B, "attention_bias": False}
    P.make_model_folder(tmp_path / "st", tied, 1)                       # tied: no output.weight
    path = export_gguf(tmp_path / "st", tmp_path / "m.gguf", merged=False)
    f = GGUFFile(path)
    tensors = {n: f.read(n).clone() for n in f.names()}
    del tensors["blk.2.ffn_up.weight"]
    tensors["blk.0.attn_k.weight"] = tensors["blk.0.attn_k.weight"][:8]
    tensors["rope_freqs.weight"] = torch.zeros(4)
    write_gguf(tmp_path / "broken.gguf", f.metadata, tensors)
    arch, cfg, g = open_model_source(tmp_path / "broken.gguf")
    assert cfg.attention_bias is False                                  # GGUF Llama has no biases
    params = declared_params(arch.model_spec(cfg))
    with pytest.raises(WeightsError) as e:
        plan_binding(params, arch.weight_sources(cfg, "gguf"), g)
    # the merged name is the canonical one, so that is what is reported as missing
    assert e.value.missing == ["blk.2.ffn_gate_up.weight"]
    assert e.value.unexpected == ["rope_freqs.weight"]
    assert e.value.wrong_shape == [("blk.0.attn_k.weight", (8, 96), (96, 96))]
    # the tied output falls back to the embedding table
    ok = plan_binding(params, arch.weight_sources(cfg, "gguf"), GGUFFile(path))
    assert ok["head.weight"] == ("=", "embed.weight")


def test_quantised_tensors_are_refused(tmp_path):
    import struct
    P.make_model_folder(tmp_path / "st", P.TINY_A, 0)
    path = export_gguf(tmp_path / "st", tmp_path / "m.gguf")
    raw = bytearray(path.read_bytes())
    key = b"blk.0.attn_output.weight"
    at = raw.index(key) + len(key) + 4 + 16           # after n_dims (u32) and two dims (u64)
    assert struct.unpack_from("<I", raw, at)[0] == 0  # F32
    struct.pack_into("<I", raw, at, 2)                # pretend it is a 4-bit block type
    (tmp_path / "q.gguf").write_bytes(bytes(raw))
    arch, cfg, f = open_model_source(tmp_path / "q.gguf")
    params = declared_params(arch.model_spec(cfg))
    with pytest.raises(WeightsError, match="unsupported dtypes"):
        plan_binding(params, arch.weight_sources(cfg, "gguf"), f)
