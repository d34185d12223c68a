"""Weights by name: one error that lists missing, unexpected and mis-shaped
tensors; storage rules; tied output; the random-weights mode."""
import json

import numpy as np
import pytest
import torch

import plain_llama as P
from transformer_amd.api import open_model_source
from transformer_amd.engine.params import declared_params
from transformer_amd.weights.loader import WeightsError, load_parameters, plan_binding
from transformer_amd.weights.random_init import write_random_model
from transformer_amd.weights.safetensors_io import (SafetensorsError, SafetensorsFile,
                                                    TensorFolder, write_safetensors)


def _rewrite(folder, change):
    w = P.read_safetensors(folder / "model.safetensors")
    change(w)
    P.write_safetensors(folder / "model.safetensors", w)


def _plan(folder):
    arch, cfg, f = open_model_source(folder)
    params = declared_params(arch.model_spec(cfg))
    return params, arch.weight_sources(cfg, f.format), f


def test_all_problems_are_listed_in_one_error(tmp_path):
    P.make_model_folder(tmp_path, P.TINY_A, 0)

    def change(w):
        del w["model.layers.1.mlp.up_proj.weight"]
        del w["model.norm.weight"]
        w["model.layers.0.self_attn.rotary_emb.inv_freq"] = np.zeros(8)
        w["model.layers.0.self_attn.k_proj.weight"] = np.zeros((16, 64))
    _rewrite(tmp_path, change)
    params, sources, f = _plan(tmp_path)
    with pytest.raises(WeightsError) as e:
        plan_binding(params, sources, f, where="tiny")
    err = e.value
    assert err.missing == ["model.layers.1.mlp.up_proj.weight", "model.norm.weight"]
    assert err.unexpected == ["model.layers.0.self_attn.rotary_emb.inv_freq"]
    assert err.wrong_shape == [("model.layers.0.self_attn.k_proj.weight", (16, 64), (32, 64))]
    for piece in ("missing", "unexpected", "wrong shapes", "up_proj", "inv_freq", "[16, 64]"):
        assert piece in str(err)


def test_untied_model_needs_its_output_matrix(tmp_path):
    P.make_model_folder(tmp_path, P.TINY_A, 0)
    _rewrite(tmp_path, lambda w: w.pop("lm_head.weight"))
    params, sources, f = _plan(tmp_path)
    with pytest.raises(WeightsError) as e:
        plan_binding(params, sources, f)
    assert e.value.missing == ["lm_head.weight"]


def test_tying_follows_the_file_when_the_config_is_silent(tmp_path):
    # models/llama/common/src/storage.rs:84
    cfg = {k: v for k, v in P.TINY_A.items() if k != "tie_word_embeddings"}
    P.make_model_folder(tmp_path, {**cfg, "tie_word_embeddings": True}, 0)
    (tmp_path / "config.json").write_text(json.dumps(cfg))
    params, sources, f = _plan(tmp_path)
    assert plan_binding(params, sources, f)["head.weight"] == ("=", "embed.weight")


def test_tied_model_tolerates_a_stored_copy(tmp_path):
    P.make_model_folder(tmp_path, P.TINY_B, 1)
    _rewrite(tmp_path, lambda w: w.__setitem__("lm_head.weight", w["model.embed_tokens.weight"]))
    params, sources, f = _plan(tmp_path)
    assert plan_binding(params, sources, f)["head.weight"] == ("=", "embed.weight")


def test_storage_rules_and_row_order(tmp_path):
    P.make_model_folder(tmp_path, P.TINY_B, 1, storage="BF16")
    params, sources, f = _plan(tmp_path)
    w = P.read_safetensors(tmp_path / "model.safetensors")
    for engine in (torch.bfloat16, torch.float32):
        t = load_parameters(params, sources, f, engine, "cpu")
        assert t["blocks.0.mixer.qkv.weight"].dtype == engine          # matrix: engine dtype
        assert t["blocks.0.norm1.weight"].dtype == torch.float32       # vector: stays 32-bit
        assert t["blocks.0.mixer.qkv.bias"].dtype == torch.float32
        assert t["head.weight"] is t["embed.weight"]                   # one buffer when tied
        qkv = t["blocks.2.mixer.qkv.weight"].double().numpy()
        want = np.concatenate([w[f"model.layers.2.self_attn.{n}_proj.weight"] for n in "qkv"])
        assert np.array_equal(qkv, want)                               # q rows, k rows, v rows
        gu = t["blocks.1.ffn.gate_up.weight"].double().numpy()
        want = np.concatenate([w["model.layers.1.mlp.gate_proj.weight"],
                               w["model.layers.1.mlp.up_proj.weight"]])
        assert np.array_equal(gu, want)                                # gate rows, up rows


def test_a_matrix_stored_in_32_bits_stays_so(tmp_path):
    """A bfloat16 engine does not narrow what its file holds in 32 bits: such a matrix stays
    float32 (and is multiplied as it is); one stored in bfloat16 is never widened either."""
    P.make_model_folder(tmp_path, P.TINY_A, 0, storage="F32")
    params, sources, f = _plan(tmp_path)
    w = P.read_safetensors(tmp_path / "model.safetensors")
    with pytest.warns(UserWarning, match="10 matrices are stored in 32 bits"):       # and it says so
        t = load_parameters(params, sources, f, torch.bfloat16, "cpu")
    assert t["blocks.0.mixer.qkv.weight"].dtype == torch.float32
    assert t["embed.weight"].dtype == torch.float32 and t["blocks.1.norm2.weight"].dtype == torch.float32
    assert np.array_equal(t["blocks.1.ffn.down.weight"].double().numpy(), w["model.layers.1.mlp.down_proj.weight"])
    # one 32-bit matrix among bfloat16 ones: only that one stays wide
    (tmp_path / "m").mkdir()
    (tmp_path / "m" / "config.json").write_text((tmp_path / "config.json").read_text())
    one = "model.layers.0.mlp.down_proj.weight"
    P.write_safetensors(tmp_path / "m" / "model.safetensors", w,
                        {n: ("F32" if n == one or a.ndim == 1 else "BF16") for n, a in w.items()})
    params, sources, f = _plan(tmp_path / "m")
    with pytest.warns(UserWarning, match=r"1 matrices .*first: blocks\.0\.ffn\.down\.weight"):
        t = load_parameters(params, sources, f, torch.bfloat16, "cpu")
    assert t["blocks.0.ffn.down.weight"].dtype == torch.float32
    assert t["blocks.1.ffn.down.weight"].dtype == torch.bfloat16
    assert t["blocks.0.mixer.qkv.weight"].dtype == torch.bfloat16


def test_random_weights_mode_writes_a_loadable_folder(tmp_path):
    a = write_random_model(tmp_path / "a", P.TINY_A, seed=5, storage="bfloat16")
    b = write_random_model(tmp_path / "b", P.TINY_A, seed=5, storage="bfloat16")
    c = write_random_model(tmp_path / "c", P.TINY_A, seed=6, storage="bfloat16")
    assert (a / "config.json").exists() and (a / "model.safetensors").exists()
    fa, fb, fc = (SafetensorsFile(x / "model.safetensors") for x in (a, b, c))
    n = "model.layers.1.mlp.down_proj.weight"
    assert torch.equal(fa.read(n), fb.read(n)) and not torch.equal(fa.read(n), fc.read(n))
    assert fa.dtype(n) == torch.bfloat16 and fa.dtype("model.norm.weight") == torch.float32
    assert abs(float(fa.read(n).float().std()) - 0.02) < 0.002
    assert abs(float(fa.read("model.norm.weight").mean()) - 1.0) < 0.05
    params, sources, f = _plan(a)
    plan_binding(params, sources, f)                                    # every tensor fits
    m = P.PlainLlama(a)                                                 # and the plain model reads it
    assert np.isfinite(m.forward([1, 2, 3])).all()
    tied = write_random_model(tmp_path / "t", P.TINY_B, seed=1, storage="float32")
    assert "lm_head.weight" not in SafetensorsFile(tied / "model.safetensors").entries


def test_safetensors_round_trip_and_errors(tmp_path):
    t = {"a": torch.randn(3, 5), "b": torch.randn(4).to(torch.bfloat16),
         "c": torch.arange(6, dtype=torch.int32).reshape(2, 3)}
    write_safetensors(tmp_path / "model.safetensors", t)
    f = TensorFolder(tmp_path)
    for k, v in t.items():
        assert torch.equal(f.read(k), v) and f.dtype(k) == v.dtype
    (tmp_path / "bad.safetensors").write_bytes(b"\xff" * 6)
    with pytest.raises(SafetensorsError):
        SafetensorsFile(tmp_path / "bad.safetensors")
    with pytest.raises(SafetensorsError, match="neither"):
        TensorFolder(tmp_path / "nothing")


def test_sharded_folder(tmp_path):
    a = {"x": torch.randn(2, 2)}
    b = {"y": torch.randn(3)}
    write_safetensors(tmp_path / "model-00001-of-00002.safetensors", a)
    write_safetensors(tmp_path / "model-00002-of-00002.safetensors", b)
    (tmp_path / "model.safetensors.index.json").write_text(json.dumps(
        {"weight_map": {"x": "model-00001-of-00002.safetensors",
                        "y": "model-00002-of-00002.safetensors"}}))
    f = TensorFolder(tmp_path)
    assert sorted(f.names()) == ["x", "y"] and torch.equal(f.read("y"), b["y"])


def test_all_parameters_lie_in_one_allocation_on_aligned_offsets(tmp_path):
    from transformer_amd.weights.loader import ALIGN, plan_placement
    P.make_model_folder(tmp_path, P.TINY_B, 1, storage="BF16")
    params, sources, f = _plan(tmp_path)
    chosen = plan_binding(params, sources, f)
    place, total = plan_placement(params, chosen, f, torch.bfloat16)
    assert "head.weight" not in place                       # shared with the embedding: no room of its own
    spans = sorted((off, off + int(np.prod(params[n].shape)) * (2 if dt == torch.bfloat16 else 4))
                   for n, (off, dt) in place.items())
    assert all(a % ALIGN == 0 for a, _ in spans) and spans[-1][1] <= total
    assert all(e <= a for (_, e), (a, _) in zip(spans, spans[1:]))          # no overlap
    t = load_parameters(params, sources, f, torch.bfloat16, "cpu", chunk_bytes=4096)
    base = {x.untyped_storage().data_ptr() for x in t.values()}
    assert len(base) == 1
    for n, (off, dt) in place.items():
        assert t[n].dtype == dt and t[n].data_ptr() - next(iter(base)) == off and t[n].is_contiguous()


def test_a_saved_model_is_the_file_it_was_loaded_from(tmp_path):
    """Parameters that were joined by rows are cut back into the file's tensors, a shared
    output matrix is not written: save(load(folder)) holds the same tensors, bit by bit."""
    from transformer_amd.weights.save import save_model_folder
    for cfg, seed in ((P.TINY_A, 0), (P.TINY_B, 1)):
        src_dir, dst_dir = tmp_path / f"s{seed}", tmp_path / f"d{seed}"
        P.make_model_folder(src_dir, cfg, seed, storage="BF16")
        params, sources, f = _plan(src_dir)
        t = load_parameters(params, sources, f, torch.bfloat16, "cpu")
        arch, typed, _ = open_model_source(src_dir)
        save_model_folder(dst_dir, typed.to_dict(), t, params, sources)
        g = TensorFolder(dst_dir)
        assert set(g.names()) == set(f.names())
        for n in f.names():
            assert g.dtype(n) == f.dtype(n) and torch.equal(g.read(n), f.read(n)), n
        # and the plain implementation reads the saved folder as it reads the first
        a, b = P.PlainLlama(src_dir), P.PlainLlama(dst_dir)
        toks = [1, 5, 9, 2]
        assert np.array_equal(a.forward(toks), b.forward(toks))


def test_parts_say_how_their_parameters_are_drawn():
    arch, cfg = __import__("transformer_amd").get_architecture("llama"), None
    cfg = arch.config_from_dict(P.TINY_B)
    params = declared_params(arch.model_spec(cfg))
    assert params["blocks.0.norm1.weight"].init == "around_one"
    assert params["final_norm.weight"].init == "around_one"
    assert params["blocks.0.mixer.qkv.bias"].init == "normal"
    assert params["blocks.0.ffn.down.weight"].init == "normal"
