"""Another architecture, added from outside the framework's files: a toy decoder defined in
this test (a typed configuration with config.json keys of its own, blocks that differ from
layer to layer, a schedule that names a block twice, a part after the embedding, its own
tensor names in the weight file) is registered, drawn, saved, loaded by the name in its
config.json, stepped, generated from and replayed by the engine's own loader, cache, step
function, generation loop and replayer. Nothing under ``transformer_amd/`` knows it.
It is no model of anyone's: even layers read a window of keys, odd layers all of them, the
embedding is scaled, and the last block runs twice."""
import dataclasses
import json
import math
from dataclasses import dataclass
from typing import Optional

import numpy as np
import pytest

import plain_llama as P

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
NAME = "ToyWindowDecoder"


@dataclass(frozen=True)
class ToyConfig:
    n_layer: int
    d_model: int
    n_head: int
    n_kv: int
    d_head: int
    d_ff: int
    n_vocab: int
    n_ctx: int
    window: int
    embed_scale: float
    eps: float = 1e-5
    theta: float = 1000.0
    tie_embeddings: Optional[bool] = True      # the output matrix is always the embedding table
    torch_dtype: Optional[str] = None

    @classmethod
    def from_dict(cls, d):
        keys = {f.name for f in dataclasses.fields(cls)} - {"tie_embeddings"}
        return cls(**{k: d[k] for k in keys if k in d})

    def to_dict(self):
        d = {k: v for k, v in dataclasses.asdict(self).items() if k != "tie_embeddings" and v is not None}
        return {"architectures": [NAME], **d}

    def with_layers(self, n):
        return dataclasses.replace(self, n_layer=n)

    def default_engine_dtype(self):
        return "float32" if self.torch_dtype == "float32" else "bfloat16"


@dataclass(frozen=True)
class EmbedScaleSpec:
    factor: float
    kind: str = "toy_embed_scale"


def _model_spec(c: ToyConfig):
    from transformer_amd.config.spec import (AttentionSpec, BlockSpec, ModelSpec, NormSpec, PositionSpec,
                                             RunSpec, SwiGLUSpec)
    blocks = tuple(
        BlockSpec(norm1=NormSpec(c.d_model, c.eps),
                  mixer=AttentionSpec(c.d_model, c.n_head, c.n_kv, c.d_head, 1 / math.sqrt(c.d_head),
                                      PositionSpec(c.d_head, c.theta, "interleaved"),
                                      window=c.window if i % 2 == 0 else None),
                  norm2=NormSpec(c.d_model, c.eps), ffn=SwiGLUSpec(c.d_model, c.d_ff))
        for i in range(c.n_layer))
    schedule = tuple(RunSpec(i) for i in range(c.n_layer)) + (RunSpec(c.n_layer - 1),)   # the last block twice
    return ModelSpec(vocab=c.n_vocab, hidden=c.d_model, blocks=blocks, schedule=schedule,
                     final_norm=NormSpec(c.d_model, c.eps), tie_embeddings=True, max_position=c.n_ctx,
                     after_embed=EmbedScaleSpec(c.embed_scale))


def _weight_sources(c: ToyConfig, file_format: str):
    from transformer_amd.weights.loader import Piece, Source
    assert file_format == "safetensors"

    def one(name, *shape):
        return Source(options=((Piece(name, tuple(shape)),),))

    width = (c.n_head + 2 * c.n_kv) * c.d_head
    src = {"embed.weight": one("tok.weight", c.n_vocab, c.d_model), "final_norm.weight": one("ln_f", c.d_model),
           "head.weight": Source(options=(), stand_in="embed.weight")}
    for i in range(c.n_layer):
        src[f"blocks.{i}.norm1.weight"] = one(f"h.{i}.ln1", c.d_model)
        src[f"blocks.{i}.norm2.weight"] = one(f"h.{i}.ln2", c.d_model)
        src[f"blocks.{i}.mixer.qkv.weight"] = one(f"h.{i}.attn.wqkv", width, c.d_model)     # stored merged
        src[f"blocks.{i}.mixer.out.weight"] = one(f"h.{i}.attn.wo", c.d_model, c.n_head * c.d_head)
        src[f"blocks.{i}.ffn.gate_up.weight"] = one(f"h.{i}.ff.w13", 2 * c.d_ff, c.d_model)
        src[f"blocks.{i}.ffn.down.weight"] = one(f"h.{i}.ff.w2", c.d_model, c.d_ff)
    return src


def _register():
    import transformer_amd as ta
    from transformer_amd.config.registry import Architecture
    from transformer_amd.parts.base import Part

    class EmbedScale(Part):
        graph_safe = True

        def __init__(self, spec, dtype, device):
            self.factor = spec.factor

        def run(self, x, ctx):
            x.mul_(self.factor)

    ta.register_part("toy_embed_scale", EmbedScale)
    ta.register_architecture(Architecture(name=NAME, config_from_dict=ToyConfig.from_dict, config_from_gguf=None,
                                          model_spec=_model_spec, weight_sources=_weight_sources), "toy_window")


CFG = {"architectures": [NAME], "n_layer": 3, "d_model": 96, "n_head": 6, "n_kv": 2, "d_head": 32, "d_ff": 136,
       "n_vocab": 211, "n_ctx": 512, "window": 40, "embed_scale": 3.0, "eps": 1e-4}


def plain_forward(w, c: ToyConfig, tokens, rounded):
    """The toy decoder out of the plain functions: whole sequence, no cache."""
    r = P.round_bf16 if rounded else (lambda a: a)
    T = len(tokens)
    pos = np.arange(T)
    x = w["tok.weight"][np.asarray(tokens)] * c.embed_scale
    for i in [*range(c.n_layer), c.n_layer - 1]:
        p = f"h.{i}."
        h = r(P.rms_norm(x, w[p + "ln1"], c.eps))
        qkv = r(P.linear(h, w[p + "attn.wqkv"])).reshape(T, c.n_head + 2 * c.n_kv, c.d_head)
        q = r(P.rope(qkv[:, :c.n_head], pos, c.theta, "interleaved"))
        k = r(P.rope(qkv[:, c.n_head:c.n_head + c.n_kv], pos, c.theta, "interleaved"))
        o = r(P.attention(q, k, qkv[:, c.n_head + c.n_kv:], 1 / math.sqrt(c.d_head),
                          window=c.window if i % 2 == 0 else None))
        x = x + P.linear(o.reshape(T, -1), w[p + "attn.wo"])
        h = r(P.rms_norm(x, w[p + "ln2"], c.eps))
        gu = r(P.linear(h, w[p + "ff.w13"]))
        x = x + P.linear(r(P.swiglu(gu[:, :c.d_ff], gu[:, c.d_ff:])), w[p + "ff.w2"])
    return P.linear(r(P.rms_norm(x, w["ln_f"], c.eps)), w["tok.weight"])


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_toy_architecture_goes_through_the_whole_engine(dtype, tmp_path):
    import transformer_amd as ta
    from transformer_amd import Entry
    from transformer_amd.engine.generate import generate
    from transformer_amd.replay import Replayer
    from transformer_amd.weights.loader import WeightsError
    _register()
    assert NAME in ta.known_architectures()
    # drawn on the GPU, written under the architecture's own names, loaded back by config.json
    drawn = ta.random_model(CFG, seed=3, dtype=dtype, architecture=NAME, std=0.05)
    folder = tmp_path / "toy"
    ta.save_model(drawn, folder)
    said = json.loads((folder / "config.json").read_text())
    assert said["architectures"] == [NAME] and said["window"] == 40 and "num_hidden_layers" not in said
    w = P.read_safetensors(folder / "model.safetensors")
    assert "h.2.attn.wqkv" in w and "tok.weight" in w and not any(n.startswith("model.") for n in w)
    model = ta.load_model(folder, dtype)
    cfg = model.config
    assert type(cfg).__name__ == "ToyConfig" and model.architecture.name == NAME
    assert model.w["head"].data_ptr() == model.w["embed"].data_ptr()              # tied by the architecture
    # four schedule entries, four cache layers in two groups (a window, everything)
    cache = model.new_cache(1024, max_slots=3)
    assert len(model.cache_needs) == 4 and [n.window for n in cache.kv_groups] == [40, None]
    for t in cache.keys + cache.values:
        t.fill_(float("nan"))
    rng = np.random.default_rng(8)
    a = [int(t) for t in rng.integers(0, cfg.n_vocab, 150)]
    b = [int(t) for t in rng.integers(0, cfg.n_vocab, 47)]
    want_a, want_b = (plain_forward(w, cfg, t, dtype == "bfloat16") for t in (a, b))
    tol = (2e-5 if dtype == "float32" else 3e-2) * max(1.0, np.abs(want_a).max())      # relative to the logits' size
    f64 = lambda t: t.float().cpu().numpy().astype(np.float64)   # noqa: E731
    sa, sb = cache.alloc_slot(), cache.alloc_slot()
    whole = f64(model.step(cache, [Entry(sa, a, range(150))]))
    assert np.abs(whole - want_a).max() < tol
    # the model that was drawn and the one that was loaded from its file are the same model
    other = drawn.new_cache(256, max_slots=1)
    again = f64(drawn.step(other, [Entry(other.alloc_slot(), a, range(150))]))
    assert np.array_equal(again, whole)
    cache.reset_slot(sa)
    # unequal prompts together, then single tokens (recorded steps); the shorter one ends earlier
    got_a, got_b = [], []
    out = f64(model.step(cache, [Entry(sa, a[:90], range(90)), Entry(sb, b[:20], range(20))]))
    got_a.append(out[:90]); got_b.append(out[90:])
    for i in range(60):
        es = [Entry(sa, [a[90 + i]], [0])] + ([Entry(sb, [b[20 + i]], [0])] if 20 + i < len(b) else [])
        out = f64(model.step(cache, es))
        got_a.append(out[:1])
        if len(es) == 2:
            got_b.append(out[1:])
    assert model._graph_safe and cache.graphs                     # the toy's own part is recorded too
    assert np.abs(np.concatenate(got_a) - want_a).max() < tol
    assert np.abs(np.concatenate(got_b) - want_b).max() < tol
    cache.pool.check()
    # the generation loop: greedy tokens are the plain model's (float32), in batches of two
    prompts = [a[:30], b[:11], a[40:47]]
    res = generate(model, prompts, max_new_tokens=5, stop_ids=[], max_batch=2)
    assert [len(t) for t in res.tokens] == [5, 5, 5] and res.batches == [[0, 1], [2]]
    if dtype == "float32":
        for p, got in zip(prompts, res.tokens):
            seq = list(p)
            for t in got:
                assert t == int(np.argmax(plain_forward(w, cfg, seq, False)[-1]))
                seq.append(t)
    # the replayer drives the same model
    rep = Replayer(model, 512, tmp_path / "trace")
    rep.run([json.dumps({"step": 0, "entries": [{"id": "x", "tokens": a[:70], "want": [0, 69]}], "end": []}),
             json.dumps({"step": 1, "entries": [{"id": "x", "tokens": [a[70]], "want": [0]}], "end": ["x"]})],
            report=open(tmp_path / "done.txt", "w"))
    first = np.fromfile(tmp_path / "trace" / "0.f32", dtype="<f4").reshape(2, -1)
    second = np.fromfile(tmp_path / "trace" / "1.f32", dtype="<f4").reshape(1, -1)
    assert np.abs(first - want_a[[0, 69]]).max() < tol and np.abs(second - want_a[70]).max() < tol
    # a file that lacks a tensor and holds a stranger is refused with both named
    from safetensors.torch import load_file, save_file
    t = load_file(str(folder / "model.safetensors"))
    t["h.9.odd"] = t.pop("h.1.ff.w2")
    bad = tmp_path / "bad"
    bad.mkdir()
    save_file(t, str(bad / "model.safetensors"))
    (bad / "config.json").write_text((folder / "config.json").read_text())
    with pytest.raises(WeightsError) as e:
        ta.load_model(bad, dtype)
    assert e.value.missing == ["h.1.ff.w2"] and e.value.unexpected == ["h.9.odd"]
    # fewer layers through the configuration's own with_layers
    short = ta.random_model(CFG, seed=3, dtype=dtype, architecture=NAME, num_layers=1)
    assert len(short.blocks) == 1 and len(short.spec.schedule) == 2
